"""MoE expert path through the C ABI against the oracle (reference dispatch order)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def rel_err(y, ref):
    return float(np.abs(y.astype(np.float64) - ref).max() / np.abs(ref).max())


def test_route_matches_reference_softmax_topk(O, tfq, gpu):
    import torch
    T, E, K = 16, 8, 2
    logits = O.rng_normal(45, T * E, 1.0).reshape(T, E)
    probs, idx, w = O.softmax_topk(logits, K)
    p_d, i_d, w_d = tfq.moe_route(torch.from_numpy(logits).to(gpu), K)
    assert np.array_equal(i_d.cpu().numpy().astype(np.int64), idx)
    assert np.abs(p_d.cpu().numpy() - probs).max() <= 2e-7
    assert np.abs(w_d.cpu().numpy() - w).max() <= 2e-7
    # closed form: rows sum to one, weights are the k largest probabilities, not renormalised
    pn = p_d.cpu().numpy()
    assert np.abs(pn.sum(axis=1) - 1).max() < 1e-6
    assert np.allclose(np.sort(pn, axis=1)[:, ::-1][:, :K], w_d.cpu().numpy(), atol=0, rtol=0)
    # k is clamped into 1..E like the reference does
    assert tfq.moe_route(torch.from_numpy(logits).to(gpu), 99)[1].shape == (T, E)


@pytest.mark.parametrize("T,E,K", [(1, 3, 2), (5, 64, 6), (16, 130, 8), (3, 257, 8), (7, 1024, 4), (2, 1100, 3)])
def test_route_many_experts_and_ties(O, tfq, gpu, T, E, K):
    """Expert counts around the wavefront width and the limit of the one-wavefront-per-token kernel (1100 experts take
    the one-lane form), against the oracle; and logits with exact duplicates: equal probabilities are picked in
    ascending expert order, the k picks of a token are distinct, and the weights are the picked probabilities."""
    import torch
    logits = O.rng_normal(70 + E, T * E, 1.0).reshape(T, E)
    probs, idx, w = O.softmax_topk(logits, K)
    p_d, i_d, w_d = tfq.moe_route(torch.from_numpy(logits).to(gpu), K)
    assert np.array_equal(i_d.cpu().numpy().astype(np.int64), idx)
    assert np.abs(p_d.cpu().numpy() - probs).max() <= 2e-7
    assert np.abs(w_d.cpu().numpy() - w).max() <= 2e-7
    tied = logits.copy()
    tied[:, 1::2] = tied[:, 0::2][:, :tied[:, 1::2].shape[1]]  # every odd expert repeats the even one before it
    probs, idx, w = O.softmax_topk(tied, K)
    p_d, i_d, w_d = tfq.moe_route(torch.from_numpy(tied).to(gpu), K)
    i_n, p_n, w_n = i_d.cpu().numpy().astype(np.int64), p_d.cpu().numpy(), w_d.cpu().numpy()
    assert np.array_equal(i_n, idx)
    for t in range(T):
        assert len(set(i_n[t].tolist())) == K
        assert np.array_equal(p_n[t, i_n[t]], w_n[t])
        order = sorted(range(E), key=lambda e: (-p_n[t, e], e))[:K]
        assert order == i_n[t].tolist()


@pytest.mark.parametrize("xdt", ["f32", "bf16"])
def test_router_linear_then_route(O, tfq, gpu, xdt):
    """tfq_moe_router: logits = x . Wr^T + b (float64 numpy as the check, 1e-5 of the largest logit), then the
    route of those very logits equals the oracle's softmax_topk of them."""
    import torch
    T, D, E, K = 16, 4096, 8, 2
    x = O.rng_normal(43, T * D, 1.0).reshape(T, D)
    if xdt == "bf16":
        x = O.bf16_round(x)
    Wr = O.rng_normal(46, E * D, 0.05).reshape(E, D)
    b = O.rng_normal(47, E, 0.1)
    xd = torch.from_numpy(x).to(gpu)
    if xdt == "bf16":
        xd = xd.bfloat16()
    logits, probs, idx, w = tfq.moe_router(xd, torch.from_numpy(Wr).to(gpu), K, bias=torch.from_numpy(b).to(gpu))
    ref = x.astype(np.float64) @ Wr.astype(np.float64).T + b
    got = logits.cpu().numpy()
    assert np.abs(got - ref).max() <= 1e-5 * np.abs(ref).max()
    p_ref, i_ref, w_ref = O.softmax_topk(got, K)
    assert np.array_equal(idx.cpu().numpy().astype(np.int64), i_ref)
    assert np.abs(probs.cpu().numpy() - p_ref).max() <= 2e-7
    assert np.abs(w.cpu().numpy() - w_ref).max() <= 2e-7


def _experts(O, tfq, fmt, E, D, F, seed):
    gate, up, down, hg, hu, hd = [], [], [], [], [], []
    for e in range(E):
        for lst, hst, n, k, off in ((gate, hg, F, D, 0), (up, hu, F, D, 1), (down, hd, D, F, 2)):
            pay = O.encode_tensor(fmt, O.rng_normal(seed + 10 * e + off, n * k, 0.02))
            hst.append(pay)
            lst.append(tfq.Weight(fmt, n, k, pay))
    return gate, up, down, hg, hu, hd


@pytest.mark.parametrize("fmt", ["Q_G_4", "B32S4"])
@pytest.mark.parametrize("xdt,mid_bf16,tol", [("bf16", True, 1e-2), ("f32", False, 1e-3)])
def test_moe_ffn_small(O, tfq, gpu, fmt, xdt, mid_bf16, tol):
    """8 experts, top-2, 16 tokens: the Mixtral-style configuration at reduced width."""
    import torch
    E, Ktop, T, D, F = 8, 2, 16, 512, 1024
    gate, up, down, hg, hu, hd = _experts(O, tfq, fmt, E, D, F, 300)
    logits = O.rng_normal(45, T * E, 1.0).reshape(T, E)
    _, idx, w = O.softmax_topk(logits, Ktop)
    x = O.rng_normal(43, T * D, 1.0).reshape(T, D)
    if xdt == "bf16":
        x = O.bf16_round(x)
        xt = torch.from_numpy(x).to(gpu).bfloat16()
    else:
        xt = torch.from_numpy(x).to(gpu)
    ref = O.moe_ffn(fmt, hg, hu, hd, D, F, idx, w, x, mid_bf16=mid_bf16)
    y = tfq.moe_ffn(gate, up, down, idx, w, xt, mid_dtype=torch.bfloat16 if mid_bf16 else torch.float32).cpu().numpy()
    assert rel_err(y, ref) <= tol
    # invariants: every (token, slot) pair is dispatched once; weights in (0, 1]
    assert sum((idx == e).sum() for e in range(E)) == T * Ktop and np.all((w > 0) & (w <= 1))
    # an expert nobody routes to, a dropped (non-positive) weight and an out-of-range id are skipped
    idx2, w2 = idx.copy(), w.copy()
    idx2[idx2 == 3] = 5
    w2[0, 0] = 0.0
    idx2[1, 1] = 99
    for t in range(T):  # keep the two slots of a token distinct
        if idx2[t, 0] == idx2[t, 1]:
            idx2[t, 1] = (idx2[t, 0] + 1) % E if (idx2[t, 0] + 1) % E != 3 else (idx2[t, 0] + 2) % E
    ref2 = O.moe_ffn(fmt, hg, hu, hd, D, F, idx2, w2, x, mid_bf16=mid_bf16)
    y2 = tfq.moe_ffn(gate, up, down, idx2, w2, xt, mid_dtype=torch.bfloat16 if mid_bf16 else torch.float32).cpu().numpy()
    assert rel_err(y2, ref2) <= tol
    yb = tfq.moe_ffn(gate, up, down, idx, w, xt, out_dtype=torch.bfloat16,
                     mid_dtype=torch.bfloat16 if mid_bf16 else torch.float32).float().cpu().numpy()
    assert rel_err(yb, ref) <= 1e-2
    for wl in gate + up + down:
        wl.close()


@pytest.mark.parametrize("fmt", ["B32S4", "Q_G_8", "Q_G_3"])
def test_moe_ffn_skewed_routing(O, tfq, gpu, fmt):
    """One expert takes most tokens (more rows than one pass of the GEMV carries, so its rows are cut into
    chunks), some experts take none; formats with the grouped launch and one without it."""
    import torch
    E, Ktop, T, D, F = 6, 2, 24, 512, 1024
    gate, up, down, hg, hu, hd = _experts(O, tfq, fmt, E, D, F, 700)
    logits = O.rng_normal(46, T * E, 1.0).reshape(T, E)
    logits[:, 2] += 6.0      # every token picks expert 2 first
    logits[:, 4] -= 20.0     # nobody picks expert 4
    _, idx, w = O.softmax_topk(logits, Ktop)
    assert (idx == 2).sum() == T and (idx == 4).sum() == 0
    x = O.bf16_round(O.rng_normal(43, T * D, 1.0).reshape(T, D))
    ref = O.moe_ffn(fmt, hg, hu, hd, D, F, idx, w, x, mid_bf16=True)
    y = tfq.moe_ffn(gate, up, down, idx, w, torch.from_numpy(x).to(gpu).bfloat16(), mid_dtype=torch.bfloat16).cpu().numpy()
    assert rel_err(y, ref) <= 1e-2
    ref32 = O.moe_ffn(fmt, hg, hu, hd, D, F, idx, w, x, mid_bf16=False)
    y32 = tfq.moe_ffn(gate, up, down, idx, w, torch.from_numpy(x).to(gpu), mid_dtype=torch.float32).cpu().numpy()
    assert rel_err(y32, ref32) <= 1e-3
    for wl in gate + up + down:
        wl.close()


@pytest.mark.parametrize("fmt,xdt,mid_bf16,tol", [("B32S4", "bf16", True, 1e-2), ("Q_G_8", "bf16", True, 1e-2),
                                                  ("Q_G_4", "f32", False, 1e-3)])
def test_moe_ffn_many_tokens_per_expert(O, tfq, gpu, fmt, xdt, mid_bf16, tol):
    """A prefill-sized call: 200 tokens over 4 experts, top-2, so every expert holds far more than 16 rows and
    the expert products go through the prefill entry (the matrix-core GEMM for bf16 rows)."""
    import torch
    E, Ktop, T, D, F = 4, 2, 200, 256, 512
    gate, up, down, hg, hu, hd = _experts(O, tfq, fmt, E, D, F, 700)
    logits = O.rng_normal(46, T * E, 1.0).reshape(T, E)
    _, idx, w = O.softmax_topk(logits, Ktop)
    assert min((idx == e).sum() for e in range(E)) > 32
    x = O.rng_normal(47, T * D, 1.0).reshape(T, D)
    if xdt == "bf16":
        x = O.bf16_round(x)
        xt = torch.from_numpy(x).to(gpu).bfloat16()
    else:
        xt = torch.from_numpy(x).to(gpu)
    ref = O.moe_ffn(fmt, hg, hu, hd, D, F, idx, w, x, mid_bf16=mid_bf16)
    y = tfq.moe_ffn(gate, up, down, idx, w, xt, mid_dtype=torch.bfloat16 if mid_bf16 else torch.float32).cpu().numpy()
    assert rel_err(y, ref) <= tol
    for W in gate + up + down:
        W.close()


@pytest.mark.parametrize("fmt", ["B32S4", "Q_G_8", "Q_G_3"])
def test_moe_ffn_prefill_sized_with_uneven_experts(O, tfq, gpu, fmt):
    """A prefill-sized call (bf16 rows and mid activations: the experts' products are grouped launches of the
    matrix-core tile kernel) in which one expert holds hundreds of rows (two token tiles), others a few dozen, one
    a handful and one none."""
    import torch
    E, Ktop, T, D, F = 6, 2, 300, 256, 512
    gate, up, down, hg, hu, hd = _experts(O, tfq, fmt, E, D, F, 1300)
    logits = O.rng_normal(54, T * E, 1.0).reshape(T, E)
    logits[:, 1] += 6.0      # every token picks expert 1 first: 300 rows
    logits[:, 4] -= 20.0     # nobody picks expert 4
    logits[:, 5] -= 3.5      # a handful pick expert 5
    _, idx, w = O.softmax_topk(logits, Ktop)
    counts = [int((idx == e).sum()) for e in range(E)]
    assert counts[1] == T and counts[4] == 0 and 0 < counts[5] <= 16, counts
    x = O.bf16_round(O.rng_normal(55, T * D, 1.0).reshape(T, D))
    ref = O.moe_ffn(fmt, hg, hu, hd, D, F, idx, w, x, mid_bf16=True)
    y = tfq.moe_ffn(gate, up, down, idx, w, torch.from_numpy(x).to(gpu).bfloat16(), mid_dtype=torch.bfloat16).cpu().numpy()
    assert rel_err(y, ref) <= 1e-2
    for W in gate + up + down:
        W.close()


@pytest.mark.parametrize("fmt", ["B32S4", "B32S8"])
def test_moe_ffn_long_down_rows_five_to_sixteen(O, tfq, gpu, fmt):
    """Experts with five to sixteen tokens and a down product too long for their staged rows (K = 5120: twenty
    block columns, so some wavefronts of the sixteen-row kernel own two): bf16 mid activations take the grouped
    sixteen-row launch, which reads every down matrix once; fp32 mid activations keep the two-row passes."""
    import torch
    E, Ktop, T, D, F = 4, 2, 18, 256, 5120
    gate, up, down, hg, hu, hd = _experts(O, tfq, fmt, E, D, F, 900)
    logits = O.rng_normal(48, T * E, 1.0).reshape(T, E)
    logits[:, 3] -= 20.0  # three experts share the tokens: twelve each
    _, idx, w = O.softmax_topk(logits, Ktop)
    counts = [int((idx == e).sum()) for e in range(E)]
    assert counts[3] == 0 and min(counts[:3]) > 4 and max(counts) <= 16, counts
    x = O.bf16_round(O.rng_normal(49, T * D, 1.0).reshape(T, D))
    ref = O.moe_ffn(fmt, hg, hu, hd, D, F, idx, w, x, mid_bf16=True)
    y = tfq.moe_ffn(gate, up, down, idx, w, torch.from_numpy(x).to(gpu).bfloat16(), mid_dtype=torch.bfloat16).cpu().numpy()
    assert rel_err(y, ref) <= 1e-2
    ref32 = O.moe_ffn(fmt, hg, hu, hd, D, F, idx, w, x, mid_bf16=False)
    y32 = tfq.moe_ffn(gate, up, down, idx, w, torch.from_numpy(x).to(gpu).bfloat16(), mid_dtype=torch.float32).cpu().numpy()
    assert rel_err(y32, ref32) <= 1e-3
    for wl in gate + up + down:
        wl.close()


@pytest.mark.parametrize("fmt,D,F,T", [("B32S4", 256, 6144, 20), ("B32S4", 768, 6400, 20), ("Q_G_4", 512, 6144, 20),
                                       ("B32S8", 256, 6144, 20), ("Q_G_8", 512, 6144, 20), ("B32S4", 512, 6144, 24),
                                       ("B32S4", 256, 6144, 40)])
def test_moe_ffn_tall_gate_up_with_five_to_eight_rows(O, tfq, gpu, fmt, D, F, T):
    """Gate / up matrices with thousands of rows and experts of five to eight tokens: enough tiles for the grouped
    launch whose wavefronts own whole tiles (a workgroup per compute unit, twelve tile pairs or more each), at one,
    two and three block columns.  Host-side and device-side routing, against the oracle.  With 24 and 40 tokens
    some experts hold nine to seventeen rows: their rows go in chunks of eight (9 and 13 problems), and the
    wavefronts take more tile pairs each so that the workgroups still fit one round."""
    import torch
    E, Ktop = 8, 2
    gate, up, down, hg, hu, hd = _experts(O, tfq, fmt, E, D, F, 1100)
    logits = O.rng_normal(52, T * E, 1.0).reshape(T, E)
    _, idx, w = O.softmax_topk(logits, Ktop)
    counts = [int((idx == e).sum()) for e in range(E)]
    assert 4 < max(counts) and (T > 20 or max(counts) <= 8), counts
    x = O.bf16_round(O.rng_normal(53, T * D, 1.0).reshape(T, D))
    ref = O.moe_ffn(fmt, hg, hu, hd, D, F, idx, w, x, mid_bf16=True)
    xt = torch.from_numpy(x).to(gpu).bfloat16()
    y = tfq.moe_ffn(gate, up, down, idx, w, xt, mid_dtype=torch.bfloat16)
    assert rel_err(y.cpu().numpy(), ref) <= 1e-2
    routed = tfq.RoutedMoe(gate, up, down, T, Ktop)
    yr = torch.empty(T, D, device=gpu)
    routed(torch.from_numpy(idx.astype(np.int32)).to(gpu), torch.from_numpy(w.astype(np.float32)).to(gpu), xt, yr)
    assert rel_err(yr.cpu().numpy(), ref) <= 1e-2
    assert float((yr - y).abs().max()) <= 1e-5 * float(y.abs().max())
    for wl in gate + up + down:
        wl.close()


@pytest.mark.parametrize("fmt", ["B32S4", "Q_G_8"])
def test_moe_ffn_routed_builds_its_lists_on_the_device(O, tfq, gpu, fmt):
    """tfq_moe_ffn_routed: routing arrays stay on the device, lists and launch tables are built there.  Skewed
    routing (an expert with more rows than one pass, an expert with none, a slot whose id is out of range) against
    the oracle and against tfq_moe_ffn with the same routing on the host."""
    import torch
    E, Ktop, T, D, F = 6, 2, 24, 512, 1024
    gate, up, down, hg, hu, hd = _experts(O, tfq, fmt, E, D, F, 800)
    logits = O.rng_normal(50, T * E, 1.0).reshape(T, E)
    logits[:, 2] += 6.0      # every token picks expert 2 first: 24 rows, three passes of eight
    logits[:, 4] -= 20.0     # nobody picks expert 4
    _, idx, w = O.softmax_topk(logits, Ktop)
    idx = idx.copy()
    idx[5, 1] = E + 3        # an id outside 0..E-1: the slot is skipped
    x = O.bf16_round(O.rng_normal(51, T * D, 1.0).reshape(T, D))
    ref = O.moe_ffn(fmt, hg, hu, hd, D, F, idx, w, x, mid_bf16=True)
    xt = torch.from_numpy(x).to(gpu).bfloat16()
    host = tfq.moe_ffn(gate, up, down, idx, w, xt, mid_dtype=torch.bfloat16)
    routed = tfq.RoutedMoe(gate, up, down, T, Ktop)
    y = torch.empty(T, D, device=gpu)
    routed(torch.from_numpy(idx.astype(np.int32)).to(gpu), torch.from_numpy(w.astype(np.float32)).to(gpu), xt, y)
    assert rel_err(y.cpu().numpy(), ref) <= 1e-2
    assert float((y - host).abs().max()) <= 1e-5 * float(host.abs().max())
    for wl in gate + up + down:
        wl.close()


@pytest.mark.parametrize("fmt,D,F", [("B32S4", 512, 1024), ("Q_G_4", 256, 768), ("B32S8", 256, 512), ("Q_G_8", 512, 512), ("B32S4", 4096, 14336)])
def test_moe_ffn_routed_single_token(O, tfq, gpu, fmt, D, F):
    """One token, top-2: the routed call is two launches that look the slots' experts up themselves and add the
    weighted down products into y with atomics.  Against the oracle (the small shapes), against the host-list
    call bit for bit, and with the irregular slots: an id outside 0..E-1, a weight that is not positive, both
    slots naming one expert, no slot with an expert at all (y = 0); ten calls in a row give the same bits."""
    import torch
    E, Ktop, T = 8, 2, 1
    small = D * F <= 1 << 20
    if small:
        gate, up, down, hg, hu, hd = _experts(O, tfq, fmt, E, D, F, 1500)
    else:
        gen = torch.Generator(device="cuda").manual_seed(3)
        gate, up, down = [], [], []
        for e in range(E):
            for lst, n, k in ((gate, F, D), (up, F, D), (down, D, F)):
                lst.append(tfq.Weight(fmt, n, k, tfq.encode(fmt, torch.randn(n * k, device=gpu, generator=gen) * 0.02)))
    x = O.bf16_round(O.rng_normal(57, T * D, 1.0).reshape(T, D))
    xt = torch.from_numpy(x).to(gpu).bfloat16()
    routed = tfq.RoutedMoe(gate, up, down, T, Ktop)
    cases = [([3, 6], [0.7, 0.3]), ([5, 0], [0.25, 0.75]), ([2, E + 1], [0.6, 0.4]), ([-1, 4], [0.5, 0.5]),
             ([1, 7], [0.0, 1.0]), ([4, 4], [0.6, 0.4]), ([-1, E + 2], [0.5, 0.5])]
    for ids, wts in cases:
        idx = np.array([ids], np.int64)
        w = np.array([wts], np.float32)
        host = tfq.moe_ffn(gate, up, down, idx, w, xt, mid_dtype=torch.bfloat16)
        y = torch.full((T, D), 7.0, device=gpu)
        di, dw = torch.from_numpy(idx.astype(np.int32)).to(gpu), torch.from_numpy(w).to(gpu)
        routed(di, dw, xt, y)
        assert torch.equal(y, host), (ids, wts, float((y - host).abs().max()))
        if not any(0 <= i < E for i in ids):
            assert float(y.abs().max()) == 0.0
        if small and ids[0] != ids[1] and any(0 <= i < E for i in ids):
            ref = O.moe_ffn(fmt, hg, hu, hd, D, F, idx, w, x, mid_bf16=True)
            assert rel_err(y.cpu().numpy(), ref) <= 1e-2
        for _ in range(10):
            y2 = torch.full((T, D), -3.0, device=gpu)
            routed(di, dw, xt, y2)
            assert torch.equal(y2, y)
    for wl in gate + up + down:
        wl.close()


@pytest.mark.parametrize("T,Ktop,E", [(1, 1, 3), (7, 3, 5), (64, 2, 4), (128, 8, 16), (5, 2, 40)])
def test_moe_ffn_routed_shapes(O, tfq, gpu, T, Ktop, E):
    """Call shapes of the routed form: one pair, odd counts, experts with several passes of eight and sixteen
    rows, the largest call it takes (1024 pairs), more experts than pairs.  Against tfq_moe_ffn with the same
    routing read back to the host (which cuts the rows into passes by its own rules: equal to rounding, or to the
    bf16 tolerance where it takes the prefill GEMM)."""
    import torch
    fmt, D, F = "B32S4", 256, 512
    gate, up, down, _, _, _ = _experts(O, tfq, fmt, E, D, F, 840)
    logits = torch.from_numpy(O.rng_normal(53, T * E, 1.0).reshape(T, E)).to(gpu)
    _, idx, w = tfq.moe_route(logits, Ktop)
    xt = torch.from_numpy(O.rng_normal(54, T * D, 1.0).reshape(T, D)).to(gpu).bfloat16()
    host = tfq.moe_ffn(gate, up, down, idx.cpu().numpy().astype(np.int64), w.cpu().numpy(), xt, mid_dtype=torch.bfloat16)
    y = torch.empty(T, D, device=gpu)
    tfq.RoutedMoe(gate, up, down, T, Ktop)(idx, w, xt, y)
    # with more than 32 rows on an expert the host-list call multiplies through the prefill GEMM, whose weights are
    # rounded to bf16; the routed call always takes the decode kernels
    counts = [int((idx == e).sum()) for e in range(E)]
    tol = 1e-2 if max(counts) > 32 else 1e-5
    assert float((y - host).abs().max()) <= tol * float(host.abs().max())
    for wl in gate + up + down:
        wl.close()


def test_moe_ffn_routed_refuses_what_it_does_not_serve(O, tfq, gpu):
    """More than 1024 pairs, or a format without the grouped kernels: no workspace size, and the call fails."""
    gate, up, down, _, _, _ = _experts(O, tfq, "B32S4", 2, 256, 512, 860)
    with pytest.raises(tfq.TfqError):
        tfq.RoutedMoe(gate, up, down, 600, 2)
    g3, u3, d3, _, _, _ = _experts(O, tfq, "Q_G_3", 2, 256, 512, 870)
    with pytest.raises(tfq.TfqError):
        tfq.RoutedMoe(g3, u3, d3, 4, 2)
    for wl in gate + up + down + g3 + u3 + d3:
        wl.close()


def test_moe_ffn_routed_in_a_graph(O, tfq, gpu):
    """The routed call captured into a graph together with the router: replays with other activations (hence other
    routing) equal the eager calls bit for bit, with eager work and synchronizations between the replays."""
    import torch
    fmt, E, Ktop, T, D, F = "B32S4", 8, 2, 16, 512, 1536
    gate, up, down, _, _, _ = _experts(O, tfq, fmt, E, D, F, 820)
    Wr = torch.from_numpy(O.rng_normal(52, E * D, 0.05).reshape(E, D).astype(np.float32)).to(gpu)
    routed = tfq.RoutedMoe(gate, up, down, T, Ktop)
    xs = [torch.from_numpy(O.rng_normal(60 + i, T * D, 1.0).reshape(T, D).astype(np.float32)).to(gpu).bfloat16() for i in range(4)]
    x = xs[0].clone()
    y = torch.zeros(T, D, device=gpu)

    def step():
        _, _, idx, wts = tfq.moe_router(x, Wr, Ktop)
        routed(idx, wts, x, y)
        return idx

    step()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        step()
    seen = set()
    for i in (1, 2, 3, 0, 2):
        x.copy_(xs[i])
        g.replay()
        torch.cuda.synchronize()
        got = y.clone()
        y.zero_()
        idx = step()
        torch.cuda.synchronize()
        seen.add(tuple(idx.cpu().numpy().reshape(-1).tolist()))
        assert torch.equal(got, y), i
    assert len(seen) >= 3  # the replays really saw different routing
    for wl in gate + up + down:
        wl.close()


def test_moe_single_token_equals_plain_mlp(O, tfq, gpu):
    """One token, one expert, weight 1: the MoE path reduces to the SwiGLU MLP step."""
    import torch
    fmt, D, F = "B32S4", 512, 768
    gate, up, down, hg, hu, hd = _experts(O, tfq, fmt, 1, D, F, 500)
    x = O.bf16_round(O.rng_normal(7, D, 1.0).reshape(1, D))
    xt = torch.from_numpy(x).to(gpu).bfloat16()
    y = tfq.moe_ffn(gate, up, down, np.zeros((1, 1), np.int64), np.ones((1, 1), np.float32), xt,
                    mid_dtype=torch.float32).cpu().numpy()
    g = O.matmul(fmt, hg[0], F, D, x)
    u = O.matmul(fmt, hu[0], F, D, x)
    want = O.matmul(fmt, hd[0], D, F, O.silu_mul(g, u))
    assert rel_err(y, want) <= 1e-3
    for wl in gate + up + down:
        wl.close()


def test_config5_mixtral_layer_full_size(tfq, gpu):
    """8 experts, top-2, 16 tokens, gate/up 14336x4096 and down 4096x14336, B32S4 weights from
    N(0, 0.02), bf16 activations: checked against a dense torch evaluation of the same decoded
    weights (the oracle takes minutes at this size), plus conservation under weight scaling."""
    import torch
    E, Ktop, T, D, F = 8, 2, 16, 4096, 14336
    g = torch.Generator(device="cuda").manual_seed(5)
    gate, up, down = [], [], []
    for e in range(E):
        for lst, n, k in ((gate, F, D), (up, F, D), (down, D, F)):
            w = torch.randn(n * k, device=gpu, generator=g) * 0.02
            lst.append(tfq.Weight("B32S4", n, k, tfq.encode("B32S4", w)))
            del w
    logits = torch.randn(T, E, device=gpu, generator=g)
    _, idx, wts = tfq.moe_route(logits, Ktop)
    idx_h, w_h = idx.cpu().numpy().astype(np.int64), wts.cpu().numpy()
    x = torch.randn(T, D, device=gpu, generator=g).bfloat16()
    y = tfq.moe_ffn(gate, up, down, idx_h, w_h, x, mid_dtype=torch.bfloat16)
    want = torch.zeros(T, D, device=gpu, dtype=torch.float64)
    xf = x.double()
    for e in range(E):
        toks = [t for t in range(T) if e in idx_h[t]]
        if not toks:
            continue
        Wg, Wu, Wd = gate[e].decode().double(), up[e].decode().double(), down[e].decode().double()
        xe = xf[toks]
        gg, uu = (xe @ Wg.T).float(), (xe @ Wu.T).float()
        h = (gg / (1 + torch.exp(-gg)) * uu).bfloat16().double()
        o = h @ Wd.T
        for i, t in enumerate(toks):
            want[t] += float(w_h[t][list(idx_h[t]).index(e)]) * o[i]
        del Wg, Wu, Wd
    err = float((y.double() - want).abs().max() / want.abs().max())
    assert err <= 1e-2, err
    # linear in the routing weights: doubling them doubles the output exactly (power of two)
    y2 = tfq.moe_ffn(gate, up, down, idx_h, 2 * w_h, x, mid_dtype=torch.bfloat16)
    assert torch.equal(y2, 2 * y)
    for wl in gate + up + down:
        wl.close()


@pytest.mark.parametrize("fmt", ["B32S4", "Q_G_4", "Q_G_8", "Q_G_6"])
@pytest.mark.parametrize("B,xdt,mid", [(1, "f32", "f32"), (3, "bf16", "bf16"), (16, "bf16", "bf16"), (20, "bf16", "f32")])
def test_mlp_step_matches_the_oracle(O, tfq, gpu, fmt, B, xdt, mid):
    """Dense SwiGLU feed-forward (Qwen35Engine::mlp_step): y = down(silu(gate x) * (up x)) against the oracle's
    block-row matmuls and silu step; formats with and without the multi-matrix kernel, decode and prefill row counts."""
    import torch
    D, F = 512, 768
    print(f"mlp_step {fmt} B={B} {xdt} mid={mid}", flush=True)
    pays = [O.encode_tensor(fmt, O.rng_normal(70 + i, n * k, 0.02)) for i, (n, k) in enumerate(((F, D), (F, D), (D, F)))]
    x = O.rng_normal(9, B * D, 1.0).reshape(B, D)
    if xdt == "bf16":
        x = O.bf16_round(x)
    g = O.matmul(fmt, pays[0], F, D, x)
    u = O.matmul(fmt, pays[1], F, D, x)
    h = O.silu_mul(g.reshape(-1), u.reshape(-1)).reshape(B, F)
    if mid == "bf16":
        h = O.bf16_round(h)
    want = O.matmul(fmt, pays[2], D, F, h)
    Ws = [tfq.Weight(fmt, n, k, p) for p, (n, k) in zip(pays, ((F, D), (F, D), (D, F)))]
    xt = torch.from_numpy(x).to(gpu)
    if xdt == "bf16":
        xt = xt.bfloat16()
    y = tfq.mlp_step(Ws[0], Ws[1], Ws[2], xt, mid_dtype=torch.bfloat16 if mid == "bf16" else torch.float32).cpu().numpy()
    tol = 1e-3 if xdt == "f32" and mid == "f32" else 1e-2
    assert float(np.abs(y - want).max()) <= tol * float(np.abs(want).max())
    for W in Ws:
        W.close()


def test_capacity_dispatch_matches_oracle(O, tfq, gpu):
    """moe_engine::plan_dispatch / gather / combine (engines/trainer/moe/dispatch.cpp:9-78) through the C ABI."""
    import torch
    fmt, E, D, F, T, K, slots = "B32S4", 4, 1024, 2048, 16, 2, 5
    gate, up, down, hg, hu, hd = _experts(O, tfq, fmt, E, D, F, 900)
    x = O.rng_normal(11, T * D, 1.0).reshape(T, D)
    rng = np.random.default_rng(12)
    idx = rng.integers(0, E, size=(T, K)).astype(np.int32)
    w = rng.standard_normal((T, K)).astype(np.float32)
    # the plan alone: the library's host-side lists equal the oracle's
    for a, b in zip(tfq.moe_plan_dispatch(idx, w, E, slots), O.moe_plan_dispatch(idx, w, E, slots)):
        assert np.array_equal(a, b)
    ref, nd_ref = O.moe_ffn_capacity(fmt, hg, hu, hd, D, F, idx, w, slots, x)
    y, nd = tfq.moe_ffn_capacity(gate, up, down, idx, w, slots, torch.from_numpy(x).to(gpu), mid_dtype=torch.float32)
    assert nd == nd_ref and nd > 0
    assert rel_err(y.cpu().numpy(), ref) <= 1e-3
    # bf16 activations and intermediate
    xb = O.bf16_round(x)
    refb, _ = O.moe_ffn_capacity(fmt, hg, hu, hd, D, F, idx, w, slots, xb, mid_bf16=True)
    yb, _ = tfq.moe_ffn_capacity(gate, up, down, idx, w, slots, torch.from_numpy(xb).to(gpu).bfloat16(), out_dtype=torch.float32)
    assert rel_err(yb.cpu().numpy(), refb) <= 1e-2
    # an expert id outside 0..E-1 is an error, as in the reference
    bad = idx.copy()
    bad[0, 0] = E
    with pytest.raises(tfq.TfqError):
        tfq.moe_ffn_capacity(gate, up, down, bad, w, slots, torch.from_numpy(x).to(gpu))
