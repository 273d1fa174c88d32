"""The persistent chain of dependent matrix-vector products (tfq_chain_*) against the oracle.

The oracle side is a composition of pinned pieces: O.matmul (block-row GEMV in the reference's loop order),
O.silu_mul (src/math/math.cpp:117-126) and O.rmsnorm (Qwen35Engine::rmsnorm,
src/adapters/tools/qwen35_engine.cpp:46-51); activations are rounded to bf16 before
every product, as the chain does.  Tolerance: max |y - y_ref| / max |y_ref| <= 1e-2 (bf16 activations).
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def rel_err(y, ref):
    return float(np.abs(y.astype(np.float64) - ref).max() / np.abs(ref).max())


def _weights(O, tfq, fmt, shapes, seed):
    out = {}
    for i, (name, N, K) in enumerate(shapes):
        pay = O.encode_tensor(fmt, O.rng_normal(seed + i, N * K, 0.02))
        out[name] = (tfq.Weight(fmt, N, K, pay), pay, N, K)
    return out


@pytest.mark.parametrize("fmt", ["B32S4", "Q_G_4"])
@pytest.mark.parametrize("D,F,B", [(1024, 2048, 1), (4096, 14336, 1), (2048, 3584, 2)])
def test_chain_mlp_step_matches_oracle(O, tfq, gpu, fmt, D, F, B):
    """Qwen35Engine::mlp_step as one launch: [gate, up] -> silu(gate) * up -> down."""
    import torch
    W = _weights(O, tfq, fmt, [("gate", F, D), ("up", F, D), ("down", D, F)], 300)
    x = O.bf16_round(O.rng_normal(43, B * D, 1.0)).reshape(B, D)
    xd = torch.from_numpy(x).to(gpu).bfloat16()
    g_d = torch.zeros(B, F, device=gpu)
    u_d = torch.zeros(B, F, device=gpu)
    y_d = torch.zeros(B, D, device=gpu)
    chain = tfq.Chain([
        {"w": [W["gate"][0], W["up"][0]], "x": xd, "y_op": tfq.Y_SWIGLU, "y": [g_d, u_d]},
        {"w": [W["down"][0]], "y": [y_d]},
    ], B=B)
    chain.run()
    torch.cuda.synchronize()
    chain.check()
    g = O.matmul(fmt, W["gate"][1], F, D, x)
    u = O.matmul(fmt, W["up"][1], F, D, x)
    h = O.bf16_round(O.silu_mul(g, u))
    y = O.matmul(fmt, W["down"][1], D, F, h)
    assert rel_err(g_d.cpu().numpy(), g) <= 1e-2
    assert rel_err(u_d.cpu().numpy(), u) <= 1e-2
    assert rel_err(y_d.cpu().numpy(), y) <= 1e-2
    # a second run gives the same bits (fixed summation order, counters back at zero)
    first = y_d.clone()
    y_d.zero_()
    chain.run()
    torch.cuda.synchronize()
    chain.check()
    assert torch.equal(first, y_d)
    chain.close()


@pytest.mark.parametrize("fmt", ["B32S4"])
def test_chain_decoder_layer_matches_oracle(O, tfq, gpu, fmt):
    """rmsnorm -> q, k, v | o(q) -> h += . | rmsnorm -> gate, up -> silu * up -> down -> h += .
    (append_token's projections; the attention between q/k/v and o is outside the path, o takes q)."""
    import torch
    D, F, KV = 2048, 4096, 512
    W = _weights(O, tfq, fmt, [("q", D, D), ("k", KV, D), ("v", KV, D), ("o", D, D), ("gate", F, D), ("up", F, D), ("down", D, F)], 500)
    h0 = O.rng_normal(7, D, 1.0)
    g1 = O.rng_normal(8, D, 0.1)
    g2 = O.rng_normal(9, D, 0.1)
    h_d = torch.from_numpy(h0.copy()).to(gpu).reshape(1, D)
    g1_d, g2_d = torch.from_numpy(g1).to(gpu), torch.from_numpy(g2).to(gpu)
    q_d, k_d, v_d = (torch.zeros(1, n, device=gpu) for n in (D, KV, KV))
    chain = tfq.Chain([
        {"w": [W["q"][0], W["k"][0], W["v"][0]], "x": h_d, "x_op": tfq.X_RMSNORM, "gamma": g1_d, "gamma_plus_one": True,
         "y": [q_d, k_d, v_d]},
        {"w": [W["o"][0]], "y_op": tfq.Y_RESIDUAL, "residual": h_d},
        {"w": [W["gate"][0], W["up"][0]], "x_op": tfq.X_RMSNORM, "gamma": g2_d, "gamma_plus_one": True, "y_op": tfq.Y_SWIGLU},
        {"w": [W["down"][0]], "y_op": tfq.Y_RESIDUAL, "residual": h_d},
    ], B=1)
    chain.run()
    torch.cuda.synchronize()
    chain.check()

    xn = O.bf16_round(O.rmsnorm(h0, g1))
    q = O.matmul(fmt, W["q"][1], D, D, xn)
    k = O.matmul(fmt, W["k"][1], KV, D, xn)
    v = O.matmul(fmt, W["v"][1], KV, D, xn)
    o = O.matmul(fmt, W["o"][1], D, D, O.bf16_round(q.reshape(-1)))
    h1 = (h0 + o.reshape(-1)).astype(np.float32)
    xn2 = O.bf16_round(O.rmsnorm(h1, g2))
    g = O.matmul(fmt, W["gate"][1], F, D, xn2)
    u = O.matmul(fmt, W["up"][1], F, D, xn2)
    hh = O.bf16_round(O.silu_mul(g, u))
    dn = O.matmul(fmt, W["down"][1], D, F, hh)
    h2 = (h1 + dn.reshape(-1)).astype(np.float32)
    assert rel_err(q_d.cpu().numpy(), q) <= 1e-2
    assert rel_err(k_d.cpu().numpy(), k) <= 1e-2
    assert rel_err(v_d.cpu().numpy(), v) <= 1e-2
    assert rel_err(h_d.cpu().numpy().reshape(-1), h2) <= 1e-2
    chain.close()


def _oracle_layer(O, fmt, W, h, g1, g2, D, F, KV):
    """One decoder layer's projections on the CPU (the order of append_token, qwen35_engine.cpp:807-835)."""
    xn = O.bf16_round(O.rmsnorm(h, g1))
    q = O.matmul(fmt, W["q"][1], D, D, xn)
    k = O.matmul(fmt, W["k"][1], KV, D, xn)
    v = O.matmul(fmt, W["v"][1], KV, D, xn)
    o = O.matmul(fmt, W["o"][1], D, D, O.bf16_round(q.reshape(-1)))
    h1 = (h + o.reshape(-1)).astype(np.float32)
    xn2 = O.bf16_round(O.rmsnorm(h1, g2))
    g = O.matmul(fmt, W["gate"][1], F, D, xn2)
    u = O.matmul(fmt, W["up"][1], F, D, xn2)
    hh = O.bf16_round(O.silu_mul(g, u))
    dn = O.matmul(fmt, W["down"][1], D, F, hh)
    return (h1 + dn.reshape(-1)).astype(np.float32), q, k, v


def test_chain_three_layers_matches_oracle_and_repeats(O, tfq, gpu):
    """Twelve phases: the link buffers are written again three phases later, the residual rows alternate between
    the kept copy in LDS and the tagged copy, and the first phase reads the very buffer the residual phases
    update.  130 runs of the one chain (the launch counter inside the tags wraps at 128) give identical bits."""
    import torch
    fmt = "B32S4"
    D, F, KV = 1024, 2048, 256
    shapes = [("q", D, D), ("k", KV, D), ("v", KV, D), ("o", D, D), ("gate", F, D), ("up", F, D), ("down", D, F)]
    layers = [_weights(O, tfq, fmt, shapes, 700 + 10 * l) for l in range(3)]
    h0 = O.rng_normal(17, D, 1.0)
    gains = [(O.rng_normal(30 + 2 * l, D, 0.1), O.rng_normal(31 + 2 * l, D, 0.1)) for l in range(3)]
    h_d = torch.from_numpy(h0.copy()).to(gpu).reshape(1, D)
    gd = [(torch.from_numpy(a).to(gpu), torch.from_numpy(b).to(gpu)) for a, b in gains]
    outs = [tuple(torch.zeros(1, n, device=gpu) for n in (D, KV, KV)) for _ in range(3)]
    phases = []
    for l, W in enumerate(layers):
        phases += [
            {"w": [W["q"][0], W["k"][0], W["v"][0]], "x": h_d if l == 0 else None, "x_op": tfq.X_RMSNORM, "gamma": gd[l][0],
             "gamma_plus_one": True, "y": list(outs[l])},
            {"w": [W["o"][0]], "y_op": tfq.Y_RESIDUAL, "residual": h_d},
            {"w": [W["gate"][0], W["up"][0]], "x_op": tfq.X_RMSNORM, "gamma": gd[l][1], "gamma_plus_one": True, "y_op": tfq.Y_SWIGLU},
            {"w": [W["down"][0]], "y_op": tfq.Y_RESIDUAL, "residual": h_d},
        ]
    chain = tfq.Chain(phases, B=1)
    chain.run()
    torch.cuda.synchronize()
    chain.check()
    h = h0
    for l, W in enumerate(layers):
        h, q, k, v = _oracle_layer(O, fmt, W, h, gains[l][0], gains[l][1], D, F, KV)
        assert rel_err(outs[l][0].cpu().numpy(), q) <= 1e-2
        assert rel_err(outs[l][1].cpu().numpy(), k) <= 1e-2
        assert rel_err(outs[l][2].cpu().numpy(), v) <= 1e-2
    assert rel_err(h_d.cpu().numpy().reshape(-1), h) <= 1e-2
    first = h_d.clone()
    firsts = [tuple(t.clone() for t in o) for o in outs]
    for _ in range(130):
        h_d.copy_(torch.from_numpy(h0).to(gpu).reshape(1, D))
        chain.run()
    torch.cuda.synchronize()
    chain.check()
    assert torch.equal(first, h_d)
    for a, b in zip(firsts, outs):
        for x, y in zip(a, b):
            assert torch.equal(x, y)
    chain.close()


def test_chain_two_rows_with_rmsnorm(O, tfq, gpu):
    """B = 2 through RMSNorm -> gate, up -> SwiGLU -> down -> residual (fp32 tagged rows, two rows per wavefront)."""
    import torch
    fmt = "Q_G_4"
    D, F, B = 1024, 2048, 2
    W = _weights(O, tfq, fmt, [("gate", F, D), ("up", F, D), ("down", D, F)], 900)
    h0 = O.rng_normal(5, B * D, 1.0).reshape(B, D)
    g = O.rng_normal(6, D, 0.1)
    h_d = torch.from_numpy(h0.copy()).to(gpu)
    x_d = h_d.clone()   # a buffer of its own for the first phase
    chain = tfq.Chain([
        {"w": [W["gate"][0], W["up"][0]], "x": x_d, "x_op": tfq.X_RMSNORM, "gamma": torch.from_numpy(g).to(gpu), "gamma_plus_one": True,
         "y_op": tfq.Y_SWIGLU},
        {"w": [W["down"][0]], "y_op": tfq.Y_RESIDUAL, "residual": h_d},
    ], B=B)
    chain.run()
    torch.cuda.synchronize()
    chain.check()
    ref = np.zeros((B, D), dtype=np.float32)
    for b in range(B):
        xn = O.bf16_round(O.rmsnorm(h0[b], g))
        gg = O.matmul(fmt, W["gate"][1], F, D, xn)
        uu = O.matmul(fmt, W["up"][1], F, D, xn)
        hh = O.bf16_round(O.silu_mul(gg, uu))
        ref[b] = h0[b] + O.matmul(fmt, W["down"][1], D, F, hh).reshape(-1)
    assert rel_err(h_d.cpu().numpy(), ref) <= 1e-2
    chain.close()


def test_chain_limits(O, tfq, gpu):
    """K above 16384 and a y_dtype outside the two served ones are refused at creation."""
    import torch
    pay = O.encode_tensor("B32S4", np.zeros(16 * 16640, dtype=np.float32))
    w = tfq.Weight("B32S4", 16, 16640, pay)
    with pytest.raises(tfq.TfqError):
        tfq.Chain([{"w": [w], "x": torch.zeros(1, 16640, device=gpu).bfloat16(), "y": [torch.zeros(1, 16, device=gpu)]}])


def test_chain_rejects_what_it_cannot_run(O, tfq, gpu):
    import torch
    pay = O.encode_tensor("Q_G_8", O.rng_normal(1, 256 * 256, 0.02))
    w8 = tfq.Weight("Q_G_8", 256, 256, pay)
    x = torch.zeros(1, 256, device=gpu).bfloat16()
    with pytest.raises(tfq.TfqError):
        tfq.Chain([{"w": [w8], "x": x, "y": [torch.zeros(1, 256, device=gpu)]}])
    pay4 = O.encode_tensor("B32S4", O.rng_normal(2, 256 * 256, 0.02))
    w4 = tfq.Weight("B32S4", 256, 256, pay4)
    with pytest.raises(tfq.TfqError):  # the first phase has no input
        tfq.Chain([{"w": [w4], "y": [torch.zeros(1, 256, device=gpu)]}])
    with pytest.raises(tfq.TfqError):  # three rows
        tfq.Chain([{"w": [w4], "x": torch.zeros(3, 256, device=gpu).bfloat16(), "y": [torch.zeros(3, 256, device=gpu)]}], B=3)
