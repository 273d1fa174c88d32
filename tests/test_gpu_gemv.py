"""Dequant-fused GEMV through the C ABI against the oracle's block-row matmul
(reference accumulation order, fp32).  Gate: max |y - y_ref| / max |y_ref|
<= 1e-3 for fp32 activations, <= 1e-2 for bf16 activations or bf16 output."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TOL_F32, TOL_BF16 = 1e-3, 1e-2
GEMV_FORMATS = ["Q_G_4", "B32S4"]
OTHER_FORMATS = ["Q_G_8", "B32S8", "Q_G_3", "Q_G_2", "SB256A3", "SB256A2", "Q_4", "Q_8", "Q_32", "Q_4_5", "Q_G_8_5",
                 "Q_2", "Q_G_6", "Q_G_6_K_M", "Q_G_2_K_L", "Q_G_3_K_H", "Q_G_4_K_M", "Q_2_5", "Q_6_5",
                 "Q_1", "Q_G_1", "Q_1_5", "Q_16", "Q_G_16", "Q_24", "Q_G_24",
                 "Q_3", "Q_6", "Q_12", "Q_G_12", "Q_G_12_K_M", "Q_G_8_K_M", "Q_4_K_H", "Q_8_K_L",
                 "Q_MX_3_5", "Q_MX_12_5", "Q_MX_16_5", "Q_G_MX_4_5", "Q_G_MX_8_5", "Q_G_MX_24_5"]


def rel_err(y, ref):
    return float(np.abs(y.astype(np.float64) - ref).max() / np.abs(ref).max())


def _case(O, fmt, N, K, B, seed=42):
    w = O.rng_normal(seed, N * K, 0.02)
    x = O.rng_normal(seed + 1, B * K, 1.0).reshape(B, K)
    return w, x, O.encode_tensor(fmt, w)


@pytest.mark.parametrize("fmt", GEMV_FORMATS)
@pytest.mark.parametrize("N,K", [(64, 256), (40, 1024), (72, 2304), (128, 4096), (33, 6400)])
@pytest.mark.parametrize("B", [1, 2, 3, 4, 8, 16])
def test_gemv_bf16_activations(O, tfq, gpu, fmt, N, K, B):
    import torch
    print(f"gemv bf16 {fmt} N={N} K={K} B={B}", flush=True)
    w, x, pay = _case(O, fmt, N, K, B)
    xb = O.bf16_round(x)
    ref = O.matmul_f64(fmt, pay, N, K, xb)
    ref32 = O.matmul(fmt, pay, N, K, xb)
    W = tfq.Weight(fmt, N, K, pay)
    y = W.gemv(torch.from_numpy(xb).to(gpu).to(torch.bfloat16)).cpu().numpy()
    assert y.shape == (B, N)
    assert rel_err(y, ref32) <= TOL_BF16
    # the kernel accumulates exact bf16 products in fp32: it should sit as close to
    # the fp64 result as the reference-order fp32 sum does (within a small factor)
    assert rel_err(y, ref) <= 1e-4
    yb = W.gemv(torch.from_numpy(xb).to(gpu).to(torch.bfloat16), out_dtype=torch.bfloat16).float().cpu().numpy()
    assert rel_err(yb, ref32) <= TOL_BF16
    W.close()


@pytest.mark.parametrize("fmt,N,K", [("B32S4", 49195, 256), ("B32S4", 49152, 768), ("Q_G_4", 49200, 512), ("B32S8", 49195, 256),
                                     ("Q_G_8", 49168, 256)])
def test_gemv_tall_matrix(O, tfq, gpu, fmt, N, K):
    """A matrix of more than 3072 row tiles (an output projection over a vocabulary) with one to eight bf16 rows
    takes the kernel whose wavefronts own whole tiles, one workgroup per compute unit; ragged last tile, fp32 and
    bf16 outputs, against the oracle."""
    import torch
    w = O.rng_normal(42, N * K, 0.02)
    pay = O.encode_tensor(fmt, w)
    W = tfq.Weight(fmt, N, K, pay)
    for B in (1, 3, 4, 5, 8):
        print(f"gemv tall {fmt} N={N} K={K} B={B}", flush=True)
        x = O.bf16_round(O.rng_normal(43 + B, B * K, 1.0).reshape(B, K))
        ref = O.matmul(fmt, pay, N, K, x)
        xt = torch.from_numpy(x).to(gpu).bfloat16()
        y = W.gemv(xt).cpu().numpy()
        assert y.shape == (B, N)
        assert rel_err(y, ref) <= (3e-4 if fmt in ("Q_G_8", "B32S8") else 1e-4)
        yb = W.gemv(xt, out_dtype=torch.bfloat16).float().cpu().numpy()
        assert rel_err(yb, ref) <= TOL_BF16
    W.close()


@pytest.mark.parametrize("fmt", GEMV_FORMATS)
@pytest.mark.parametrize("N,K,B", [(64, 256, 1), (48, 2048, 1), (96, 4096, 1), (40, 1280, 4), (24, 4096, 16),
                                   (72, 2304, 3), (33, 6400, 7), (40, 14336, 5), (1040, 14336, 8), (2000, 4096, 13), (272, 8192, 3)])
def test_gemv_fp32_activations(O, tfq, gpu, fmt, N, K, B):
    import torch
    print(f"gemv f32 {fmt} N={N} K={K} B={B}", flush=True)
    w, x, pay = _case(O, fmt, N, K, B, seed=7)
    ref = O.matmul(fmt, pay, N, K, x)
    W = tfq.Weight(fmt, N, K, pay)
    y = W.gemv(torch.from_numpy(x).to(gpu)).cpu().numpy()
    assert rel_err(y, ref) <= TOL_F32
    W.close()


@pytest.mark.parametrize("fmt", GEMV_FORMATS)
def test_config1_single_gemv_4096(O, tfq, gpu, fmt):
    """W 4096x4096 from N(0,0.02) seed 42, x fp32 [1,4096] seed 43: codes/decoded
    weights bit-exact, then y within 1e-3."""
    import torch
    N = K = 4096
    w = O.rng_normal(42, N * K, 0.02)
    x = O.rng_normal(43, K, 1.0).reshape(1, K)
    pay = O.encode_tensor(fmt, w)
    W = tfq.Weight(fmt, N, K, pay)
    dec = W.decode().cpu().numpy().reshape(-1)
    assert np.array_equal(dec.view(np.uint32), O.decode_tensor(fmt, pay, N * K).view(np.uint32))
    if fmt == "B32S4":
        assert np.array_equal(tfq.encode(fmt, torch.from_numpy(w).to(gpu)).cpu().numpy(), pay)
    ref = O.matmul(fmt, pay, N, K, x)
    y = W.gemv(torch.from_numpy(x).to(gpu)).cpu().numpy()
    assert rel_err(y, ref) <= TOL_F32
    W.close()


def test_gemv_linearity_and_row_independence(O, tfq, gpu):
    """Size-independent properties at a full Llama shape: y(x1 + x2) = y(x1) + y(x2)
    for bf16-exact inputs, and rows computed alone equal rows computed together."""
    import torch
    N, K = 14336, 4096
    fmt = "B32S4"
    g = torch.Generator(device="cuda").manual_seed(1)
    wt = torch.randn(N, K, device=gpu, generator=g) * 0.02
    pay = tfq.encode(fmt, wt)
    W = tfq.Weight(fmt, N, K, pay)
    x1 = torch.randint(-64, 64, (1, K), device=gpu, generator=g).float()
    x2 = torch.randint(-64, 64, (1, K), device=gpu, generator=g).float()
    y1 = W.gemv(x1.bfloat16()); y2 = W.gemv(x2.bfloat16()); y12 = W.gemv((x1 + x2).bfloat16())
    scale = float(y12.abs().max())
    assert float((y12 - (y1 + y2)).abs().max()) <= 2e-5 * scale
    # batch of 4 equals four single calls bit for bit in fp32 accumulation order per row
    xb = torch.cat([x1, x2, x1 - x2, x2 * 0.5]).bfloat16()
    yb = W.gemv(xb)
    for i in range(4):
        assert float((yb[i] - W.gemv(xb[i:i + 1])[0]).abs().max()) <= 2e-5 * scale
    # against a dense torch matmul of the decoded matrix
    dense = W.decode()
    want = (xb.float().double() @ dense.double().T).float()
    assert float((yb - want).abs().max()) <= 1e-4 * float(want.abs().max())
    W.close()


def test_gemv_rejects_bad_arguments(O, tfq, gpu):
    import torch
    pay = O.encode_tensor("Q_G_4", O.rng_normal(1, 8 * 256, 0.02))
    with pytest.raises(tfq.TfqError):
        tfq.Weight("Q_G_4", 8, 256, pay[:-1])
    with pytest.raises(tfq.TfqError):
        tfq.Weight("Q_G_4", 8, 255, pay)
    W = tfq.Weight("Q_G_4", 8, 256, pay)
    x = torch.zeros(17, 256, device=gpu, dtype=torch.bfloat16)
    with pytest.raises(tfq.TfqError):
        W.gemv(x)
    W.close()


@pytest.mark.parametrize("fmt", GEMV_FORMATS)
@pytest.mark.parametrize("B", [1, 4])
def test_gemv_multi_matches_single_launches(O, tfq, gpu, fmt, B):
    """q/k/v style: three matrices of different heights on one input, one launch."""
    import torch
    K = 2048
    shapes = [72, 24, 33]
    x = torch.from_numpy(O.bf16_round(O.rng_normal(5, B * K, 1.0).reshape(B, K))).to(gpu).bfloat16()
    Ws, singles = [], []
    for i, N in enumerate(shapes):
        pay = O.encode_tensor(fmt, O.rng_normal(60 + i, N * K, 0.02))
        W = tfq.Weight(fmt, N, K, pay)
        Ws.append(W)
        singles.append(W.gemv(x))
    outs = [torch.zeros(B, N, device=gpu) for N in shapes]
    tfq.gemv_multi(Ws, x, outs)
    for got, want in zip(outs, singles):
        assert torch.equal(got, want)
    for W in Ws:
        W.close()


@pytest.mark.parametrize("fmt", GEMV_FORMATS)
@pytest.mark.parametrize("B", [3, 4, 8, 11])
def test_gemv_multi_fp32_rows(O, tfq, gpu, fmt, B):
    """Three matrices on one fp32 input of several rows (four rows per pass on the two-set kernel, eight on the
    sixteen-row kernel): the same bits as single launches, and the oracle's result."""
    import torch
    K = 2048
    shapes = [72, 24, 33]
    xh = O.rng_normal(5, B * K, 1.0).reshape(B, K)
    x = torch.from_numpy(xh).to(gpu)
    Ws, singles, pays = [], [], []
    for i, N in enumerate(shapes):
        pay = O.encode_tensor(fmt, O.rng_normal(60 + i, N * K, 0.02))
        W = tfq.Weight(fmt, N, K, pay)
        Ws.append(W)
        pays.append(pay)
        singles.append(W.gemv(x))
    outs = [torch.zeros(B, N, device=gpu) for N in shapes]
    tfq.gemv_multi(Ws, x, outs)
    for got, want, pay, N in zip(outs, singles, pays, shapes):
        assert torch.equal(got, want)
        assert rel_err(got.cpu().numpy(), O.matmul(fmt, pay, N, K, xh)) <= TOL_F32
    for W in Ws:
        W.close()


@pytest.mark.parametrize("fmt", OTHER_FORMATS)
@pytest.mark.parametrize("N,K,B,xdt", [(48, 512, 1, "bf16"), (33, 1024, 3, "bf16"), (20, 2304, 8, "f32"), (16, 4096, 16, "bf16")])
def test_gemv_other_formats(O, tfq, gpu, fmt, N, K, B, xdt):
    """8-bit, 3-bit, 2-bit, plain lattice and raw blocks: every registered format the
    codec handles also runs through the matmul entry point."""
    import torch
    print(f"gemv {fmt} N={N} K={K} B={B} {xdt}", flush=True)
    dist = O.rng_laplace(44, N * K, 0.015) if fmt.startswith("SB256") or fmt in ("Q_G_3", "Q_G_2") else O.rng_normal(42, N * K, 0.02)
    x = O.rng_normal(43, B * K, 1.0).reshape(B, K)
    pay = O.encode_tensor(fmt, dist)
    W = tfq.Weight(fmt, N, K, pay)
    if xdt == "bf16":
        x = O.bf16_round(x)
        y = W.gemv(torch.from_numpy(x).to(gpu).bfloat16()).cpu().numpy()
        tol = TOL_BF16
    else:
        y = W.gemv(torch.from_numpy(x).to(gpu)).cpu().numpy()
        tol = TOL_F32
    ref = O.matmul(fmt, pay, N, K, x)
    # exact weights and (bf16-split) products: only the summation order differs.  The companded 8-bit grid is
    # multiplied through a line fitted to its 256 levels (7.5e-5 relative per weight), so those get a wider gate.
    assert rel_err(y, ref) <= (3e-4 if fmt in ("Q_G_8", "Q_8", "Q_8_5", "Q_G_8_5") else 1e-4)
    assert np.array_equal(W.decode().cpu().numpy().reshape(-1).view(np.uint32),
                          O.decode_tensor(fmt, pay, N * K).view(np.uint32))
    W.close()


@pytest.mark.parametrize("fmt,bits", [("SB256A3", 3), ("SB256A2", 2), ("Q_G_3", 3), ("Q_G_2", 2)])
def test_config4_lowbit_superblock_shapes(O, tfq, gpu, fmt, bits):
    """Laplace(0, 0.015) weights, 14336-wide rows (a slice of the 14336x4096 matrix), batch 1 and 8."""
    import torch
    N, K = 256, 4096
    w = O.rng_laplace(44, N * K, 0.015)
    pay = O.encode_tensor(fmt, w)
    W = tfq.Weight(fmt, N, K, pay)
    for B in (1, 8):
        x = O.bf16_round(O.rng_normal(43, B * K, 1.0).reshape(B, K))
        y = W.gemv(torch.from_numpy(x).to(gpu).bfloat16()).cpu().numpy()
        assert rel_err(y, O.matmul(fmt, pay, N, K, x)) <= 1e-4
    W.close()


@pytest.mark.parametrize("fmt", ["SB256A3", "SB256A2"])
def test_config4_lowbit_superblock_full_size(tfq, gpu, fmt):
    """The whole 14336x4096 matrix of the benchmark's low-bit configuration (Laplace(0, 0.015) weights encoded on
    the device), batch 1 and batch 8, against the float64 product of the device-decoded matrix; the decoded matrix
    itself is pinned bit for bit against the oracle by the tests above."""
    import torch
    N, K = 14336, 4096
    g = torch.Generator(device="cuda").manual_seed(44)
    u = torch.rand(N * K, device=gpu, generator=g) - 0.5
    w = -0.015 * torch.sign(u) * torch.log1p(-2 * u.abs().clamp(max=0.4999999))
    W = tfq.Weight(fmt, N, K, tfq.encode(fmt, w))
    dense = W.decode().double()
    for B in (1, 8):
        x = torch.randn(B, K, device=gpu, generator=g).bfloat16()
        want = x.double() @ dense.T
        y = W.gemv(x)
        assert float((y.double() - want).abs().max() / want.abs().max()) <= 1e-4
        yb = W.gemv(x, out_dtype=torch.bfloat16)
        assert float((yb.double() - want).abs().max() / want.abs().max()) <= 1e-2
    W.close()


@pytest.mark.parametrize("fmt", ["SB256A3", "SB256A2", "Q_G_2"])
@pytest.mark.parametrize("N,K", [(4200, 1024), (40, 14336), (1000, 2304)])
def test_one_row_of_the_byte_header_formats(O, tfq, gpu, fmt, N, K):
    """One bf16 row of the formats with sixteen 16-weight groups runs the kernel variant in which every lane row
    decodes the scales of its own 32 weights: several tiles per workgroup with a partial last tile, two fetches in
    flight, uneven block columns per wavefront; the same matrix at two rows (the other variant) as a cross-check."""
    import torch
    w = O.rng_laplace(44, N * K, 0.015)
    pay = O.encode_tensor(fmt, w)
    W = tfq.Weight(fmt, N, K, pay)
    x = O.bf16_round(O.rng_normal(43, 2 * K, 1.0).reshape(2, K))
    ref = O.matmul(fmt, pay, N, K, x)
    xg = torch.from_numpy(x).to(gpu).bfloat16()
    y1 = W.gemv(xg[:1].contiguous()).cpu().numpy()
    y2 = W.gemv(xg).cpu().numpy()
    assert rel_err(y1, ref[:1]) <= 1e-4
    assert rel_err(y2, ref) <= 1e-4
    assert rel_err(y1, y2[:1]) <= 1e-5
    W.close()


@pytest.mark.parametrize("fmt", ["Q_G_8", "Q_8", "B32S8"])
@pytest.mark.parametrize("N,K", [(256, 4096), (48, 14336), (1040, 1024)])
def test_config2_eight_bit_formats(O, tfq, gpu, fmt, N, K):
    """8-bit formats at the projection widths, batch 1, 4, 8, 16 with bf16 activations and batch 1, 3 with
    fp32 activations.  Q_G_8 / Q_8 multiply through the fitted line of the companded grid: the error
    against the exact-table oracle stays under a third of the fp32 gate."""
    import torch
    w = O.rng_normal(42, N * K, 0.02)
    pay = O.encode_tensor(fmt, w)
    W = tfq.Weight(fmt, N, K, pay)
    assert np.array_equal(W.decode().cpu().numpy().reshape(-1).view(np.uint32), O.decode_tensor(fmt, pay, N * K).view(np.uint32))
    for B in (1, 4, 8, 16):
        print(f"gemv 8-bit {fmt} N={N} K={K} B={B} bf16", flush=True)
        x = O.bf16_round(O.rng_normal(43, B * K, 1.0).reshape(B, K))
        y = W.gemv(torch.from_numpy(x).to(gpu).bfloat16()).cpu().numpy()
        assert rel_err(y, O.matmul(fmt, pay, N, K, x)) <= 3e-4
    for B in (1, 3):
        print(f"gemv 8-bit {fmt} N={N} K={K} B={B} f32", flush=True)
        x = O.rng_normal(45, B * K, 1.0).reshape(B, K)
        y = W.gemv(torch.from_numpy(x).to(gpu)).cpu().numpy()
        assert rel_err(y, O.matmul(fmt, pay, N, K, x)) <= 3e-4
    # all-positive activations and weights: nothing cancels, the systematic part of the line fit shows in full
    wp = np.abs(w)
    payp = O.encode_tensor(fmt, wp)
    Wp = tfq.Weight(fmt, N, K, payp)
    x = np.abs(O.bf16_round(O.rng_normal(43, K, 1.0))).reshape(1, K)
    y = Wp.gemv(torch.from_numpy(x).to(gpu).bfloat16()).cpu().numpy()
    assert rel_err(y, O.matmul(fmt, payp, N, K, x)) <= 3e-4
    W.close()
    Wp.close()


@pytest.mark.parametrize("fmt", GEMV_FORMATS)
@pytest.mark.parametrize("N,K,B", [(16 * 256 * 2, 256, 1), (16 * 256 * 7, 256, 3), (16 * 256 * 5 + 40, 512, 4),
                                   (16 * 300, 4096, 2), (48, 14336, 4), (16 * 256 * 3, 1024, 16)])
def test_gemv_many_tiles_per_workgroup(O, tfq, gpu, fmt, N, K, B):
    """More than 256 row tiles (a workgroup then walks several tiles, in groups of fetches with a
    partial last group) and K = 14336 (four block columns per wavefront): checked against a dense
    torch product of the device-decoded matrix, which the codec tests hold bit-exact."""
    import torch
    print(f"gemv tiles {fmt} N={N} K={K} B={B}", flush=True)
    g = torch.Generator(device="cuda").manual_seed(N + K + B)
    if fmt == "B32S4":
        w = torch.randn(N * K, device=gpu, generator=g) * 0.02
        pay = tfq.encode(fmt, w)
    else:  # random valid payloads: any code bytes, small finite binary16 d and dm
        bb = tfq.block_bytes(fmt)
        pay = torch.randint(0, 256, (N * K // 256, bb), device=gpu, dtype=torch.uint8, generator=g)
        pay[:, -4:] = torch.tensor([0x00, 0x20, 0x00, 0x20], dtype=torch.uint8, device=gpu)
        pay = pay.reshape(-1)
    W = tfq.Weight(fmt, N, K, pay)
    x = torch.randn(B, K, device=gpu, generator=g).bfloat16()
    y = W.gemv(x)
    want = x.double() @ W.decode().double().T
    err = float((y.double() - want).abs().max() / want.abs().max())
    assert err <= 1e-4, err
    W.close()


@pytest.mark.parametrize("fmt", ["B32S4", "Q_G_4", "B32S8", "Q_G_8", "Q_8"])
@pytest.mark.parametrize("N,K,B", [(16 * 256 * 3 + 40, 512, 16), (16 * 300, 4096, 9), (4096, 14336, 16), (1040, 4608, 5),
                                   (16 * 256 * 9, 256, 13), (24, 7168, 8)])
def test_gemv_five_to_sixteen_rows(O, tfq, gpu, fmt, N, K, B):
    """Five or more bf16 rows take the sixteen-row kernel (one block column per wavefront, K parts over workgroups
    above sixteen block columns): a single block column, sixteen, a partial last part, four parts, rows not a
    multiple of four, more tiles than one round of workgroups holds.  Checked against a dense product of the
    device-decoded matrix (bit-exact by the codec tests), fp32 and bf16 outputs."""
    import torch
    print(f"gemv rows {fmt} N={N} K={K} B={B}", flush=True)
    g = torch.Generator(device="cuda").manual_seed(N + K + B)
    if fmt in ("B32S4", "B32S8"):
        pay = tfq.encode(fmt, torch.randn(N * K, device=gpu, generator=g) * 0.02)
    else:
        bb = tfq.block_bytes(fmt)
        pay = torch.randint(0, 256, (N * K // 256, bb), device=gpu, dtype=torch.uint8, generator=g)
        if fmt == "Q_G_4":
            pay[:, -4:] = torch.tensor([0x00, 0x20, 0x00, 0x20], dtype=torch.uint8, device=gpu)
        elif fmt == "Q_G_8":
            pay[:, -16:] = torch.tensor([0x00, 0x20] * 8, dtype=torch.uint8, device=gpu)
        else:
            pay[:, :2] = torch.tensor([0x00, 0x20], dtype=torch.uint8, device=gpu)
        pay = pay.reshape(-1)
    W = tfq.Weight(fmt, N, K, pay)
    x = torch.randn(B, K, device=gpu, generator=g).bfloat16()
    want = x.double() @ W.decode().double().T
    scale = float(want.abs().max())
    y = W.gemv(x)
    tol = 1e-4 if fmt in ("B32S4", "Q_G_4", "B32S8") else 1e-3  # the companded formats multiply through a line fit
    assert float((y.double() - want).abs().max()) <= tol * scale
    yb = W.gemv(x, out_dtype=torch.bfloat16)
    assert float((yb.double() - want).abs().max()) <= 1e-2 * scale
    # every row equals the single-row product of the same kernel family to rounding
    one = W.gemv(x[B - 1:B])
    assert float((y[B - 1] - one[0]).abs().max()) <= 2e-5 * scale
    W.close()


def test_gemv_multi_with_eight_rows(O, tfq, gpu):
    """q/k/v style launch with more than four rows: three matrices, one launch of the sixteen-row kernel."""
    import torch
    K, B = 4096, 8
    shapes = [4096, 1024, 1040]
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(B, K, device=gpu, generator=g).bfloat16()
    Ws = [tfq.Weight("B32S4", N, K, tfq.encode("B32S4", torch.randn(N * K, device=gpu, generator=g) * 0.02)) for N in shapes]
    outs = [torch.zeros(B, N, device=gpu) for N in shapes]
    tfq.gemv_multi(Ws, x, outs)
    for W, got in zip(Ws, outs):
        want = x.double() @ W.decode().double().T
        assert float((got.double() - want).abs().max()) <= 1e-4 * float(want.abs().max())
        assert torch.equal(got, W.gemv(x))
        W.close()


@pytest.mark.parametrize("fmt", ["B32S4", "B32S8"])
def test_gemv_rows_with_k_split_repeated_calls(O, tfq, gpu, fmt):
    """K above 4096 with five or more rows: the workgroups of a row group split K, write their partial sums to the
    call's workspace, and a second launch adds the parts in part order.  Calls in a row on one handle (other
    activations, fewer rows, bf16 output, 40 rows through tfq_gemm) each match a dense product of the decoded
    matrix, a repeated call gives the same bits, and two matrices of such a K in one launch (no split there)
    agree with the single launches."""
    import torch
    N, K = 1000, 14336  # 63 tiles, the last one short; 56 block columns in 4 parts of 14
    g = torch.Generator(device="cuda").manual_seed(77)
    W = tfq.Weight(fmt, N, K, tfq.encode(fmt, torch.randn(N * K, device=gpu, generator=g) * 0.02))
    dense = W.decode().double()
    first = None
    for i, B in enumerate((16, 16, 5, 12, 9)):
        print(f"gemv k-split {fmt} call {i} B={B}", flush=True)
        x = torch.randn(B, K, device=gpu, generator=torch.Generator(device="cuda").manual_seed(5 if i < 2 else 5 + i)).bfloat16()
        want = x.double() @ dense.T
        scale = float(want.abs().max())
        y = W.gemv(x)
        assert float((y.double() - want).abs().max()) <= 1e-4 * scale
        if i == 0:
            first = y.clone()
        if i == 1:
            assert torch.equal(y, first)
        yb = W.gemv(x, out_dtype=torch.bfloat16)
        assert float((yb.double() - want).abs().max()) <= 1e-2 * scale
    x = torch.randn(40, K, device=gpu, generator=g).bfloat16()
    want = x.double() @ dense.T
    # (tfq_gemm may take the matrix-core tile kernel, which rounds the decoded weights to bf16: 1e-2 is the bar there)
    assert float((W.gemm(x).double() - want).abs().max()) <= 1e-2 * float(want.abs().max())
    W2 = tfq.Weight(fmt, 48, K, tfq.encode(fmt, torch.randn(48 * K, device=gpu, generator=g) * 0.02))
    x = torch.randn(8, K, device=gpu, generator=g).bfloat16()
    outs = [torch.zeros(8, N, device=gpu), torch.zeros(8, 48, device=gpu)]
    tfq.gemv_multi([W, W2], x, outs)
    for Wi, got in zip((W, W2), outs):
        want = x.double() @ Wi.decode().double().T
        assert float((got.double() - want).abs().max()) <= 1e-4 * float(want.abs().max())
    W.close()
    W2.close()


def test_gemv_k_split_in_graph_replays(O, tfq, gpu):
    """The K-split launches (the parts' kernel and the kernel that adds them) inside a captured graph: every replay
    (with eager launches on the same handle between replays) gives the bits of the eager result."""
    import torch
    N, K, B = 4096, 14336, 16
    g = torch.Generator(device="cuda").manual_seed(11)
    W = tfq.Weight("B32S4", N, K, tfq.encode("B32S4", torch.randn(N * K, device=gpu, generator=g) * 0.02))
    xs = [torch.randn(B, K, device=gpu, generator=g).bfloat16() for _ in range(3)]
    eager = [W.gemv(x).clone() for x in xs]
    outs = [torch.empty(B, N, device=gpu) for _ in xs]
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for x, y in zip(xs, outs):
            W.gemv(x, out=y)
    for rep in range(5):
        print(f"gemv k-split graph replay {rep}", flush=True)
        for y in outs:
            y.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for want, got in zip(eager, outs):
            assert torch.equal(want, got)
        assert torch.equal(W.gemv(xs[rep % 3]), eager[rep % 3])  # eager work between the replays
    W.close()


def test_gemv_one_handle_on_two_streams(O, tfq, gpu):
    """Qwen35Engine::gemm is const and may run concurrently on one matrix (qwen35_engine.cpp:54-75): calls on
    one handle overlap on two streams, each with a workspace of its own, and give the bits of the serial
    result; so does the call without a workspace (unsplit) to the matmul tolerance."""
    import torch
    N, K, B = 4096, 14336, 16
    g = torch.Generator(device="cuda").manual_seed(21)
    W = tfq.Weight("B32S4", N, K, tfq.encode("B32S4", torch.randn(N * K, device=gpu, generator=g) * 0.02))
    xs = [torch.randn(B, K, device=gpu, generator=g).bfloat16() for _ in range(2)]
    need = W.gemv_workspace_bytes(tfq.BF16, B)
    assert need > 0
    wss = [torch.empty(need, dtype=torch.uint8, device=gpu) for _ in range(2)]
    serial = [W.gemv(x, workspace=wss[0]).clone() for x in xs]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [torch.empty(B, N, device=gpu) for _ in range(2)]
    for rep in range(50):
        for i, st in enumerate(streams):
            with torch.cuda.stream(st):
                W.gemv(xs[i], out=outs[i], workspace=wss[i])
        torch.cuda.synchronize()
        for want, got in zip(serial, outs):
            assert torch.equal(want, got), rep
    # no workspace: the unsplit kernel, the same product to the tolerance of bf16 activations
    y = torch.empty(B, N, device=gpu)
    rc = tfq.lib().tfq_gemv(W.handle, xs[0].data_ptr(), tfq.BF16, B, y.data_ptr(), tfq.F32, None)
    assert rc == 0
    torch.cuda.synchronize()
    assert float((y - serial[0]).abs().max()) <= 1e-4 * float(serial[0].abs().max())
    W.close()


def test_gemv_k_split_soak(O, tfq, gpu):
    """A bounded soak of the K split: 3000 replays of a graph holding three K-split products, each compared bit
    for bit with the eager result on the device; the loop stops at the first block of replays that holds a
    mismatch.  (Partial sums pass from the workgroups of one launch, on different XCDs, to the launch that adds
    them; a lost or late partial sum would change bits.)"""
    import torch
    N, K, B = 4096, 14336, 16
    g = torch.Generator(device="cuda").manual_seed(12)
    W = tfq.Weight("B32S4", N, K, tfq.encode("B32S4", torch.randn(N * K, device=gpu, generator=g) * 0.02))
    xs = [torch.randn(B, K, device=gpu, generator=g).bfloat16() for _ in range(3)]
    eager = [W.gemv(x).clone() for x in xs]
    outs = [torch.empty(B, N, device=gpu) for _ in xs]
    bad = torch.zeros((), device=gpu, dtype=torch.int64)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for x, y in zip(xs, outs):
            W.gemv(x, out=y)
    for block in range(30):
        for _ in range(100):
            graph.replay()
            for want, got in zip(eager, outs):
                bad += (want != got).sum()
        torch.cuda.synchronize()
        assert int(bad.item()) == 0, f"mismatch within replays {block * 100}..{block * 100 + 99}"
    W.close()


@pytest.mark.parametrize("fmt", ["B32S4", "Q_G_4", "B32S8"])
@pytest.mark.parametrize("K,B,xdt", [(65536, 1, "bf16"), (65536, 3, "bf16"), (40960, 1, "f32"), (65536, 2, "f32")])
def test_very_long_k(O, tfq, gpu, fmt, K, B, xdt):
    """K beyond what one staged activation row leaves room for in LDS (61440 for a bf16 row, 32768 for an fp32
    row): the product goes through the kernel whose wavefronts fetch their own activation fragments."""
    import torch
    N = 48
    pay = O.encode_tensor(fmt, O.rng_normal(63, N * K, 0.02))
    W = tfq.Weight(fmt, N, K, pay)
    x = O.rng_normal(64, B * K, 1.0).reshape(B, K)
    if xdt == "bf16":
        x = O.bf16_round(x)
        y = W.gemv(torch.from_numpy(x).to(gpu).bfloat16()).cpu().numpy()
    else:
        y = W.gemv(torch.from_numpy(x).to(gpu)).cpu().numpy()
    ref = O.matmul(fmt, pay, N, K, x)
    assert float(np.abs(y - ref).max() / np.abs(ref).max()) <= (1e-4 if xdt == "bf16" else 1e-3)
    W.close()


@pytest.mark.parametrize("fmt,K,xdt,one_launch", [("SB256A2", 49152, "bf16", True), ("SB256A2", 49408, "bf16", False),
                                                  ("Q_G_3", 61440, "bf16", True), ("Q_G_3", 61696, "bf16", False),
                                                  ("SB256A3", 28672, "f32", True), ("SB256A3", 28928, "f32", False)])
def test_k_ceiling_of_the_staged_formats(O, tfq, gpu, fmt, K, xdt, one_launch):
    """The tiled formats outside the sixteen-row kernel stage a whole activation row up to a K that depends on the
    format; one block more and the row is walked in windows of K that add into an fp32 output.  Both sides of the
    step match the oracle; a bf16 output, which cannot be added to, is refused above the step before any launch."""
    import torch
    N = 16
    pay = O.encode_tensor(fmt, O.rng_laplace(65, N * K, 0.015))
    W = tfq.Weight(fmt, N, K, pay)
    x = O.rng_normal(66, K, 1.0).reshape(1, K)
    xg = torch.from_numpy(O.bf16_round(x)).to(gpu).bfloat16() if xdt == "bf16" else torch.from_numpy(x).to(gpu)
    y = W.gemv(xg).cpu().numpy()
    ref = O.matmul(fmt, pay, N, K, O.bf16_round(x) if xdt == "bf16" else x)
    assert float(np.abs(y - ref).max() / np.abs(ref).max()) <= 1e-3
    if one_launch:
        assert W.gemv(xg, out_dtype=torch.bfloat16).shape == (1, N)
    else:
        with pytest.raises(Exception, match="K too large"):
            W.gemv(xg, out_dtype=torch.bfloat16)
    W.close()


@pytest.mark.parametrize("fmt", ["SB256A2", "SB256A3", "Q_G_3", "Q_G_2", "Q_G_6"])
@pytest.mark.parametrize("K,B,xdt", [(65536, 1, "bf16"), (65536, 8, "bf16"), (65536, 3, "f32"), (70400, 5, "bf16")])
def test_k_above_the_staging_ceiling_in_windows(O, tfq, gpu, fmt, K, B, xdt):
    """K = 65536 and a K that no even split divides, one row to eight: windows of block columns, each a round of
    launches that adds into y, against the oracle's product.  (Q_G_6 is not held as tiles and takes the generic
    kernel, which has no K limit: it rides along as the control.)"""
    import torch
    N = 40
    pay = O.encode_tensor(fmt, O.rng_laplace(67, N * K, 0.015))
    W = tfq.Weight(fmt, N, K, pay)
    x = O.rng_normal(68, B * K, 1.0).reshape(B, K)
    if xdt == "bf16":
        x = O.bf16_round(x)
        xg = torch.from_numpy(x).to(gpu).bfloat16()
    else:
        xg = torch.from_numpy(x).to(gpu)
    y = W.gemv(xg).cpu().numpy()
    ref = O.matmul(fmt, pay, N, K, x)
    assert float(np.abs(y - ref).max() / np.abs(ref).max()) <= 1e-3
    # the same call adds nothing to a second run's result (every window but the first accumulates: y must be
    # overwritten by the first window, not added to)
    out = torch.full((B, N), 7.0, device=gpu)
    W.gemv(xg, out=out)
    assert np.array_equal(out.cpu().numpy(), y)
    W.close()


@pytest.mark.parametrize("K,B,xdt", [(28672, 4, "bf16"), (28672, 2, "f32"), (20480, 4, "bf16"), (32768, 3, "f32")])
def test_long_k_takes_fewer_rows_per_pass(O, tfq, gpu, K, B, xdt):
    """K above 16384 leaves LDS room for fewer staged rows per pass; the product must still run (and match)."""
    import torch
    fmt, N = "B32S4", 64
    pay = O.encode_tensor(fmt, O.rng_normal(61, N * K, 0.02))
    W = tfq.Weight(fmt, N, K, pay)
    x = O.rng_normal(62, B * K, 1.0).reshape(B, K)
    if xdt == "bf16":
        x = O.bf16_round(x)
        y = W.gemv(torch.from_numpy(x).to(gpu).bfloat16()).cpu().numpy()
        tol = 1e-2
    else:
        y = W.gemv(torch.from_numpy(x).to(gpu)).cpu().numpy()
        tol = 1e-3
    ref = O.matmul(fmt, pay, N, K, x)
    assert float(np.abs(y - ref).max() / np.abs(ref).max()) <= tol
    # the prefill entry with fp32 rows slices through the same path
    if xdt == "f32":
        ym = W.gemm(torch.from_numpy(np.concatenate([x, x])).to(gpu), workspace=False).cpu().numpy()
        assert float(np.abs(ym[:B] - ref).max() / np.abs(ref).max()) <= tol
    W.close()


@pytest.mark.parametrize("fmt", ["B32S4", "Q_G_4", "B32S8", "SB256A3"])
@pytest.mark.parametrize("B,plus_one", [(1, True), (2, False), (5, True)])
def test_rmsnorm_prologue_matches_oracle(O, tfq, gpu, fmt, B, plus_one):
    """rmsnorm -> q, k, v in one launch against the oracle's rmsnorm + fp32 matmul; fp32 activations, 1e-3."""
    import torch
    K = 2048
    shapes = [("q", 1024, K), ("k", 256, K), ("v", 272, K)]
    pays = {n: O.encode_tensor(fmt, O.rng_normal(60 + i, N * K, 0.02)) for i, (n, N, _) in enumerate(shapes)}
    Ws = [tfq.Weight(fmt, N, K, pays[n]) for n, N, _ in shapes]
    x = O.rng_normal(43, B * K, 1.5).reshape(B, K)
    gamma = O.rng_normal(44, K, 0.2)
    outs = [torch.zeros(B, N, device=gpu) for _, N, _ in shapes]
    tfq.gemv_multi_fused(Ws, torch.from_numpy(x).to(gpu), outs, rmsnorm=torch.from_numpy(gamma).to(gpu), eps=1e-6,
                         gamma_plus_one=plus_one)
    xn = np.stack([O.rmsnorm(x[b], gamma, 1e-6, plus_one) for b in range(B)])
    for (n, N, _), o in zip(shapes, outs):
        ref = O.matmul(fmt, pays[n], N, K, xn)
        got = o.cpu().numpy()
        assert np.abs(got - ref).max() / np.abs(ref).max() <= 1e-3, (n, fmt)


@pytest.mark.parametrize("fmt", ["B32S4", "Q_G_4"])
@pytest.mark.parametrize("B,mid", [(1, "f32"), (2, "bf16"), (3, "f32")])
def test_swiglu_prologue_matches_oracle(O, tfq, gpu, fmt, B, mid):
    """down(silu(g) * u) with the elementwise step inside the down launch (Qwen35Engine::mlp_step)."""
    import torch
    F, D = 3584, 1024
    pay = O.encode_tensor(fmt, O.rng_normal(70, D * F, 0.02))
    W = tfq.Weight(fmt, D, F, pay)
    g = O.rng_normal(71, B * F, 1.0).reshape(B, F)
    u = O.rng_normal(72, B * F, 1.0).reshape(B, F)
    y = torch.zeros(B, D, device=gpu)
    tfq.gemv_multi_fused([W], torch.from_numpy(g).to(gpu), [y], swiglu_up=torch.from_numpy(u).to(gpu),
                         mid_dtype=torch.bfloat16 if mid == "bf16" else torch.float32)
    h = O.silu_mul(g.reshape(-1), u.reshape(-1)).reshape(B, F)
    if mid == "bf16":
        h = O.bf16_round(h)
    ref = O.matmul(fmt, pay, D, F, h)
    tol = 1e-2 if mid == "bf16" else 1e-3
    assert np.abs(y.cpu().numpy() - ref).max() / np.abs(ref).max() <= tol


def test_prologue_rejects_untiled_formats(O, tfq, gpu):
    import torch
    pay = O.encode_tensor("Q_4", O.rng_normal(1, 256 * 256, 0.02))
    W = tfq.Weight("Q_4", 256, 256, pay)
    with pytest.raises(tfq.TfqError):
        tfq.gemv_multi_fused([W], torch.zeros(1, 256, device=gpu), [torch.zeros(1, 256, device=gpu)],
                             rmsnorm=torch.zeros(256, device=gpu))


@pytest.mark.parametrize("xdt,B", [("bf16", 1), ("bf16", 4), ("f32", 2)])
def test_accumulate_epilogue_adds_into_y(O, tfq, gpu, xdt, B):
    """ys += W x (the residual addition of a decoder layer) in the launch's epilogue."""
    import torch
    fmt, N, K = "B32S4", 1040, 2048
    pay = O.encode_tensor(fmt, O.rng_normal(80, N * K, 0.02))
    W = tfq.Weight(fmt, N, K, pay)
    x = O.rng_normal(81, B * K, 1.0).reshape(B, K)
    y0 = O.rng_normal(82, B * N, 1.0).reshape(B, N)
    if xdt == "bf16":
        x = O.bf16_round(x)
        xd = torch.from_numpy(x).to(gpu).bfloat16()
    else:
        xd = torch.from_numpy(x).to(gpu)
    y = torch.from_numpy(y0.copy()).to(gpu)
    tfq.gemv_multi_fused([W], xd, [y], accumulate=True)
    ref = y0 + O.matmul(fmt, pay, N, K, x)
    assert np.abs(y.cpu().numpy() - ref).max() / np.abs(ref).max() <= (1e-2 if xdt == "bf16" else 1e-3)
    with pytest.raises(tfq.TfqError):  # more rows than one pass carries
        tfq.gemv_multi_fused([W], torch.zeros(8, K, device=gpu).bfloat16(), [torch.zeros(8, N, device=gpu)], accumulate=True)


@pytest.mark.parametrize("fmt", ["B32S4", "Q_G_4", "B32S8"])
@pytest.mark.parametrize("xdt,B,norm,ydt", [("bf16", 1, False, "f32"), ("bf16", 4, False, "bf16"), ("f32", 2, False, "f32"),
                                          ("f32", 1, True, "bf16")])
def test_paired_gate_up_with_swiglu_epilogue(O, tfq, gpu, fmt, xdt, B, norm, ydt):
    """gate and up in one launch, silu(gate x) * (up x) written by its epilogue (Qwen35Engine::mlp_step), with and
    without RMSNorm in front; F = 1040 leaves a partial last tile."""
    import torch
    F, D = 1040, 2048
    pg = O.encode_tensor(fmt, O.rng_normal(90, F * D, 0.02))
    pu = O.encode_tensor(fmt, O.rng_normal(91, F * D, 0.02))
    Wg, Wu = tfq.Weight(fmt, F, D, pg), tfq.Weight(fmt, F, D, pu)
    x = O.rng_normal(92, B * D, 1.0).reshape(B, D)
    gamma = O.rng_normal(93, D, 0.2)
    if xdt == "bf16":
        x = O.bf16_round(x)
        xd = torch.from_numpy(x).to(gpu).bfloat16()
    else:
        xd = torch.from_numpy(x).to(gpu)
    xin = np.stack([O.rmsnorm(x[b], gamma) for b in range(B)]) if norm else x
    h = torch.zeros(B, F, device=gpu, dtype=torch.bfloat16 if ydt == "bf16" else torch.float32)
    tfq.gemv_multi_fused([Wg, Wu], xd, [h], pair_swiglu=True, rmsnorm=torch.from_numpy(gamma).to(gpu) if norm else None)
    ref = O.silu_mul(O.matmul(fmt, pg, F, D, xin).reshape(-1), O.matmul(fmt, pu, F, D, xin).reshape(-1)).reshape(B, F)
    tol = 1e-2 if (xdt == "bf16" or ydt == "bf16") else 1e-3
    assert np.abs(h.float().cpu().numpy() - ref).max() / np.abs(ref).max() <= tol
