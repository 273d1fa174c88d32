"""Prefill GEMM (MFMA path) through the C ABI.  Gate: max |y - y_ref| / max |y_ref| <= 1e-2
(bf16 activations, bf16 or fp32 output, fp32 accumulate)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOL = 1e-2


def rel_err(y, ref):
    return float(np.abs(y.astype(np.float64) - ref).max() / np.abs(ref).max())


@pytest.mark.parametrize("fmt", ["Q_G_4", "B32S4", "Q_G_3", "B32S8", "Q_G_8", "Q_8"])
@pytest.mark.parametrize("M,N,K", [(17, 48, 256), (64, 128, 512), (300, 200, 1024), (512, 33, 2304), (256, 384, 4096)])
def test_gemm_against_oracle(O, tfq, gpu, fmt, M, N, K):
    import torch
    print(f"gemm {fmt} M={M} N={N} K={K}", flush=True)
    w = O.rng_normal(42, N * K, 0.02)
    x = O.bf16_round(O.rng_normal(43, M * K, 1.0).reshape(M, K))
    pay = O.encode_tensor(fmt, w)
    ref = O.matmul(fmt, pay, N, K, x)
    W = tfq.Weight(fmt, N, K, pay)
    xt = torch.from_numpy(x).to(gpu).bfloat16()
    y = W.gemm(xt).cpu().numpy()
    assert y.shape == (M, N)
    assert rel_err(y, ref) <= TOL
    yb = W.gemm(xt, out_dtype=torch.bfloat16).float().cpu().numpy()
    assert rel_err(yb, ref) <= TOL
    # without scratch memory (no K split) the sums are the same up to the order of the fp32 additions
    y0 = W.gemm(xt, workspace=False).cpu().numpy()
    assert rel_err(y0, ref) <= TOL and rel_err(y, y0) <= 1e-5
    # the tile kernel and the 16-row GEMV path agree to the bf16 rounding of the decoded weights
    y16 = torch.cat([W.gemv(xt[i:i + 16]) for i in range(0, M, 16)]).cpu().numpy()
    assert rel_err(y, y16) <= 5e-3
    W.close()


def test_gemm_fp32_activations_take_the_exact_path(O, tfq, gpu):
    import torch
    M, N, K = 40, 64, 512
    w = O.rng_normal(42, N * K, 0.02)
    x = O.rng_normal(43, M * K, 1.0).reshape(M, K)
    pay = O.encode_tensor("Q_G_4", w)
    W = tfq.Weight("Q_G_4", N, K, pay)
    y = W.gemm(torch.from_numpy(x).to(gpu)).cpu().numpy()
    assert rel_err(y, O.matmul("Q_G_4", pay, N, K, x)) <= 1e-3
    W.close()


@pytest.mark.parametrize("fmt", ["B32S4", "Q_G_4", "Q_G_3", "B32S8", "Q_G_8"])
@pytest.mark.parametrize("N,K", [(14336, 4096), (4096, 14336)])
def test_config3_prefill_shapes(tfq, gpu, N, K, fmt):
    """M = 2048 tokens, bf16 activations N(0,1), block-32 weights from N(0, 0.02), bf16 output:
    against a dense fp32 torch matmul of the decoded matrix (for the companded 8-bit grid that also
    checks the line that stands for the grid in the matmul against the exact table of the decode)."""
    import torch
    M = 2048
    g = torch.Generator(device="cuda").manual_seed(3)
    w = torch.randn(N * K, device=gpu, generator=g) * 0.02
    print(f"prefill {fmt} M={M} N={N} K={K}", flush=True)
    W = tfq.Weight(fmt, N, K, tfq.encode(fmt, w))
    del w
    x = torch.randn(M, K, device=gpu, generator=g).bfloat16()
    y = W.gemm(x, out_dtype=torch.bfloat16)
    dense = W.decode()
    want = x.float() @ dense.T
    err = float((y.float() - want).abs().max() / want.abs().max())
    assert err <= TOL, err
    # linearity in x for power-of-two factors is exact
    y2 = W.gemm((x.float() * 2).bfloat16(), out_dtype=torch.float32)
    y1 = W.gemm(x, out_dtype=torch.float32)
    assert torch.equal(y2, 2 * y1)
    W.close()


@pytest.mark.parametrize("fmt", ["B32S4", "B32S8"])
def test_prefill_full_grid_is_repeatable(tfq, gpu, fmt):
    """On a full grid the step of the tile kernel runs in two barrier-separated phases with the two halves of a
    workgroup one phase apart, on LDS buffers that are reused every other step: forty launches of the gate shape
    give the same bits every time, and the rows of a tile do not depend on what the other rows hold (a call with
    half the tokens equals the first half of the whole call)."""
    import torch
    N, K, M = 14336, 4096, 2048
    g = torch.Generator(device="cuda").manual_seed(9)
    W = tfq.Weight(fmt, N, K, tfq.encode(fmt, torch.randn(N * K, device=gpu, generator=g) * 0.02))
    x = torch.randn(M, K, device=gpu, generator=g).bfloat16()
    ref = W.gemm(x, out_dtype=torch.float32).clone()
    for _ in range(40):
        assert torch.equal(W.gemm(x, out_dtype=torch.float32), ref)
    half = W.gemm(x[:M // 2], out_dtype=torch.float32)
    assert torch.equal(half, ref[:M // 2])
    W.close()
