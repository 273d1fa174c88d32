"""tfq_gemm_static (the entry point that allocates nothing) against tfq_gemm_ws, bit for bit: same kernels, the K-split
scratch in the library's static device array instead of a caller workspace.  Two calls in a row, the second with
a smaller input, so that what the first call left in the array is there when the second runs."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fmt", ["B32S4", "Q_G_4"])
def test_gemm_static_equals_workspace_form(O, tfq, gpu, fmt):
    import torch
    N, K = 1024, 4096  # few weight rows and a long K: the tile kernel splits K and uses the scratch
    pay = O.encode_tensor(fmt, O.rng_normal(91, N * K, 0.02))
    W = tfq.Weight(fmt, N, K, pay)
    lib = tfq.lib()
    assert lib.tfq_gemm_static_scratch_bytes() == 32 << 20
    for M in (384, 128):  # the second call is the smaller one
        x = torch.from_numpy(O.bf16_round(O.rng_normal(92 + M, M * K, 1.0)).reshape(M, K)).to(gpu).bfloat16()
        need = int(lib.tfq_gemm_workspace_bytes(W.handle, tfq.BF16, M))
        assert 0 < need <= 32 << 20, "the case must exercise the split"
        y_ws = W.gemm(x, out_dtype=torch.float32, workspace=True)
        y_st = torch.full((M, N), float("nan"), device=gpu)
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.tfq_gemm_static(W.handle, x.data_ptr(), tfq.BF16, M, y_st.data_ptr(), tfq.F32, stream)
        assert rc == 0, lib.tfq_last_error().decode()
        torch.cuda.synchronize()
        assert torch.equal(y_ws, y_st)
        # and both are the product: against the oracle on a few rows
        rows = [0, M // 2, M - 1]
        ref = O.matmul(fmt, pay, N, K, x[rows].float().cpu().numpy())
        got = y_st[rows].cpu().numpy()
        assert np.abs(got - ref).max() / np.abs(ref).max() <= 1e-2
    W.close()


def test_gemm_static_refuses_what_does_not_fit(O, tfq, gpu):
    """4096x14336 at 2048 rows splits K in two: 64 MiB of partial tiles, more than the static area holds.  The call
    is refused with TFQ_ERR_SHAPE before anything is launched, and y stays as it was."""
    import torch
    fmt, N, K, M = "B32S4", 4096, 14336, 2048
    lib = tfq.lib()
    w = torch.randn(N * K, device=gpu) * 0.02
    W = tfq.Weight(fmt, N, K, tfq.encode(fmt, w))
    need = int(lib.tfq_gemm_workspace_bytes(W.handle, tfq.BF16, M))
    assert need > 32 << 20, "the case must ask for more than the static area"
    x = torch.zeros(M, K, device=gpu).bfloat16()
    y = torch.full((M, N), 3.0, device=gpu)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.tfq_gemm_static(W.handle, x.data_ptr(), tfq.BF16, M, y.data_ptr(), tfq.F32, stream)
    assert rc == 3 and b"static area" in lib.tfq_last_error()
    torch.cuda.synchronize()
    assert bool((y == 3.0).all())
    W.close()
