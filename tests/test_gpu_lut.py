"""Codebook-lookup operators on the device against the oracle's scalar restatements.
Gate: max |y - y_ref| / max |y_ref| <= 1e-3 (fp32 activations, fp32 accumulate)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOL = 1e-3


def rel_err(y, ref):
    return float(np.abs(y.astype(np.float64) - ref).max() / np.abs(ref).max())


def half_bits(values):
    return np.asarray(values, np.float16).view(np.uint16)


@pytest.mark.parametrize("M,N,K", [(1, 1, 32), (3, 5, 64), (2, 7, 256), (4, 16, 4096), (3, 5, 50), (2, 3, 33)])
def test_lut4_gemm(O, tfq, gpu, M, N, K):
    import torch
    print(f"lut4_gemm M={M} N={N} K={K}", flush=True)
    rs = np.random.RandomState(K)
    nbytes = (M * N * K + 1) // 2
    packed = rs.randint(0, 256, nbytes).astype(np.uint8)
    cb = half_bits(rs.randn(16))
    act = rs.randn(N, K).astype(np.float32)
    ref = O.quant4_gemm(packed, cb, act, M, N, K)
    y = tfq.lut4_gemm(torch.from_numpy(packed).to(gpu), cb, torch.from_numpy(act).to(gpu), M, N, K).cpu().numpy()
    assert rel_err(y, ref) <= TOL


@pytest.mark.parametrize("M,N,K", [(1, 1, 16), (4, 6, 50), (5, 64, 256), (16, 128, 4096), (33, 20, 1000)])
def test_lut8_gemm(O, tfq, gpu, M, N, K):
    import torch
    print(f"lut8_gemm M={M} N={N} K={K}", flush=True)
    rs = np.random.RandomState(K + 1)
    idx = rs.randint(0, 256, (N, K)).astype(np.uint8)
    cb = rs.randn(256).astype(np.float32)
    act = rs.randn(M, K).astype(np.float32)
    ref = O.quant8_gemm(idx, cb, act, M, N, K)
    y = tfq.lut8_gemm(torch.from_numpy(idx).to(gpu), cb, torch.from_numpy(act).to(gpu), M, N, K).cpu().numpy()
    assert rel_err(y, ref) <= TOL


@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("M,N,K", [(7, 1, 64), (7, 3, 37), (100, 5, 1024), (4096, 1, 4096), (512, 16, 4096)])
def test_lut_gemv_batch(O, tfq, gpu, bits, M, N, K):
    import torch
    print(f"lut_gemv_batch bits={bits} M={M} N={N} K={K}", flush=True)
    rs = np.random.RandomState(bits * 1000 + K)
    row_bytes = (K * bits + 7) // 8
    packed = rs.randint(0, 256, (M, row_bytes)).astype(np.uint8)
    X = rs.randn(N, K).astype(np.float32)
    cb = None if bits == 2 else half_bits(rs.randn(16)) if bits == 4 else rs.randn(256).astype(np.float32)
    ref = O.lut_gemv_batch(bits, packed, cb, 0.37, X, M, N, K)
    y = tfq.lut_gemv_batch(bits, torch.from_numpy(packed).to(gpu), cb, 0.37, torch.from_numpy(X).to(gpu), M, N, K)
    assert rel_err(y.cpu().numpy(), ref) <= TOL


def test_lut_rejects_bad_arguments(tfq, gpu):
    import torch
    x = torch.zeros(64, device=gpu)
    w = torch.zeros(64, dtype=torch.uint8, device=gpu)
    with pytest.raises(tfq.TfqError):
        tfq.lut_gemv_batch(3, w, np.zeros(16, np.uint16), 1.0, x, 1, 1, 64)
    with pytest.raises(tfq.TfqError):
        tfq.lut4_gemm(w, np.zeros(16, np.uint16), x, 0, 1, 64)


def test_device_memory_helpers_round_trip(tfq, gpu):
    import ctypes as C
    lib = tfq.lib()
    src = np.arange(1000, dtype=np.float32)
    dst = np.zeros_like(src)
    p = lib.tfq_malloc(src.nbytes)
    assert p
    assert lib.tfq_copy_to_device(p, src.ctypes.data, src.nbytes) == 0
    assert lib.tfq_copy_to_host(dst.ctypes.data, p, src.nbytes) == 0
    assert lib.tfq_stream_sync(None) == 0
    lib.tfq_free(p)
    assert np.array_equal(src, dst)
