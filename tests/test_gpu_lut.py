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


@pytest.mark.parametrize("bits", [3, 6, 12, 24])
@pytest.mark.parametrize("M,N,K", [(1, 1, 8), (3, 4, 64), (3, 4, 37), (2, 16, 4096), (5, 3, 1000), (64, 8, 512)])
def test_lutn_gemm(O, tfq, gpu, bits, M, N, K):
    """kernel::q3_gemm / q6_gemm / q12_gemm / q24_gemm (include/quant/kernel.h:36-54)."""
    import torch
    print(f"lutn_gemm bits={bits} M={M} N={N} K={K}", flush=True)
    rs = np.random.RandomState(bits * 100 + K)
    row_bytes = (K * bits + 7) // 8
    act = rs.randn(N, K).astype(np.float32)
    if bits == 24:
        packed, cb = O.fp24_encode(rs.randn(M * N * K).astype(np.float32)), None
    else:
        packed = rs.randint(0, 256, M * N * row_bytes).astype(np.uint8)
        cb = half_bits(rs.randn(4096)) if bits == 12 else rs.randn(1 << bits).astype(np.float32)
    ref = O.lutn_gemm(bits, packed, cb, act, M, N, K)
    y = tfq.lutn_gemm(bits, torch.from_numpy(packed).to(gpu), cb, torch.from_numpy(act).to(gpu), M, N, K)
    assert rel_err(y.cpu().numpy(), ref) <= TOL


@pytest.mark.parametrize("count", [1, 255, 4096, 1000003])
def test_fp24_encode_decode_bit_exact(O, tfq, gpu, count):
    import torch
    print(f"fp24 count={count}", flush=True)
    rs = np.random.RandomState(count % 1000)
    w = (rs.randn(count) * 10.0 ** rs.randint(-10, 10, count)).astype(np.float32)
    packed = tfq.fp24_encode(torch.from_numpy(w).to(gpu))
    assert np.array_equal(packed.cpu().numpy(), O.fp24_encode(w))
    back = tfq.fp24_decode(packed).cpu().numpy()
    assert np.array_equal(back.view(np.uint32), O.fp24_decode(O.fp24_encode(w)).view(np.uint32))


def test_lut_rejects_bad_arguments(tfq, gpu):
    import torch
    x = torch.zeros(64, device=gpu)
    w = torch.zeros(64, dtype=torch.uint8, device=gpu)
    with pytest.raises(tfq.TfqError):
        tfq.lut_gemv_batch(3, w, np.zeros(16, np.uint16), 1.0, x, 1, 1, 64)
    with pytest.raises(tfq.TfqError):
        tfq.lut4_gemm(w, np.zeros(16, np.uint16), x, 0, 1, 64)
    with pytest.raises(tfq.TfqError):
        tfq.lutn_gemm(5, w, np.zeros(32, np.float32), x, 1, 1, 64)


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
