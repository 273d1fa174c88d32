"""The dense fp32 operators behind a GPU_HIP ComputeBackend (tfq_dense_*, tfq::HipBackend) against the
arithmetic of the reference's CPU backend (src/math/math.cpp:50-309) restated in numpy: float64 where the
reference accumulates in double, float32 sequential order otherwise.  Tolerance 1e-5 relative to the largest
output (fp32 sums in a different order); elementwise operators 2 ulp-level (1e-6)."""
import ctypes as C
import math
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
f32p = C.POINTER(C.c_float)


def pf(a):
    return a.ctypes.data_as(f32p)


def close(got, ref, tol):
    return float(np.abs(got.astype(np.float64) - ref).max()) <= tol * max(1e-30, float(np.abs(ref).max()))


@pytest.fixture(scope="module")
def drv(gpu):
    d = C.CDLL(os.path.join(ROOT, "tests", "libshim_driver.so"))
    ll = C.c_longlong
    d.drv_backend_memory_total.restype = ll
    d.drv_backend_gemm.argtypes = [C.c_float, f32p, f32p, C.c_float, f32p, ll, ll, ll]
    d.drv_backend_gemv.argtypes = [C.c_float, f32p, f32p, C.c_float, f32p, ll, ll]
    d.drv_backend_softmax.argtypes = [f32p, f32p, ll, ll, ll]
    d.drv_backend_norm.argtypes = [C.c_int, f32p, f32p, f32p, C.c_float, f32p, ll, ll]
    d.drv_backend_unary.argtypes = [C.c_int, C.c_float, f32p, f32p, ll]
    d.drv_backend_binary.argtypes = [C.c_int, f32p, f32p, f32p, ll]
    return d


def test_backend_reports_the_device(drv):
    assert drv.drv_backend_available() == 1
    assert drv.drv_backend_memory_total() > 100 * 2**30  # 288 GB of HBM3E


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (33, 65, 17), (128, 128, 16), (300, 257, 515), (1024, 512, 2048)])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (0.5, -1.5)])
def test_gemm(O, drv, M, N, K, alpha, beta):
    A = O.rng_normal(1, M * K, 1.0).reshape(M, K)
    B = O.rng_normal(2, K * N, 1.0).reshape(K, N)
    C0 = O.rng_normal(3, M * N, 1.0).reshape(M, N)
    out = C0.copy()
    assert drv.drv_backend_gemm(alpha, pf(A), pf(B), beta, pf(out), M, N, K) == 1
    ref = alpha * (A.astype(np.float64) @ B.astype(np.float64)) + beta * C0
    assert close(out, ref, 1e-5)


def test_gemm_with_beta_zero_ignores_what_c_held(O, drv):
    A = O.rng_normal(1, 64 * 32, 1.0).reshape(64, 32)
    B = O.rng_normal(2, 32 * 48, 1.0).reshape(32, 48)
    out = np.full((64, 48), np.nan, np.float32)
    assert drv.drv_backend_gemm(1.0, pf(A), pf(B), 0.0, pf(out), 64, 48, 32) == 1
    assert close(out, A.astype(np.float64) @ B.astype(np.float64), 1e-5)


@pytest.mark.parametrize("M,N", [(1, 1), (77, 300), (4096, 1024)])
def test_gemv(O, drv, M, N):
    A = O.rng_normal(4, M * N, 1.0).reshape(M, N)
    x = O.rng_normal(5, N, 1.0)
    y0 = O.rng_normal(6, M, 1.0)
    y = y0.copy()
    assert drv.drv_backend_gemv(2.0, pf(A), pf(x), 0.25, pf(y), M, N) == 1
    assert close(y, 2.0 * (A.astype(np.float64) @ x) + 0.25 * y0, 1e-5)


@pytest.mark.parametrize("shape,axis", [((7, 129), 1), ((5, 33, 6), 1), ((4, 3, 1000), 2), ((50, 8), 0)])
def test_softmax_along_an_axis(O, drv, shape, axis):
    x = O.rng_normal(7, int(np.prod(shape)), 3.0).reshape(shape)
    y = np.zeros_like(x)
    outer = int(np.prod(shape[:axis]))
    inner = int(np.prod(shape[axis + 1:]))
    assert drv.drv_backend_softmax(pf(x), pf(y), outer, shape[axis], inner) == 1
    e = np.exp((x - x.max(axis=axis, keepdims=True)).astype(np.float32)).astype(np.float64)
    ref = e / e.sum(axis=axis, keepdims=True)
    assert close(y, ref, 1e-6)
    assert np.allclose(y.sum(axis=axis), 1.0, atol=1e-5)


@pytest.mark.parametrize("rows,n", [(1, 1), (9, 100), (64, 4096)])
def test_norms(O, drv, rows, n):
    x = O.rng_normal(8, rows * n, 2.0).reshape(rows, n) + np.float32(0.5)
    g = O.rng_normal(9, n, 1.0)
    b = O.rng_normal(10, n, 1.0)
    y = np.zeros_like(x)
    x64 = x.astype(np.float64)
    assert drv.drv_backend_norm(1, pf(x), pf(g), pf(b), 1e-5, pf(y), rows, n) == 1
    mu = x64.mean(axis=1, keepdims=True)
    var = ((x64 - mu) ** 2).mean(axis=1, keepdims=True)
    ref = ((x64 - mu) / np.sqrt(var + 1e-5)).astype(np.float32) * g + b
    assert close(y, ref.astype(np.float64), 1e-5)
    assert drv.drv_backend_norm(0, pf(x), pf(g), pf(b), 1e-6, pf(y), rows, n) == 1
    ref = (x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-6)).astype(np.float32) * g
    assert close(y, ref.astype(np.float64), 1e-5)


def test_elementwise(O, drv):
    n = 100003
    a = O.rng_normal(11, n, 2.0)
    b = O.rng_normal(12, n, 2.0)
    y = np.zeros_like(a)
    a64 = a.astype(np.float64)
    erf = np.vectorize(math.erf)
    for op, ref in ((0, np.maximum(a64, 0.0)), (1, 0.5 * a64 * (1.0 + erf(a64 * 0.7071067811865475))),
                    (2, a64 / (1.0 + np.exp(-a64))), (3, -1.75 * a64)):
        assert drv.drv_backend_unary(op, -1.75, pf(a), pf(y), n) == 1
        assert close(y, ref, 1e-6), op
    assert drv.drv_backend_binary(0, pf(a), pf(b), pf(y), n) == 1
    assert np.array_equal(y, a + b)
    assert drv.drv_backend_binary(1, pf(a), pf(b), pf(y), n) == 1
    assert np.array_equal(y, a * b)


def test_device_pointer_forms_fill_copy_and_errors(tfq, gpu):
    import torch
    L = tfq.lib()
    for name, args in (("tfq_dense_unary", [C.c_int, C.c_void_p, C.c_float, C.c_void_p, C.c_int64, C.c_void_p]),
                       ("tfq_dense_binary", [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]),
                       ("tfq_dense_gemm", [C.c_float, C.c_void_p, C.c_void_p, C.c_float, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_void_p])):
        getattr(L, name).argtypes = args
        getattr(L, name).restype = C.c_int
    y = torch.zeros(1000, device=gpu)
    assert L.tfq_dense_unary(5, None, 2.5, y.data_ptr(), 1000, None) == 0  # fill
    x = torch.arange(1000, device=gpu, dtype=torch.float32)
    z = torch.zeros(1000, device=gpu)
    assert L.tfq_dense_unary(4, x.data_ptr(), 0.0, z.data_ptr(), 1000, None) == 0  # copy
    torch.cuda.synchronize()
    assert bool((y == 2.5).all()) and torch.equal(x, z)
    assert L.tfq_dense_unary(99, x.data_ptr(), 0.0, z.data_ptr(), 1000, None) != 0
    assert L.tfq_dense_binary(0, x.data_ptr(), None, z.data_ptr(), 1000, None) != 0
    assert L.tfq_dense_gemm(1.0, x.data_ptr(), x.data_ptr(), 0.0, z.data_ptr(), 0, 10, 10, None) != 0
