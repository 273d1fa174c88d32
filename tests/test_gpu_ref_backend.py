"""The reference's ComputeBackend interface (include/quant/backend.h:77-108) subclassed for GPU_HIP over this
library's operators, COMPILED against the reference's own headers and Tensor (oracle/ref_backend_glue.cpp ->
oracle/_ref/libref_backend.so, built where the reference tree is present) and driven through a ComputeBackend
pointer: every virtual operator against numpy (float64 sums; the arithmetic of src/math/math.cpp).  The file is
skipped where the library was never built."""
import ctypes as C
import math
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "oracle", "_ref", "libref_backend.so")
f32p = C.POINTER(C.c_float)


def pf(a):
    return a.ctypes.data_as(f32p)


def close(got, ref, tol):
    return float(np.abs(got.astype(np.float64) - ref).max()) <= tol * max(1e-30, float(np.abs(ref).max()))


@pytest.fixture(scope="module")
def glue(gpu):
    if not os.path.exists(LIB):
        pytest.skip("oracle/_ref/libref_backend.so was not built (it needs the reference tree)")
    d = C.CDLL(LIB)
    ll = C.c_longlong
    d.refglue_name.restype = C.c_char_p
    d.refglue_memory_total.restype = ll
    d.refglue_gemm.argtypes = [C.c_float, f32p, f32p, C.c_float, f32p, ll, ll, ll]
    d.refglue_gemv.argtypes = [C.c_float, f32p, f32p, C.c_float, f32p, ll, ll]
    d.refglue_softmax.argtypes = [f32p, f32p, ll, ll, ll, C.c_int]
    d.refglue_layer_norm.argtypes = [f32p, f32p, f32p, C.c_float, f32p, ll, ll]
    d.refglue_rms_norm.argtypes = [f32p, f32p, C.c_float, f32p, ll, ll]
    d.refglue_unary.argtypes = [C.c_int, C.c_float, f32p, f32p, ll]
    d.refglue_binary.argtypes = [C.c_int, f32p, f32p, f32p, ll]
    return d


def test_identity(glue):
    assert glue.refglue_name() == b"GPU_HIP"
    assert glue.refglue_is_gpu_hip() == 1
    assert glue.refglue_available() == 1
    assert glue.refglue_memory_total() > 100 * 2**30


@pytest.mark.parametrize("M,N,K,alpha,beta", [(1, 1, 1, 1.0, 0.0), (33, 65, 17, 0.5, -1.5), (300, 257, 515, 1.0, 1.0)])
def test_gemm_and_gemv(O, glue, M, N, K, alpha, beta):
    A = O.rng_normal(1, M * K, 1.0).reshape(M, K)
    B = O.rng_normal(2, K * N, 1.0).reshape(K, N)
    C0 = O.rng_normal(3, M * N, 1.0).reshape(M, N)
    out = C0.copy()
    assert glue.refglue_gemm(alpha, pf(A), pf(B), beta, pf(out), M, N, K) == 1
    assert close(out, alpha * (A.astype(np.float64) @ B.astype(np.float64)) + beta * C0, 1e-5)
    x = O.rng_normal(4, K, 1.0)
    y0 = O.rng_normal(5, M, 1.0)
    y = y0.copy()
    assert glue.refglue_gemv(alpha, pf(A), pf(x), beta, pf(y), M, K) == 1
    assert close(y, alpha * (A.astype(np.float64) @ x.astype(np.float64)) + beta * y0, 1e-5)


@pytest.mark.parametrize("axis", [0, 1, 2, -1])
def test_softmax_over_any_axis(O, glue, axis):
    shape = (5, 33, 7)
    x = O.rng_normal(6, int(np.prod(shape)), 2.0).reshape(shape)
    y = np.zeros(shape, np.float32)
    assert glue.refglue_softmax(pf(x), pf(y), *shape, axis) == 1
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(axis=axis, keepdims=True))
    assert close(y, e / e.sum(axis=axis, keepdims=True), 1e-5)


def test_norms(O, glue):
    rows, n = 19, 515
    x = O.rng_normal(7, rows * n, 1.5).reshape(rows, n)
    g = O.rng_normal(8, n, 1.0)
    b = O.rng_normal(9, n, 1.0)
    y = np.zeros((rows, n), np.float32)
    x64 = x.astype(np.float64)
    assert glue.refglue_rms_norm(pf(x), pf(g), 1e-6, pf(y), rows, n) == 1
    assert close(y, x64 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + 1e-6) * g, 1e-5)
    assert glue.refglue_layer_norm(pf(x), pf(g), pf(b), 1e-5, pf(y), rows, n) == 1
    mu = x64.mean(axis=1, keepdims=True)
    var = ((x64 - mu) ** 2).mean(axis=1, keepdims=True)
    assert close(y, (x64 - mu) / np.sqrt(var + 1e-5) * g + b, 1e-5)


def test_elementwise(O, glue):
    n = 100003
    a = O.rng_normal(10, n, 2.0)
    b = O.rng_normal(11, n, 2.0)
    y = np.zeros(n, np.float32)
    a64 = a.astype(np.float64)
    assert glue.refglue_unary(0, 0.0, pf(a), pf(y), n) == 1
    assert np.array_equal(y, np.maximum(a, 0.0))
    assert glue.refglue_unary(2, 0.0, pf(a), pf(y), n) == 1
    assert close(y, a64 / (1.0 + np.exp(-a64)), 1e-6)
    assert glue.refglue_unary(1, 0.0, pf(a), pf(y), n) == 1  # gelu, the erf form
    assert close(y, 0.5 * a64 * (1.0 + np.vectorize(math.erf)(a64 * 0.7071067811865475)), 1e-6)
    assert glue.refglue_unary(3, -2.5, pf(a), pf(y), n) == 1
    assert np.array_equal(y, (np.float32(-2.5) * a).astype(np.float32))
    assert glue.refglue_binary(0, pf(a), pf(b), pf(y), n) == 1
    assert np.array_equal(y, a + b)
    assert glue.refglue_binary(1, pf(a), pf(b), pf(y), n) == 1
    assert np.array_equal(y, a * b)
