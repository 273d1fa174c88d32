"""The reference-named C++ entry points (libtfq_shims.so) driven from host buffers, against the
oracle.  Codes and decoded weights bit-exact; matmul outputs max |y - y_ref| / max |y_ref| <= 1e-3
(fp32 activations)."""
import ctypes as C
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = 1e-3

u8p, f32p = C.POINTER(C.c_uint8), C.POINTER(C.c_float)


def p8(a):
    return a.ctypes.data_as(u8p)


def pf(a):
    return a.ctypes.data_as(f32p)


def rel_err(y, ref):
    return float(np.abs(y.astype(np.float64) - ref).max() / np.abs(ref).max())


@pytest.fixture(scope="module")
def drv(gpu):
    path = os.path.join(ROOT, "tests", "libshim_driver.so")
    if not os.path.exists(path):
        pytest.fail("tests/libshim_driver.so is missing: run __graft_entry__.build()")
    d = C.CDLL(path)
    d.drv_quantize_block.restype = C.c_long
    d.drv_quantize_block.argtypes = [C.c_uint8, f32p, C.c_int, u8p, C.c_size_t]
    d.drv_dequantize_block.argtypes = [C.c_uint8, u8p, C.c_size_t, C.c_uint32, f32p]
    d.drv_claimed_bytes.restype = C.c_size_t
    d.drv_claimed_bytes.argtypes = [C.c_uint8, C.c_uint32]
    d.drv_quant4_gemm.argtypes = [u8p, C.POINTER(C.c_uint16), f32p, f32p, C.c_int, C.c_int, C.c_int]
    d.drv_quant8_gemm.argtypes = [u8p, f32p, f32p, f32p, C.c_int, C.c_int, C.c_int]
    d.drv_lutn_gemm.argtypes = [C.c_int, u8p, C.c_void_p, f32p, f32p, C.c_int, C.c_int, C.c_int]
    d.drv_q24_encode.argtypes = [f32p, u8p, C.c_int]
    d.drv_q24_decode.argtypes = [u8p, f32p, C.c_int]
    d.drv_gemv_quant_tiled.argtypes = [u8p, C.c_float, f32p, f32p, C.c_int, C.c_int]
    d.drv_gemv_quant4_tiled.argtypes = [u8p, C.POINTER(C.c_uint16), C.c_float, f32p, f32p, C.c_int, C.c_int]
    d.drv_gemv_quant8_tiled.argtypes = [u8p, f32p, C.c_float, f32p, f32p, C.c_int, C.c_int]
    d.drv_gemv_quant_batch.argtypes = [u8p, C.c_float, f32p, f32p, C.c_int, C.c_int, C.c_int]
    d.drv_gemv_quant4_batch.argtypes = [u8p, C.POINTER(C.c_uint16), C.c_float, f32p, f32p, C.c_int, C.c_int, C.c_int]
    d.drv_gemv_quant8_batch.argtypes = [u8p, f32p, C.c_float, f32p, f32p, C.c_int, C.c_int, C.c_int]
    d.drv_blockrow_gemm.argtypes = [C.c_uint8, C.c_int64, C.c_int64, u8p, C.c_size_t, f32p, f32p, C.c_int]
    d.drv_mlp_step.argtypes = [C.c_uint8, C.c_int64, C.c_int64, u8p, u8p, u8p, C.c_size_t, C.c_size_t, f32p, f32p]
    d.drv_tensor_round_trip.restype = C.c_long
    d.drv_tensor_round_trip.argtypes = [C.c_uint8, f32p, C.c_int64, u8p, C.c_size_t, C.POINTER(C.c_uint32), f32p]
    return d


def test_claimed_bytes_are_ceil_of_bpw(O, drv):
    for name, want in [("Q_G_4", 144), ("Q_4", 128), ("Q_G_8", 272), ("Q_G_3", 112), ("Q_G_2", 84), ("B32S4", 144)]:
        assert drv.drv_claimed_bytes(O.FMT[name], 256) == want


@pytest.mark.parametrize("fmt", ["B32S4", "B32S8", "Q_32", "Q_G_4", "Q_G_3", "Q_G_2", "SB256A3", "Q_16", "Q_G_24", "Q_1", "Q_G_1_K_H"])
def test_quantize_block_all_codes_bit_exact(O, drv, fmt):
    w = O.rng_normal(7, 256, 0.02)
    want = O.encode_block(fmt, w)
    out = np.zeros(2048, np.uint8)
    n = drv.drv_quantize_block(O.FMT[fmt], pf(w), 256, p8(out), out.size)
    assert n == len(want)
    assert np.array_equal(out[:n], want)


def test_quantize_block_all_reports_failure_like_the_reference(O, drv):
    w = O.rng_normal(7, 256, 0.02)
    out = np.zeros(2048, np.uint8)
    # unknown wire id: false, both vectors left empty
    assert drv.drv_quantize_block(200, pf(w), 256, p8(out), out.size) == -1


@pytest.mark.parametrize("fmt", ["Q_G_4", "Q_4", "Q_8", "Q_G_8", "Q_G_3", "Q_G_2", "B32S4", "B32S8", "SB256A3", "SB256A2"])
def test_dequantize_block_all_bit_exact(O, drv, fmt):
    w = O.rng_normal(11, 256, 0.02)
    pay = O.encode_block(fmt, w)
    want = O.decode_block(fmt, pay, 256)
    got = np.full(256, 7.0, np.float32)
    drv.drv_dequantize_block(O.FMT[fmt], p8(pay), pay.size, 256, pf(got))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # a truncated payload decodes as if the missing bytes were zero
    cut = pay[: pay.size // 2].copy()
    want = O.decode_block(fmt, np.concatenate([cut, np.zeros(pay.size - cut.size, np.uint8)]), 256)
    drv.drv_dequantize_block(O.FMT[fmt], p8(cut), cut.size, 256, pf(got))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dequantize_block_all_unhandled_format_leaves_zeros(drv):
    got = np.full(256, 7.0, np.float32)
    pay = np.ones(64, np.uint8)
    drv.drv_dequantize_block(200, p8(pay), pay.size, 256, pf(got))
    assert not got.any()


def test_lookup_gemms(O, drv):
    rs = np.random.RandomState(3)
    M, N, K = 3, 5, 256
    packed = rs.randint(0, 256, M * N * K // 2).astype(np.uint8)
    cb16 = rs.randn(16).astype(np.float16).view(np.uint16)
    act = rs.randn(N, K).astype(np.float32)
    out = np.zeros((M, N), np.float32)
    drv.drv_quant4_gemm(p8(packed), cb16.ctypes.data_as(C.POINTER(C.c_uint16)), pf(act), pf(out), M, N, K)
    assert rel_err(out, O.quant4_gemm(packed, cb16, act, M, N, K)) <= TOL
    idx = rs.randint(0, 256, (N, K)).astype(np.uint8)
    cb = rs.randn(256).astype(np.float32)
    act8 = rs.randn(M, K).astype(np.float32)
    drv.drv_quant8_gemm(p8(idx), pf(cb), pf(act8), pf(out), M, N, K)
    assert rel_err(out, O.quant8_gemm(idx, cb, act8, M, N, K)) <= TOL


def test_wide_lookup_gemms_and_fp24(O, drv):
    """q3_gemm / q6_gemm / q12_gemm / q24_gemm / q24_encode / q24_decode (include/quant/kernel.h:36-54)."""
    rs = np.random.RandomState(8)
    M, N, K = 3, 5, 200
    act = rs.randn(N, K).astype(np.float32)
    w = rs.randn(M * N * K).astype(np.float32)
    packed24 = np.zeros(3 * w.size, np.uint8)
    drv.drv_q24_encode(pf(w), p8(packed24), w.size)
    assert np.array_equal(packed24, O.fp24_encode(w))
    back = np.zeros_like(w)
    drv.drv_q24_decode(p8(packed24), pf(back), w.size)
    assert np.array_equal(back.view(np.uint32), O.fp24_decode(packed24).view(np.uint32))
    for bits in (3, 6, 12, 24):
        print(f"shim lutn bits={bits}", flush=True)
        if bits == 24:
            packed, cb, cbp = packed24, None, None
        else:
            packed = rs.randint(0, 256, M * N * ((K * bits + 7) // 8)).astype(np.uint8)
            cb = rs.randn(4096).astype(np.float16).view(np.uint16) if bits == 12 else rs.randn(1 << bits).astype(np.float32)
            cbp = cb.ctypes.data
        out = np.zeros((M, N), np.float32)
        drv.drv_lutn_gemm(bits, p8(packed), cbp, pf(act), pf(out), M, N, K)
        assert rel_err(out, O.lutn_gemm(bits, packed, cb, act, M, N, K)) <= TOL


def test_production_gemvs(O, drv):
    rs = np.random.RandomState(5)
    M, N, K = 96, 3, 512
    X = rs.randn(N, K).astype(np.float32)
    Y = np.zeros((N, M), np.float32)
    y = np.zeros(M, np.float32)
    cb16 = rs.randn(16).astype(np.float16).view(np.uint16)
    cb16p = cb16.ctypes.data_as(C.POINTER(C.c_uint16))
    cb8 = rs.randn(256).astype(np.float32)
    w2 = rs.randint(0, 256, (M, K // 4)).astype(np.uint8)
    w4 = rs.randint(0, 256, (M, K // 2)).astype(np.uint8)
    w8 = rs.randint(0, 256, (M, K)).astype(np.uint8)
    drv.drv_gemv_quant_batch(p8(w2), 0.5, pf(X), pf(Y), M, N, K)
    assert rel_err(Y, O.lut_gemv_batch(2, w2, None, 0.5, X, M, N, K)) <= TOL
    drv.drv_gemv_quant4_batch(p8(w4), cb16p, 0.5, pf(X), pf(Y), M, N, K)
    assert rel_err(Y, O.lut_gemv_batch(4, w4, cb16, 0.5, X, M, N, K)) <= TOL
    drv.drv_gemv_quant8_batch(p8(w8), pf(cb8), 0.5, pf(X), pf(Y), M, N, K)
    assert rel_err(Y, O.lut_gemv_batch(8, w8, cb8, 0.5, X, M, N, K)) <= TOL
    drv.drv_gemv_quant_tiled(p8(w2), 2.0, pf(X[0]), pf(y), M, K)
    assert rel_err(y, O.lut_gemv_batch(2, w2, None, 2.0, X[:1], M, 1, K)[0]) <= TOL
    drv.drv_gemv_quant4_tiled(p8(w4), cb16p, 2.0, pf(X[0]), pf(y), M, K)
    assert rel_err(y, O.lut_gemv_batch(4, w4, cb16, 2.0, X[:1], M, 1, K)[0]) <= TOL
    drv.drv_gemv_quant8_tiled(p8(w8), pf(cb8), 2.0, pf(X[0]), pf(y), M, K)
    assert rel_err(y, O.lut_gemv_batch(8, w8, cb8, 2.0, X[:1], M, 1, K)[0]) <= TOL


@pytest.mark.parametrize("fmt", ["Q_G_4", "B32S4", "Q_G_8"])
@pytest.mark.parametrize("B", [1, 5, 40, 512])
def test_block_row_matmul_like_the_engine_gemm(O, drv, fmt, B):
    """B = 40 and 512 (the engine's MAX_BATCH): fp32 rows go through the 16-row decode kernel as a bf16 high and low part."""
    N, K = 96, 1024
    w = O.rng_normal(42, N * K, 0.02)
    X = O.rng_normal(43, B * K, 1.0).reshape(B, K)
    pay = O.encode_tensor(fmt, w)
    Y = np.zeros((B, N), np.float32)
    assert drv.drv_blockrow_gemm(O.FMT[fmt], N, K, p8(pay), pay.size, pf(X), pf(Y), B) == 1
    assert rel_err(Y, O.matmul(fmt, pay, N, K, X)) <= TOL
    # K not a multiple of 256: construction fails, nothing is written (the engine returns silently)
    Y[:] = 7.0
    assert drv.drv_blockrow_gemm(O.FMT[fmt], N, K - 1, p8(pay), pay.size, pf(X), pf(Y), B) == 0
    assert (Y == 7.0).all()


def test_mlp_step(O, drv):
    D, F = 512, 768
    fmt = "B32S4"
    g = O.encode_tensor(fmt, O.rng_normal(1, F * D, 0.05))
    u = O.encode_tensor(fmt, O.rng_normal(2, F * D, 0.05))
    d = O.encode_tensor(fmt, O.rng_normal(3, D * F, 0.05))
    x = O.rng_normal(4, D, 1.0)
    out = np.zeros(D, np.float32)
    assert drv.drv_mlp_step(O.FMT[fmt], D, F, p8(g), p8(u), p8(d), g.size, d.size, pf(x), pf(out)) == 1
    gate = O.matmul(fmt, g, F, D, x[None])[0]
    up = O.matmul(fmt, u, F, D, x[None])[0]
    mid = O.silu_mul(gate, up)
    want = O.matmul(fmt, d, D, F, mid[None])[0]
    assert rel_err(out, want) <= TOL


def test_tensor_codec_round_trip(O, drv):
    n = 256 * 37
    w = O.rng_normal(9, n, 0.02)
    fmt = "B32S4"
    want = O.encode_tensor(fmt, w)
    pay = np.zeros(want.size + 16, np.uint8)
    sizes = np.zeros(n // 256, np.uint32)
    dec = np.zeros(n, np.float32)
    got = drv.drv_tensor_round_trip(O.FMT[fmt], pf(w), n, p8(pay), pay.size, sizes.ctypes.data_as(C.POINTER(C.c_uint32)), pf(dec))
    assert got == want.size
    assert np.array_equal(pay[:got], want)
    assert (sizes == 144).all()
    assert np.array_equal(dec.view(np.uint32), O.decode_tensor(fmt, want, n).view(np.uint32))


@pytest.mark.parametrize("fmt,tail", [("Q_G_4", 100), ("Q_4", 33), ("Q_G_8", 160), ("B32S4", 96)])
def test_tensor_codec_short_last_block(O, drv, fmt, tail):
    """A tensor whose size is not a multiple of 256: the last block is short
    (FormatRegistry::quantize, src/codec/format_registry.cpp:168-207)."""
    n = 256 * 5 + tail
    w = O.rng_normal(11, n, 0.02)
    want = O.encode_tensor(fmt, w)
    pay = np.zeros(want.size + 16, np.uint8)
    sizes = np.zeros(6, np.uint32)
    dec = np.zeros(n, np.float32)
    got = drv.drv_tensor_round_trip(O.FMT[fmt], pf(w), n, p8(pay), pay.size, sizes.ctypes.data_as(C.POINTER(C.c_uint32)), pf(dec))
    assert got == want.size
    assert np.array_equal(pay[:got], want)
    assert (sizes[:5] == O.block_bytes(fmt, 256)).all() and sizes[5] == O.block_bytes(fmt, tail)
    assert np.array_equal(dec.view(np.uint32), O.decode_tensor(fmt, want, n).view(np.uint32))
