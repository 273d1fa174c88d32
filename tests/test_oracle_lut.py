"""Pins of the oracle's codebook-lookup operators (kernel::quant4_gemm, kernel::quant8_gemm,
prod::gemv_quant*_batch) without running the reference: brute-force numpy restatements from the
index conventions, closed forms, and (where it is built) the compiled reference."""
import numpy as np
import pytest


def half_bits(values):
    return np.asarray(values, np.float16).view(np.uint16)


def test_quant4_gemm_row_per_output_pair(O):
    """out[m][n] uses packed row (m*N+n) and activation row n (src/kernel/kernel_quant4.cpp:24-43)."""
    rs = np.random.RandomState(0)
    M, N, K = 3, 5, 64
    packed = rs.randint(0, 256, M * N * K // 2).astype(np.uint8)
    cb = half_bits(rs.randn(16))
    act = rs.randn(N, K).astype(np.float32)
    nib = np.stack([packed & 15, packed >> 4], -1).reshape(M, N, K)
    want = (cb.view(np.float16).astype(np.float64)[nib] * act[None].astype(np.float64)).sum(-1)
    got = O.quant4_gemm(packed, cb, act, M, N, K)
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()
    # a transposed activation index (m instead of n) must not pass
    wrong = (cb.view(np.float16).astype(np.float64)[nib] * act[:M, None].astype(np.float64)).sum(-1)
    assert np.abs(got - wrong).max() > 1e-2 * np.abs(want).max()


def test_quant8_gemm_conventional(O):
    rs = np.random.RandomState(1)
    M, N, K = 4, 6, 50
    idx = rs.randint(0, 256, (N, K)).astype(np.uint8)
    cb = rs.randn(256).astype(np.float32)
    act = rs.randn(M, K).astype(np.float32)
    want = act.astype(np.float64) @ cb.astype(np.float64)[idx].T
    got = O.quant8_gemm(idx, cb, act, M, N, K)
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()


@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("K", [64, 37])
def test_lut_gemv_batch_brute_force(O, bits, K):
    """Y[n][m] = scale * sum_k value(m,k) X[n][k], rows of ceil(K*bits/8) bytes, low bits first
    (src/kernel/kernel_production.cpp:68-117)."""
    rs = np.random.RandomState(2 + bits)
    M, N = 7, 3
    row_bytes = (K * bits + 7) // 8
    packed = rs.randint(0, 256, (M, row_bytes)).astype(np.uint8)
    X = rs.randn(N, K).astype(np.float32)
    if bits == 2:
        cb, table = None, np.array([-1.0, 0.0, 1.0, 1.0])
    elif bits == 4:
        cb = half_bits(rs.randn(16))
        table = cb.view(np.float16).astype(np.float64)
    else:
        cb = rs.randn(256).astype(np.float32)
        table = cb.astype(np.float64)
    per = 8 // bits
    k = np.arange(K)
    codes = (packed[:, k // per] >> ((k % per) * bits)) & ((1 << bits) - 1)
    want = 0.37 * (X.astype(np.float64) @ table[codes].T)
    got = O.lut_gemv_batch(bits, packed, cb, 0.37, X, M, N, K)
    assert got.shape == (N, M)
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()


def test_constant_codebook_closed_form(O):
    """Every centroid = c  =>  y = scale * c * sum(x), whatever the indices are."""
    rs = np.random.RandomState(9)
    M, N, K = 5, 2, 96
    packed = rs.randint(0, 256, (M, K // 2)).astype(np.uint8)
    X = rs.randn(N, K).astype(np.float32)
    got = O.lut_gemv_batch(4, packed, half_bits(np.full(16, 0.5)), 2.0, X, M, N, K)
    want = np.repeat(X.astype(np.float64).sum(1)[:, None], M, 1)
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()


def test_lookup_gemms_equal_the_compiled_reference(O):
    if not O.have_ref():
        pytest.skip("compiled reference not built on this machine")
    rs = np.random.RandomState(4)
    M, N, K = 3, 4, 128
    packed = rs.randint(0, 256, M * N * K // 2).astype(np.uint8)
    cb16 = half_bits(rs.randn(16))
    act = rs.randn(N, K).astype(np.float32)
    a, b = O.quant4_gemm(packed, cb16, act, M, N, K), O.ref_quant4_gemm(packed, cb16, act, M, N, K)
    assert np.abs(a - b).max() <= 1e-5 * np.abs(b).max()  # the reference's AVX2 path sums in another order
    idx = rs.randint(0, 256, (N, K)).astype(np.uint8)
    cb = rs.randn(256).astype(np.float32)
    act8 = rs.randn(M, K).astype(np.float32)
    a, b = O.quant8_gemm(idx, cb, act8, M, N, K), O.ref_quant8_gemm(idx, cb, act8, M, N, K)
    assert np.abs(a - b).max() <= 1e-5 * np.abs(b).max()


def unpack_bits(rows, bits, K):
    """Codes of `bits` bits, low bits first, from byte rows [..., row_bytes] (brute force, bit by bit)."""
    b = np.unpackbits(rows, axis=-1, bitorder="little")[..., : K * bits].reshape(rows.shape[:-1] + (K, bits))
    return (b.astype(np.int64) << np.arange(bits)).sum(-1)


@pytest.mark.parametrize("bits", [3, 6, 12])
@pytest.mark.parametrize("K", [64, 37])
def test_lutn_gemm_brute_force(O, bits, K):
    """out[m][n] = sum_k codebook[code(m,n,k)] act[n][k], rows of ceil(K*bits/8) bytes per (m, n)
    (src/kernel/kernel_q3.cpp:18-44, kernel_q6.cpp:18-43, kernel_q12.cpp:24-50)."""
    rs = np.random.RandomState(20 + bits)
    M, N = 3, 4
    row_bytes = (K * bits + 7) // 8
    packed = rs.randint(0, 256, (M, N, row_bytes)).astype(np.uint8)
    act = rs.randn(N, K).astype(np.float32)
    if bits == 12:
        cb = half_bits(rs.randn(4096))
        table = cb.view(np.float16).astype(np.float64)
    else:
        cb = rs.randn(1 << bits).astype(np.float32)
        table = cb.astype(np.float64)
    want = (table[unpack_bits(packed, bits, K)] * act[None].astype(np.float64)).sum(-1)
    got = O.lutn_gemm(bits, packed, cb, act, M, N, K)
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()


def test_fp24_is_the_top_three_bytes_of_binary32(O):
    """float_to_fp24 / fp24_to_float (src/kernel/kernel_q24.cpp:28-45): truncation to 16 mantissa bits,
    most significant byte first; the round trip is exact for values with <= 16 mantissa bits."""
    rs = np.random.RandomState(5)
    w = np.concatenate([rs.randn(1000).astype(np.float32) * 10.0 ** rs.randint(-20, 20, 1000),
                        np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, 1e-45, 3.4e38], np.float32)]).astype(np.float32)
    packed = O.fp24_encode(w)
    be = w.view(np.uint32).astype(">u4").view(np.uint8).reshape(-1, 4)[:, :3]
    assert np.array_equal(packed.reshape(-1, 3), be)
    back = O.fp24_decode(packed)
    assert np.array_equal(back.view(np.uint32), w.view(np.uint32) & np.uint32(0xFFFFFF00))
    exact = np.float32(np.arange(-300, 300)) / np.float32(64)
    assert np.array_equal(O.fp24_decode(O.fp24_encode(exact)), exact)
    # truncation, never away from zero
    assert np.all(np.abs(back[np.isfinite(back)]) <= np.abs(w[np.isfinite(back)]))


def test_q24_gemm_brute_force(O):
    rs = np.random.RandomState(6)
    M, N, K = 3, 4, 50
    w = rs.randn(M, N, K).astype(np.float32)
    packed = O.fp24_encode(w)
    act = rs.randn(N, K).astype(np.float32)
    wt = (w.view(np.uint32) & np.uint32(0xFFFFFF00)).view(np.float32).astype(np.float64)
    want = (wt * act[None].astype(np.float64)).sum(-1)
    got = O.lutn_gemm(24, packed, None, act, M, N, K)
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()


def test_wide_lookup_gemms_equal_the_compiled_reference(O):
    if not O.have_ref():
        pytest.skip("compiled reference not built on this machine")
    rs = np.random.RandomState(7)
    M, N = 3, 5
    for bits, K in [(3, 64), (3, 40), (6, 64), (6, 36), (12, 64), (12, 30), (24, 64), (24, 19)]:
        row_bytes = (K * bits + 7) // 8
        act = rs.randn(N, K).astype(np.float32)
        if bits == 24:
            packed, cb = O.fp24_encode(rs.randn(M * N * K).astype(np.float32)), None
        else:
            packed = rs.randint(0, 256, M * N * row_bytes).astype(np.uint8)
            cb = half_bits(rs.randn(4096)) if bits == 12 else rs.randn(1 << bits).astype(np.float32)
        a, b = O.lutn_gemm(bits, packed, cb, act, M, N, K), O.ref_lutn_gemm(bits, packed, cb, act, M, N, K)
        assert np.abs(a - b).max() <= 1e-5 * np.abs(b).max(), (bits, K)
    w = rs.randn(777).astype(np.float32)
    packed, back = O.ref_fp24_round_trip(w)
    assert np.array_equal(packed, O.fp24_encode(w))
    assert np.array_equal(back, O.fp24_decode(packed))
