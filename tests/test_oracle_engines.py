"""Pins of the oracle's in-memory engine restatements (engines::Q4Engine / Q8Engine, quant8 codec and
activation quantizer) without the reference: numpy brute force from the definitions, invariants, and
(where it is built) the compiled reference, bit for bit.  CPU only."""
import numpy as np
import pytest


def nearest_first(cb, v):
    """index of the first centroid at the smallest |v - c| (strict '<' scan)"""
    d = np.abs(v[:, None].astype(np.float32) - cb[None, :].astype(np.float32))
    return d.argmin(1)


@pytest.mark.parametrize("bits", [4, 8])
def test_quantize_per_block_brute_force(O, bits):
    """src/codec/quant_engines_quant4.cpp:102-133, quant_engines_quant8.cpp:92-117"""
    rs = np.random.RandomState(bits)
    cb = np.sort(rs.randn(1 << bits)).astype(np.float32) * np.float32(0.5)
    data = (rs.randn(700) * 0.05 + 0.02).astype(np.float32)
    bs = 256
    idx, scales = O.engine_quantize_per_block(bits, cb, data, bs)
    for b in range(3):
        x = data[b * bs:(b + 1) * bs]
        if bits == 4:
            half = (x.max() - x.min()) * np.float32(0.5)
            center = (x.max() + x.min()) * np.float32(0.5)
            assert scales[2 * b] == center and scales[2 * b + 1] == half
            want = nearest_first(cb, (x - center) / half)
            back = cb[want] * half + center
        else:
            amax = np.abs(x).max()
            assert scales[b] == amax
            want = nearest_first(cb, x / amax)
            back = cb[want] * amax
        assert np.array_equal(idx[b * bs:(b + 1) * bs], want)
        got = O.engine_dequantize_per_block(bits, cb, idx, scales, bs)[b * bs:(b + 1) * bs]
        assert np.abs(got - back).max() <= 1e-6 * np.abs(back).max()
    # a flat block: half_range < 1e-10 is replaced by 1 (4-bit), absmax < 1e-10 by 1 (8-bit)
    flat = np.full(64, 0.25 if bits == 4 else 0.0, np.float32)
    _, sc = O.engine_quantize_per_block(bits, cb, flat, 64)
    assert sc[-1] == 1.0


@pytest.mark.parametrize("bits", [4, 8])
def test_quantize_tensor_and_gemm_brute_force(O, bits):
    """nearest centroid per value, 4-bit packed low nibble first (:213-224); quant_gemm with the code
    matrix laid out [K][N] (:226-249, quant_engines_quant8.cpp:201-219)"""
    rs = np.random.RandomState(10 + bits)
    cb = rs.randn(1 << bits).astype(np.float32)
    data = rs.randn(101).astype(np.float32)
    want = nearest_first(cb, data)
    got = O.engine_quantize_tensor(bits, cb, data)
    codes = np.stack([got & 15, got >> 4], 1).reshape(-1)[:101] if bits == 4 else got
    assert np.array_equal(codes, want)
    assert np.array_equal(O.engine_dequant_tensor(bits, cb, got, 101), cb[want])
    M, N, K = 3, 10, 17
    a = rs.randn(M, K).astype(np.float32)
    a[1, 4] = 0.0
    kn = rs.randint(0, 1 << bits, (K, N))
    flat = kn.reshape(-1)
    packed = (flat[0::2] | (flat[1::2] << 4)).astype(np.uint8) if bits == 4 else flat.astype(np.uint8)
    want = a.astype(np.float64) @ cb.astype(np.float64)[kn]
    got = O.engine_quant_gemm(bits, cb, a, packed, M, N, K)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    # B as [N][K] instead of [K][N] must not pass
    wrong = a.astype(np.float64) @ cb.astype(np.float64)[flat.reshape(N, K)].T
    assert np.abs(got - wrong).max() > 1e-2 * np.abs(want).max()


def test_q8codec_is_lossless_up_to_256_distinct_weights(O):
    """Every weight seeds its own centroid when the block has at most 256 weights
    (src/codec/codebook.cpp:73-88), so Lloyd's fixed point reproduces the block exactly."""
    rs = np.random.RandomState(3)
    for n in (1, 17, 255, 256):
        w = rs.randn(n).astype(np.float32)
        cent, idx, dec = O.q8codec_block(w)
        assert np.array_equal(dec, w), n
        assert np.array_equal(cent[idx], w)
        assert np.array_equal(cent[n:], np.full(256 - n, w[0], np.float32))
    # duplicates collapse onto the first of the equal centroids
    w = np.array([0.5, -1.0, 0.5, 0.5, 2.0], np.float32)
    cent, idx, dec = O.q8codec_block(w)
    assert idx.tolist() == [0, 1, 0, 0, 4] and np.array_equal(dec, w)


def test_q8_affine_rows_closed_form(O):
    """engines/quant/quantize.cpp:14-58: inv_scale = range / 255, scale = 1 / inv_scale, zero_point = -min * scale,
    q = clamp(round(x * scale + zero_point), 0, 255); dequantize = (q - zero_point) * inv_scale."""
    rs = np.random.RandomState(4)
    src = (rs.randn(3, 500) * 2 + 1).astype(np.float32)
    q, params = O.q8_quantize_rows(src)
    for b in range(3):
        lo, hi = src[b].min(), src[b].max()
        inv = (hi - lo) / np.float32(255)
        assert params[b, 1] == inv and params[b, 0] == np.float32(1) / inv and params[b, 2] == -lo * params[b, 0]
        assert q[b, src[b].argmin()] == 0 and q[b, src[b].argmax()] == 255
        back = O.q8_dequantize(q[b], params[b])
        assert np.abs(back - src[b]).max() <= 0.5001 * inv
    f, p = O.q8_quantize_rows(src, dst_f32=True)
    for b in range(3):
        amax = np.abs(src[b]).max()
        assert p[b, 0] == np.float32(127) / amax and p[b, 2] == 0
        assert np.array_equal(f[b], src[b] * p[b, 0])
        assert np.abs(O.q8_dequantize(f[b], p[b]) - src[b]).max() <= 1e-6 * amax
    # constant row: range < 1e-12 is replaced by 1
    _, p = O.q8_quantize_rows(np.full((1, 8), 0.3, np.float32))
    assert p[0, 1] == np.float32(1) / np.float32(255)


def test_engines_equal_the_compiled_reference(O):
    if not O.have_ref():
        pytest.skip("compiled reference not built on this machine")
    rs = np.random.RandomState(5)
    same = lambda a, b: np.array_equal(np.ascontiguousarray(a).view(np.uint8), np.ascontiguousarray(b).view(np.uint8))
    for bits in (4, 8):
        cb = (np.sort(rs.randn(1 << bits)) * 0.5).astype(np.float32)
        for n, bs in ((1000, 256), (256, 64), (777, 100), (5, 8)):
            data = (rs.randn(n) * 0.05 + 0.01).astype(np.float32)
            a, b = O.engine_quantize_per_block(bits, cb, data, bs), O.engine_quantize_per_block(bits, cb, data, bs, use_ref=True)
            assert same(a[0], b[0]) and same(a[1], b[1])
            assert same(O.engine_dequantize_per_block(bits, cb, a[0], a[1], bs),
                        O.engine_dequantize_per_block(bits, cb, a[0], a[1], bs, use_ref=True))
            t = O.engine_quantize_tensor(bits, cb, data)
            assert same(t, O.engine_quantize_tensor(bits, cb, data, use_ref=True))
            assert same(O.engine_dequant_tensor(bits, cb, t, n), O.engine_dequant_tensor(bits, cb, t, n, use_ref=True))
        for M, N, K in ((3, 8, 16), (5, 7, 33), (2, 64, 128)):
            a = rs.randn(M, K).astype(np.float32)
            a[0, 3] = 0
            bidx = rs.randint(0, 256, (K * N + 1) // 2 if bits == 4 else K * N).astype(np.uint8)
            assert same(O.engine_quant_gemm(bits, cb, a, bidx, M, N, K), O.engine_quant_gemm(bits, cb, a, bidx, M, N, K, use_ref=True))
    for n in (256, 100, 1, 17, 255):
        w = (rs.randn(n) * 0.02).astype(np.float32)
        if n == 100:
            w[::3] = w[0]
        for x, y in zip(O.q8codec_block(w), O.q8codec_block(w, use_ref=True)):
            assert same(x, y)
    for shape in ((1, 1000), (4, 300), (3, 1)):
        src = (rs.randn(*shape) * 3 + 0.5).astype(np.float32)
        for f32 in (False, True):
            a, b = O.q8_quantize_rows(src, f32), O.q8_quantize_rows(src, f32, use_ref=True)
            assert same(a[0], b[0]) and same(a[1], b[1])
            assert same(O.q8_dequantize(a[0][0], a[1][0]), O.q8_dequantize(a[0][0], a[1][0], use_ref=True))
