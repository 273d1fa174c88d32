"""The oracle beside the compiled reference (oracle/_ref, built from the
reference's own sources) on fresh seeded inputs.  Skipped where the compiled
reference is absent.  CPU only."""
import numpy as np
import pytest


@pytest.fixture(scope="module")
def R(O):
    if not O.have_ref():
        pytest.skip("oracle/_ref/libref.so not built")
    return O


def _blocks(O, nblk):
    rng = np.random.default_rng(2024)
    yield O.rng_normal(142, nblk * 256, 0.02)
    yield O.rng_laplace(144, nblk * 256, 0.015)
    yield rng.standard_normal(nblk * 256).astype(np.float32)
    yield (np.abs(rng.standard_normal(nblk * 256)) * 0.1 + 0.5).astype(np.float32)
    h = (rng.standard_normal(nblk * 256) * 0.02).astype(np.float32)
    h[::97] *= 40
    yield h


@pytest.mark.parametrize("fmt", ["Q_4", "Q_8", "Q_32", "Q_G_2", "Q_G_3", "Q_G_4", "Q_G_8",
                                 "Q_3_5", "Q_4_5", "Q_8_5", "Q_G_3_5", "Q_G_4_5", "Q_G_8_5"])
def test_codec_bit_exact(R, fmt):
    nblk = 24 if "8" in fmt else 60
    for data in _blocks(R, nblk):
        for b in range(nblk):
            w = data[b * 256:(b + 1) * 256]
            mine, theirs = R.encode_block(fmt, w), R.ref_encode_block(fmt, w)
            assert np.array_equal(mine, theirs)
            assert np.array_equal(R.decode_block(fmt, theirs).view(np.uint32),
                                  R.ref_decode_block(fmt, theirs).view(np.uint32))


def test_decode_of_arbitrary_payloads(R):
    # decoders are pure functions of the payload: random bytes must decode identically
    rng = np.random.default_rng(5)
    for fmt in ("Q_4", "Q_8", "Q_G_2", "Q_G_3", "Q_G_4", "Q_G_8"):
        nb = R.block_bytes(fmt)
        for _ in range(64):
            p = rng.integers(0, 256, nb, dtype=np.uint8)
            if fmt in ("Q_G_8", "Q_8"):  # keep scales finite so NaN payload bits do not matter
                p[-16:] &= 0x7B
                p[:2] &= 0x7B
            else:
                p[-4:] &= 0x7B
            a, b = R.decode_block(fmt, p), R.ref_decode_block(fmt, p)
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), fmt


def test_registry_path_concatenates_blocks(R):
    w = R.rng_normal(77, 256 * 9, 0.02)
    for name, fmt in (("Q_G_4", "Q_G_4"), ("QG4", "Q_G_4"), ("qg8", "Q_G_8"), ("Q_4", "Q_4"), ("Q_G_3", "Q_G_3")):
        pay, per = R.ref_registry_quantize(name, w)
        assert np.all(per == R.block_bytes(fmt))
        assert np.array_equal(pay, R.encode_tensor(fmt, w))


def test_generator_bit_exact(R):
    for seed in (42, 43, 44, 45, 0, 2 ** 63 + 5):
        assert np.array_equal(R.rng_normal(seed, 5000, 0.02).view(np.uint32),
                              R.ref_rng_normal(seed, 5000, 0.02).view(np.uint32))
        assert np.array_equal(R.rng_uniform(seed, 5000).view(np.uint32), R.ref_rng_uniform(seed, 5000).view(np.uint32))


def test_codebook_gemm_operators(R):
    rng = np.random.default_rng(9)
    M, N, K = 3, 5, 64
    w4 = rng.integers(0, 256, M * N * K // 2, dtype=np.uint8)
    cb16 = (rng.standard_normal(16) * 0.1).astype(np.float16).view(np.uint16)
    act4 = rng.standard_normal(N * K).astype(np.float32)
    a, b = R.quant4_gemm(w4, cb16, act4, M, N, K), R.ref_quant4_gemm(w4, cb16, act4, M, N, K)
    assert np.abs(a - b).max() <= 1e-5 * np.abs(b).max()
    idx = rng.integers(0, 256, N * K, dtype=np.uint8)
    cb = rng.standard_normal(256).astype(np.float32)
    act8 = rng.standard_normal(M * K).astype(np.float32)
    a, b = R.quant8_gemm(idx, cb, act8, M, N, K), R.ref_quant8_gemm(idx, cb, act8, M, N, K)
    assert np.abs(a - b).max() <= 1e-5 * np.abs(b).max()
    # brute force in numpy (the semantics, independent of both)
    lut = cb16.view(np.float16).astype(np.float32)
    nib = np.stack([w4 & 15, w4 >> 4], axis=1).reshape(M * N, K)
    want = (lut[nib] * act4.reshape(N, K)[np.arange(M * N) % N]).sum(axis=1).reshape(M, N)
    assert np.abs(R.quant4_gemm(w4, cb16, act4, M, N, K) - want).max() <= 1e-5 * np.abs(want).max()
