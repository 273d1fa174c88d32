"""The oracle against the golden fixtures written from the compiled reference
(tests/golden/make_golden.py) and against what the mathematics fixes.  CPU only."""
import os

import numpy as np
import pytest

G = os.path.join(os.path.dirname(__file__), "golden")
FORMATS = ["Q_4", "Q_8", "Q_G_2", "Q_G_3", "Q_G_4", "Q_G_8", "Q_32"]
# bytes per 256-block printed by the reference's tests/test_format_audit.cpp
AUDIT_BYTES = {"Q_4": 128, "Q_8": 256, "Q_G_2": 84, "Q_G_3": 112, "Q_G_4": 144, "Q_G_8": 272, "Q_32": 1024,
               "B32S4": 144, "B32S8": 272, "SB256A3": 124, "SB256A2": 92}
# NMSE caps of the reference's tests/test_fuzz_codec.cpp:118-240
NMSE_CAP = {"Q_4": 0.60, "Q_G_4": 0.60, "Q_8": 0.08, "Q_G_8": 0.10, "Q_G_3": 0.80, "Q_G_2": 1.60}


@pytest.fixture(scope="module")
def codec():
    return np.load(os.path.join(G, "codec.npz"))


@pytest.mark.parametrize("fmt", FORMATS)
def test_encode_matches_reference_payload(O, codec, fmt):
    w = codec["w"].reshape(-1, 256)
    want = codec[f"{fmt}_payload"]
    for i, blk in enumerate(w):
        got = O.encode_block(fmt, blk)
        assert got.size == want[i].size == AUDIT_BYTES[fmt]
        assert np.array_equal(got, want[i]), f"{fmt} block {i}"


@pytest.mark.parametrize("fmt", FORMATS)
def test_decode_matches_reference_values(O, codec, fmt):
    pay, want = codec[f"{fmt}_payload"], codec[f"{fmt}_decoded"]
    for i in range(pay.shape[0]):
        got = O.decode_block(fmt, pay[i])
        assert np.array_equal(got.view(np.uint32), want[i].view(np.uint32)), f"{fmt} block {i}"


@pytest.mark.parametrize("alias,base", [("Q_4_5", "Q_G_4"), ("Q_G_4_5", "Q_G_4"), ("Q_3_5", "Q_G_3"),
                                        ("Q_G_3_5", "Q_G_3"), ("Q_8_5", "Q_G_8"), ("Q_G_8_5", "Q_G_8")])
def test_half_bpw_aliases_share_the_payload(O, codec, alias, base):
    w = codec["w"].reshape(-1, 256)[:8]
    for blk in w:
        assert np.array_equal(O.encode_block(alias, blk), O.encode_block(base, blk))


def test_comp8_levels(O, codec):
    lv = O.comp8_table()
    assert np.array_equal(lv.view(np.uint32), codec["comp8_levels"].view(np.uint32))
    # closed form: odd symmetry, end points +-1, strictly increasing, tanh compander
    assert lv[0] == -1.0 and lv[255] == 1.0
    assert np.all(np.diff(lv) > 0)
    assert np.abs(lv + lv[::-1]).max() < 2e-7  # odd up to the rounding of j/127.5 - 1
    j = np.arange(256, dtype=np.float64)
    exact = np.tanh(0.02 * (j / 127.5 - 1.0)) / np.tanh(0.02)
    assert np.abs(lv - exact).max() < 2e-7


def test_f16_to_f32_all_patterns(O, codec):
    want = codec["f16_all_decoded"]
    got = np.array([O.f16_to_f32(h) for h in range(65536)], np.float32).view(np.uint32)
    # level 1.0 * scale == scale, except that NaN payloads need not survive a multiply
    h = np.arange(65536)
    nan = ((h >> 10) & 31 == 31) & (h & 1023 != 0)
    assert np.array_equal(got[~nan], want[~nan])
    # and against numpy's IEEE binary16
    ieee = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32).view(np.uint32)
    assert np.array_equal(got[~nan], ieee[~nan])


def test_f32_to_f16_is_ieee_rne_with_two_quirks(O):
    rng = np.random.default_rng(7)
    u = rng.integers(0, 2**32, 200000, dtype=np.uint64).astype(np.uint32)
    # add every binary16 value, its neighbours and the exact midpoints
    h = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    h = h[np.isfinite(h)]
    mids = ((h[:-1].astype(np.float64) + h[1:].astype(np.float64)) / 2).astype(np.float32)
    f = np.concatenate([u.view(np.float32), h, np.nextafter(h, np.float32(np.inf)),
                        np.nextafter(h, np.float32(-np.inf)), mids])
    got = np.array([O.f32_to_f16(v) for v in f], np.uint16)
    with np.errstate(over="ignore"):
        ieee = f.astype(np.float16).view(np.uint16)
    a = np.abs(f.astype(np.float64))
    quirk = np.isnan(f) | ((a < 2.0**-24) & (a > 0))
    assert np.array_equal(got[~quirk], ieee[~quirk])
    # quirk 1: NaN collapses to infinity of the same sign; quirk 2: below 2^-24 flushes to zero
    assert O.f32_to_f16(float("nan")) & 0x7FFF == 0x7C00
    assert O.f32_to_f16(2.0**-24 * 0.75) == 0 and O.f32_to_f16(-(2.0**-24) * 0.75) == 0x8000
    assert O.f32_to_f16(2.0**-24) == 1


def test_generator(O):
    r = np.load(os.path.join(G, "rng.npz"))
    assert np.array_equal(O.rng_u64(42, 4096), r["u64_42"])
    assert np.array_equal(O.rng_uniform(42, 4096).view(np.uint32), r["uniform_42"].view(np.uint32))
    assert np.array_equal(O.rng_normal(42, 4096, 0.02).view(np.uint32), r["normal_42_002"].view(np.uint32))
    assert np.array_equal(O.rng_normal(43, 4096, 1.0).view(np.uint32), r["normal_43"].view(np.uint32))
    # xoroshiro128+ seeded by splitmix64: first output for seed 0 from the published algorithms
    def splitmix(s):
        s = (s + 0x9E3779B97F4A7C15) & (2**64 - 1)
        z = s
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & (2**64 - 1)
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & (2**64 - 1)
        return s, z ^ (z >> 31)
    s, a = splitmix(0)
    s, b = splitmix(s)
    assert int(O.rng_u64(0, 1)[0]) == (a + b) & (2**64 - 1)


@pytest.mark.parametrize("fmt", ["Q_G_4", "Q_G_8", "Q_4"])
def test_matmul_fixture(O, fmt):
    m = np.load(os.path.join(G, "matmul.npz"))
    N, K = 48, 512
    y = O.matmul(fmt, m[f"{fmt}_payload"], N, K, m["X"].reshape(3, K), threads=2)
    ref = m[f"{fmt}_y"]
    # same products, different summation order (256-blocks vs one 512 run): fp32 rounding only
    assert np.abs(y - ref).max() <= 2e-6 * np.abs(ref).max()
    # the oracle re-encodes W to the same payload
    assert np.array_equal(O.encode_tensor(fmt, m["W"]), m[f"{fmt}_payload"])


@pytest.mark.parametrize("fmt", list(AUDIT_BYTES))
def test_block_bytes_and_nmse(O, fmt):
    assert O.block_bytes(fmt, 256) == AUDIT_BYTES[fmt]
    w = O.rng_normal(99, 256 * 64, 1.0)
    dec = O.decode_tensor(fmt, O.encode_tensor(fmt, w), w.size)
    nmse = float(((dec - w) ** 2).sum() / (w ** 2).sum())
    cap = NMSE_CAP.get(fmt, {"B32S4": 0.02, "B32S8": 1e-4, "SB256A3": 0.05, "SB256A2": 0.2, "Q_32": 0.0}.get(fmt))
    assert nmse <= cap, (fmt, nmse)


def test_quality_ordering_like_reference_proof(O):
    # tests/test_grp_quality_proof.cpp:90-99: Q_G_4 > Q_G_3 > Q_G_2 in PSNR on N(0, 0.1)
    w = O.rng_normal(5, 8192, 0.1)
    def psnr(fmt):
        d = O.decode_tensor(fmt, O.encode_tensor(fmt, w), w.size)
        return 10 * np.log10(float(np.abs(w).max()) ** 2 / float(((d - w) ** 2).mean()))
    p4, p3, p2 = psnr("Q_G_4"), psnr("Q_G_3"), psnr("Q_G_2")
    assert p4 > p3 > p2 and p3 >= 24.0


def test_matmul_equals_dense_product_of_decoded_matrix(O):
    N, K, B = 40, 768, 5
    w = O.rng_normal(11, N * K, 0.02)
    x = O.rng_normal(12, B * K, 1.0).reshape(B, K)
    for fmt in ("Q_G_4", "B32S4", "Q_G_8", "B32S8", "Q_G_3", "Q_G_2", "SB256A3", "SB256A2", "Q_4", "Q_8"):
        p = O.encode_tensor(fmt, w)
        dense = O.decode_tensor(fmt, p, N * K).reshape(N, K).astype(np.float64)
        want = x.astype(np.float64) @ dense.T
        got = O.matmul(fmt, p, N, K, x, threads=2)
        got64 = O.matmul_f64(fmt, p, N, K, x, threads=2)
        assert np.abs(got64 - want).max() <= 1e-12 * np.abs(want).max() + 1e-15
        assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    # all-ones x all-twos closed form (tests/test_kernel.cpp:16-25), through Q_32 blocks
    ones = np.full(4 * 256, 2.0, np.float32)
    y = O.matmul("Q_32", O.encode_tensor("Q_32", ones), 4, 256, np.ones((1, 256), np.float32))
    assert np.all(y == 512.0)
