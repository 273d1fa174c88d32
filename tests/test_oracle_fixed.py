"""Fixed-codebook formats (Q_3 / Q_6 / Q_12), the 12-bit compound (Q_G_12 family) and the searched
_K tiers of the plain lattices and of Q_G_8 in the oracle: the level tables against the fixture read
off the compiled reference and against scipy's normal quantile function, payload layouts against
hand-built blocks, tier ordering, and every block size against the compiled reference where it is
built.  The fixture rows for these ids in tests/golden/tails.npz are covered by test_oracle_tails.py.
CPU only."""
import math
import os

import numpy as np
import pytest

G = os.path.join(os.path.dirname(__file__), "golden")
Q3 = np.array([-3.0776, -2.1479, -1.2879, -0.4240, 0.4240, 1.2879, 2.1479, 3.0776], np.float32)


def put_bits(buf, pos, value, count):
    for i in range(count):
        if (value >> i) & 1:
            buf[(pos + i) >> 3] |= 1 << ((pos + i) & 7)
    return pos + count


def is_slot(i, n, slots=16):
    return ((i + 1) * slots) // n != (i * slots) // n


def test_level_tables_match_the_reference_and_the_normal_quantiles(O):
    """src/codec/block_codec.cpp:563-588: mid-quantiles of N(0,1), odd-symmetric, ascending.  The
    reference builds them from a rational erf (error about 1.2e-7) inverted by Newton steps; the
    library quantile function agrees to that accuracy, the fixture bit for bit."""
    from scipy.special import ndtri
    fix = np.load(os.path.join(G, "fixed_levels.npz"))
    for bits in (6, 12):
        t = O.fixed_table(bits)
        assert np.array_equal(t.view(np.uint32), fix[f"t{bits}"])
        count = 1 << bits
        assert np.array_equal(t, -t[::-1]) and np.all(np.diff(t) > 0)
        want = ndtri((np.arange(count) + 0.5) / count)
        assert np.abs(t - want).max() < 2e-6 * np.abs(want).max()
    assert np.array_equal(O.fixed_table(3), Q3)


def test_fixed_codebook_layout_by_hand(O):
    """Full block: binary16 scale, then a code per weight; the sixteen slot positions store code >> 1 in
    bits - 1 bits and decode to the even code (src/codec/block_codec.cpp:646-662, :727-734)."""
    rs = np.random.RandomState(0)
    for fmt, bits, nbytes in (("Q_3", 3, 96), ("Q_6", 6, 192), ("Q_12", 12, 384)):
        table = O.fixed_table(bits)
        codes = rs.randint(0, 1 << bits, 256)
        buf = np.zeros(nbytes, np.uint8)
        pos = put_bits(buf, 0, 0x3400, 16)  # 0.25
        for i, c in enumerate(codes):
            if is_slot(i, 256):
                codes[i] = c & ~1
                pos = put_bits(buf, pos, int(c) >> 1, bits - 1)
            else:
                pos = put_bits(buf, pos, int(c), bits)
        assert pos == nbytes * 8 and O.block_bytes(fmt, 256) == nbytes
        assert np.array_equal(O.decode_block(fmt, buf), table[codes] * np.float32(0.25))
        for tier in ("_K_L", "_K_M", "_K_H"):
            assert np.array_equal(O.decode_block(fmt + tier, buf), table[codes] * np.float32(0.25))
        # fewer than 16 weights: raw codes, implied scale 1
        small = np.zeros(math.ceil(bits * 11 / 8), np.uint8)
        pos = 0
        for c in codes[:11]:
            pos = put_bits(small, pos, int(c), bits)
        assert np.array_equal(O.decode_block(fmt, small, 11), table[codes[:11]])


def test_compound_12_bit_layout_by_hand(O):
    """n 12-bit codes, then one binary16 scale per 32 weights (src/codec/block_codec.cpp:969-1040);
    400 bytes for a full block whatever the id claims."""
    rs = np.random.RandomState(1)
    table = O.fixed_table(12)
    codes = rs.randint(0, 4096, 256)
    scales = np.array([0.5, 0.25, 1.0, 2.0, 0.125, 4.0, 0.0625, 1.5], np.float16)
    buf = np.zeros(400, np.uint8)
    pos = 0
    for c in codes:
        pos = put_bits(buf, pos, int(c), 12)
    buf[384:] = scales.view(np.uint8)
    want = np.repeat(scales.astype(np.float32), 32) * table[codes]
    for fmt in ("Q_G_12", "Q_G_12_K_L", "Q_G_12_K_H", "Q_12_5", "Q_G_12_5"):
        assert O.block_bytes(fmt, 256) == 400
        assert np.array_equal(O.decode_block(fmt, buf), want), fmt
    # other block sizes: Q_G_12 takes the grouped-lattice fallback, the others the fixed codebook
    assert O.block_bytes("Q_G_12", 100) == 150 + 5 + 2 and O.block_bytes("Q_12_5", 100) == 150
    assert O.block_bytes("Q_G_12_K_M", 100) == 150 and O.block_bytes("Q_G_12", 96) == 150


def test_round_trip_error_is_what_the_code_width_allows(O):
    rs = np.random.RandomState(2)
    w = (rs.randn(16, 256) * 0.02).astype(np.float32)
    for fmt, cap in (("Q_3", 0.15), ("Q_6", 6e-3), ("Q_12", 5e-4), ("Q_G_12", 1.5e-4)):
        nmse = []
        for blk in w:
            d = O.decode_block(fmt, O.encode_block(fmt, blk))
            nmse.append(float(((d - blk).astype(np.float64) ** 2).sum() / (blk.astype(np.float64) ** 2).sum()))
        assert max(nmse) < cap, (fmt, max(nmse))
    zero = np.zeros(256, np.float32)
    for fmt in ("Q_3", "Q_6", "Q_12", "Q_G_12", "Q_G_12_K_H"):
        assert not O.decode_block(fmt, O.encode_block(fmt, zero)).any()


@pytest.mark.parametrize("base", ["Q_2", "Q_3", "Q_4", "Q_6", "Q_8", "Q_12", "Q_G_8", "Q_G_12"])
def test_tier_search_never_loses(O, base):
    """_K_L is the base encoder's payload (Q_G_12_K_L equals Q_G_12 on full blocks), and
    MSE(_K_H) <= MSE(_K_M) <= MSE(_K_L) (src/codec/block_codec.cpp:2378-2388)."""
    rs = np.random.RandomState(3)
    for trial in range(6):
        w = (rs.standard_t(4, 256) * 0.02).astype(np.float32)
        err = []
        for tier in ("_K_L", "_K_M", "_K_H"):
            d = O.decode_block(base + tier, O.encode_block(base + tier, w))
            err.append(float(((d - w).astype(np.float64) ** 2).mean()))
        assert err[2] <= err[1] <= err[0], (trial, err)
        assert np.array_equal(O.encode_block(base, w), O.encode_block(base + "_K_L", w))


def test_every_block_size_equals_the_compiled_reference(O):
    if not O.have_ref():
        pytest.skip("compiled reference not built on this machine")
    rs = np.random.RandomState(4)
    ids = ["Q_3", "Q_6", "Q_12", "Q_G_12", "Q_12_5", "Q_G_12_5"] + [
        b + t for b in ("Q_2", "Q_3", "Q_4", "Q_6", "Q_8", "Q_12", "Q_G_8", "Q_G_12") for t in ("_K_L", "_K_M", "_K_H")]
    for fmt in ids:
        for n in list(range(1, 70, 2)) + [96, 100, 128, 192, 224, 250, 255, 256, 256]:
            w = (rs.randn(n) * 0.02).astype(np.float32) if n % 3 else (rs.laplace(0, 0.015, n) + 0.01).astype(np.float32)
            pay = O.ref_encode_block(fmt, w)
            assert O.block_bytes(fmt, n) == pay.size, (fmt, n)
            assert np.array_equal(O.encode_block(fmt, w), pay), (fmt, n)
            rnd = rs.randint(0, 256, pay.size).astype(np.uint8)
            a, b = O.decode_block(fmt, rnd, n), O.ref_decode_block(fmt, rnd, n)
            keep = ~(np.isnan(a) & np.isnan(b))
            assert np.array_equal(a.view(np.uint32)[keep], b.view(np.uint32)[keep]), (fmt, n)
