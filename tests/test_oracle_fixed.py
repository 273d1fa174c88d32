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


# ---------------------------------------------------------------- four-tier mixes
MIX = {"Q_MX_3_5": (3.5, [(1, 92.0), (2, 1.5), (4, 6.0), (32, 0.5)], False),
       "Q_MX_12_5": (12.5, [(1, 0.5), (3, 2.0), (8, 87.5), (32, 10.0)], False),
       "Q_G_MX_6_5": (6.5, [(1, 0.5), (3, 5.0), (4, 93.0), (32, 1.5)], True),
       "Q_G_MX_16_5": (16.5, [(1, 10.0), (2, 1.0), (16, 88.0), (32, 1.0)], True)}
GRID2 = np.array([-1.5104, -0.4528, 0.4528, 1.5104], np.float32)
GRID4 = np.array([-2.7178, -2.0522, -1.5995, -1.2392, -0.9275, -0.6508, -0.3976, -0.1260,
                  0.1260, 0.3976, 0.6508, 0.9275, 1.2392, 1.5995, 2.0522, 2.7178], np.float32)


def mix_value(O, bits, code, s):
    if bits == 1:
        return np.float32(s) * np.float32(1.0 if code else -1.0)
    if bits == 2:
        return GRID2[code] * np.float32(s)
    if bits == 4:
        return GRID4[code] * np.float32(s)
    if bits == 8:
        return (np.float32(-8.0) + np.float32(16.0) * np.float32(code) / np.float32(255)) * np.float32(s)
    if bits == 3:
        return Q3[code] * np.float32(s)
    if bits == 16:
        return np.array([code], np.uint16).view(np.float16).astype(np.float32)[0]
    return np.array([code], np.uint32).view(np.float32)[0]


@pytest.mark.parametrize("fmt", sorted(MIX))
def test_mix_layout_by_hand(O, fmt):
    """Full block of a four-tier mix (src/codec/block_codec.cpp:1875-1995, :2207-2263): tier counts are the
    rounded shares (the widest tier takes the rest), the stream is 256 2-bit tiers then the four value
    runs, the scales follow byte aligned: one per tier narrower than 16 bits, one per 32 values for the
    most populated tier of a grouped id.  A hand-built payload decodes to the values the layout implies."""
    claim, tiers, grouped = MIX[fmt]
    n = 256
    c = [max(1, int(math.floor(p * 0.01 * n + 0.5))) for _, p in tiers[:3]]
    c.append(n - sum(c))
    bits = [b for b, _ in tiers]

    def shape():
        dom = int(np.argmax(c))
        nsc = [0 if b >= 16 else ((c[t] + 31) // 32 if grouped and t == dom else 1) for t, b in enumerate(bits)]
        return nsc, 2 * n + sum(ct * b for ct, b in zip(c, bits))

    # while the layout is over the claim, one weight moves from the widest tier that can spare one to the next narrower
    while shape()[1] + 16 * sum(shape()[0]) > math.ceil(claim * n):
        t = max(t for t in (1, 2, 3) if c[t] > 1 and bits[t] > bits[t - 1])
        c[t] -= 1
        c[t - 1] += 1
    nsc, payload_bits = shape()
    total = (payload_bits + 7) // 8 + 2 * sum(nsc)
    assert O.block_bytes(fmt, n) == total
    rs = np.random.RandomState(len(fmt))
    tier = np.repeat(np.arange(4), c)
    rs.shuffle(tier)
    buf = np.zeros(total, np.uint8)
    pos = 0
    for t in tier:
        pos = put_bits(buf, pos, int(t), 2)
    codes = [rs.randint(0, 1 << min(b, 31), ct).astype(np.uint64) for ct, b in zip(c, bits)]
    for t in range(4):
        if bits[t] == 32:
            codes[t] = rs.randn(c[t]).astype(np.float32).view(np.uint32).astype(np.uint64)
        for code in codes[t]:
            pos = put_bits(buf, pos, int(code), bits[t])
    assert pos == payload_bits
    scales = [np.float16(2.0 ** -rs.randint(1, 6, k)) for k in nsc]
    at = (payload_bits + 7) // 8
    for t in range(4):
        for s in scales[t]:
            buf[at:at + 2] = np.array([s], np.float16).view(np.uint8)
            at += 2
    want = np.zeros(n, np.float32)
    seen = [0, 0, 0, 0]
    for i, t in enumerate(tier):
        j = seen[t]
        seen[t] += 1
        s = float(scales[t][min(j // 32, nsc[t] - 1)]) if nsc[t] else 1.0
        want[i] = mix_value(O, bits[t], int(codes[t][j]), s)
    got = O.decode_block(fmt, buf)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_mix_round_trip_properties(O):
    """The widest tier is lossless for the largest magnitudes (raw binary32), every payload is within
    ceil(bpw n / 8) + 1 bytes for every n (tests/test_format_audit.cpp:52-77), and tails too small for the
    map plus scales collapse to bare signs."""
    rs = np.random.RandomState(9)
    w = (rs.standard_t(3, 256) * 0.02).astype(np.float32)
    order = np.argsort(-np.abs(w))
    for fmt, claim in (("Q_MX_3_5", 3.5), ("Q_MX_8_5", 8.5), ("Q_G_MX_12_5", 12.5), ("Q_G_MX_24_5", 24.5), ("Q_G_MX_3_5", 3.78125)):
        d = O.decode_block(fmt, O.encode_block(fmt, w))
        assert np.array_equal(d[order[:1]], w[order[:1]])
        for n in range(1, 257):
            assert O.block_bytes(fmt, n) <= math.ceil(claim * n / 8) + 1, (fmt, n)
    small = np.array([0.3, -0.2, 0.0, -5.0], np.float32)
    pay = O.encode_block("Q_MX_3_5", small)
    assert pay.size == 2 and np.array_equal(O.decode_block("Q_MX_3_5", pay, 4), np.array([1, -1, 1, -1], np.float32))


def test_mix_equals_the_compiled_reference(O):
    if not O.have_ref():
        pytest.skip("compiled reference not built on this machine")
    rs = np.random.RandomState(10)
    for fid in range(91, 105):
        for n in list(range(1, 70, 3)) + [96, 100, 128, 200, 250, 255, 256, 256]:
            w = (rs.randn(n) * 0.02).astype(np.float32) if n % 2 else (rs.standard_t(3, n) * 0.5).astype(np.float32)
            pay = O.ref_encode_block(fid, w)
            assert O.block_bytes(fid, n) == pay.size, (fid, n)
            assert np.array_equal(O.encode_block(fid, w), pay), (fid, n)
            rnd = rs.randint(0, 256, pay.size).astype(np.uint8)
            a, b = O.decode_block(fid, rnd, n), O.ref_decode_block(fid, rnd, n)
            keep = ~(np.isnan(a) & np.isnan(b))
            assert np.array_equal(a.view(np.uint32)[keep], b.view(np.uint32)[keep]), (fid, n)
