"""Short blocks (n < 256), Q_2, Q_G_6 and the grouped-lattice fallback layout in the oracle:
against the fixture written from the compiled reference (tests/golden/tails.npz), against the
byte budgets the reference's audit test fixes (tests/test_format_audit.cpp:52-77), and against
hand-built payloads whose decoded values follow from the layout alone.  CPU only."""
import math
import os

import numpy as np
import pytest

G = os.path.join(os.path.dirname(__file__), "golden")
BPW = {"Q_2": 2.0, "Q_4": 4.0, "Q_8": 8.0, "Q_G_2": 2.625, "Q_G_3": 3.5, "Q_G_4": 4.5, "Q_G_6": 6.5625,
       "Q_G_8": 8.5, "Q_G_2_K_H": 2.4375, "Q_G_3_K_L": 3.4375, "Q_G_4_K_M": 4.4375, "Q_G_6_K_H": 6.5625,
       "Q_2_5": 2.5, "Q_6_5": 6.5, "Q_1": 1.0, "Q_G_1_K_H": 1.0, "Q_1_5": 1.5, "Q_16": 16.0, "Q_G_16": 16.5,
       "Q_24": 24.0, "Q_G_24": 24.5}
GRID2 = np.array([-1.5104, -0.4528, 0.4528, 1.5104], np.float32)
GRID4 = np.array([-2.7178, -2.0522, -1.5995, -1.2392, -0.9275, -0.6508, -0.3976, -0.1260,
                  0.1260, 0.3976, 0.6508, 0.9275, 1.2392, 1.5995, 2.0522, 2.7178], np.float32)


@pytest.fixture(scope="module")
def tails():
    return np.load(os.path.join(G, "tails.npz"))


def rows(t):
    for fmt, n, which, poff, plen, doff in t["index"]:
        yield int(fmt), int(n), int(which), t["payloads"][poff:poff + plen], t["decoded"][doff:doff + n]


def test_encode_and_decode_match_the_reference_for_every_block_size(O, tails):
    seen = 0
    for fmt, n, which, pay, dec in rows(tails):
        w = tails["src"][which][:n]
        assert O.block_bytes(fmt, n) == pay.size, (fmt, n)
        assert np.array_equal(O.encode_block(fmt, w), pay), (fmt, n, which)
        assert np.array_equal(O.decode_block(fmt, pay, n).view(np.uint32), dec.view(np.uint32)), (fmt, n, which)
        seen += 1
    assert seen == 42 * 13 * 2


@pytest.mark.parametrize("fmt", sorted(BPW))
def test_payload_never_exceeds_the_claimed_budget(O, fmt):
    """bytes <= ceil(bpw * n / 8) + 1 for every n (the audit's rule, tests/test_format_audit.cpp:52-77);
    a full block is exactly the claim except for the ids claiming less than their layout needs."""
    for n in range(1, 257):
        assert O.block_bytes(fmt, n) <= math.ceil(BPW[fmt] * n / 8) + 1, n
    full = {"Q_2": 64, "Q_4": 128, "Q_8": 256, "Q_G_2": 84, "Q_G_3": 112, "Q_G_4": 144, "Q_G_6": 210, "Q_G_8": 272,
            "Q_G_2_K_H": 78, "Q_G_3_K_L": 110, "Q_G_4_K_M": 142, "Q_G_6_K_H": 210, "Q_2_5": 78, "Q_6_5": 206,
            "Q_1": 32, "Q_G_1_K_H": 32, "Q_1_5": 48, "Q_16": 512, "Q_G_16": 528, "Q_24": 768, "Q_G_24": 784}
    assert O.block_bytes(fmt, 256) == full[fmt]


def put_bits(buf, pos, value, count):
    for i in range(count):
        if (value >> i) & 1:
            buf[(pos + i) >> 3] |= 1 << ((pos + i) & 7)
    return pos + count


def test_grouped_lattice_layout_by_hand(O):
    """Q_G_4_K_L, 256 weights: 128 B of 4-bit levels, 32 3-bit scales, binary16 d in one bit stream;
    value = grid[level] * d * scale (src/codec/block_codec.cpp:916-945)."""
    rs = np.random.RandomState(0)
    lev = rs.randint(0, 16, 256)
    sc = rs.randint(0, 8, 32)
    buf = np.zeros(142, np.uint8)
    pos = 0
    for v in lev:
        pos = put_bits(buf, pos, int(v), 4)
    for v in sc:
        pos = put_bits(buf, pos, int(v), 3)
    put_bits(buf, pos, 0x3800, 16)  # d = 0.5
    want = (GRID4[lev] * np.float32(0.5)) * sc[np.arange(256) // 8].astype(np.float32)
    assert np.array_equal(O.decode_block("Q_G_4_K_L", buf), want)
    # 2-bit and 3-bit widths: Lloyd-Max grid of 4, and the uniform grid -8 + 16 i / 7
    for fmt, bits, nbytes in (("Q_G_2_K_M", 2, 78), ("Q_G_3_K_H", 3, 110)):
        lev = rs.randint(0, 1 << bits, 256)
        buf = np.zeros(nbytes, np.uint8)
        pos = 0
        for v in lev:
            pos = put_bits(buf, pos, int(v), bits)
        for v in sc:
            pos = put_bits(buf, pos, int(v), 3)
        put_bits(buf, pos, 0x4000, 16)  # d = 2
        grid = GRID2[lev] if bits == 2 else (np.float32(-8.0) + np.float32(16.0) * lev.astype(np.float32) / np.float32(7))
        want = (grid * np.float32(2.0)) * sc[np.arange(256) // 8].astype(np.float32)
        assert np.array_equal(O.decode_block(fmt, buf), want), fmt


def test_q_g_6_layout_by_hand(O):
    """192 B of 6-bit levels stored +32, 16 int8 scales, binary16 d: value = (d * scale) * (level - 32)
    (src/codec/block_codec.cpp:1240-1303)."""
    rs = np.random.RandomState(1)
    lev = rs.randint(0, 64, 256)
    sc = rs.randint(-127, 128, 16)
    buf = np.zeros(210, np.uint8)
    pos = 0
    for v in lev:
        pos = put_bits(buf, pos, int(v), 6)
    buf[192:208] = sc.astype(np.int8).view(np.uint8)
    buf[208], buf[209] = 0x00, 0x34  # d = 0.25
    want = (np.float32(0.25) * sc[np.arange(256) // 16].astype(np.float32)) * (lev - 32).astype(np.float32)
    got = O.decode_block("Q_G_6", buf)
    assert np.array_equal(got, want)
    assert not np.signbit(got[want == 0]).any()  # full groups never produce -0
    for alias in ("Q_G_6_K_L", "Q_G_6_K_M", "Q_G_6_K_H"):
        assert np.array_equal(O.decode_block(alias, buf), want)


def test_q_g_6_round_trip_quality_and_tier_order(O):
    """NMSE far below the 6-bit cap of tests/test_fuzz_codec.cpp, and MSE(H) <= MSE(M) <= MSE(L) by
    construction of the tier search (src/codec/block_codec.cpp:2378-2388)."""
    rs = np.random.RandomState(2)
    for _ in range(8):
        w = (rs.randn(256) * 0.02).astype(np.float32)
        err = []
        for fmt in ("Q_G_6_K_L", "Q_G_6_K_M", "Q_G_6_K_H"):
            d = O.decode_block(fmt, O.encode_block(fmt, w))
            err.append(float(((d - w).astype(np.float64) ** 2).mean()))
        assert err[2] <= err[1] <= err[0]
        assert err[0] / float((w.astype(np.float64) ** 2).mean()) < 2e-3
        assert np.array_equal(O.encode_block("Q_G_6", w), O.encode_block("Q_G_6_K_L", w))


def test_sign_and_wide_formats_by_hand(O):
    """Q_1: binary16 scale, then a sign bit per weight except every 16th (zero), src/codec/block_codec.cpp:1526-1618.
    Q_24: bytes 1..3 of the binary32 (:1809-1873).  Q_16: binary32 min and max, 63-bit groups of 16+16+16+15-bit
    uniform codes (:1690-1807).  Q_G_16 / Q_G_24 add a binary16 mean per 32 weights."""
    rs = np.random.RandomState(7)
    bits = rs.randint(0, 2, 240)
    buf = np.zeros(32, np.uint8)
    put_bits(buf, 0, 0x3800, 16)  # 0.5
    pos = 16
    for b in bits:
        pos = put_bits(buf, pos, int(b), 1)
    want = np.zeros(256, np.float32)
    kept = [i for i in range(256) if i % 16 != 15]
    want[kept] = np.where(bits == 1, 0.5, -0.5)
    assert np.array_equal(O.decode_block("Q_1", buf), want)
    assert np.array_equal(O.decode_block("Q_G_1_K_M", buf), want)

    w = rs.randn(256).astype(np.float32)
    pay = O.encode_block("Q_24", w)
    assert np.array_equal(pay.reshape(256, 3), w.view(np.uint8).reshape(256, 4)[:, 1:])
    assert np.array_equal(O.decode_block("Q_24", pay).view(np.uint32), w.view(np.uint32) & np.uint32(0xFFFFFF00))
    g = O.encode_block("Q_G_24", w)
    assert g.size == 784 and np.array_equal(g[:768], pay)
    resid = (w.astype(np.float64) - O.decode_block("Q_24", pay)).reshape(8, 32).mean(1)
    assert np.array_equal(g[768:].view(np.float16), resid.astype(np.float32).astype(np.float16))
    assert np.array_equal(O.decode_block("Q_G_24", g), O.decode_block("Q_24", pay) + np.repeat(g[768:].view(np.float16).astype(np.float32), 32))

    buf = np.zeros(512, np.uint8)
    buf[:8] = np.array([-1.0, 1.0], np.float32).view(np.uint8)
    codes = rs.randint(0, 65536, 256)
    codes[3::4] >>= 1
    codes[:8] = [0, 65535, 32768, 32767, 1, 2, 3, 0]
    pos = 64
    for i, c in enumerate(codes):
        pos = put_bits(buf, pos, int(c), 15 if i % 4 == 3 else 16)
    got = O.decode_block("Q_16", buf)
    step = np.where(np.arange(256) % 4 == 3, np.float32(2.0) / np.float32(32767), np.float32(2.0) / np.float32(65535))
    exact = -1.0 + codes.astype(np.float64) * step.astype(np.float64)
    assert np.abs(got - exact).max() <= 2.0 ** -24 and got[0] == -1.0 and got[1] == 1.0 and got[3] == 1.0
    # a uniform 16-bit grid over the block's range: error at most half a step
    w = (rs.randn(256) * 0.02).astype(np.float32)
    back = O.decode_block("Q_16", O.encode_block("Q_16", w))
    assert np.abs(back - w).max() <= 0.51 * (w.max() - w.min()) / 32767
    # pieces that are not 256 weights long are raw binary16
    assert np.array_equal(O.encode_block("Q_16", w[:100]).view(np.float16), w[:100].astype(np.float16))


def test_tiny_blocks_are_raw_levels(O):
    """n < 8: no header, implied scale 1 (src/codec/block_codec.cpp:812-817, :1085-1090)."""
    w = np.array([0.4, -1.6, 2.0, -0.1, 31.2], np.float32)
    assert np.array_equal(O.decode_block("Q_G_6", O.encode_block("Q_G_6", w), 5), np.array([0, -2, 2, 0, 31], np.float32))
    got = O.decode_block("Q_G_4", O.encode_block("Q_G_4", w), 5)
    assert np.array_equal(got, GRID4[[9, 2, 14, 7, 15]])


def test_every_tail_size_equals_the_compiled_reference(O):
    if not O.have_ref():
        pytest.skip("compiled reference not built on this machine")
    rs = np.random.RandomState(3)
    for fmt in ("Q_2", "Q_4", "Q_8", "Q_G_2", "Q_G_3", "Q_G_4", "Q_G_6", "Q_G_8", "Q_G_4_K_H", "Q_G_6_K_H", "Q_6_5"):
        for n in list(range(1, 70)) + [95, 96, 127, 129, 191, 192, 224, 240, 249, 251]:
            w = (rs.randn(n) * 0.02).astype(np.float32)
            pay = O.ref_encode_block(fmt, w)
            assert np.array_equal(O.encode_block(fmt, w), pay), (fmt, n)
            rnd = rs.randint(0, 256, pay.size).astype(np.uint8)
            a, b = O.decode_block(fmt, rnd, n), O.ref_decode_block(fmt, rnd, n)
            keep = ~(np.isnan(a) & np.isnan(b))
            assert np.array_equal(a.view(np.uint32)[keep], b.view(np.uint32)[keep]), (fmt, n)
