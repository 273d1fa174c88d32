"""Device codec through the C ABI against the oracle: decoded weights and
device-encoded codes must be bit-exact."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

G = os.path.join(os.path.dirname(__file__), "golden")
DECODE_FORMATS = ["Q_2", "Q_4", "Q_8", "Q_32", "Q_G_2", "Q_G_3", "Q_G_4", "Q_G_6", "Q_G_8", "Q_4_5", "Q_G_8_5",
                  "Q_G_2_K_M", "Q_G_3_K_L", "Q_G_4_K_H", "Q_G_6_K_H", "Q_2_5", "Q_G_6_5",
                  "Q_1", "Q_G_1", "Q_G_1_K_H", "Q_1_5", "Q_16", "Q_16_5", "Q_G_16", "Q_G_16_K_M", "Q_24", "Q_G_24_5", "Q_G_24",
                  "Q_G_24_K_L", "Q_3", "Q_6", "Q_12", "Q_3_K_M", "Q_4_K_H", "Q_12_K_L", "Q_G_12", "Q_G_12_K_H", "Q_12_5",
                  "Q_G_8_K_M", "Q_MX_3_5", "Q_MX_4_5", "Q_MX_6_5", "Q_MX_8_5", "Q_MX_12_5", "Q_MX_16_5", "Q_MX_24_5",
                  "Q_G_MX_3_5", "Q_G_MX_4_5", "Q_G_MX_6_5", "Q_G_MX_8_5", "Q_G_MX_12_5", "Q_G_MX_16_5", "Q_G_MX_24_5",
                  "B32S4", "B32S8", "SB256A3", "SB256A2"]


def _inputs(O, nblk):
    rng = np.random.default_rng(31)
    w = np.concatenate([O.rng_normal(42, nblk * 256, 0.02), O.rng_laplace(44, nblk * 256, 0.015),
                        rng.standard_normal(nblk * 256).astype(np.float32)])
    w[256:512] = 0.0
    w[512:544] = 0.0
    w[1024:1280] = 0.75
    return w


@pytest.mark.parametrize("fmt", DECODE_FORMATS)
def test_decode_bit_exact(O, tfq, gpu, fmt):
    import torch
    print(f"decode {fmt}", flush=True)
    w = _inputs(O, 64)
    pay = O.encode_tensor(fmt, w)
    want = O.decode_tensor(fmt, pay, w.size)
    got = tfq.decode(fmt, torch.from_numpy(pay).to(gpu), w.size).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("fmt", ["Q_4", "Q_8", "Q_G_2", "Q_G_3", "Q_G_4", "Q_G_8"])
def test_decode_golden_payloads(tfq, gpu, fmt):
    import torch
    c = np.load(os.path.join(G, "codec.npz"))
    pay, want = c[f"{fmt}_payload"], c[f"{fmt}_decoded"]
    got = tfq.decode(fmt, torch.from_numpy(pay.reshape(-1)).to(gpu), want.size).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.reshape(-1).view(np.uint32))


@pytest.mark.parametrize("fmt", ["Q_2", "Q_4", "Q_8", "Q_G_2", "Q_G_3", "Q_G_4", "Q_G_6", "Q_G_8", "Q_G_2_K_L", "Q_G_3_K_M",
                                 "Q_G_4_K_L", "Q_6_5", "SB256A3", "SB256A2", "Q_1", "Q_1_5", "Q_16", "Q_G_16", "Q_24",
                                 "Q_G_24"])
def test_decode_arbitrary_payload_bits(O, tfq, gpu, fmt):
    # every payload bit pattern is legal input: random bytes, finite scales
    import torch
    rng = np.random.default_rng(17)
    nb = O.block_bytes(fmt)
    pay = rng.integers(0, 256, (256, nb), dtype=np.uint8)
    if fmt in ("Q_G_8",):
        pay[:, -16:] &= 0x7B
    elif fmt in ("Q_16", "Q_G_16"):   # binary32 min / max with small exponents, finite residual means
        pay[:, [3, 7]] &= 0x3F
        pay[:, -16:] &= 0x7B
    elif fmt in ("Q_24", "Q_G_24"):   # the top byte of every weight, finite residual means
        pay[:, 2:768:3] &= 0xBF
        pay[:, -16:] &= 0x7B
    elif fmt in ("Q_1", "Q_2", "Q_4", "Q_8"):
        pay[:, :2] &= 0x7B
    else:
        pay[:, -4:] &= 0x7B
    want = O.decode_tensor(fmt, pay.reshape(-1), 256 * 256)
    got = tfq.decode(fmt, torch.from_numpy(pay.reshape(-1)).to(gpu), 256 * 256).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


TAIL_FORMATS = ["Q_2", "Q_4", "Q_8", "Q_32", "Q_G_2", "Q_G_3", "Q_G_4", "Q_G_6", "Q_G_8", "Q_G_2_K_H", "Q_G_4_K_M",
                "Q_G_6_K_L", "Q_6_5", "SB256A3", "Q_1", "Q_G_1_K_M", "Q_1_5", "Q_16", "Q_G_16", "Q_16_5", "Q_24", "Q_G_24",
                "Q_G_24_K_H", "Q_3", "Q_6_K_M", "Q_12", "Q_G_12", "Q_G_12_K_L", "Q_G_12_5", "Q_G_8_K_H", "Q_2_K_L",
                "Q_MX_3_5", "Q_MX_12_5", "Q_MX_24_5", "Q_G_MX_3_5", "Q_G_MX_6_5", "Q_G_MX_8_5", "Q_G_MX_16_5"]


@pytest.mark.parametrize("fmt", TAIL_FORMATS)
def test_decode_with_a_short_last_block(O, tfq, gpu, fmt):
    """Tensors whose size is not a multiple of 256: the last block uses the layout the codec chooses
    for its size (no header, one scale, grouped-lattice fallback, ...)."""
    import torch
    w = _inputs(O, 2)
    for n in (1, 5, 8, 15, 16, 17, 31, 32, 33, 64, 100, 160, 200, 224, 250, 255, 256 + 7, 512 + 250):
        print(f"decode {fmt} n={n}", flush=True)
        pay = O.encode_tensor(fmt, w[:n])
        assert tfq.block_bytes(fmt, n % 256 or 256) == O.block_bytes(fmt, n % 256 or 256)
        want = O.decode_tensor(fmt, pay, n)
        got = tfq.decode(fmt, torch.from_numpy(pay).to(gpu), n).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), n
        rnd = np.random.default_rng(n).integers(0, 256, pay.size, dtype=np.uint8)
        want = O.decode_tensor(fmt, rnd, n)
        got = tfq.decode(fmt, torch.from_numpy(rnd).to(gpu), n).cpu().numpy()
        keep = ~(np.isnan(want) & np.isnan(got))
        assert np.array_equal(got.view(np.uint32)[keep], want.view(np.uint32)[keep]), n


def test_decode_short_blocks_golden(tfq, gpu):
    """The fixture written from the compiled reference (tests/golden/tails.npz)."""
    import torch
    t = np.load(os.path.join(G, "tails.npz"))
    for fmt, n, which, poff, plen, doff in t["index"]:
        pay = np.ascontiguousarray(t["payloads"][poff:poff + plen])
        want = t["decoded"][doff:doff + n]
        assert tfq.block_bytes(int(fmt), int(n)) == plen, (fmt, n)
        got = tfq.decode(int(fmt), torch.from_numpy(pay).to(gpu), int(n)).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (fmt, n, which)


def test_encode_short_blocks_golden(O, tfq, gpu):
    """The device encoder of a short block against the payloads the compiled reference wrote
    (tests/golden/tails.npz: 42 ids x 13 block sizes x 2 inputs), and a tensor of full blocks plus a
    short one against the oracle."""
    import torch
    t = np.load(os.path.join(G, "tails.npz"))
    for fmt, n, which, poff, plen, doff in t["index"]:
        w = np.ascontiguousarray(t["src"][which][:n])
        want = t["payloads"][poff:poff + plen]
        got = tfq.encode(int(fmt), torch.from_numpy(w).to(gpu)).cpu().numpy()
        assert np.array_equal(got, want), (fmt, n, which)
    for fmt in ("Q_G_4", "Q_4", "Q_G_8", "Q_G_6_K_H", "Q_8_K_H", "Q_G_12", "Q_MX_4_5", "B32S4"):
        n = 3 * 256 + 160
        w = O.rng_normal(77, n, 0.05)
        want = O.encode_tensor(fmt, w)
        got = tfq.encode(fmt, torch.from_numpy(w).to(gpu)).cpu().numpy()
        assert np.array_equal(got, want), fmt
        back = tfq.decode(fmt, torch.from_numpy(want).to(gpu), n).cpu().numpy()
        assert np.array_equal(back.view(np.uint32), O.decode_tensor(fmt, want, n).view(np.uint32)), fmt


def test_encode_short_blocks_every_id_against_oracle(O, tfq, gpu):
    """Every id the library serves x tail sizes on both sides of each layout switch (bare codes, one scale, group
    headers, whole 32-groups) x a gaussian, a heavy-tailed, an all-zero and a constant block: the wavefront
    encoder of a short block gives the oracle's bytes (the oracle itself is pinned by tails.npz)."""
    import torch
    sizes = [1, 5, 7, 8, 9, 15, 16, 17, 24, 31, 32, 33, 40, 48, 63, 64, 65, 96, 100, 127, 128, 160, 192, 200, 224, 254, 255]
    ids = [i for i in range(0, 109) if tfq.lib().tfq_format_supported(i)]
    srcs = [O.rng_normal(901, 256, 0.05), (O.rng_normal(902, 256, 1.0) ** 3 * 0.02).astype(np.float32),
            np.zeros(256, np.float32), np.full(256, -0.37, np.float32)]
    bad, checked = [], 0
    for fmt in ids:
        name = tfq.lib().tfq_format_name(fmt).decode()
        mixed = name.startswith("Q_MX") or name.startswith("Q_G_MX")
        for n in sizes:
            try:
                tfq.block_bytes(fmt, n)
            except tfq.TfqError:
                continue  # the literal block-32 formats hold whole 32-groups only
            for k, src in enumerate(srcs):
                if mixed and k >= 2:
                    continue  # equal magnitudes across a tier boundary: the reference's order is its sort's
                w = np.ascontiguousarray(src[:n])
                want = O.encode_tensor(fmt, w)
                got = tfq.encode(fmt, torch.from_numpy(w).to(gpu)).cpu().numpy()
                checked += 1
                if not np.array_equal(got, want):
                    bad.append((name, n, k))
    assert not bad, bad[:40]
    assert checked > 8000, checked


def test_half_subnormal_scales_decode_exactly(O, tfq, gpu):
    import torch
    pay = np.zeros((128, 272), np.uint8)
    pay[:, :256] = 255
    hs = np.concatenate([np.arange(0, 512), np.arange(0x8000, 0x8000 + 512)]).astype(np.uint16)
    pay[:, 256:] = hs.reshape(128, 8).view(np.uint8).reshape(128, 16)
    want = O.decode_tensor("Q_G_8", pay.reshape(-1), 128 * 256)
    got = tfq.decode("Q_G_8", torch.from_numpy(pay.reshape(-1)).to(gpu), 128 * 256).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("fmt", ["B32S4", "B32S8", "Q_32", "Q_24", "Q_24_5", "Q_G_24", "Q_G_24_K_M", "Q_16", "Q_G_16_5", "Q_G_16",
                                 "Q_G_16_K_L", "Q_1", "Q_G_1", "Q_1_K_M", "Q_G_1_K_H",
                                 "Q_G_4", "Q_4_5", "Q_G_3", "Q_G_2", "SB256A3", "SB256A2", "Q_1_5",
                                 "Q_G_8", "Q_8_5", "Q_8", "Q_4", "Q_2",
                                 "Q_G_2_K_L", "Q_G_3_K_M", "Q_G_4_K_H", "Q_2_5", "Q_G_6_5", "Q_G_6", "Q_G_6_K_L", "Q_G_6_K_M",
                                 "Q_G_6_K_H", "Q_3", "Q_6", "Q_12", "Q_G_12", "Q_12_5", "Q_2_K_M", "Q_2_K_H", "Q_4_K_M", "Q_4_K_H",
                                 "Q_8_K_M", "Q_8_K_H", "Q_3_K_M", "Q_3_K_H", "Q_6_K_M", "Q_6_K_H", "Q_12_K_M", "Q_12_K_H",
                                 "Q_G_8_K_L", "Q_G_8_K_M", "Q_G_8_K_H", "Q_G_12_K_L", "Q_G_12_K_M", "Q_G_12_K_H"])
def test_device_encoder_codes_bit_exact(O, tfq, gpu, fmt):
    import torch
    w = _inputs(O, 64)
    w[2048:2080] = 1e-9          # scale underflows binary16
    w[4096] = 3.0e5              # scale overflows binary16 -> inf -> codes 0
    want = O.encode_tensor(fmt, w)
    got = tfq.encode(fmt, torch.from_numpy(w).to(gpu)).cpu().numpy()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("fmt", ["Q_G_4", "Q_G_3", "Q_G_2", "SB256A3", "SB256A2", "Q_G_8", "Q_8", "Q_4", "Q_2",
                                 "Q_G_2_K_L", "Q_G_3_K_L", "Q_G_4_K_L", "Q_6_5", "Q_G_6", "Q_G_6_K_H",
                                 "Q_3", "Q_6", "Q_12", "Q_G_12", "Q_4_K_H", "Q_6_K_H", "Q_G_12_K_H", "Q_G_8_K_H"])
def test_iterative_encoders_many_blocks(O, tfq, gpu, fmt):
    """The iterative encoders (affine: per-group Lloyd fit + joint refinement; companded 8-bit: golden-section
    scale search; lattice: least-squares refits) on thousands of blocks of four distributions: every payload
    byte equals the oracle's."""
    import torch
    print(f"encode many {fmt}", flush=True)
    rs = np.random.RandomState(11)
    n = (512 if fmt in ("Q_G_8", "Q_8", "Q_G_8_K_H", "Q_12", "Q_G_12", "Q_G_12_K_H", "Q_6_K_H") else 2048) * 256
    w = np.concatenate([(rs.randn(n) * 0.02), rs.randn(n), rs.laplace(0, 0.015, n) + 0.01, np.abs(rs.randn(n)) * 0.3]).astype(np.float32)
    got = tfq.encode(fmt, torch.from_numpy(w).to(gpu)).cpu().numpy()
    want = O.encode_tensor(fmt, w)
    bb = O.block_bytes(fmt)
    bad = np.nonzero((got.reshape(-1, bb) != want.reshape(-1, bb)).any(1))[0]
    assert bad.size == 0, f"{bad.size} of {w.size // 256} blocks differ, first {bad[:5]}"


MIX_FORMATS = ["Q_MX_3_5", "Q_MX_4_5", "Q_MX_6_5", "Q_MX_8_5", "Q_MX_12_5", "Q_MX_16_5", "Q_MX_24_5",
               "Q_G_MX_3_5", "Q_G_MX_4_5", "Q_G_MX_6_5", "Q_G_MX_8_5", "Q_G_MX_12_5", "Q_G_MX_16_5", "Q_G_MX_24_5"]


@pytest.mark.parametrize("fmt", MIX_FORMATS)
def test_mix_encoder_bit_exact_on_distinct_magnitudes(O, tfq, gpu, fmt):
    """Four-tier mixes: tiers by magnitude rank, per-tier scales, values.  Every payload byte equals the
    oracle's on blocks whose magnitudes are pairwise distinct; for equal magnitudes the reference's order is
    whatever its unstable sort leaves, so such blocks are only required to round-trip no worse."""
    import torch
    print(f"encode mix {fmt}", flush=True)
    rs = np.random.RandomState(21)
    nblk = 1024
    w = np.concatenate([(rs.randn(nblk * 256) * 0.02), rs.standard_t(3, nblk * 256) * 0.5, rs.laplace(0, 0.015, nblk * 256) + 0.01]).astype(np.float32)
    blocks = w.reshape(-1, 256)
    distinct = np.array([np.unique(np.abs(b)).size == 256 for b in blocks])
    assert distinct.mean() > 0.95
    got = tfq.encode(fmt, torch.from_numpy(w).to(gpu)).cpu().numpy()
    want = O.encode_tensor(fmt, w)
    bb = O.block_bytes(fmt)
    same = (got.reshape(-1, bb) == want.reshape(-1, bb)).all(1)
    bad = np.nonzero(~same & distinct)[0]
    assert bad.size == 0, f"{bad.size} of {int(distinct.sum())} tie-free blocks differ, first {bad[:5]}"
    # blocks with ties (and an all-zero and a constant block): same size, decoded error not worse than the oracle's
    odd = np.concatenate([blocks[~distinct][:8], np.zeros((1, 256), np.float32), np.full((1, 256), 0.25, np.float32)])
    pay = tfq.encode(fmt, torch.from_numpy(odd.reshape(-1)).to(gpu)).cpu().numpy()
    dec = O.decode_tensor(fmt, pay, odd.size).reshape(-1, 256)
    ref = O.decode_tensor(fmt, O.encode_tensor(fmt, odd.reshape(-1)), odd.size).reshape(-1, 256)
    e_dev = ((dec - odd).astype(np.float64) ** 2).sum(1)
    e_ref = ((ref - odd).astype(np.float64) ** 2).sum(1)
    assert np.all(e_dev <= e_ref * 1.05 + 1e-12)


def test_host_pointer_codec_entry_points(O, tfq, gpu):
    import ctypes as C
    w = O.rng_normal(42, 256 * 8, 0.02)
    L = tfq.lib()
    dst = np.zeros(8 * 144, np.uint8)
    per = np.zeros(8, np.uint32)
    rc = L.tfq_encode_blocks_host(105, w.ctypes.data, w.size, dst.ctypes.data, dst.size, per.ctypes.data)
    assert rc == 0 and np.all(per == 144)
    assert np.array_equal(dst, O.encode_tensor("B32S4", w))
    pay = O.encode_tensor("Q_G_4", w)
    out = np.zeros(w.size, np.float32)
    assert L.tfq_decode_blocks_host(40, pay.ctypes.data, pay.size, w.size, out.ctypes.data) == 0
    assert np.array_equal(out.view(np.uint32), O.decode_tensor("Q_G_4", pay, w.size).view(np.uint32))
    # a format this build does not handle must say so, not encode on the CPU
    assert L.tfq_encode_blocks_host(119, w.ctypes.data, w.size, dst.ctypes.data, dst.size, None) in (2, 3)
