"""The literal block-32 formats against an independent brute-force statement
(numpy, one line per step of the definition).  CPU only."""
import numpy as np
import pytest


def brute_b32(w, bits):
    qmax = 7.0 if bits == 4 else 127.0
    lo, hi = (-8, 7) if bits == 4 else (-127, 127)
    w = w.reshape(-1, 32).astype(np.float32)
    amax = np.abs(w).max(axis=1)
    d16 = (amax / np.float32(qmax)).astype(np.float32).astype(np.float16)  # IEEE RNE
    d = d16.astype(np.float32)
    q = np.zeros_like(w, dtype=np.int32)
    live = (d > 0) & np.isfinite(d)
    r = w[live] / d[live][:, None]
    r = np.sign(r) * np.floor(np.abs(r) + np.float32(0.5))  # half away from zero
    q[live] = np.clip(r, lo, hi).astype(np.int32)
    return q, d16


@pytest.mark.parametrize("fmt,bits", [("B32S4", 4), ("B32S8", 8)])
def test_sym32_against_brute_force(O, fmt, bits):
    rng = np.random.default_rng(3)
    w = np.concatenate([O.rng_normal(42, 256 * 40, 0.02), rng.standard_normal(256 * 8).astype(np.float32),
                        np.zeros(256, np.float32), np.full(256, 0.25, np.float32)])
    w[5 * 256:5 * 256 + 32] = 0.0
    q, d16 = brute_b32(w, bits)
    q = q.reshape(-1, 256)
    d16 = d16.reshape(-1, 8)
    pay = O.encode_tensor(fmt, w).reshape(-1, 144 if bits == 4 else 272)
    for b in range(pay.shape[0]):
        if bits == 4:
            nib = np.stack([pay[b, :128] & 15, pay[b, :128] >> 4], axis=1).reshape(-1).astype(np.int32) - 8
            assert np.array_equal(nib, q[b])
            sc = pay[b, 128:].view(np.uint16)
        else:
            assert np.array_equal(pay[b, :256].view(np.int8).astype(np.int32), q[b])
            sc = pay[b, 256:].view(np.uint16)
        assert np.array_equal(sc, d16[b].view(np.uint16))
        dec = O.decode_block(fmt, pay[b])
        want = (q[b].astype(np.float32).reshape(8, 32) * d16[b].astype(np.float32)[:, None]).reshape(-1)
        assert np.array_equal(dec.view(np.uint32), want.view(np.uint32))
    # idempotence: re-encoding a decoded block reproduces the codes when the absmax code is +-qmax
    dec = O.decode_tensor(fmt, pay.reshape(-1), w.size)
    assert np.array_equal(O.decode_tensor(fmt, O.encode_tensor(fmt, dec), w.size), dec)


@pytest.mark.parametrize("fmt,bits,bytes_", [("SB256A3", 3, 124), ("SB256A2", 2, 92)])
def test_superblock_layout(O, fmt, bits, bytes_):
    # 16 sub-blocks of 16, 6-bit scale + 6-bit min each, binary16 super scale / min
    assert bits * 32 + 12 + 12 + 4 == bytes_ == O.block_bytes(fmt, 256)
    w = O.rng_laplace(44, 256 * 16, 0.015)
    pay = O.encode_tensor(fmt, w).reshape(-1, bytes_)
    dec = O.decode_tensor(fmt, pay.reshape(-1), w.size).reshape(-1, 256)
    top = float(2 ** bits - 1)
    for b in range(pay.shape[0]):
        bits_le = np.unpackbits(pay[b], bitorder="little")
        idx = bits_le[:256 * bits].reshape(256, bits) @ (1 << np.arange(bits))
        sc = bits_le[256 * bits:256 * bits + 96].reshape(16, 6) @ (1 << np.arange(6))
        mc = bits_le[256 * bits + 96:256 * bits + 192].reshape(16, 6) @ (1 << np.arange(6)) - 32
        d = pay[b, -4:-2].view(np.float16).astype(np.float32)[0]
        dm = pay[b, -2:].view(np.float16).astype(np.float32)[0]
        lv = idx.astype(np.float32) * np.float32(1.0 / top)
        es = (d * sc.astype(np.float32)).astype(np.float32)
        neg = -(dm * mc.astype(np.float32)).astype(np.float32)
        want = (es.repeat(16).astype(np.float64) * lv.astype(np.float64) + neg.repeat(16).astype(np.float64)).astype(np.float32)
        assert np.array_equal(dec[b].view(np.uint32), want.view(np.uint32))


def test_laplace_generator_moments(O):
    w = O.rng_laplace(44, 400000, 0.015)
    assert abs(float(w.mean())) < 2e-4
    assert abs(float(np.abs(w).mean()) - 0.015) < 2e-4          # E|x| = b
    assert abs(float(w.var()) - 2 * 0.015 ** 2) < 2e-5          # Var = 2 b^2
