"""Writes the golden fixtures from the COMPILED REFERENCE (oracle/_ref/libref.so,
built from the reference's own sources by oracle/Makefile).  Run it where the
reference tree exists; the fixtures it writes are what travels.

    python tests/golden/make_golden.py

codec.npz
    w            [4 distributions x 8 blocks x 256] fp32 inputs (seeded with the
                 reference generator: N(0,0.02) seed 42, N(0,1) seed 43,
                 Laplace(0,0.015) seed 44, heavy-tail mix seed 46)
    <fmt>_payload  uint8 payload of every block, reference quantize_block_all
    <fmt>_decoded  fp32 output of reference dequantize_block_all on that payload
    comp8_levels  the 256-entry companded grid (decoded from a Q_G_8 payload
                 with codes 0..255 and scale 1.0)
    f16_all_decoded  binary32 bit patterns the reference decodes all 65,536
                 binary16 patterns to (each pattern placed as a Q_G_8 group scale
                 over code 255, whose level is exactly 1.0)
rng.npz
    u64_42, uniform_42, normal_42_002, normal_43: first 4096 draws of RNG(seed)
tails.npz
    blocks of n <= 256 weights (the first n of two of the inputs above) through the
    reference codec, one row of `index` = (wire id, n, input, payload offset, payload
    bytes, decoded offset) into the flat `payloads` / `decoded` arrays: the short-block
    layouts (raw levels, one scale, grouped-lattice fallback), Q_2, Q_G_6, the ids
    whose claim is below the affine header's size, the sign formats, the 16- and
    24-bit formats, the fixed-codebook formats, the 12-bit compound, searched tiers and
    four-tier mixes
sample.quant, sample_quant.npz
    a container written by the reference's QUANTWriter (header with a 5-byte config,
    format table, tensor table, block records): tensor "blk.0.ffn_gate" 4 x 512 in Q_G_4,
    "mixed" whose blocks alternate formats, "tail" of 300 weights in Q_G_8 and "raw" of 40
    weights in Q_32; the npz holds what QUANTReader::read_tensor returns for each name
fixed_levels.npz, ../../transformers-fusion_amd/csrc/fixed{6,12}_levels.inc
    the 64- and 4096-entry level tables of Q_6 / Q_12 as binary32 bit patterns, read off
    the reference by decoding blocks of fewer than 16 weights (raw codes, implied scale 1)
    that hold every code once; the .inc files carry the same words for the device build
matmul.npz
    for Q_G_4 and Q_G_8: y = x.W^T with W 48x512 from the fixture generator,
    computed by the reference scalar_gemm_bt on the reference-decoded matrix
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle as O  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
FORMATS = ["Q_4", "Q_8", "Q_G_2", "Q_G_3", "Q_G_4", "Q_G_8", "Q_32"]


def inputs():
    nb = 8
    a = O.ref_rng_normal(42, nb * 256, 0.02)
    b = O.ref_rng_normal(43, nb * 256, 1.0)
    u = O.ref_rng_uniform(44, nb * 256) - np.float32(0.5)
    c = (-np.float32(0.015) * np.sign(u) * np.log(np.float32(1) - np.float32(2) * np.abs(u))).astype(np.float32)
    d = O.ref_rng_normal(46, nb * 256, 0.02)
    d[::37] *= np.float32(25.0)
    d[256:512] = 0.0              # an all-zero block
    d[512:768] = np.float32(0.5)  # a constant block
    d[768:800] = 0.0              # one zero group inside a live block
    return np.stack([a, b, c, d]).reshape(4, nb, 256)


TAIL_FORMATS = ["Q_2", "Q_4", "Q_8", "Q_G_2", "Q_G_3", "Q_G_4", "Q_G_6", "Q_G_8", "Q_G_2_K_H", "Q_G_3_K_L",
                "Q_G_4_K_M", "Q_G_6_K_M", "Q_G_6_K_H", "Q_2_5", "Q_6_5",
                "Q_1", "Q_G_1_K_H", "Q_1_5", "Q_16", "Q_G_16", "Q_24", "Q_G_24",
                "Q_3", "Q_6", "Q_12", "Q_2_K_H", "Q_4_K_M", "Q_8_K_H", "Q_3_K_H", "Q_6_K_M", "Q_12_K_H", "Q_G_12",
                "Q_G_8_K_H", "Q_G_12_K_H", "Q_12_5", "Q_MX_3_5", "Q_MX_12_5", "Q_MX_24_5", "Q_G_MX_3_5", "Q_G_MX_6_5",
                "Q_G_MX_8_5", "Q_G_MX_16_5"]
TAIL_SIZES = [1, 7, 8, 15, 16, 31, 32, 33, 100, 160, 250, 255, 256]


def tails(w):
    src = [w[0].reshape(-1), w[2].reshape(-1) + np.float32(0.01)]
    index, pays, decs, poff, doff = [], [], [], 0, 0
    for fmt in TAIL_FORMATS:
        for n in TAIL_SIZES:
            for which, x in enumerate(src):
                p = O.ref_encode_block(fmt, x[300:300 + n])
                index.append((O.FMT[fmt], n, which, poff, p.size, doff))
                pays.append(p)
                decs.append(O.ref_decode_block(fmt, p, n))
                poff += p.size
                doff += n
    np.savez_compressed(os.path.join(HERE, "tails.npz"), src=np.stack([s[300:556] for s in src]),
                        index=np.array(index, np.int64), payloads=np.concatenate(pays),
                        decoded=np.concatenate(decs))


def container(w):
    flat = w.reshape(-1)
    tensors = [("blk.0.ffn_gate", flat[:2048]), ("mixed", flat[2048:2048 + 1280]), ("tail", flat[4096:4396]),
               ("raw", flat[5000:5040])]
    fmts = ["Q_G_4"] * 8 + ["Q_G_4", "Q_G_8", "Q_4", "Q_G_6", "Q_G_3_K_L"] + ["Q_G_8", "Q_G_8"] + ["Q_32"]
    path = os.path.join(HERE, "sample.quant")
    assert O.ref_container_write(path, tensors, fmts, config=b"hello") == len(fmts)
    np.savez_compressed(os.path.join(HERE, "sample_quant.npz"),
                        **{name: O.ref_container_read_tensor(path, name) for name, _ in tensors})


def pack_lsb_first(codes, bits):
    """Codes into a byte string, each `bits` wide, least significant bit first."""
    out = np.zeros((len(codes) * bits + 7) // 8, np.uint8)
    pos = 0
    for c in codes:
        for b in range(bits):
            if (int(c) >> b) & 1:
                out[pos >> 3] |= 1 << (pos & 7)
            pos += 1
    return out


def fixed_levels():
    tables = {}
    for bits, fmt in ((6, "Q_6"), (12, "Q_12")):
        count = 1 << bits
        vals = np.empty(count, np.float32)
        for c0 in range(0, count, 15):
            codes = np.arange(c0, min(c0 + 15, count))
            vals[c0:c0 + len(codes)] = O.ref_decode_block(fmt, pack_lsb_first(codes, bits), len(codes))
        tables[f"t{bits}"] = vals.view(np.uint32)
        inc = os.path.join(ROOT, "transformers-fusion_amd", "csrc", f"fixed{bits}_levels.inc")
        with open(inc, "w") as f:
            f.write(f"// {count} levels of the fixed {bits}-bit codebook as binary32 bit patterns: mid-quantiles of N(0,1),\n"
                    f"// levels[j] = -levels[{count - 1} - j] = RN(sqrt(2) * erfinv(2 (j + 0.5) / {count} - 1)) for j < {count // 2}, with the\n"
                    "// reference's own erf approximation and Newton inverse (src/codec/block_codec.cpp:542-588).\n"
                    "// Shipped as data so that no transcendental is evaluated on the device.\n")
            words = [f"0x{int(v):08x}u" for v in vals.view(np.uint32)]
            for i in range(0, count, 8):
                f.write("    " + ", ".join(words[i:i + 8]) + ",\n")
    np.savez_compressed(os.path.join(HERE, "fixed_levels.npz"), **tables)


def main():
    assert O.have_ref(), "build oracle/_ref first (make -C oracle)"
    w = inputs()
    fixed_levels()
    tails(w)
    container(w)
    out = {"w": w}
    for fmt in FORMATS:
        pays, decs = [], []
        for blk in w.reshape(-1, 256):
            p = O.ref_encode_block(fmt, blk)
            pays.append(p)
            decs.append(O.ref_decode_block(fmt, p))
        out[f"{fmt}_payload"] = np.stack(pays)
        out[f"{fmt}_decoded"] = np.stack(decs)
    p = np.zeros(272, np.uint8)
    p[:256] = np.arange(256)
    p[257:272:2] = 0x3C
    out["comp8_levels"] = O.ref_decode_block("Q_G_8", p)
    # binary16 -> binary32 seen through the codec: every 16-bit pattern as a
    # Q_G_8 group scale over code 255 (level exactly 1.0).
    dec = np.empty(65536, np.float32)
    for h0 in range(0, 65536, 8):
        q = np.zeros(272, np.uint8)
        q[:256] = 255
        for g in range(8):
            q[256 + 2 * g] = (h0 + g) & 0xFF
            q[256 + 2 * g + 1] = (h0 + g) >> 8
        dec[h0:h0 + 8] = O.ref_decode_block("Q_G_8", q)[::32]
    out["f16_all_decoded"] = dec.view(np.uint32)
    np.savez_compressed(os.path.join(HERE, "codec.npz"), **out)

    rng = {
        "u64_42": np.empty(4096, np.uint64),
        "uniform_42": O.ref_rng_uniform(42, 4096),
        "normal_42_002": O.ref_rng_normal(42, 4096, 0.02),
        "normal_43": O.ref_rng_normal(43, 4096, 1.0),
    }
    import ctypes as C
    O.ref.ref_rng_u64(42, 4096, rng["u64_42"].ctypes.data_as(C.POINTER(C.c_uint64)))
    np.savez_compressed(os.path.join(HERE, "rng.npz"), **rng)

    N, K, B = 48, 512, 3
    W = O.ref_rng_normal(47, N * K, 0.02)
    X = O.ref_rng_normal(48, B * K, 1.0)
    mm = {"W": W, "X": X}
    for fmt in ("Q_G_4", "Q_G_8", "Q_4"):
        pays = np.concatenate([O.ref_encode_block(fmt, W[i:i + 256]) for i in range(0, N * K, 256)])
        dec = np.concatenate([O.ref_decode_block(fmt, pays[i:i + len(pays) // (N * K // 256)])
                              for i in range(0, len(pays), len(pays) // (N * K // 256))])
        Y = np.empty((B, N), np.float32)
        _f = C.POINTER(C.c_float)
        O.ref.ref_scalar_gemm_bt(X.ctypes.data_as(_f), dec.ctypes.data_as(_f), Y.ctypes.data_as(_f), B, N, K)
        mm[f"{fmt}_payload"] = pays
        mm[f"{fmt}_y"] = Y
    np.savez_compressed(os.path.join(HERE, "matmul.npz"), **mm)
    for f in ("codec.npz", "rng.npz", "matmul.npz", "tails.npz", "sample.quant", "sample_quant.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)))


if __name__ == "__main__":
    main()
