"""The .quant container: the oracle's restatement (oracle/container.py) and the library's reader
(tfq_container_*, host-side parsing; no compute here) against
  * the byte layout the reference's own test spells out (tests/test_protected.cpp:618-621) and its
    fail-closed cases (:606-680),
  * a file written by the reference's QUANTWriter (tests/golden/sample.quant),
  * the compiled reference's QUANTReader where it is built."""
import os
import struct

import numpy as np
import pytest

from oracle import container as OC

G = os.path.join(os.path.dirname(__file__), "golden")
NAMES = ["blk.0.ffn_gate", "mixed", "tail", "raw"]


def p6b_image():
    """write_p6b_valid (tests/test_protected.cpp:581-607): one Q_32 block of 8 weights, tensor "w"."""
    vals = np.arange(1, 9, dtype=np.float32).tobytes()
    return OC.write_image([("w", [(9, 8, b"", vals)])])


@pytest.fixture(scope="module")
def sample():
    with open(os.path.join(G, "sample.quant"), "rb") as f:
        return f.read()


def test_writer_offsets_match_the_reference_test(O):
    img = p6b_image()
    # header 16 B | ft-count @16 | ft-entry @20 (9 B) | tt-count @29 | name_len @33 | name @35 | start @36 | count @40
    assert img[:4] == b"QUA1" and struct.unpack_from("<I", img, 4)[0] == 1 << 22
    assert struct.unpack_from("<I", img, 16)[0] == 1
    assert struct.unpack_from("<IBI", img, 20) == (0, 9, 0)
    assert struct.unpack_from("<I", img, 29)[0] == 1
    assert struct.unpack_from("<H", img, 33)[0] == 1 and img[35:36] == b"w"
    assert struct.unpack_from("<II", img, 36) == (0, 1)
    assert struct.unpack_from("<II", img, 44) == (8, 0) and struct.unpack_from("<I", img, 52)[0] == 32
    assert len(img) == 56 + 32


def readers(tfq, image):
    return OC.Reader(image), tfq.Container(image=image)


def test_fail_closed_cases_of_the_reference_test(tfq):
    img = bytearray(p6b_image())
    r, c = readers(tfq, bytes(img))
    assert r.valid and c.valid and r.tensor_blocks("w") == (0, 1) == c.tensor_blocks("w")
    assert c.block(0)[:3] == (9, 8, 0) and np.frombuffer(c.block(0)[3], np.float32).tolist() == list(range(1, 9))
    # A: tensor (start 7, count 5) beyond the single block
    a = bytearray(img)
    struct.pack_into("<II", a, 36, 7, 5)
    r, c = readers(tfq, bytes(a))
    assert r.valid and c.valid
    assert r.tensor_blocks("w") is None
    with pytest.raises(tfq.TfqError):
        c.tensor_blocks("w")
    assert r.record(7) is None
    with pytest.raises(tfq.TfqError):
        c.block(7)
    # start + count wrapping past 2^32 must not alias block 0
    struct.pack_into("<II", a, 36, 0xFFFFFFFF, 2)
    r, c = readers(tfq, bytes(a))
    assert r.tensor_blocks("w") is None
    with pytest.raises(tfq.TfqError):
        c.tensor_blocks("w")
    # B: format-table count 0xFFFFFFFF -> invalid, no walk
    b = bytearray(img)
    struct.pack_into("<I", b, 16, 0xFFFFFFFF)
    r, c = readers(tfq, bytes(b))
    assert not r.valid and not c.valid and c.num_blocks == 0
    # wrong magic, short file
    for bad in (b"QUA2" + bytes(img[4:]), bytes(img[:10]), b""):
        r, c = readers(tfq, bad)
        assert not r.valid and not c.valid


def test_sample_file_tables(tfq, sample):
    r, c = readers(tfq, sample)
    assert r.valid and c.valid
    assert r.tensor_names() == NAMES == c.tensor_names()
    assert c.header() == (1 << 22, 0, b"hello") and r.config() == b"hello"
    assert r.blocks == 16 == c.num_blocks
    want = {"blk.0.ffn_gate": (0, 8), "mixed": (8, 5), "tail": (13, 2), "raw": (15, 1)}
    for name, rng in want.items():
        assert r.tensor_blocks(name) == rng == c.tensor_blocks(name)
    fmts = [40] * 8 + [40, 42, 3, 41, 52] + [42, 42] + [9]
    sizes = [144] * 8 + [144, 272, 128, 210, 110] + [272, 46] + [160]
    for b in range(16):
        nw, cb, idx = r.record(b)
        f, nw2, cb2, idx2 = c.block(b)
        assert (OC.clamp_format(r.format[b]), nw, len(cb), idx) == (f, nw2, cb2, idx2)
        assert f == fmts[b] and len(idx) == sizes[b], b
        assert nw == (44 if b == 14 else 40 if b == 15 else 256)
    with pytest.raises(tfq.TfqError):
        c.tensor_blocks("absent")


def test_oracle_decodes_the_sample_like_the_reference(O, sample):
    want = np.load(os.path.join(G, "sample_quant.npz"))
    r = OC.Reader(sample)
    for name in NAMES:
        got = np.array(r.tensor(name, lambda f, pay, n: O.decode_block(f, np.frombuffer(pay, np.uint8), n)), np.float32)
        assert np.array_equal(got.view(np.uint32), want[name].view(np.uint32)), name


def test_format_byte_clamp(tfq, sample):
    """ids outside the enum and id 19 read as Q_32 (src/codec/quant_format.cpp:430-434); the four appended
    ids stay themselves in this library's reader."""
    assert [OC.clamp_format(b) for b in (0, 18, 19, 20, 104, 105, 200, 255)] == [0, 18, 9, 20, 104, 9, 9, 9]
    img = bytearray(sample)
    ft = 16 + 5 + 4
    for blk, byte in ((0, 19), (1, 200), (2, 105), (3, 109)):
        img[ft + 9 * blk + 4] = byte
    c = tfq.Container(image=bytes(img))
    assert [c.block(b)[0] for b in range(4)] == [9, 9, 105, 9]


def test_every_truncation_is_handled(tfq, sample):
    """No prefix of a good file may crash a reader; both agree on what is still reachable."""
    for cut in list(range(0, 120)) + list(range(120, len(sample), 37)) + [len(sample) - 1]:
        r, c = readers(tfq, sample[:cut])
        assert r.valid == c.valid, cut
        if not r.valid:
            continue
        assert r.tensor_names() == c.tensor_names(), cut
        for b in range(r.blocks):
            rec = r.record(b)
            if rec is None:
                with pytest.raises(tfq.TfqError):
                    c.block(b)
            else:
                assert c.block(b)[1:] == (rec[0], len(rec[1]), rec[2]), (cut, b)


def test_against_the_compiled_reference_reader(O, tfq, tmp_path):
    if not O.have_ref():
        pytest.skip("compiled reference not built on this machine")
    rs = np.random.RandomState(0)
    tensors = [("a", rs.randn(700).astype(np.float32) * 0.02), ("b.weight", rs.randn(512).astype(np.float32)),
               ("", rs.randn(5).astype(np.float32))]
    fmts = ["Q_G_4", "Q_G_2", "Q_G_4"] + ["Q_8", "Q_G_6_K_M"] + ["Q_G_4"]
    path = str(tmp_path / "t.quant")
    assert O.ref_container_write(path, tensors, fmts, config=b"\x01\x02", version=7) == 6
    image = open(path, "rb").read()
    info = O.ref_container_info(path)
    r, c = readers(tfq, image)
    assert info == dict(valid=True, blocks=r.blocks, tensors=len(r.tensor_names()), version=7, config_size=2)
    assert c.header() == (7, 0, b"\x01\x02")
    for name, w in tensors:
        assert O.ref_container_tensor_blocks(path, name) == r.tensor_blocks(name) == c.tensor_blocks(name)
        want = O.ref_container_read_tensor(path, name)
        got = np.array(r.tensor(name, lambda f, pay, n: O.decode_block(f, np.frombuffer(pay, np.uint8), n)), np.float32)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), name
    for b in range(6):
        rb = O.ref_container_block(path, b)
        assert (rb["weights"], rb["cb_bytes"], rb["idx_bytes"]) == (c.block(b)[1], c.block(b)[2], len(c.block(b)[3]))
        assert rb["format"] == c.block(b)[0] and rb["offset"] == r.offset[b]
    # the same image rewritten by the restated writer is byte-identical
    blocks = [(O.FMT[f], 0, b"", b"") for f in fmts]
    recs = [r.record(b) for b in range(6)]
    rebuilt = OC.write_image([("a", [(O.FMT[fmts[b]], recs[b][0], recs[b][1], recs[b][2]) for b in range(3)]),
                              ("b.weight", [(O.FMT[fmts[b]], recs[b][0], recs[b][1], recs[b][2]) for b in (3, 4)]),
                              ("", [(O.FMT[fmts[5]], recs[5][0], recs[5][1], recs[5][2])])],
                             version=7, config=b"\x01\x02")
    assert rebuilt == image
    # truncations: the reference's reader and both of ours agree on validity and block reachability
    for cut in range(0, len(image), 53):
        open(path, "wb").write(image[:cut])
        info = O.ref_container_info(path)
        r, c = readers(tfq, image[:cut])
        assert info["valid"] == r.valid == c.valid, cut
        if r.valid:
            assert info["blocks"] == r.blocks and info["tensors"] == len(r.tensor_names()), cut
            for b in range(r.blocks):
                assert (O.ref_container_block(path, b) is None) == (r.record(b) is None), (cut, b)
