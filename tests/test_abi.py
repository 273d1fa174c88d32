"""The C-ABI library loads on a CPU-only machine and exports every symbol that
include/tfq.h declares; argument errors are reported without a GPU."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "tfq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tfq_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(tfq):
    lib = C.CDLL(tfq.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/tfq.h but not exported"


def test_registry_mirror_without_gpu(tfq):
    L = tfq.lib()
    for spelling in (b"Q_G_4", b"QG4", b"qg4", b"Q.G.4"):
        assert L.tfq_format_id(spelling) == 40
    assert L.tfq_format_id(b"Q_G_8") == 42 and L.tfq_format_id(b"b32s4") == 105
    assert L.tfq_format_id(b"nope") == -1
    assert L.tfq_format_name(40) == b"Q_G_4" and L.tfq_format_name(200) == b"unknown"
    # wire-truth bpw table (include/quant/types.h:197-230 of the reference)
    for fid, bpw in ((3, 4.0), (5, 8.0), (38, 2.625), (39, 3.5), (40, 4.5), (42, 8.5), (105, 4.5), (106, 8.5),
                     (107, 3.875), (108, 2.875), (2, 3.0), (6, 12.0), (43, 12.5), (74, 2.4375), (77, 6.4375), (61, 8.5),
                     (64, 12.5), (83, 2.4375), (25, 8.0), (91, 3.5), (98, 3.78125), (104, 24.5)):
        assert L.tfq_format_bpw(fid) == pytest.approx(bpw)
    for fmt, nbytes in (("Q_4", 128), ("Q_8", 256), ("Q_G_2", 84), ("Q_G_3", 112), ("Q_G_4", 144), ("Q_G_8", 272),
                        ("Q_3", 96), ("Q_6_K_H", 192), ("Q_12", 384), ("Q_G_12", 400), ("Q_G_12_K_M", 400), ("Q_G_8_K_L", 272)):
        assert tfq.block_bytes(fmt) == nbytes


def test_errors_are_reported_not_swallowed(tfq):
    L = tfq.lib()
    out = C.c_size_t(0)
    assert L.tfq_block_bytes(19 + 100, 256, C.byref(out)) == 2     # TFQ_ERR_FORMAT: no such wire id
    assert b"not handled" in L.tfq_last_error()
    assert L.tfq_block_bytes(40, 100, C.byref(out)) == 0 and out.value == 57   # short block: grouped-lattice fallback
    assert L.tfq_block_bytes(40, 257, C.byref(out)) == 3           # TFQ_ERR_SHAPE
    assert L.tfq_block_bytes(105, 100, C.byref(out)) == 3          # literal formats need whole groups of 32
    assert L.tfq_gemv(None, None, 0, 1, None, 0, None) == 1        # TFQ_ERR_ARG
    assert L.tfq_weight_upload(40, 4, 100, None, 0) is None        # null payload
    with pytest.raises(tfq.TfqError):
        tfq.block_bytes("Q_G_4", 300)


def test_no_cpu_fallback_without_device(tfq):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    L = tfq.lib()
    buf = (C.c_uint8 * (144 * 4))()
    h = L.tfq_weight_upload(40, 4, 256, buf, len(buf))
    assert h is None and L.tfq_last_error() != b""
    src = (C.c_float * 256)()
    dst = (C.c_uint8 * 144)()
    assert L.tfq_encode_blocks_host(105, src, 256, dst, 144, None) == 4   # TFQ_ERR_DEVICE


def test_block_sizes_equal_the_oracle_for_every_id_and_length(O, tfq):
    """The host-side layout rules (which short-block layout a length takes) against the oracle's, which is
    pinned to the compiled reference: all handled wire ids, every n up to a full block."""
    L = tfq.lib()
    out = C.c_size_t(0)
    for name, fid in sorted(tfq.FMT.items()):
        for n in range(1, 257):
            want = O.block_bytes(fid, n)
            rc = L.tfq_block_bytes(fid, n, C.byref(out))
            if want < 0:
                assert rc != 0, (name, n)
            else:
                assert rc == 0 and out.value == want, (name, n, out.value, want)
