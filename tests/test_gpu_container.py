"""Tensors of a .quant container decoded and multiplied on the device (tfq_container_read_tensor,
tfq_container_weight) against the fixture written and read back by the compiled reference
(tests/golden/sample.quant, sample_quant.npz) and against the oracle."""
import os

import numpy as np
import pytest

from oracle import container as OC

pytestmark = pytest.mark.gpu
G = os.path.join(os.path.dirname(__file__), "golden")


def test_read_tensor_bit_exact(tfq, gpu):
    want = np.load(os.path.join(G, "sample_quant.npz"))
    c = tfq.Container(path=os.path.join(G, "sample.quant"))
    assert c.valid
    for name in c.tensor_names():
        print(f"container read_tensor {name}", flush=True)
        got = c.read_tensor(name).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want[name].view(np.uint32)), name
    # host-pointer variant
    out = np.zeros(2048, np.float32)
    assert tfq.lib().tfq_container_read_tensor_host(c.handle, b"blk.0.ffn_gate", out.ctypes.data, out.size) == 0
    assert np.array_equal(out.view(np.uint32), want["blk.0.ffn_gate"].view(np.uint32))
    assert tfq.lib().tfq_container_read_tensor_host(c.handle, b"blk.0.ffn_gate", out.ctypes.data, 100) == 3


def test_weight_from_container_runs_the_matmul(O, tfq, gpu):
    import torch
    c = tfq.Container(path=os.path.join(G, "sample.quant"))
    r = OC.Reader(open(os.path.join(G, "sample.quant"), "rb").read())
    W = c.weight("blk.0.ffn_gate", 4, 512)
    assert (W.fmt, W.N, W.K) == (40, 4, 512)
    pay = np.frombuffer(b"".join(r.record(b)[2] for b in range(8)), np.uint8)
    x = O.rng_normal(43, 3 * 512, 1.0).reshape(3, 512)
    y = W.gemv(torch.from_numpy(x).to(gpu)).cpu().numpy()
    ref = O.matmul("Q_G_4", pay, 4, 512, x)
    assert float(np.abs(y - ref).max() / np.abs(ref).max()) <= 1e-3
    assert np.array_equal(W.decode().cpu().numpy().reshape(-1).view(np.uint32),
                          np.load(os.path.join(G, "sample_quant.npz"))["blk.0.ffn_gate"].view(np.uint32))
    # a smaller shape takes the tensor's first rows * cols / 256 blocks (Qwen35Engine::resolve accepts count >= need)
    W2 = c.weight("blk.0.ffn_gate", 2, 512)
    assert np.array_equal(W2.decode().cpu().numpy(), W.decode().cpu().numpy()[:2])
    for bad in (("blk.0.ffn_gate", 5, 512), ("blk.0.ffn_gate", 4, 500), ("tail", 1, 512), ("absent", 1, 256)):
        with pytest.raises(tfq.TfqError):
            c.weight(*bad)


def test_mixed_format_tensor_runs_the_matmul(O, tfq, gpu):
    """The reference-written tensor whose five blocks carry five wire ids: Qwen35Engine::gemm decodes each block by
    its own format byte (decode_block, src/adapters/tools/qwen35_engine.cpp:19-35) and multiplies.  Expected: the
    decoded values the compiled reference wrote into the fixture, bit for bit, and the block-row product of exactly
    those values (the oracle's matmul over them as a Q_32 matrix)."""
    import torch
    c = tfq.Container(path=os.path.join(G, "sample.quant"))
    want = np.load(os.path.join(G, "sample_quant.npz"))["mixed"]
    W = c.weight("mixed", 1, 1280)
    assert (W.N, W.K) == (1, 1280)
    assert np.array_equal(W.decode().cpu().numpy().reshape(-1).view(np.uint32), want.view(np.uint32))
    x = O.rng_normal(43, 4 * 1280, 1.0).reshape(4, 1280)
    ref = O.matmul("Q_32", want.view(np.uint8), 1, 1280, x)
    y = W.gemv(torch.from_numpy(x).to(gpu)).cpu().numpy()
    assert float(np.abs(y - ref).max() / np.abs(ref).max()) <= 1e-3
    xb = O.bf16_round(x)
    yb = W.gemv(torch.from_numpy(xb).to(gpu).bfloat16()).cpu().numpy()
    refb = O.matmul("Q_32", want.view(np.uint8), 1, 1280, xb)
    assert float(np.abs(yb - refb).max() / np.abs(refb).max()) <= 1e-2


def test_mixed_upload_every_wire_id(O, tfq, gpu):
    """A 6 x 4608 matrix whose 108 blocks walk through every wire id the library encodes (0..108 without the
    container's id-19 quirk): decode equals the oracle's per-block decode bit for bit, the product equals the
    block-row product of the decoded matrix."""
    import torch
    ids = [i for i in range(109) if tfq.lib().tfq_format_supported(i)]
    N, K = 6, 4608
    nblocks = N * K // 256
    fmts = [ids[b % len(ids)] for b in range(nblocks)]
    w = O.rng_normal(77, N * K, 0.05)
    pays, dec = [], []
    for b, f in enumerate(fmts):
        p = O.encode_block(f, w[b * 256:(b + 1) * 256])
        pays.append(p)
        dec.append(O.decode_block(f, p))
    W = tfq.Weight.mixed(N, K, fmts, np.concatenate(pays))
    dense = np.concatenate(dec).astype(np.float32)
    assert np.array_equal(W.decode().cpu().numpy().reshape(-1).view(np.uint32), dense.view(np.uint32))
    x = O.rng_normal(78, 5 * K, 1.0).reshape(5, K)
    ref = O.matmul("Q_32", dense.view(np.uint8), N, K, x)
    y = W.gemv(torch.from_numpy(x).to(gpu)).cpu().numpy()
    assert float(np.abs(y - ref).max() / np.abs(ref).max()) <= 1e-3
    # the prefill entry slices through the same kernel
    xm = O.rng_normal(79, 20 * K, 1.0).reshape(20, K)
    refm = O.matmul("Q_32", dense.view(np.uint8), N, K, xm)
    ym = W.gemm(torch.from_numpy(xm).to(gpu), workspace=False).cpu().numpy()
    assert float(np.abs(ym - refm).max() / np.abs(refm).max()) <= 1e-3
    with pytest.raises(tfq.TfqError):  # payload size must match the blocks
        tfq.Weight.mixed(N, K, fmts, np.concatenate(pays)[:-1])


def test_larger_container_from_the_restated_writer(O, tfq, gpu):
    """A file built by the oracle's writer: 64 x 1024 matrix in B32S4 (an appended id) next to a Q_G_8 one."""
    import torch
    w = O.rng_normal(42, 64 * 1024, 0.02)
    tensors = []
    for name, fmt in (("ffn_up", "B32S4"), ("ffn_down", "Q_G_8")):
        pay = O.encode_tensor(fmt, w)
        nb = O.block_bytes(fmt)
        tensors.append((name, [(O.FMT[fmt], 256, b"", pay[i:i + nb].tobytes()) for i in range(0, pay.size, nb)]))
    c = tfq.Container(image=OC.write_image(tensors))
    x = O.bf16_round(O.rng_normal(43, 2 * 1024, 1.0).reshape(2, 1024))
    for name, fmt in (("ffn_up", "B32S4"), ("ffn_down", "Q_G_8")):
        print(f"container weight {name}", flush=True)
        W = c.weight(name, 64, 1024)
        y = W.gemv(torch.from_numpy(x).to(gpu).bfloat16()).cpu().numpy()
        ref = O.matmul(fmt, O.encode_tensor(fmt, w), 64, 1024, x)
        assert float(np.abs(y - ref).max() / np.abs(ref).max()) <= 1e-2
        got = c.read_tensor(name).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), O.decode_tensor(fmt, O.encode_tensor(fmt, w), w.size).view(np.uint32))
