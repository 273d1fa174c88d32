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
    for bad in (("blk.0.ffn_gate", 5, 512), ("blk.0.ffn_gate", 4, 500), ("mixed", 1, 1280), ("tail", 1, 512), ("absent", 1, 256)):
        with pytest.raises(tfq.TfqError):
            c.weight(*bad)


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
