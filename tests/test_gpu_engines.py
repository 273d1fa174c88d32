"""The in-memory engines on the device (tfq_engine_*, tfq_q8codec_*, tfq_q8_*) against the oracle:
indices, scales, centroids and decoded values bit-exact; quant_gemm within 1e-3 of max |ref|."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def same(a, b):
    return np.array_equal(np.ascontiguousarray(a).view(np.uint8), np.ascontiguousarray(b).view(np.uint8))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("n,bs", [(1000, 256), (256, 64), (777, 100), (5, 8), (70000, 256), (5000, 5000)])
def test_per_block_and_tensor_codes_bit_exact(O, tfq, gpu, bits, n, bs):
    import torch
    print(f"engine bits={bits} n={n} bs={bs}", flush=True)
    rs = np.random.RandomState(n + bits)
    cb = (np.sort(rs.randn(1 << bits)) * 0.5).astype(np.float32)
    data = (rs.randn(n) * 0.05 + 0.01).astype(np.float32)
    if n >= 1000:
        data[256:512] = 0.125     # a flat block
    eng = tfq.CodebookEngine(bits, cb)
    d = torch.from_numpy(data).to(gpu)
    idx, scales = eng.quantize_per_block(d, bs)
    want_idx, want_scales = O.engine_quantize_per_block(bits, cb, data, bs)
    assert same(idx.cpu().numpy(), want_idx) and same(scales.cpu().numpy(), want_scales)
    back = eng.dequantize_per_block(idx, scales, bs).cpu().numpy()
    assert same(back, O.engine_dequantize_per_block(bits, cb, want_idx, want_scales, bs))
    packed = eng.quantize_tensor(d)
    want = O.engine_quantize_tensor(bits, cb, data)
    assert same(packed.cpu().numpy(), want)
    assert same(eng.dequant_tensor(packed, n).cpu().numpy(), O.engine_dequant_tensor(bits, cb, want, n))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (3, 8, 16), (5, 7, 33), (2, 64, 128), (9, 300, 200), (16, 4096, 512)])
def test_quant_gemm(O, tfq, gpu, bits, M, N, K):
    import torch
    print(f"engine gemm bits={bits} M={M} N={N} K={K}", flush=True)
    rs = np.random.RandomState(M * N + K)
    cb = rs.randn(1 << bits).astype(np.float32)
    a = rs.randn(M, K).astype(np.float32)
    a[0, 0] = 0.0
    bidx = rs.randint(0, 256, (K * N + 1) // 2 if bits == 4 else K * N).astype(np.uint8)
    ref = O.engine_quant_gemm(bits, cb, a, bidx, M, N, K)
    got = tfq.CodebookEngine(bits, cb).quant_gemm(torch.from_numpy(a).to(gpu), torch.from_numpy(bidx).to(gpu), M, N, K)
    assert float(np.abs(got.cpu().numpy() - ref).max()) <= 1e-3 * float(np.abs(ref).max())


@pytest.mark.parametrize("total,bs", [(256, 256), (1000, 256), (100, 100), (77, 32), (4096, 128), (1, 256)])
def test_q8codec_bit_exact(O, tfq, gpu, total, bs):
    import torch
    print(f"q8codec total={total} bs={bs}", flush=True)
    rs = np.random.RandomState(total)
    w = (rs.randn(total) * 0.02).astype(np.float32)
    w[::7] = w[0]   # duplicates: several weights share a centroid, the update step has real sums
    cent, idx = tfq.q8codec_encode(torch.from_numpy(w).to(gpu), bs)
    dec = tfq.q8codec_decode(cent, idx, bs).cpu().numpy()
    cent, idx = cent.cpu().numpy(), idx.cpu().numpy()
    for b in range((total + bs - 1) // bs):
        wc, wi, wd = O.q8codec_block(w[b * bs:(b + 1) * bs])
        assert same(cent[b], wc), b
        assert same(idx[b * bs:(b + 1) * bs], wi) and same(dec[b * bs:(b + 1) * bs], wd), b
    with pytest.raises(tfq.TfqError):
        tfq.q8codec_encode(torch.from_numpy(w).to(gpu), 257)


@pytest.mark.parametrize("shape", [(1, 1000), (4, 300), (3, 1), (16, 4096)])
def test_q8_affine_rows_bit_exact(O, tfq, gpu, shape):
    import torch
    rs = np.random.RandomState(shape[1])
    src = (rs.randn(*shape) * 3 + 0.5).astype(np.float32)
    for f32 in (False, True):
        q, p = tfq.q8_quantize_rows(torch.from_numpy(src).to(gpu), f32)
        wq, wp = O.q8_quantize_rows(src, f32)
        assert same(q.cpu().numpy(), wq) and same(p.cpu().numpy(), wp)
        back = tfq.q8_dequantize(q[0], p[0]).cpu().numpy()
        assert same(back, O.q8_dequantize(wq[0], wp[0]))


def test_engine_argument_errors(tfq, gpu):
    import torch
    x = torch.zeros(16, device=gpu)
    with pytest.raises(tfq.TfqError):
        tfq.lib() and tfq._check(tfq.lib().tfq_engine_quantize_tensor(5, x.data_ptr(), x.data_ptr(), 16, x.data_ptr(), None))
    with pytest.raises(tfq.TfqError):
        tfq._check(tfq.lib().tfq_engine_quant_gemm(4, None, x.data_ptr(), x.data_ptr(), 1, 1, 1, x.data_ptr(), None))
