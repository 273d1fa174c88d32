"""CPU pins of the oracle's mixture-of-experts helpers, each against an independent statement of what the
reference computes: softmax_with_topk (src/model/moe_core.cpp:98-149) against numpy exp / argsort, silu(g) * u
(src/math/math.cpp:117-126) against float64, the inference dispatch (moe_core.cpp:289-343) and the
capacity-limited dispatch (engines/trainer/moe/dispatch.cpp:9-78) against a dense float64 product of the decoded
expert matrices and a pure-Python walk of the slots."""
import numpy as np


def test_softmax_topk_against_numpy(O):
    T, E, K = 33, 8, 2
    logits = O.rng_normal(45, T * E, 1.0).reshape(T, E)
    probs, idx, w = O.softmax_topk(logits, K)
    z = np.exp(logits.astype(np.float64) - logits.max(axis=1, keepdims=True))
    p = z / z.sum(axis=1, keepdims=True)
    assert np.abs(probs - p).max() < 3e-7
    order = np.argsort(-p, axis=1, kind="stable")[:, :K]  # descending, lowest index first on ties
    assert np.array_equal(idx, order)
    assert np.abs(w - np.take_along_axis(p, order, axis=1)).max() < 3e-7
    assert np.abs(probs.sum(axis=1) - 1).max() < 1e-6
    # k is clamped into 1..E
    assert O.softmax_topk(logits, 99)[1].shape == (T, E)
    # ties: equal logits keep the lower expert id first
    tied = np.zeros((1, 4), np.float32)
    assert O.softmax_topk(tied, 3)[1].tolist() == [[0, 1, 2]]


def test_silu_mul_against_float64(O):
    g = O.rng_normal(1, 4096, 3.0)
    u = O.rng_normal(2, 4096, 1.0)
    ref = g.astype(np.float64) / (1.0 + np.exp(-g.astype(np.float64))) * u.astype(np.float64)
    got = O.silu_mul(g, u)
    assert np.abs(got - ref).max() <= 1e-6 * max(1.0, np.abs(ref).max())
    assert O.silu_mul(np.zeros(3, np.float32), np.ones(3, np.float32)).tolist() == [0.0, 0.0, 0.0]
    # large negative gate: silu -> 0 without overflow trouble
    assert abs(float(O.silu_mul(np.array([-80.0], np.float32), np.array([2.0], np.float32))[0])) < 1e-30


def _experts(O, fmt, E, D, F, seed):
    pk, dense = {"gate": [], "up": [], "down": []}, {"gate": [], "up": [], "down": []}
    for e in range(E):
        for j, (name, n, k) in enumerate((("gate", F, D), ("up", F, D), ("down", D, F))):
            pay = O.encode_tensor(fmt, O.rng_normal(seed + 10 * e + j, n * k, 0.05))
            pk[name].append(pay)
            dense[name].append(O.decode_tensor(fmt, pay, n * k).reshape(n, k).astype(np.float64))
    return pk, dense


def _ffn64(dense, e, x):
    g = dense["gate"][e] @ x
    u = dense["up"][e] @ x
    return dense["down"][e] @ (g / (1.0 + np.exp(-g)) * u)


def test_moe_ffn_inference_dispatch_against_dense_float64(O):
    fmt, E, D, F, T, K = "B32S4", 4, 256, 512, 6, 2
    pk, dense = _experts(O, fmt, E, D, F, 700)
    x = O.rng_normal(3, T * D, 1.0).reshape(T, D)
    _, idx, w = O.softmax_topk(O.rng_normal(4, T * E, 1.0).reshape(T, E), K)
    w[1, 0] = 0.0  # a slot whose weight is not positive is skipped
    out = O.moe_ffn(fmt, pk["gate"], pk["up"], pk["down"], D, F, idx, w, x)
    ref = np.zeros((T, D))
    for t in range(T):
        for j in range(K):
            if w[t, j] > 0:
                ref[t] += float(w[t, j]) * _ffn64(dense, int(idx[t, j]), x[t].astype(np.float64))
    assert np.abs(out - ref).max() / np.abs(ref).max() < 2e-5


def test_plan_dispatch_against_python_walk(O):
    T, K, E, slots = 9, 2, 3, 4
    rng = np.random.default_rng(5)
    idx = rng.integers(0, E, size=(T, K)).astype(np.int32)
    w = rng.standard_normal((T, K)).astype(np.float32)
    first, tok, wt, dropped = O.moe_plan_dispatch(idx, w, E, slots)
    lists, drop = [[] for _ in range(E)], []
    for t in range(T):
        for j in range(K):
            e = int(idx[t, j])
            (lists[e] if len(lists[e]) < slots else drop).append((t, j))
    assert dropped.tolist() == [t * K + j for t, j in drop]
    for e in range(E):
        sl = slice(int(first[e]), int(first[e + 1]))
        assert tok[sl].tolist() == [t for t, _ in lists[e]]
        assert wt[sl].tolist() == [float(w[t, j]) for t, j in lists[e]]
    assert int(first[E]) + len(drop) == T * K           # every slot is kept or dropped
    assert all(len(l) <= slots for l in lists)
    # a capacity that holds everything drops nothing
    assert O.moe_plan_dispatch(idx, w, E, T * K)[3].size == 0


def test_moe_ffn_capacity_against_dense_float64(O):
    fmt, E, D, F, T, K, slots = "B32S4", 3, 256, 512, 7, 2, 3
    pk, dense = _experts(O, fmt, E, D, F, 800)
    x = O.rng_normal(6, T * D, 1.0).reshape(T, D)
    rng = np.random.default_rng(7)
    idx = rng.integers(0, E, size=(T, K)).astype(np.int32)
    w = rng.standard_normal((T, K)).astype(np.float32)  # negative weights are kept in this form
    out, nd = O.moe_ffn_capacity(fmt, pk["gate"], pk["up"], pk["down"], D, F, idx, w, slots, x)
    ref, cnt, drop = np.zeros((T, D)), [0] * E, 0
    for t in range(T):
        for j in range(K):
            e = int(idx[t, j])
            if cnt[e] < slots:
                cnt[e] += 1
                ref[t] += float(w[t, j]) * _ffn64(dense, e, x[t].astype(np.float64))
            else:
                drop += 1
    assert nd == drop and drop > 0
    assert np.abs(out - ref).max() / np.abs(ref).max() < 2e-5


def test_rmsnorm_closed_forms(O):
    """O.rmsnorm (Qwen35Engine::rmsnorm, src/adapters/tools/qwen35_engine.cpp:46-51) against what the formula fixes:
    a constant row, unit root-mean-square of the output for zero gains, scale invariance, the (1 + w) gain (not w),
    and float64 numpy on a random row."""
    n = 384
    c = np.full(n, 3.0, np.float32)
    out = O.rmsnorm(c, np.zeros(n, np.float32))
    assert np.allclose(out, 3.0 / np.sqrt(9.0 + 1e-6), rtol=1e-6)
    x = O.rng_normal(5, n, 2.0)
    out = O.rmsnorm(x, np.zeros(n, np.float32))
    assert abs(np.sqrt(np.mean(out.astype(np.float64) ** 2)) - 1.0) < 1e-5  # eps is 1e-6 against mean(x^2) of 4
    assert np.allclose(O.rmsnorm(8.0 * x, np.zeros(n, np.float32)), out, rtol=1e-5, atol=1e-6)
    w = O.rng_normal(6, n, 0.3)
    x64 = x.astype(np.float64)
    ref = x64 / np.sqrt(np.mean(x64 ** 2) + 1e-6) * (1.0 + w.astype(np.float64))
    assert np.abs(O.rmsnorm(x, w) - ref).max() <= 2e-6 * np.abs(ref).max()
    ref_plain = x64 / np.sqrt(np.mean(x64 ** 2) + 1e-6) * w.astype(np.float64)
    assert np.abs(O.rmsnorm(x, w, plus_one=False) - ref_plain).max() <= 2e-6 * np.abs(ref).max()
    # a dropped eps would turn a zero row into NaN
    assert np.array_equal(O.rmsnorm(np.zeros(n, np.float32), w), np.zeros(n, np.float32))
