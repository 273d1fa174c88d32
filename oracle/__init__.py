"""numpy front-end of the CPU oracle (liboracle.so) and of the compiled
reference (_ref/libref.so, when it has been built).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
CPU-baseline leg of the benchmark.  The shipped library never imports it.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "liboracle.so")
_REF = os.path.join(_HERE, "_ref", "libref.so")

# wire ids (include/quant/types.h:22-66 of the reference) + appended literal formats
FMT = {
    "Q_1": 0, "Q_2": 1, "Q_4": 3, "Q_8": 5, "Q_16": 7, "Q_24": 8, "Q_32": 9,
    "Q_1_K_L": 10, "Q_1_K_M": 11, "Q_1_K_H": 12, "Q_16_K_L": 31, "Q_16_K_M": 32, "Q_16_K_H": 33,
    "Q_24_K_L": 34, "Q_24_K_M": 35, "Q_24_K_H": 36, "Q_G_1": 37, "Q_G_16": 44, "Q_G_24": 45,
    "Q_G_1_K_L": 46, "Q_G_1_K_M": 47, "Q_G_1_K_H": 48, "Q_G_16_K_L": 67, "Q_G_16_K_M": 68, "Q_G_16_K_H": 69,
    "Q_G_24_K_L": 70, "Q_G_24_K_M": 71, "Q_G_24_K_H": 72, "Q_1_5": 73, "Q_16_5": 80, "Q_24_5": 81,
    "Q_G_1_5": 82, "Q_G_16_5": 89, "Q_G_24_5": 90,
    "Q_G_2": 38, "Q_G_3": 39, "Q_G_4": 40, "Q_G_6": 41, "Q_G_8": 42,
    "Q_G_2_K_L": 49, "Q_G_2_K_M": 50, "Q_G_2_K_H": 51, "Q_G_3_K_L": 52, "Q_G_3_K_M": 53, "Q_G_3_K_H": 54,
    "Q_G_4_K_L": 55, "Q_G_4_K_M": 56, "Q_G_4_K_H": 57, "Q_G_6_K_L": 58, "Q_G_6_K_M": 59, "Q_G_6_K_H": 60,
    "Q_2_5": 74, "Q_3_5": 75, "Q_4_5": 76, "Q_6_5": 77, "Q_8_5": 78,
    "Q_G_2_5": 83, "Q_G_3_5": 84, "Q_G_4_5": 85, "Q_G_6_5": 86, "Q_G_8_5": 87,
    "B32S4": 105, "B32S8": 106, "SB256A3": 107, "SB256A2": 108,
    "Q_3": 2, "Q_6": 4, "Q_12": 6, "Q_2_K_L": 13, "Q_2_K_M": 14, "Q_2_K_H": 15, "Q_3_K_L": 16, "Q_3_K_M": 17,
    "Q_3_K_H": 18, "Q_4_K_L": 19, "Q_4_K_M": 20, "Q_4_K_H": 21, "Q_6_K_L": 22, "Q_6_K_M": 23, "Q_6_K_H": 24,
    "Q_8_K_L": 25, "Q_8_K_M": 26, "Q_8_K_H": 27, "Q_12_K_L": 28, "Q_12_K_M": 29, "Q_12_K_H": 30, "Q_G_12": 43,
    "Q_G_8_K_L": 61, "Q_G_8_K_M": 62, "Q_G_8_K_H": 63, "Q_G_12_K_L": 64, "Q_G_12_K_M": 65, "Q_G_12_K_H": 66,
    "Q_12_5": 79, "Q_G_12_5": 88,
    "Q_MX_3_5": 91, "Q_MX_4_5": 92, "Q_MX_6_5": 93, "Q_MX_8_5": 94, "Q_MX_12_5": 95, "Q_MX_16_5": 96, "Q_MX_24_5": 97,
    "Q_G_MX_3_5": 98, "Q_G_MX_4_5": 99, "Q_G_MX_6_5": 100, "Q_G_MX_8_5": 101, "Q_G_MX_12_5": 102, "Q_G_MX_16_5": 103, "Q_G_MX_24_5": 104,
}
# formats that exist in the reference (the compiled reference can run them)
REF_FORMATS = [k for k, v in FMT.items() if v < 105]

_u8p = C.POINTER(C.c_uint8)
_f32p = C.POINTER(C.c_float)


def build(force: bool = False) -> None:
    """Compile liboracle.so (and _ref/libref.so where the reference tree exists)."""
    if force or not os.path.exists(_LIB):
        subprocess.check_call(["make", "-s", "-C", _HERE, "all"])


def _load(path):
    return C.CDLL(path) if os.path.exists(path) else None


build()
lib = _load(_LIB)
ref = _load(_REF)


def have_ref() -> bool:
    return ref is not None


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _ptr(a, t):
    return a.ctypes.data_as(t)


lib.orc_f32_to_f16.restype = C.c_uint16
lib.orc_f32_to_f16.argtypes = [C.c_float]
lib.orc_f16_to_f32.restype = C.c_float
lib.orc_f16_to_f32.argtypes = [C.c_uint16]
lib.orc_block_bytes.restype = C.c_long
lib.orc_block_bytes.argtypes = [C.c_uint8, C.c_int]
lib.orc_encode_block.restype = C.c_long
lib.orc_encode_block.argtypes = [C.c_uint8, _f32p, C.c_int, _u8p, C.c_size_t]
lib.orc_decode_block.restype = C.c_int
lib.orc_decode_block.argtypes = [C.c_uint8, _u8p, C.c_size_t, C.c_int, _f32p]
lib.orc_encode_tensor.restype = C.c_long
lib.orc_encode_tensor.argtypes = [C.c_uint8, _f32p, C.c_int64, _u8p, C.c_size_t, C.c_int]
lib.orc_decode_tensor.restype = C.c_int
lib.orc_decode_tensor.argtypes = [C.c_uint8, _u8p, C.c_size_t, C.c_int64, _f32p, C.c_int]
lib.orc_matmul.restype = C.c_int
lib.orc_matmul.argtypes = [C.c_uint8, _u8p, C.c_int64, C.c_int64, _f32p, C.c_int, _f32p, C.c_int]
lib.orc_matmul_f64.restype = C.c_int
lib.orc_matmul_f64.argtypes = [C.c_uint8, _u8p, C.c_int64, C.c_int64, _f32p, C.c_int,
                               C.POINTER(C.c_double), C.c_int]
lib.orc_rng_normal.argtypes = [C.c_uint64, C.c_int64, C.c_float, _f32p]
lib.orc_rng_uniform.argtypes = [C.c_uint64, C.c_int64, _f32p]
lib.orc_rng_u64.argtypes = [C.c_uint64, C.c_int64, C.POINTER(C.c_uint64)]
lib.orc_rng_laplace.argtypes = [C.c_uint64, C.c_int64, C.c_float, _f32p]
lib.orc_softmax_topk.argtypes = [_f32p, C.c_int64, C.c_int64, C.c_int64, _f32p,
                                 C.POINTER(C.c_int64), _f32p]
lib.orc_silu_mul.argtypes = [_f32p, _f32p, C.c_int64, _f32p]
lib.orc_moe_ffn.restype = C.c_int
lib.orc_moe_ffn.argtypes = [C.c_uint8, C.POINTER(_u8p), C.POINTER(_u8p), C.POINTER(_u8p), C.c_int,
                            C.c_int64, C.c_int64, C.POINTER(C.c_int64), _f32p, C.c_int64, C.c_int64,
                            _f32p, _f32p, C.c_int, C.c_int]
lib.orc_quant4_gemm.argtypes = [_u8p, C.POINTER(C.c_uint16), _f32p, _f32p, C.c_int, C.c_int, C.c_int]
lib.orc_quant8_gemm.argtypes = [_u8p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
lib.orc_lut_gemv_batch.argtypes = [C.c_int, _u8p, C.c_void_p, C.c_float, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
lib.orc_lutn_gemm.argtypes = [C.c_int, _u8p, C.c_void_p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
lib.orc_fp24_encode.argtypes = [_f32p, _u8p, C.c_int64]
lib.orc_fp24_decode.argtypes = [_u8p, _f32p, C.c_int64]
lib.orc_comp8_table.argtypes = [_f32p]

THREADS = min(16, os.cpu_count() or 1)


def fmt_id(fmt) -> int:
    return FMT[fmt] if isinstance(fmt, str) else int(fmt)


def f32_to_f16(v: float) -> int:
    return int(lib.orc_f32_to_f16(float(v)))


def f16_to_f32(h: int) -> float:
    return float(lib.orc_f16_to_f32(int(h)))


def comp8_table() -> np.ndarray:
    out = np.empty(256, np.float32)
    lib.orc_comp8_table(_ptr(out, _f32p))
    return out


def fixed_table(bits: int) -> np.ndarray:
    out = np.empty(1 << bits, np.float32)
    lib.orc_fixed_table(int(bits), _ptr(out, _f32p))
    return out


def block_bytes(fmt, n: int = 256) -> int:
    return int(lib.orc_block_bytes(fmt_id(fmt), n))


def encode_block(fmt, w) -> np.ndarray:
    w = _f32(w)
    need = block_bytes(fmt, w.size)
    if need < 0:
        raise ValueError(f"format {fmt} cannot encode a block of {w.size}")
    out = np.zeros(need, np.uint8)
    r = lib.orc_encode_block(fmt_id(fmt), _ptr(w, _f32p), w.size, _ptr(out, _u8p), need)
    if r != need:
        raise RuntimeError("oracle encode failed")
    return out


def decode_block(fmt, payload, n: int = 256) -> np.ndarray:
    payload = np.ascontiguousarray(payload, np.uint8)
    out = np.empty(n, np.float32)
    if lib.orc_decode_block(fmt_id(fmt), _ptr(payload, _u8p), payload.size, n, _ptr(out, _f32p)) != 0:
        raise RuntimeError("oracle decode failed")
    return out


def encode_tensor(fmt, w, threads: int = THREADS) -> np.ndarray:
    w = _f32(w).reshape(-1)
    nb = (w.size + 255) // 256
    tail = w.size - (nb - 1) * 256
    cap = (nb - 1) * max(block_bytes(fmt, 256), 0) + block_bytes(fmt, tail)
    out = np.zeros(cap, np.uint8)
    r = lib.orc_encode_tensor(fmt_id(fmt), _ptr(w, _f32p), w.size, _ptr(out, _u8p), cap, threads)
    if r != cap:
        raise RuntimeError("oracle encode_tensor failed")
    return out


def decode_tensor(fmt, payload, total: int, threads: int = THREADS) -> np.ndarray:
    payload = np.ascontiguousarray(payload, np.uint8)
    out = np.empty(total, np.float32)
    if lib.orc_decode_tensor(fmt_id(fmt), _ptr(payload, _u8p), payload.size, total, _ptr(out, _f32p), threads):
        raise RuntimeError("oracle decode_tensor failed")
    return out


def matmul(fmt, packed, N: int, K: int, X, threads: int = THREADS) -> np.ndarray:
    """Y[B][N] = X[B][K] . W^T in the reference engine's accumulation order (fp32)."""
    packed = np.ascontiguousarray(packed, np.uint8)
    X = _f32(X).reshape(-1, K)
    Y = np.empty((X.shape[0], N), np.float32)
    if lib.orc_matmul(fmt_id(fmt), _ptr(packed, _u8p), N, K, _ptr(X, _f32p), X.shape[0], _ptr(Y, _f32p), threads):
        raise RuntimeError("oracle matmul failed")
    return Y


def matmul_f64(fmt, packed, N: int, K: int, X, threads: int = THREADS) -> np.ndarray:
    packed = np.ascontiguousarray(packed, np.uint8)
    X = _f32(X).reshape(-1, K)
    Y = np.empty((X.shape[0], N), np.float64)
    if lib.orc_matmul_f64(fmt_id(fmt), _ptr(packed, _u8p), N, K, _ptr(X, _f32p), X.shape[0],
                          Y.ctypes.data_as(C.POINTER(C.c_double)), threads):
        raise RuntimeError("oracle matmul_f64 failed")
    return Y


def rng_normal(seed: int, n: int, scale: float = 1.0) -> np.ndarray:
    out = np.empty(n, np.float32)
    lib.orc_rng_normal(seed, n, scale, _ptr(out, _f32p))
    return out


def rng_uniform(seed: int, n: int) -> np.ndarray:
    out = np.empty(n, np.float32)
    lib.orc_rng_uniform(seed, n, _ptr(out, _f32p))
    return out


def rng_u64(seed: int, n: int) -> np.ndarray:
    out = np.empty(n, np.uint64)
    lib.orc_rng_u64(seed, n, out.ctypes.data_as(C.POINTER(C.c_uint64)))
    return out


def rng_laplace(seed: int, n: int, b: float) -> np.ndarray:
    out = np.empty(n, np.float32)
    lib.orc_rng_laplace(seed, n, b, _ptr(out, _f32p))
    return out


def rmsnorm(x, w, eps: float = 1e-6, plus_one: bool = True) -> np.ndarray:
    """Qwen35Engine::rmsnorm (src/adapters/tools/qwen35_engine.cpp:46-51) for one row:
    s = sum x_i^2 accumulated in fp32 in index order, r = 1 / sqrt(s / n + eps), out_i = x_i * r * (1 + w_i),
    every operation in fp32 (plus_one=False: * w_i, the plain form of math::rms_norm)."""
    x = _f32(x).reshape(-1)
    w = _f32(w).reshape(-1)
    s = np.float32(0)
    for v in x:
        s = np.float32(s + np.float32(v * v))
    r = np.float32(1.0) / np.sqrt(np.float32(np.float32(s / np.float32(x.size)) + np.float32(eps)), dtype=np.float32)
    g = (np.float32(1) + w) if plus_one else w
    return (np.float32(1) * (x * r) * g).astype(np.float32)


def bf16_round(a) -> np.ndarray:
    """fp32 -> nearest-even bf16 -> fp32 (the reference has no bf16 type; this is
    how 'bf16 activations' enter its fp32 matmul)."""
    a = _f32(a)
    u = a.view(np.uint32).astype(np.uint64)
    finite = (u & 0x7F800000) != 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
    return np.where(finite, r, a.view(np.uint32)).astype(np.uint32).view(np.float32).reshape(a.shape)


def softmax_topk(logits, k: int):
    logits = _f32(logits)
    T, E = logits.shape
    k = max(1, min(k, E))
    probs = np.empty((T, E), np.float32)
    idx = np.empty((T, k), np.int64)
    w = np.empty((T, k), np.float32)
    lib.orc_softmax_topk(_ptr(logits, _f32p), T, E, k, _ptr(probs, _f32p),
                         idx.ctypes.data_as(C.POINTER(C.c_int64)), _ptr(w, _f32p))
    return probs, idx, w


def silu_mul(g, u) -> np.ndarray:
    g, u = _f32(g), _f32(u)
    out = np.empty_like(g)
    lib.orc_silu_mul(_ptr(g, _f32p), _ptr(u, _f32p), g.size, _ptr(out, _f32p))
    return out


def moe_ffn(fmt, gate, up, down, D: int, F: int, topk_idx, topk_w, x, mid_bf16: bool = False,
            threads: int = THREADS) -> np.ndarray:
    E = len(gate)
    keep = [np.ascontiguousarray(a, np.uint8) for a in list(gate) + list(up) + list(down)]
    arr = lambda xs: (_u8p * E)(*[_ptr(a, _u8p) for a in xs])
    topk_idx = np.ascontiguousarray(topk_idx, np.int64)
    topk_w = _f32(topk_w)
    x = _f32(x)
    T, Kk = topk_idx.shape
    out = np.empty((T, D), np.float32)
    r = lib.orc_moe_ffn(fmt_id(fmt), arr(keep[:E]), arr(keep[E:2 * E]), arr(keep[2 * E:]), E, D, F,
                        topk_idx.ctypes.data_as(C.POINTER(C.c_int64)), _ptr(topk_w, _f32p), T, Kk,
                        _ptr(x, _f32p), _ptr(out, _f32p), int(mid_bf16), threads)
    if r:
        raise RuntimeError("oracle moe_ffn failed")
    return out


def moe_plan_dispatch(topk_idx, topk_w, E: int, slots: int):
    """plan_dispatch (engines/trainer/moe/dispatch.cpp:9-38): (expert_first [E + 1], item_token, item_weight, dropped slots)."""
    idx = np.ascontiguousarray(topk_idx, np.int32)
    w = _f32(topk_w)
    T, Kk = idx.shape
    first = np.zeros(E + 1, np.int32)
    tok = np.zeros(T * Kk, np.int32)
    wt = np.zeros(T * Kk, np.float32)
    dr = np.zeros(T * Kk, np.int32)
    i32p = C.POINTER(C.c_int32)
    lib.orc_moe_plan_dispatch.restype = C.c_int64
    lib.orc_moe_plan_dispatch.argtypes = [i32p, _f32p, C.c_int64, C.c_int64, C.c_int64, C.c_int64, i32p, i32p, _f32p, i32p]
    nd = lib.orc_moe_plan_dispatch(idx.ctypes.data_as(i32p), _ptr(w, _f32p), T, Kk, E, slots, first.ctypes.data_as(i32p),
                                   tok.ctypes.data_as(i32p), _ptr(wt, _f32p), dr.ctypes.data_as(i32p))
    if nd < 0:
        raise RuntimeError("oracle plan_dispatch: expert id out of range")
    n = int(first[E])
    return first, tok[:n], wt[:n], dr[:nd]


def moe_ffn_capacity(fmt, gate, up, down, D: int, F: int, topk_idx, topk_w, slots: int, x, mid_bf16: bool = False,
                     threads: int = THREADS):
    """(out [T][D], dropped count): plan_dispatch + gather + expert FFN + combine_expert_outputs (dispatch.cpp:9-78)."""
    E = len(gate)
    keep = [np.ascontiguousarray(a, np.uint8) for a in list(gate) + list(up) + list(down)]
    arr = lambda xs: (_u8p * E)(*[_ptr(a, _u8p) for a in xs])
    idx = np.ascontiguousarray(topk_idx, np.int32)
    topk_w = _f32(topk_w)
    x = _f32(x)
    T, Kk = idx.shape
    out = np.empty((T, D), np.float32)
    i32p = C.POINTER(C.c_int32)
    lib.orc_moe_ffn_capacity.restype = C.c_int64
    lib.orc_moe_ffn_capacity.argtypes = [C.c_uint8, C.POINTER(_u8p), C.POINTER(_u8p), C.POINTER(_u8p), C.c_int, C.c_int64, C.c_int64,
                                         i32p, _f32p, C.c_int64, C.c_int64, C.c_int64, _f32p, _f32p, C.c_int, C.c_int]
    nd = lib.orc_moe_ffn_capacity(fmt_id(fmt), arr(keep[:E]), arr(keep[E:2 * E]), arr(keep[2 * E:]), E, D, F,
                                  idx.ctypes.data_as(i32p), _ptr(topk_w, _f32p), T, Kk, slots, _ptr(x, _f32p), _ptr(out, _f32p),
                                  int(mid_bf16), threads)
    if nd < 0:
        raise RuntimeError("oracle moe_ffn_capacity failed")
    return out, int(nd)


def quant4_gemm(w, cb16, act, M: int, N: int, K: int) -> np.ndarray:
    w = np.ascontiguousarray(w, np.uint8)
    cb16 = np.ascontiguousarray(cb16, np.uint16)
    act = _f32(act)
    out = np.empty((M, N), np.float32)
    lib.orc_quant4_gemm(_ptr(w, _u8p), cb16.ctypes.data_as(C.POINTER(C.c_uint16)), _ptr(act, _f32p),
                        _ptr(out, _f32p), M, N, K)
    return out


def quant8_gemm(idx, cb256, act, M: int, N: int, K: int) -> np.ndarray:
    idx = np.ascontiguousarray(idx, np.uint8)
    cb256, act = _f32(cb256), _f32(act)
    out = np.empty((M, N), np.float32)
    lib.orc_quant8_gemm(_ptr(idx, _u8p), _ptr(cb256, _f32p), _ptr(act, _f32p), _ptr(out, _f32p), M, N, K)
    return out


def lut_gemv_batch(bits: int, packed, cb, scale: float, X, M: int, N: int, K: int) -> np.ndarray:
    """Y[N][M] of the production batch GEMV (scalar semantics); cb: 16 uint16 (bits 4), 256 float (bits 8), None (bits 2)."""
    packed = np.ascontiguousarray(packed, np.uint8)
    X = _f32(X)
    out = np.empty((N, M), np.float32)
    if bits == 4:
        cb = np.ascontiguousarray(cb, np.uint16)
    elif bits == 8:
        cb = _f32(cb)
    cbp = C.c_void_p(cb.ctypes.data) if bits != 2 else C.c_void_p(0)
    lib.orc_lut_gemv_batch(bits, _ptr(packed, _u8p), cbp, C.c_float(scale), _ptr(X, _f32p), _ptr(out, _f32p), M, N, K)
    return out


def _lutn_codebook(bits, cb):
    if bits == 24:
        return None, C.c_void_p(0)
    cb = np.ascontiguousarray(cb, np.uint16 if bits == 12 else np.float32)
    assert cb.size == 1 << bits
    return cb, C.c_void_p(cb.ctypes.data)


def lutn_gemm(bits: int, packed, cb, act, M: int, N: int, K: int) -> np.ndarray:
    """q3_gemm / q6_gemm / q12_gemm / q24_gemm (scalar semantics): packed row per (m, n), activation row n."""
    packed = np.ascontiguousarray(packed, np.uint8)
    act = _f32(act)
    keep, cbp = _lutn_codebook(bits, cb)
    out = np.empty((M, N), np.float32)
    lib.orc_lutn_gemm(bits, _ptr(packed, _u8p), cbp, _ptr(act, _f32p), _ptr(out, _f32p), M, N, K)
    return out


def fp24_encode(w) -> np.ndarray:
    w = _f32(w).reshape(-1)
    out = np.empty(3 * w.size, np.uint8)
    lib.orc_fp24_encode(_ptr(w, _f32p), _ptr(out, _u8p), w.size)
    return out


def fp24_decode(packed) -> np.ndarray:
    packed = np.ascontiguousarray(packed, np.uint8)
    out = np.empty(packed.size // 3, np.float32)
    lib.orc_fp24_decode(_ptr(packed, _u8p), _ptr(out, _f32p), out.size)
    return out


# ------------------------------------------------------------ compiled reference
if ref is not None:
    ref.ref_quantize_block.restype = C.c_long
    ref.ref_quantize_block.argtypes = [C.c_uint8, _f32p, C.c_int, _u8p, C.c_size_t]
    ref.ref_dequantize_block.argtypes = [C.c_uint8, _u8p, C.c_size_t, C.c_uint32, _f32p]
    ref.ref_block_claimed_bytes.restype = C.c_size_t
    ref.ref_block_claimed_bytes.argtypes = [C.c_uint8, C.c_uint32]
    ref.ref_format_bpw.restype = C.c_float
    ref.ref_format_bpw.argtypes = [C.c_uint8]
    ref.ref_format_name.restype = C.c_char_p
    ref.ref_format_name.argtypes = [C.c_uint8]
    ref.ref_registry_quantize.restype = C.c_long
    ref.ref_registry_quantize.argtypes = [C.c_char_p, _f32p, C.c_int64, _u8p, C.c_size_t,
                                          C.POINTER(C.c_uint32), C.c_int64]
    ref.ref_registry_roundtrip.restype = C.c_int
    ref.ref_registry_roundtrip.argtypes = [C.c_char_p, _f32p, C.c_int64, _f32p]
    ref.ref_parse_format_id.restype = C.c_int
    ref.ref_parse_format_id.argtypes = [C.c_char_p]
    ref.ref_rng_normal.argtypes = [C.c_uint64, C.c_int64, C.c_float, _f32p]
    ref.ref_rng_uniform.argtypes = [C.c_uint64, C.c_int64, _f32p]
    ref.ref_rng_u64.argtypes = [C.c_uint64, C.c_int64, C.POINTER(C.c_uint64)]
    ref.ref_quant4_gemm.argtypes = [_u8p, C.POINTER(C.c_uint16), _f32p, _f32p, C.c_int, C.c_int, C.c_int]
    ref.ref_quant8_gemm.argtypes = [_u8p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
    ref.ref_scalar_gemm_bt.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
    ref.ref_gemv_quant4_tiled.argtypes = [_u8p, C.POINTER(C.c_uint16), C.c_float, _f32p, _f32p, C.c_int, C.c_int]
    ref.ref_gemv_quant8_tiled.argtypes = [_u8p, _f32p, C.c_float, _f32p, _f32p, C.c_int, C.c_int]
    ref.ref_detect_cpu_isa.restype = C.c_int


def ref_encode_block(fmt, w) -> np.ndarray:
    w = _f32(w)
    out = np.zeros(w.size * 4 + 64, np.uint8)
    r = ref.ref_quantize_block(fmt_id(fmt), _ptr(w, _f32p), w.size, _ptr(out, _u8p), out.size)
    if r < 0:
        raise RuntimeError(f"reference quantize failed ({r})")
    return out[:r].copy()


def ref_decode_block(fmt, payload, n: int = 256) -> np.ndarray:
    payload = np.ascontiguousarray(payload, np.uint8)
    out = np.empty(n, np.float32)
    ref.ref_dequantize_block(fmt_id(fmt), _ptr(payload, _u8p), payload.size, n, _ptr(out, _f32p))
    return out


def ref_rng_normal(seed: int, n: int, scale: float = 1.0) -> np.ndarray:
    out = np.empty(n, np.float32)
    ref.ref_rng_normal(seed, n, scale, _ptr(out, _f32p))
    return out


def ref_rng_uniform(seed: int, n: int) -> np.ndarray:
    out = np.empty(n, np.float32)
    ref.ref_rng_uniform(seed, n, _ptr(out, _f32p))
    return out


def ref_registry_quantize(name: str, data):
    data = _f32(data).reshape(-1)
    nb = (data.size + 255) // 256
    out = np.zeros(data.size * 4 + 64 * nb, np.uint8)
    per = np.zeros(nb, np.uint32)
    r = ref.ref_registry_quantize(name.encode(), _ptr(data, _f32p), data.size, _ptr(out, _u8p), out.size,
                                  per.ctypes.data_as(C.POINTER(C.c_uint32)), nb)
    if r < 0:
        raise RuntimeError(f"reference registry quantize failed ({r})")
    return out[:r].copy(), per


def ref_quant4_gemm(w, cb16, act, M, N, K) -> np.ndarray:
    w = np.ascontiguousarray(w, np.uint8)
    cb16 = np.ascontiguousarray(cb16, np.uint16)
    act = _f32(act)
    out = np.empty((M, N), np.float32)
    ref.ref_quant4_gemm(_ptr(w, _u8p), cb16.ctypes.data_as(C.POINTER(C.c_uint16)), _ptr(act, _f32p),
                        _ptr(out, _f32p), M, N, K)
    return out


def ref_quant8_gemm(idx, cb256, act, M, N, K) -> np.ndarray:
    idx = np.ascontiguousarray(idx, np.uint8)
    cb256, act = _f32(cb256), _f32(act)
    out = np.empty((M, N), np.float32)
    ref.ref_quant8_gemm(_ptr(idx, _u8p), _ptr(cb256, _f32p), _ptr(act, _f32p), _ptr(out, _f32p), M, N, K)
    return out


def ref_lutn_gemm(bits: int, packed, cb, act, M, N, K) -> np.ndarray:
    packed = np.ascontiguousarray(packed, np.uint8)
    act = _f32(act)
    keep, cbp = _lutn_codebook(bits, cb)
    out = np.empty((M, N), np.float32)
    ref.ref_lutn_gemm.argtypes = [C.c_int, _u8p, C.c_void_p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
    ref.ref_lutn_gemm(bits, _ptr(packed, _u8p), cbp, _ptr(act, _f32p), _ptr(out, _f32p), M, N, K)
    return out


def ref_fp24_round_trip(w):
    w = _f32(w).reshape(-1)
    packed = np.empty(3 * w.size, np.uint8)
    back = np.empty(w.size, np.float32)
    ref.ref_fp24_encode.argtypes = [_f32p, _u8p, C.c_int]
    ref.ref_fp24_decode.argtypes = [_u8p, _f32p, C.c_int]
    ref.ref_fp24_encode(_ptr(w, _f32p), _ptr(packed, _u8p), w.size)
    ref.ref_fp24_decode(_ptr(packed, _u8p), _ptr(back, _f32p), w.size)
    return packed, back


def ref_container_write(path: str, tensors, block_fmt, config: bytes = b"", version: int = 1 << 22) -> int:
    """tensors: list of (name, fp32 array); block_fmt: wire id of every 256-block of the file, in order."""
    names = (C.c_char_p * len(tensors))(*[n.encode() for n, _ in tensors])
    data = np.concatenate([_f32(w).reshape(-1) for _, w in tensors])
    sizes = np.array([np.size(w) for _, w in tensors], np.int64)
    offsets = np.concatenate([[0], np.cumsum(sizes)[:-1]]).astype(np.int64)
    fm = np.array([fmt_id(f) for f in block_fmt], np.uint8)
    assert fm.size == int(((sizes + 255) // 256).sum())
    i64p = C.POINTER(C.c_int64)
    ref.ref_container_write.argtypes = [C.c_char_p, C.c_int, C.POINTER(C.c_char_p), _f32p, i64p, i64p, _u8p,
                                        C.c_char_p, C.c_uint32, C.c_uint32]
    return ref.ref_container_write(path.encode(), len(tensors), names, _ptr(data, _f32p), offsets.ctypes.data_as(i64p),
                                   sizes.ctypes.data_as(i64p), _ptr(fm, _u8p), config, len(config), version)


def ref_container_info(path: str):
    out = np.zeros(5, np.int64)
    ref.ref_container_info.argtypes = [C.c_char_p, C.POINTER(C.c_int64)]
    ref.ref_container_info(path.encode(), out.ctypes.data_as(C.POINTER(C.c_int64)))
    return dict(valid=bool(out[0]), blocks=int(out[1]), tensors=int(out[2]), version=int(out[3]), config_size=int(out[4]))


def ref_container_tensor_blocks(path: str, name: str):
    s, k = C.c_uint32(0), C.c_uint32(0)
    ref.ref_container_tensor_blocks.argtypes = [C.c_char_p, C.c_char_p, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]
    ok = ref.ref_container_tensor_blocks(path.encode(), name.encode(), C.byref(s), C.byref(k))
    return (s.value, k.value) if ok else None


def ref_container_block(path: str, block_id: int):
    out = np.zeros(5, np.int64)
    ref.ref_container_block.argtypes = [C.c_char_p, C.c_uint32, C.POINTER(C.c_int64)]
    if ref.ref_container_block(path.encode(), block_id, out.ctypes.data_as(C.POINTER(C.c_int64))) != 0:
        return None
    return dict(format=int(out[0]), weights=int(out[1]), cb_bytes=int(out[2]), idx_bytes=int(out[3]), offset=int(out[4]))


def ref_container_read_tensor(path: str, name: str, cap: int = 1 << 22) -> np.ndarray:
    out = np.empty(cap, np.float32)
    ref.ref_container_read_tensor.restype = C.c_int64
    ref.ref_container_read_tensor.argtypes = [C.c_char_p, C.c_char_p, _f32p, C.c_int64]
    n = ref.ref_container_read_tensor(path.encode(), name.encode(), _ptr(out, _f32p), cap)
    if n < 0:
        raise RuntimeError("reference read_tensor: destination too small")
    return out[:n].copy()


# ---- in-memory codebook engines (Q4Engine / Q8Engine, quant8 codec): oracle and compiled reference share signatures
def _engine_lib(use_ref):
    return ref if use_ref else lib


def _pfx(use_ref):
    return "ref_" if use_ref else "orc_"


def engine_quantize_per_block(bits, cb, data, block_size, use_ref=False):
    cb, data = _f32(cb), _f32(data).reshape(-1)
    nb = (data.size + block_size - 1) // block_size
    idx = np.zeros(data.size, np.uint8)
    scales = np.zeros(nb * (2 if bits == 4 else 1), np.float32)
    fn = getattr(_engine_lib(use_ref), _pfx(use_ref) + "engine_quantize_per_block")
    fn.argtypes = [C.c_int, _f32p, _f32p, C.c_int64, C.c_int64, _u8p, _f32p]
    fn(bits, _ptr(cb, _f32p), _ptr(data, _f32p), data.size, block_size, _ptr(idx, _u8p), _ptr(scales, _f32p))
    return idx, scales


def engine_dequantize_per_block(bits, cb, idx, scales, block_size, use_ref=False):
    cb, scales = _f32(cb), _f32(scales)
    idx = np.ascontiguousarray(idx, np.uint8)
    out = np.zeros(idx.size, np.float32)
    fn = getattr(_engine_lib(use_ref), _pfx(use_ref) + "engine_dequantize_per_block")
    fn.argtypes = [C.c_int, _f32p, _u8p, _f32p, C.c_int64, C.c_int64, _f32p]
    fn(bits, _ptr(cb, _f32p), _ptr(idx, _u8p), _ptr(scales, _f32p), idx.size, block_size, _ptr(out, _f32p))
    return out


def engine_quantize_tensor(bits, cb, data, use_ref=False):
    cb, data = _f32(cb), _f32(data).reshape(-1)
    out = np.zeros(data.size if bits == 8 else (data.size + 1) // 2, np.uint8)
    fn = getattr(_engine_lib(use_ref), _pfx(use_ref) + "engine_quantize_tensor")
    fn.argtypes = [C.c_int, _f32p, _f32p, C.c_int64, _u8p]
    fn(bits, _ptr(cb, _f32p), _ptr(data, _f32p), data.size, _ptr(out, _u8p))
    return out


def engine_dequant_tensor(bits, cb, idx, n, use_ref=False):
    cb = _f32(cb)
    idx = np.ascontiguousarray(idx, np.uint8)
    out = np.zeros(n, np.float32)
    fn = getattr(_engine_lib(use_ref), _pfx(use_ref) + "engine_dequant_tensor")
    fn.argtypes = [C.c_int, _f32p, _u8p, C.c_int64, _f32p]
    fn(bits, _ptr(cb, _f32p), _ptr(idx, _u8p), n, _ptr(out, _f32p))
    return out


def engine_quant_gemm(bits, cb, a, b_idx, M, N, K, use_ref=False):
    cb, a = _f32(cb), _f32(a)
    b_idx = np.ascontiguousarray(b_idx, np.uint8)
    out = np.zeros((M, N), np.float32)
    fn = getattr(_engine_lib(use_ref), _pfx(use_ref) + "engine_quant_gemm")
    fn.argtypes = [C.c_int, _f32p, _f32p, _u8p, C.c_int64, C.c_int64, C.c_int64, _f32p]
    fn(bits, _ptr(cb, _f32p), _ptr(a, _f32p), _ptr(b_idx, _u8p), M, N, K, _ptr(out, _f32p))
    return out


def q8codec_block(w, use_ref=False):
    """(centroids[256], indices, decoded) of Q8Encoder::encode / Q8Decoder::decode on one block of <= 256 weights."""
    w = _f32(w).reshape(-1)
    cent, idx, dec = np.zeros(256, np.float32), np.zeros(w.size, np.uint8), np.zeros(w.size, np.float32)
    fn = getattr(_engine_lib(use_ref), _pfx(use_ref) + "q8codec_block")
    fn.argtypes = [_f32p, C.c_uint32, _f32p, _u8p, _f32p]
    fn(_ptr(w, _f32p), w.size, _ptr(cent, _f32p), _ptr(idx, _u8p), _ptr(dec, _f32p))
    return cent, idx, dec


def q8_quantize_rows(src, dst_f32=False, use_ref=False):
    src = _f32(src)
    batch, per = src.shape
    dst = np.zeros((batch, per), np.float32 if dst_f32 else np.uint8)
    params = np.zeros((batch, 3), np.float32)
    fn = getattr(_engine_lib(use_ref), _pfx(use_ref) + "q8_quantize_rows")
    fn.argtypes = [_f32p, C.c_int64, C.c_int64, C.c_int, C.c_void_p, _f32p]
    fn(_ptr(src, _f32p), batch, per, int(dst_f32), dst.ctypes.data, _ptr(params, _f32p))
    return dst, params


def q8_dequantize(src, params3, use_ref=False):
    src = np.ascontiguousarray(src)
    params3 = _f32(params3)
    out = np.zeros(src.size, np.float32)
    fn = getattr(_engine_lib(use_ref), _pfx(use_ref) + "q8_dequantize")
    fn.argtypes = [C.c_void_p, C.c_int64, C.c_int, _f32p, _f32p]
    fn(src.ctypes.data, src.size, int(src.dtype == np.float32), _ptr(params3, _f32p), _ptr(out, _f32p))
    return out
