"""ctypes binding of libtfq.so, the gfx950 backend for the block-quantized
weight matmul.  PyTorch is used only to own device memory and streams; every
computation is a hand-written HIP kernel reached through the C ABI declared in
include/tfq.h.  There is no fallback: importing works without a GPU (so the
symbol table can be inspected), but every compute call raises TfqError when
the library or the device is missing.

The directory name contains a hyphen, so import it with
``importlib.import_module("transformers-fusion_amd")``.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtfq.so")

F32, BF16 = 0, 1

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


class TfqError(RuntimeError):
    pass


def _load():
    if not os.path.exists(LIB_PATH):
        raise TfqError(f"{LIB_PATH} is missing: run __graft_entry__.build() (hipcc) first")
    lib = C.CDLL(LIB_PATH)
    vp, u8, i32, i64, sz = C.c_void_p, C.c_uint8, C.c_int, C.c_int64, C.c_size_t
    sig = {
        "tfq_init": (i32, [i32]),
        "tfq_last_error": (C.c_char_p, []),
        "tfq_version": (C.c_char_p, []),
        "tfq_format_id": (i32, [C.c_char_p]),
        "tfq_format_name": (C.c_char_p, [u8]),
        "tfq_format_bpw": (C.c_float, [u8]),
        "tfq_format_supported": (i32, [u8]),
        "tfq_block_bytes": (i32, [u8, C.c_uint32, C.POINTER(sz)]),
        "tfq_encode_blocks": (i32, [u8, vp, i64, vp, sz, vp]),
        "tfq_decode_blocks": (i32, [u8, vp, sz, i64, vp, vp]),
        "tfq_encode_blocks_host": (i32, [u8, vp, i64, vp, sz, vp]),
        "tfq_decode_blocks_host": (i32, [u8, vp, sz, i64, vp]),
        "tfq_weight_upload": (vp, [u8, i64, i64, vp, sz]),
        "tfq_weight_wrap": (vp, [u8, i64, i64, vp, sz]),
        "tfq_weight_upload_mixed": (vp, [i64, i64, vp, vp, sz]),
        "tfq_weight_free": (None, [vp]),
        "tfq_weight_info": (i32, [vp, C.POINTER(u8), C.POINTER(i64), C.POINTER(i64), C.POINTER(sz)]),
        "tfq_weight_decode": (i32, [vp, vp, vp]),
        "tfq_gemv": (i32, [vp, vp, i32, i32, vp, i32, vp]),
        "tfq_gemm": (i32, [vp, vp, i32, i32, vp, i32, vp]),
        "tfq_gemv_workspace_bytes": (sz, [vp, i32, i32]),
        "tfq_gemv_ws": (i32, [vp, vp, i32, i32, vp, i32, vp, sz, vp]),
        "tfq_gemm_workspace_bytes": (sz, [vp, i32, i32]),
        "tfq_gemm_ws": (i32, [vp, vp, i32, i32, vp, i32, vp, sz, vp]),
        "tfq_gemm_static": (i32, [vp, vp, i32, i32, vp, i32, vp]),
        "tfq_gemm_static_scratch_bytes": (sz, []),
        "tfq_gemv_multi": (i32, [vp, i32, vp, i32, i32, vp, i32, vp]),
        "tfq_matmul_host": (i32, [vp, vp, vp, i32]),
        "tfq_mlp_workspace_bytes": (sz, [i32, i64]),
        "tfq_mlp_step": (i32, [vp, vp, vp, vp, i32, i32, vp, i32, i32, vp, sz, vp]),
        "tfq_moe_route": (i32, [vp, i32, i32, i32, vp, vp, vp, vp]),
        "tfq_moe_workspace_bytes": (sz, [i32, i32, i64, i64]),
        "tfq_moe_ffn": (i32, [vp, vp, vp, i32, vp, vp, i32, i32, vp, i32, vp, i32, i32, vp, sz, vp]),
        "tfq_moe_expert_table": (i32, [vp, vp, vp, i32, vp]),
        "tfq_moe_routed_workspace_bytes": (sz, [vp, vp, vp, i32, i32, i32]),
        "tfq_moe_ffn_routed": (i32, [vp, vp, vp, i32, vp, vp, vp, i32, i32, vp, i32, vp, i32, i32, vp, sz, vp]),
        "tfq_moe_plan_dispatch": (i32, [vp, vp, i32, i32, i32, i64, vp, vp, vp, vp, vp]),
        "tfq_moe_ffn_capacity": (i32, [vp, vp, vp, i32, vp, vp, i32, i32, i64, vp, i32, vp, i32, i32, vp, sz, vp, vp]),
        "tfq_lut4_gemm": (i32, [vp, vp, vp, vp, i32, i32, i32, vp]),
        "tfq_lut8_gemm": (i32, [vp, vp, vp, vp, i32, i32, i32, vp]),
        "tfq_lut_gemv_batch": (i32, [i32, vp, vp, C.c_float, vp, vp, i32, i32, i32, vp]),
        "tfq_lutn_gemm": (i32, [i32, vp, vp, vp, vp, i32, i32, i32, vp]),
        "tfq_fp24_encode": (i32, [vp, vp, i64, vp]),
        "tfq_fp24_decode": (i32, [vp, vp, i64, vp]),
        "tfq_engine_quantize_per_block": (i32, [i32, vp, vp, i64, i64, vp, vp, vp]),
        "tfq_engine_dequantize_per_block": (i32, [i32, vp, vp, vp, i64, i64, vp, vp]),
        "tfq_engine_quantize_tensor": (i32, [i32, vp, vp, i64, vp, vp]),
        "tfq_engine_dequant_tensor": (i32, [i32, vp, vp, i64, vp, vp]),
        "tfq_engine_quant_gemm": (i32, [i32, vp, vp, vp, i64, i64, i64, vp, vp]),
        "tfq_q8codec_encode": (i32, [vp, i64, i32, vp, vp, vp]),
        "tfq_q8codec_decode": (i32, [vp, vp, i64, i32, vp, vp]),
        "tfq_q8_quantize_rows": (i32, [vp, i64, i64, i32, vp, vp, vp]),
        "tfq_q8_dequantize": (i32, [vp, i64, i32, vp, vp, vp]),
        "tfq_container_open": (vp, [C.c_char_p]),
        "tfq_container_from_memory": (vp, [vp, sz]),
        "tfq_container_close": (None, [vp]),
        "tfq_container_valid": (i32, [vp]),
        "tfq_container_header": (i32, [vp, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(vp), C.POINTER(sz)]),
        "tfq_container_num_blocks": (i64, [vp]),
        "tfq_container_num_tensors": (i32, [vp]),
        "tfq_container_tensor_name": (i32, [vp, i32, C.c_char_p, sz]),
        "tfq_container_tensor_blocks": (i32, [vp, C.c_char_p, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
        "tfq_container_block": (i32, [vp, C.c_uint32, C.POINTER(u8), C.POINTER(C.c_uint32), C.POINTER(C.c_uint32),
                                      C.POINTER(C.c_uint32), C.POINTER(vp)]),
        "tfq_container_tensor_weights": (i64, [vp, C.c_char_p]),
        "tfq_container_read_tensor": (i32, [vp, C.c_char_p, vp, i64, vp]),
        "tfq_container_read_tensor_host": (i32, [vp, C.c_char_p, vp, i64]),
        "tfq_container_weight": (vp, [vp, C.c_char_p, i64, i64]),
        "tfq_chain_create": (vp, [vp, i32, i32]),
        "tfq_chain_run": (i32, [vp, vp]),
        "tfq_chain_check": (i32, [vp]),
        "tfq_chain_weight_bytes": (sz, [vp]),
        "tfq_chain_free": (None, [vp]),
        "tfq_malloc": (vp, [sz]),
        "tfq_free": (None, [vp]),
        "tfq_copy_to_device": (i32, [vp, vp, sz]),
        "tfq_copy_to_host": (i32, [vp, vp, sz]),
        "tfq_stream_sync": (i32, [vp]),
        "tfq_gemv_multi_fused": (i32, [vp, i32, vp, i32, i32, vp, i32, vp, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


SHIMS_PATH = os.path.join(_HERE, "libtfq_shims.so")
_shims = None


def shims():
    """libtfq_shims.so: the reference-named host C++ entry points and the seeded generator."""
    global _shims
    if _shims is None:
        lib()  # libtfq.so first: the shim library links against it
        if not os.path.exists(SHIMS_PATH):
            raise TfqError(f"{SHIMS_PATH} is missing: run __graft_entry__.build() first")
        s = C.CDLL(SHIMS_PATH)
        s.tfq_rng_normal.argtypes = [C.c_uint64, C.c_int64, C.c_float, C.c_void_p]
        s.tfq_rng_normal.restype = None
        s.tfq_rng_uniform.argtypes = [C.c_uint64, C.c_int64, C.c_void_p]
        s.tfq_rng_uniform.restype = None
        _shims = s
    return _shims


def rng_normal(seed: int, n: int, scale: float = 1.0):
    """n draws of quant::RNG(seed).normal() * scale as a float32 numpy array (src/core/random.cpp:45-81)."""
    import numpy as np
    out = np.empty(n, np.float32)
    shims().tfq_rng_normal(seed, n, scale, out.ctypes.data)
    return out


def rng_uniform(seed: int, n: int):
    import numpy as np
    out = np.empty(n, np.float32)
    shims().tfq_rng_uniform(seed, n, out.ctypes.data)
    return out


def _check(rc: int):
    if rc != 0:
        raise TfqError(f"tfq error {rc}: {lib().tfq_last_error().decode()}")


def fmt_id(fmt) -> int:
    return FMT[fmt] if isinstance(fmt, str) else int(fmt)


def block_bytes(fmt, n: int = 256) -> int:
    out = C.c_size_t(0)
    _check(lib().tfq_block_bytes(fmt_id(fmt), n, C.byref(out)))
    return out.value


def _stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dtype_code(t):
    import torch
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise TfqError(f"unsupported dtype {t.dtype}")


def init(device: int = 0):
    _check(lib().tfq_init(device))


def encode(fmt, w):
    """fp32 device tensor -> uint8 device tensor of payloads (256-weight blocks, the last one possibly short)."""
    import torch
    w = w.contiguous()
    assert w.is_cuda and w.dtype == torch.float32
    n = w.numel()
    nbytes = (n // 256) * block_bytes(fmt) + (block_bytes(fmt, n % 256) if n % 256 else 0)
    out = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
    _check(lib().tfq_encode_blocks(fmt_id(fmt), w.data_ptr(), n, out.data_ptr(), out.numel(), _stream()))
    return out


def decode(fmt, payload, n: int):
    import torch
    assert payload.is_cuda and payload.dtype == torch.uint8
    out = torch.empty(n, dtype=torch.float32, device=payload.device)
    _check(lib().tfq_decode_blocks(fmt_id(fmt), payload.data_ptr(), payload.numel(), n, out.data_ptr(), _stream()))
    return out


class Weight:
    """Device-resident packed matrix W[N][K] (N rows of K/256 wire blocks)."""

    def __init__(self, fmt, N: int, K: int, packed, handle=None):
        import numpy as np
        import torch
        self.fmt, self.N, self.K = fmt_id(fmt), int(N), int(K)
        if handle is not None:  # adopted from tfq_container_weight
            self.handle = C.c_void_p(handle)
            return
        if isinstance(packed, torch.Tensor) and packed.is_cuda:
            # device payload: copied into the handle's own layout, the caller may drop its tensor
            h = lib().tfq_weight_wrap(self.fmt, N, K, packed.data_ptr(), packed.numel())
        else:
            arr = np.ascontiguousarray(packed.cpu().numpy() if isinstance(packed, torch.Tensor) else packed,
                                       dtype=np.uint8)
            h = lib().tfq_weight_upload(self.fmt, N, K, arr.ctypes.data, arr.size)
        if not h:
            raise TfqError(lib().tfq_last_error().decode())
        self.handle = C.c_void_p(h)

    @classmethod
    def mixed(cls, N: int, K: int, block_formats, packed):
        """A matrix whose blocks carry their own wire ids (tfq_weight_upload_mixed): block_formats uint8 [N * K / 256]
        (names or ids), packed the concatenated payloads (host array)."""
        import numpy as np
        fm = np.ascontiguousarray([fmt_id(f) for f in block_formats], dtype=np.uint8)
        arr = np.ascontiguousarray(packed, dtype=np.uint8)
        h = lib().tfq_weight_upload_mixed(N, K, fm.ctypes.data, arr.ctypes.data, arr.size)
        if not h:
            raise TfqError(lib().tfq_last_error().decode())
        return cls(int(fm[0]), N, K, None, handle=h)

    def close(self):
        if getattr(self, "handle", None):
            lib().tfq_weight_free(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def decode(self):
        import torch
        out = torch.empty((self.N, self.K), dtype=torch.float32, device="cuda")
        _check(lib().tfq_weight_decode(self.handle, out.data_ptr(), _stream()))
        return out

    def _mm(self, fn, x, out_dtype):
        import torch
        x = x.contiguous()
        assert x.is_cuda and x.shape[-1] == self.K
        B = x.numel() // self.K
        y = torch.empty((B, self.N), dtype=out_dtype or torch.float32, device=x.device)
        _check(fn(self.handle, x.data_ptr(), _dtype_code(x), B, y.data_ptr(), _dtype_code(y), _stream()))
        return y

    def gemv(self, x, out_dtype=None, out=None, workspace=None):
        """y[B][N] = x[B][K] . W^T for 1 <= B <= 16 (decode).  Calls that cut K into parts (five or more rows, K above
        4096) go through tfq_gemv_ws; `workspace` is a uint8 tensor of tfq_gemv_workspace_bytes or more (one is made
        per call when none is given; pass one when the call is captured into a graph and replayed)."""
        import torch
        x = x.contiguous()
        assert x.is_cuda and x.shape[-1] == self.K
        B = x.numel() // self.K
        if out is None:
            out = torch.empty((B, self.N), dtype=out_dtype or torch.float32, device=x.device)
        need = int(lib().tfq_gemv_workspace_bytes(self.handle, _dtype_code(x), B))
        if need == 0:
            _check(lib().tfq_gemv(self.handle, x.data_ptr(), _dtype_code(x), B, out.data_ptr(), _dtype_code(out), _stream()))
            return out
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
        assert workspace.numel() >= need and workspace.data_ptr() % 256 == 0
        _check(lib().tfq_gemv_ws(self.handle, x.data_ptr(), _dtype_code(x), B, out.data_ptr(), _dtype_code(out),
                                 workspace.data_ptr(), workspace.numel(), _stream()))
        return out

    def gemv_workspace_bytes(self, x_dtype_code: int, B: int) -> int:
        return int(lib().tfq_gemv_workspace_bytes(self.handle, x_dtype_code, B))

    def gemm(self, x, out_dtype=None, workspace=True):
        """y[M][N] = x[M][K] . W^T for any M (prefill).  With `workspace` the call goes through tfq_gemm_ws with
        as much scratch memory as tfq_gemm_workspace_bytes asks for (the K split of the prefill kernel)."""
        import torch
        if not workspace:
            return self._mm(lib().tfq_gemm, x, out_dtype)
        x = x.contiguous()
        assert x.is_cuda and x.shape[-1] == self.K
        M = x.numel() // self.K
        y = torch.empty((M, self.N), dtype=out_dtype or torch.float32, device=x.device)
        need = int(lib().tfq_gemm_workspace_bytes(self.handle, _dtype_code(x), M))
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device=x.device)
        _check(lib().tfq_gemm_ws(self.handle, x.data_ptr(), _dtype_code(x), M, y.data_ptr(), _dtype_code(y),
                                 ws.data_ptr(), need, _stream()))
        return y


class _ChainPhase(C.Structure):
    """tfq_chain_phase_t (include/tfq.h)."""
    _fields_ = [("w", C.c_void_p * 4), ("count", C.c_int), ("x", C.c_void_p), ("x_dtype", C.c_int),
                ("x_op", C.c_int), ("gamma", C.c_void_p), ("eps", C.c_float),
                ("gamma_plus_one", C.c_int), ("y_op", C.c_int), ("y", C.c_void_p * 4), ("y_dtype", C.c_int),
                ("residual", C.c_void_p)]


X_PLAIN, X_RMSNORM = 0, 1
Y_PLAIN, Y_SWIGLU, Y_RESIDUAL = 0, 1, 2


class Chain:
    """A sequence of dependent matrix-vector products in one persistent launch (tfq_chain_*).

    phases: list of dicts with keys
      w (list of Weight), x (tensor [B][K] for the first phase; None afterwards = the previous phase's result),
      x_op (X_PLAIN / X_RMSNORM), gamma (fp32 tensor), eps, gamma_plus_one,
      y_op (Y_PLAIN / Y_SWIGLU / Y_RESIDUAL), y (list of tensors or None), residual (fp32 tensor [B][N]).
    The tensors and Weight objects are kept alive by the chain."""

    def __init__(self, phases, B: int = 1):
        arr = (_ChainPhase * len(phases))()
        self._keep = []
        for i, ph in enumerate(phases):
            d = arr[i]
            ws = ph["w"]
            d.count = len(ws)
            for m, w in enumerate(ws):
                d.w[m] = w.handle
                self._keep.append(w)
            x = ph.get("x")
            if x is not None:
                d.x = x.data_ptr()
                d.x_dtype = _dtype_code(x)
                self._keep.append(x)
            d.x_op = ph.get("x_op", X_PLAIN)
            g = ph.get("gamma")
            if g is not None:
                d.gamma = g.data_ptr()
                self._keep.append(g)
            d.eps = float(ph.get("eps", 1e-6))
            d.gamma_plus_one = 1 if ph.get("gamma_plus_one") else 0
            d.y_op = ph.get("y_op", Y_PLAIN)
            ys = ph.get("y") or []
            d.y_dtype = F32
            kinds = {_dtype_code(y) for y in ys if y is not None}
            if len(kinds) > 1:
                raise TfqError("Chain: the outputs of one phase must share a dtype")
            for m, y in enumerate(ys):
                if y is not None:
                    d.y[m] = y.data_ptr()
                    d.y_dtype = _dtype_code(y)
                    self._keep.append(y)
            r = ph.get("residual")
            if r is not None:
                d.residual = r.data_ptr()
                self._keep.append(r)
        h = lib().tfq_chain_create(C.cast(arr, C.c_void_p), len(phases), B)
        if not h:
            raise TfqError(lib().tfq_last_error().decode())
        self.handle = C.c_void_p(h)

    @property
    def weight_bytes(self) -> int:
        return int(lib().tfq_chain_weight_bytes(self.handle))

    def run(self):
        _check(lib().tfq_chain_run(self.handle, _stream()))

    def check(self):
        """Call after synchronising: raises if a wait inside the last runs ran out."""
        _check(lib().tfq_chain_check(self.handle))

    def close(self):
        if getattr(self, "handle", None):
            lib().tfq_chain_free(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Container:
    """A .quant file (QUANTReader, include/quant/quant_format.h:64-149): host-side tables, tensors decoded or
    uploaded on the device."""

    def __init__(self, path=None, image=None):
        if path is not None:
            h = lib().tfq_container_open(os.fsencode(path))
        else:
            image = bytes(image)
            h = lib().tfq_container_from_memory(image, len(image))
        if not h:
            raise TfqError(lib().tfq_last_error().decode())
        self.handle = C.c_void_p(h)

    def close(self):
        if getattr(self, "handle", None):
            lib().tfq_container_close(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def valid(self) -> bool:
        return bool(lib().tfq_container_valid(self.handle))

    @property
    def num_blocks(self) -> int:
        return int(lib().tfq_container_num_blocks(self.handle))

    def header(self):
        ver, flags, cfg, n = C.c_uint32(0), C.c_uint32(0), C.c_void_p(0), C.c_size_t(0)
        _check(lib().tfq_container_header(self.handle, C.byref(ver), C.byref(flags), C.byref(cfg), C.byref(n)))
        return ver.value, flags.value, (C.string_at(cfg.value, n.value) if n.value else b"")

    def tensor_names(self):
        buf = C.create_string_buffer(1 << 16)
        out = []
        for i in range(lib().tfq_container_num_tensors(self.handle)):
            n = lib().tfq_container_tensor_name(self.handle, i, buf, len(buf))
            if n < 0:
                raise TfqError(lib().tfq_last_error().decode())
            out.append(buf.raw[:n].decode("utf-8", "replace"))
        return out

    def tensor_blocks(self, name: str):
        s, k = C.c_uint32(0), C.c_uint32(0)
        _check(lib().tfq_container_tensor_blocks(self.handle, name.encode(), C.byref(s), C.byref(k)))
        return s.value, k.value

    def block(self, block_id: int):
        """(format as the readers see it, weights, cb_bytes, payload bytes)"""
        f, nw, cb, ib, p = C.c_uint8(0), C.c_uint32(0), C.c_uint32(0), C.c_uint32(0), C.c_void_p(0)
        _check(lib().tfq_container_block(self.handle, block_id, C.byref(f), C.byref(nw), C.byref(cb), C.byref(ib), C.byref(p)))
        return f.value, nw.value, cb.value, C.string_at(p.value, ib.value)

    def read_tensor(self, name: str, device="cuda"):
        import torch
        n = lib().tfq_container_tensor_weights(self.handle, name.encode())
        if n < 0:
            raise TfqError(lib().tfq_last_error().decode())
        out = torch.empty(n, dtype=torch.float32, device=device)
        _check(lib().tfq_container_read_tensor(self.handle, name.encode(), out.data_ptr(), n, _stream()))
        return out

    def weight(self, name: str, rows: int, cols: int) -> "Weight":
        h = lib().tfq_container_weight(self.handle, name.encode(), rows, cols)
        if not h:
            raise TfqError(lib().tfq_last_error().decode())
        f, n, k, b = C.c_uint8(0), C.c_int64(0), C.c_int64(0), C.c_size_t(0)
        lib().tfq_weight_info(h, C.byref(f), C.byref(n), C.byref(k), C.byref(b))
        return Weight(f.value, n.value, k.value, None, handle=h)


def gemv_multi(weights, x, outs):
    """One launch for up to four matrices that share K, format and x (q/k/v, gate/up)."""
    n = len(weights)
    hs = (C.c_void_p * n)(*[w.handle for w in weights])
    ys = (C.c_void_p * n)(*[o.data_ptr() for o in outs])
    B = x.numel() // weights[0].K
    _check(lib().tfq_gemv_multi(hs, n, x.data_ptr(), _dtype_code(x), B, ys, _dtype_code(outs[0]), _stream()))
    return outs


class _Prologue(C.Structure):
    """tfq_prologue_t (include/tfq.h)."""
    _fields_ = [("op", C.c_int), ("gamma", C.c_void_p), ("eps", C.c_float), ("gamma_plus_one", C.c_int),
                ("up", C.c_void_p), ("mid_dtype", C.c_int), ("pair_swiglu", C.c_int), ("accumulate", C.c_int)]


PRO_NONE, PRO_RMSNORM, PRO_SWIGLU = 0, 1, 2


def gemv_multi_fused(ws, x, outs, *, rmsnorm=None, swiglu_up=None, eps=1e-6, gamma_plus_one=True, mid_dtype=None, accumulate=False,
                     pair_swiglu=False):
    """tfq_gemv_multi_fused: up to four matrices on fp32 x [B][K] with RMSNorm (rmsnorm = the fp32 gain vector)
    or SwiGLU (x = the gate product, swiglu_up = the up product) applied while the activations are staged."""
    import torch
    n = len(ws)
    assert x.is_contiguous()
    B = x.shape[0]
    hs = (C.c_void_p * n)(*[w.handle for w in ws])
    ys = (C.c_void_p * n)(*[o.data_ptr() for o in outs])
    pro = _Prologue()
    pro.accumulate = 1 if accumulate else 0
    pro.pair_swiglu = 1 if pair_swiglu else 0
    if pair_swiglu and len(outs) == 1:  # ys[1] is not written; the C call still wants two pointers
        ys = (C.c_void_p * n)(outs[0].data_ptr(), outs[0].data_ptr())
    if rmsnorm is not None:
        assert rmsnorm.dtype == torch.float32
        pro.op, pro.gamma, pro.eps, pro.gamma_plus_one = PRO_RMSNORM, rmsnorm.data_ptr(), eps, 1 if gamma_plus_one else 0
    elif swiglu_up is not None:
        assert swiglu_up.dtype == torch.float32 and swiglu_up.shape == x.shape and swiglu_up.is_contiguous()
        pro.op, pro.up = PRO_SWIGLU, swiglu_up.data_ptr()
        pro.mid_dtype = BF16 if mid_dtype == torch.bfloat16 else F32
    _check(lib().tfq_gemv_multi_fused(hs, n, x.data_ptr(), _dtype_code(x), B, ys, _dtype_code(outs[0]), C.byref(pro), _stream()))
    return outs


def moe_router(x, router_w, k: int, bias=None):
    """Router Linear + softmax + top-k on the device: returns (logits, probs, idx int32, weights)."""
    import torch
    T, D = x.shape
    E = router_w.shape[0]
    assert router_w.dtype == torch.float32 and router_w.is_contiguous() and x.is_contiguous()
    logits = torch.empty(T, E, device=x.device)
    probs = torch.empty(T, E, device=x.device)
    kk = max(1, min(k, E))
    idx = torch.empty(T, kk, device=x.device, dtype=torch.int32)
    w = torch.empty(T, kk, device=x.device)
    L = lib()
    L.tfq_moe_router.restype = C.c_int
    L.tfq_moe_router.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int,
                                 C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    _check(L.tfq_moe_router(x.data_ptr(), _dtype_code(x), router_w.data_ptr(), bias.data_ptr() if bias is not None else None,
                            T, D, E, k, logits.data_ptr(), probs.data_ptr(), idx.data_ptr(), w.data_ptr(), _stream()))
    return logits, probs, idx, w


def moe_route(logits, k: int):
    """Device softmax + top-k: returns (probs [T][E], idx [T][k] int32, weights [T][k])."""
    import torch
    logits = logits.contiguous().float()
    T, E = logits.shape
    k = max(1, min(k, E))
    probs = torch.empty_like(logits)
    idx = torch.empty((T, k), dtype=torch.int32, device=logits.device)
    w = torch.empty((T, k), dtype=torch.float32, device=logits.device)
    _check(lib().tfq_moe_route(logits.data_ptr(), T, E, k, probs.data_ptr(), idx.data_ptr(), w.data_ptr(), _stream()))
    return probs, idx, w


def mlp_step(gate, up, down, x, out_dtype=None, mid_dtype=None):
    """Dense SwiGLU feed-forward y = down(silu(gate x) * (up x)) for x [B][D] on the device."""
    import torch
    x = x.contiguous()
    B = x.numel() // gate.K
    y = torch.empty((B, down.N), dtype=out_dtype or torch.float32, device=x.device)
    mid = BF16 if (mid_dtype or x.dtype) == torch.bfloat16 else F32
    nbytes = lib().tfq_mlp_workspace_bytes(B, gate.N)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    _check(lib().tfq_mlp_step(gate.handle, up.handle, down.handle, x.data_ptr(), _dtype_code(x), B, y.data_ptr(),
                              _dtype_code(y), mid, ws.data_ptr(), nbytes, _stream()))
    return y


def moe_ffn(gate, up, down, topk_idx, topk_w, x, out_dtype=None, mid_dtype=None):
    """MoE expert FFN.  gate/up/down: lists of Weight; topk_idx/topk_w: host arrays [T][k]; x: device [T][D]."""
    import numpy as np
    import torch
    E = len(gate)
    idx = np.ascontiguousarray(topk_idx, np.int64)
    wts = np.ascontiguousarray(topk_w, np.float32)
    T, k = idx.shape
    D, F = gate[0].K, gate[0].N
    x = x.contiguous()
    y = torch.empty((T, D), dtype=out_dtype or torch.float32, device=x.device)
    mid = BF16 if (mid_dtype or x.dtype) == torch.bfloat16 else F32
    nbytes = lib().tfq_moe_workspace_bytes(T, k, D, F)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    arr = lambda ws_: (C.c_void_p * E)(*[w.handle for w in ws_])
    _check(lib().tfq_moe_ffn(arr(gate), arr(up), arr(down), E, idx.ctypes.data, wts.ctypes.data, T, k,
                             x.data_ptr(), _dtype_code(x), y.data_ptr(), _dtype_code(y), mid,
                             ws.data_ptr(), nbytes, _stream()))
    return y


class RoutedMoe:
    """tfq_moe_ffn_routed for one set of experts and one call shape: the experts' address table and the workspace
    are made once, so a call allocates nothing and can be captured into a graph.  idx (int32) and weights are device
    tensors [T][k] as moe_route returns them."""

    def __init__(self, gate, up, down, T: int, k: int, device="cuda"):
        import torch
        self.E = len(gate)
        self.gate, self.up, self.down = list(gate), list(up), list(down)
        self.T, self.k, self.D, self.F = T, k, gate[0].K, gate[0].N
        arr = lambda ws_: (C.c_void_p * self.E)(*[w.handle for w in ws_])
        self._g, self._u, self._d = arr(gate), arr(up), arr(down)
        self.table = torch.empty(3 * self.E * 8, dtype=torch.uint8, device=device)
        _check(lib().tfq_moe_expert_table(self._g, self._u, self._d, self.E, self.table.data_ptr()))
        self.nbytes = int(lib().tfq_moe_routed_workspace_bytes(self._g, self._u, self._d, self.E, T, k))
        if self.nbytes == 0:
            raise TfqError("tfq_moe_ffn_routed does not take this configuration")
        self.ws = torch.empty(self.nbytes, dtype=torch.uint8, device=device)

    def __call__(self, idx, wts, x, y):
        assert idx.is_cuda and wts.is_cuda and idx.dtype.itemsize == 4 and x.is_contiguous() and y.is_contiguous()
        _check(lib().tfq_moe_ffn_routed(self._g, self._u, self._d, self.E, self.table.data_ptr(), idx.data_ptr(), wts.data_ptr(),
                                        self.T, self.k, x.data_ptr(), _dtype_code(x), y.data_ptr(), _dtype_code(y), BF16,
                                        self.ws.data_ptr(), self.nbytes, _stream()))
        return y


def moe_plan_dispatch(topk_idx, topk_w, E: int, slots_per_expert: int):
    """moe_engine::plan_dispatch on the host side of the library: (expert_first, item_token, item_weight, dropped slots)."""
    import numpy as np
    idx = np.ascontiguousarray(topk_idx, np.int32)
    wts = np.ascontiguousarray(topk_w, np.float32)
    T, k = idx.shape
    first = np.zeros(E + 1, np.int32)
    tok = np.zeros(T * k, np.int32)
    wt = np.zeros(T * k, np.float32)
    dr = np.zeros(T * k, np.int32)
    nd = C.c_int64(0)
    _check(lib().tfq_moe_plan_dispatch(idx.ctypes.data, wts.ctypes.data, T, k, E, slots_per_expert, first.ctypes.data,
                                       tok.ctypes.data, wt.ctypes.data, dr.ctypes.data, C.addressof(nd)))
    n = int(first[E])
    return first, tok[:n], wt[:n], dr[:nd.value]


def moe_ffn_capacity(gate, up, down, topk_idx, topk_w, slots_per_expert: int, x, out_dtype=None, mid_dtype=None):
    """Capacity-limited MoE FFN (tfq_moe_ffn_capacity): returns (y [T][D], dropped count)."""
    import numpy as np
    import torch
    E = len(gate)
    idx = np.ascontiguousarray(topk_idx, np.int32)
    wts = np.ascontiguousarray(topk_w, np.float32)
    T, k = idx.shape
    D, F = gate[0].K, gate[0].N
    x = x.contiguous()
    y = torch.empty((T, D), dtype=out_dtype or torch.float32, device=x.device)
    mid = BF16 if (mid_dtype or x.dtype) == torch.bfloat16 else F32
    nbytes = lib().tfq_moe_workspace_bytes(T, k, D, F)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    arr = lambda ws_: (C.c_void_p * E)(*[w.handle for w in ws_])
    nd = C.c_int64(0)
    _check(lib().tfq_moe_ffn_capacity(arr(gate), arr(up), arr(down), E, idx.ctypes.data, wts.ctypes.data, T, k,
                                      slots_per_expert, x.data_ptr(), _dtype_code(x), y.data_ptr(), _dtype_code(y), mid,
                                      ws.data_ptr(), nbytes, C.addressof(nd), _stream()))
    return y, int(nd.value)


def lut4_gemm(packed, codebook16, act, M: int, N: int, K: int):
    """kernel::quant4_gemm on the device: packed (uint8) and act (fp32 [N][K]) are device tensors, codebook16 a host uint16[16]."""
    import numpy as np
    import torch
    cb = np.ascontiguousarray(codebook16, np.uint16)
    out = torch.empty((M, N), dtype=torch.float32, device=act.device)
    _check(lib().tfq_lut4_gemm(packed.data_ptr(), cb.ctypes.data, act.data_ptr(), out.data_ptr(), M, N, K, _stream()))
    return out


def lut8_gemm(idx, codebook256, act, M: int, N: int, K: int):
    """kernel::quant8_gemm on the device: idx uint8 [N][K], act fp32 [M][K] device tensors, codebook256 a host float[256]."""
    import numpy as np
    import torch
    cb = np.ascontiguousarray(codebook256, np.float32)
    out = torch.empty((M, N), dtype=torch.float32, device=act.device)
    _check(lib().tfq_lut8_gemm(idx.data_ptr(), cb.ctypes.data, act.data_ptr(), out.data_ptr(), M, N, K, _stream()))
    return out


def lut_gemv_batch(bits: int, packed, codebook, scale: float, X, M: int, N: int, K: int):
    """prod::gemv_quant{,4,8}_batch on the device: Y[N][M] = scale * W . X^T."""
    import numpy as np
    import torch
    cbp = None
    if bits == 4:
        cb = np.ascontiguousarray(codebook, np.uint16)
        cbp = cb.ctypes.data
    elif bits == 8:
        cb = np.ascontiguousarray(codebook, np.float32)
        cbp = cb.ctypes.data
    out = torch.empty((N, M), dtype=torch.float32, device=X.device)
    _check(lib().tfq_lut_gemv_batch(bits, packed.data_ptr(), cbp, scale, X.data_ptr(), out.data_ptr(), M, N, K, _stream()))
    return out


def lutn_gemm(bits: int, packed, codebook, act, M: int, N: int, K: int):
    """kernel::q3_gemm / q6_gemm / q12_gemm / q24_gemm on the device (bits = 3, 6, 12, 24): packed uint8 and
    act fp32 [N][K] are device tensors, codebook a host array (float32, or uint16 binary16 bits for 12; None for 24)."""
    import numpy as np
    import torch
    cbp = None
    if bits != 24:
        cb = np.ascontiguousarray(codebook, np.uint16 if bits == 12 else np.float32)
        cbp = cb.ctypes.data
    out = torch.empty((M, N), dtype=torch.float32, device=act.device)
    _check(lib().tfq_lutn_gemm(bits, packed.data_ptr(), cbp, act.data_ptr(), out.data_ptr(), M, N, K, _stream()))
    return out


def fp24_encode(w):
    import torch
    w = w.contiguous().float()
    out = torch.empty(3 * w.numel(), dtype=torch.uint8, device=w.device)
    _check(lib().tfq_fp24_encode(w.data_ptr(), out.data_ptr(), w.numel(), _stream()))
    return out


def fp24_decode(packed):
    import torch
    out = torch.empty(packed.numel() // 3, dtype=torch.float32, device=packed.device)
    _check(lib().tfq_fp24_decode(packed.data_ptr(), out.data_ptr(), out.numel(), _stream()))
    return out


class CodebookEngine:
    """engines::Q4Engine (bits=4) / Q8Engine (bits=8) with the given centroids; tensors live on the device."""

    def __init__(self, bits: int, codebook):
        import numpy as np
        self.bits = bits
        self.cb = np.ascontiguousarray(codebook, np.float32)
        assert self.cb.size == 1 << bits

    def quantize_per_block(self, data, block_size: int):
        import torch
        data = data.contiguous().float()
        n = data.numel()
        nb = (n + block_size - 1) // block_size
        idx = torch.empty(n, dtype=torch.uint8, device=data.device)
        scales = torch.empty(nb * (2 if self.bits == 4 else 1), dtype=torch.float32, device=data.device)
        _check(lib().tfq_engine_quantize_per_block(self.bits, self.cb.ctypes.data, data.data_ptr(), n, block_size,
                                                   idx.data_ptr(), scales.data_ptr(), _stream()))
        return idx, scales

    def dequantize_per_block(self, idx, scales, block_size: int):
        import torch
        out = torch.empty(idx.numel(), dtype=torch.float32, device=idx.device)
        _check(lib().tfq_engine_dequantize_per_block(self.bits, self.cb.ctypes.data, idx.data_ptr(), scales.data_ptr(),
                                                     idx.numel(), block_size, out.data_ptr(), _stream()))
        return out

    def quantize_tensor(self, data):
        import torch
        data = data.contiguous().float()
        n = data.numel()
        out = torch.empty(n if self.bits == 8 else (n + 1) // 2, dtype=torch.uint8, device=data.device)
        _check(lib().tfq_engine_quantize_tensor(self.bits, self.cb.ctypes.data, data.data_ptr(), n, out.data_ptr(), _stream()))
        return out

    def dequant_tensor(self, idx, n: int):
        import torch
        out = torch.empty(n, dtype=torch.float32, device=idx.device)
        _check(lib().tfq_engine_dequant_tensor(self.bits, self.cb.ctypes.data, idx.data_ptr(), n, out.data_ptr(), _stream()))
        return out

    def quant_gemm(self, a, b_idx, M: int, N: int, K: int):
        import torch
        a = a.contiguous().float()
        out = torch.empty((M, N), dtype=torch.float32, device=a.device)
        _check(lib().tfq_engine_quant_gemm(self.bits, self.cb.ctypes.data, a.data_ptr(), b_idx.data_ptr(), M, N, K,
                                           out.data_ptr(), _stream()))
        return out


def q8codec_encode(data, block_size: int = 256):
    """Q8Encoder::encode_tensor: (centroids [blocks][256], indices)."""
    import torch
    data = data.contiguous().float()
    n = data.numel()
    nb = (n + block_size - 1) // block_size
    cent = torch.empty((nb, 256), dtype=torch.float32, device=data.device)
    idx = torch.empty(n, dtype=torch.uint8, device=data.device)
    _check(lib().tfq_q8codec_encode(data.data_ptr(), n, block_size, cent.data_ptr(), idx.data_ptr(), _stream()))
    return cent, idx


def q8codec_decode(cent, idx, block_size: int = 256):
    import torch
    out = torch.empty(idx.numel(), dtype=torch.float32, device=idx.device)
    _check(lib().tfq_q8codec_decode(cent.data_ptr(), idx.data_ptr(), idx.numel(), block_size, out.data_ptr(), _stream()))
    return out


def q8_quantize_rows(src, dst_f32: bool = False):
    """quant8::quantize_activations: (quantized [batch][per], params [batch][3] = scale, inv_scale, zero_point)."""
    import torch
    src = src.contiguous().float()
    batch, per = src.shape
    dst = torch.empty((batch, per), dtype=torch.float32 if dst_f32 else torch.uint8, device=src.device)
    params = torch.empty((batch, 3), dtype=torch.float32, device=src.device)
    _check(lib().tfq_q8_quantize_rows(src.data_ptr(), batch, per, int(dst_f32), dst.data_ptr(), params.data_ptr(), _stream()))
    return dst, params


def q8_dequantize(src, params3):
    import torch
    out = torch.empty(src.numel(), dtype=torch.float32, device=src.device)
    _check(lib().tfq_q8_dequantize(src.data_ptr(), src.numel(), int(src.dtype == torch.float32), params3.data_ptr(),
                                   out.data_ptr(), _stream()))
    return out
