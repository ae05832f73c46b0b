"""ctypes binding of libmagi_attn.so (the C-ABI declared in include/magi_attn.h).

The library is the only compute path: when it is missing, loading raises, there is no
fallback to PyTorch ops.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmagi_attn.so")

MAGI_DTYPE_BF16 = 0
MAGI_DTYPE_FP8_E4M3 = 1
MAGI_RANGES_PAIRS = 0
MAGI_RANGES_CU = 1
MAGI_NORM_LAYERNORM_1P = 0
MAGI_NORM_RMSNORM_1P = 1
MAGI_NORM_NONE = 2
MAGI_ATTN_FP8_POW2_PRESCALED = 1
MAGI_ATTN_Q_PRESCALED = 2
MAGI_ATTN_FP8_FAST_EXP2 = 4
MAGI_ATTN_BOUNDED_MFMA32 = 8
MAGI_ATTN_AUTO_BOUND = 16
MAGI_SCORE_BOUND_MAX = 64.0


class MagiError(RuntimeError):
    """A C-ABI call returned a negative code; .code holds it."""

    def __init__(self, code: int, msg: str):
        super().__init__(f"libmagi_attn error {code}: {msg}")
        self.code = code


class _SizedStructure(C.Structure):
    """Every argument struct of the C-ABI starts with its own size (struct_size), filled in here."""

    def __init__(self, *args, **kw):
        super().__init__(*args, **kw)
        self.struct_size = C.sizeof(type(self))


class AttnArgs(_SizedStructure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("k2", C.c_void_p), ("v2", C.c_void_p),
        ("out", C.c_void_p), ("lse", C.c_void_p), ("q_ranges", C.c_void_p), ("k_ranges", C.c_void_p),
        ("q_scale", C.c_void_p), ("k_scale", C.c_void_p), ("v_scale", C.c_void_p),
        ("q_stride_t", C.c_int64), ("q_stride_h", C.c_int64), ("k_stride_t", C.c_int64), ("k_stride_h", C.c_int64),
        ("v_stride_t", C.c_int64), ("v_stride_h", C.c_int64), ("o_stride_t", C.c_int64), ("o_stride_h", C.c_int64),
        ("total_q", C.c_int32), ("total_k", C.c_int32), ("k_split", C.c_int32),
        ("n_ranges", C.c_int32), ("ranges_mode", C.c_int32),
        ("max_seqlen_q", C.c_int32), ("max_seqlen_k", C.c_int32),
        ("Hq", C.c_int32), ("Hkv", C.c_int32), ("D", C.c_int32),
        ("dtype", C.c_int32), ("scale_chunk_tokens", C.c_int32),
        ("softmax_scale", C.c_float), ("flags", C.c_int32),
        ("out_group_heads", C.c_int32), ("o_stride_g", C.c_int64), ("score_bound", C.c_float),
        ("q_tile_rows", C.c_int32),
        ("q_norm_gamma", C.c_void_p), ("q_norm_beta", C.c_void_p), ("q_norm_eps", C.c_float), ("q_norm_kind", C.c_int32),
        ("k2_scale", C.c_void_p), ("v2_scale", C.c_void_p),
        ("workspace", C.c_void_p),
    ]


class PrologueArgs(_SizedStructure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("q_raw", C.c_void_p), ("k_raw", C.c_void_p), ("v_raw", C.c_void_p), ("rope", C.c_void_p),
        ("gq", C.c_void_p), ("bq", C.c_void_p), ("gk", C.c_void_p), ("bk", C.c_void_p),
        ("q_out", C.c_void_p), ("kv_out", C.c_void_p), ("kv_tail", C.c_void_p),
        ("q_raw_stride_t", C.c_int64), ("k_raw_stride_t", C.c_int64), ("v_raw_stride_t", C.c_int64),
        ("kv_stride_t", C.c_int64), ("kv_tail_stride_t", C.c_int64),
        ("S", C.c_int32), ("n_cache_rows", C.c_int32),
        ("Hq", C.c_int32), ("Hkv", C.c_int32), ("D", C.c_int32), ("R2", C.c_int32),
        ("norm_kind", C.c_int32), ("eps", C.c_float), ("batch", C.c_int32), ("q_premul", C.c_float),
        ("out_dtype", C.c_int32), ("q_quant_scale", C.c_float), ("k_quant_scale", C.c_float),
    ]


class QkvProjArgs(_SizedStructure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("x", C.c_void_p), ("w", C.c_void_p), ("x_stride", C.c_int64), ("w_stride", C.c_int64),
        ("S", C.c_int32), ("K", C.c_int32),
        ("Hq", C.c_int32), ("Hkv", C.c_int32), ("Hqx", C.c_int32), ("D", C.c_int32),
        ("rope", C.c_void_p), ("R2", C.c_int32),
        ("gq", C.c_void_p), ("bq", C.c_void_p), ("gk", C.c_void_p), ("bk", C.c_void_p),
        ("norm_kind", C.c_int32), ("eps", C.c_float), ("batch", C.c_int32), ("q_premul", C.c_float),
        ("q_out", C.c_void_p), ("kv_out", C.c_void_p), ("kv_tail", C.c_void_p),
        ("kv_stride_t", C.c_int64), ("kv_tail_stride_t", C.c_int64), ("n_cache_rows", C.c_int32),
        ("qx_out", C.c_void_p),
    ]


class QuantizeArgs(_SizedStructure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("x", C.c_void_p), ("x_stride_t", C.c_int64), ("x_stride_h", C.c_int64),
        ("T", C.c_int32), ("H", C.c_int32), ("D", C.c_int32), ("chunk_tokens", C.c_int32),
        ("premul", C.c_float), ("pow2_scales", C.c_int32),
        ("y", C.c_void_p), ("scales", C.c_void_p), ("n_rows_first", C.c_int32),
        ("y2", C.c_void_p), ("scales2", C.c_void_p),
    ]


ABI_VERSION = 103  # magi_version() of the library these mirrors were written for

EXPORTS = ("magi_version", "magi_last_error", "magi_launch_count", "magi_attn_fwd", "magi_attn_fwd_static_scratch",
           "magi_qk_prologue", "magi_head_norm",
           "magi_apply_rotary", "magi_quantize_fp8", "magi_quantize_fp8_split", "magi_layer_norm", "magi_qkv_proj_prologue", "magi_div_clamp_to_e4m3")

_lib = None


def lib() -> C.CDLL:
    """Load (once) and return the shared library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C magi-1_amd/csrc` (or __graft_entry__.build()); "
                "there is no fallback path")
        l = C.CDLL(LIB_PATH)
        l.magi_version.restype = C.c_int
        if l.magi_version() != ABI_VERSION:
            raise RuntimeError(f"{LIB_PATH} reports version {l.magi_version()}, this package binds version {ABI_VERSION}: "
                               "rebuild the library (`make -C magi-1_amd/csrc`)")
        l.magi_launch_count.restype = C.c_uint64
        l.magi_last_error.restype = C.c_char_p
        l.magi_attn_fwd.argtypes = [C.POINTER(AttnArgs), C.c_void_p]
        l.magi_attn_fwd.restype = C.c_int
        l.magi_attn_fwd_static_scratch.argtypes = [C.POINTER(AttnArgs), C.c_void_p]
        l.magi_attn_fwd_static_scratch.restype = C.c_int
        l.magi_qk_prologue.argtypes = [C.POINTER(PrologueArgs), C.c_void_p]
        l.magi_qk_prologue.restype = C.c_int
        l.magi_head_norm.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32,
                                     C.c_int32, C.c_int32, C.c_int32, C.c_float, C.c_void_p]
        l.magi_head_norm.restype = C.c_int
        l.magi_layer_norm.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p, C.c_int64,
                                      C.c_int64, C.c_int32, C.c_float, C.c_void_p]
        l.magi_layer_norm.restype = C.c_int
        l.magi_div_clamp_to_e4m3.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_int32, C.c_void_p, C.c_int64, C.c_int64,
                                             C.c_int32, C.c_void_p]
        l.magi_div_clamp_to_e4m3.restype = C.c_int
        l.magi_apply_rotary.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32,
                                        C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p]
        l.magi_apply_rotary.restype = C.c_int
        l.magi_quantize_fp8.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_int32,
                                        C.c_int32, C.c_int32, C.c_int32, C.c_float, C.c_int32, C.c_void_p]
        l.magi_quantize_fp8.restype = C.c_int
        l.magi_qkv_proj_prologue.argtypes = [C.POINTER(QkvProjArgs), C.c_void_p]
        l.magi_qkv_proj_prologue.restype = C.c_int
        l.magi_quantize_fp8_split.argtypes = [C.POINTER(QuantizeArgs), C.c_void_p]
        l.magi_quantize_fp8_split.restype = C.c_int
        _lib = l
    return _lib


def check(code: int) -> None:
    if code != 0:
        raise MagiError(code, lib().magi_last_error().decode("utf-8", "replace"))
