"""MI355X-native attention hot path of the MAGI-1 DiT (host side over libmagi_attn.so)."""
from ._lib import (MAGI_DTYPE_BF16, MAGI_DTYPE_FP8_E4M3, MAGI_NORM_LAYERNORM_1P, MAGI_NORM_NONE, MAGI_NORM_RMSNORM_1P,
                   MAGI_RANGES_CU, MAGI_RANGES_PAIRS, MAGI_SCORE_BOUND_MAX, MagiError, lib)
from .functional import (apply_rotary_emb, div_clamp_to, flash_attn_func, flash_attn_varlen_func, flex_flash_attn_func, head_norm,
                         layer_norm, pow2_scale_for, qk_norm_score_bound, qk_prologue, qk_prologue_fp8, qkv_proj_prologue, quantize_fp8,
                         quantize_fp8_split,
                         range_attention)

__all__ = [
    "MAGI_DTYPE_BF16", "MAGI_DTYPE_FP8_E4M3", "MAGI_NORM_LAYERNORM_1P", "MAGI_NORM_NONE", "MAGI_NORM_RMSNORM_1P",
    "MAGI_RANGES_CU", "MAGI_RANGES_PAIRS", "MAGI_SCORE_BOUND_MAX", "MagiError", "lib", "apply_rotary_emb", "div_clamp_to", "flash_attn_func",
    "flash_attn_varlen_func", "flex_flash_attn_func", "head_norm", "layer_norm", "pow2_scale_for", "qk_norm_score_bound", "qk_prologue", "qk_prologue_fp8", "qkv_proj_prologue",
    "quantize_fp8", "quantize_fp8_split", "range_attention",
]
