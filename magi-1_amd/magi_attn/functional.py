"""Reference-shaped callables over the C-ABI.

The four functions the reference's DiT module imports from third-party CUDA packages
(inference/model/dit/dit_module.py:27-37) keep their names, argument meaning and return
shapes here, so the module-level code reads the same:

  flex_flash_attn_func   (MagiAttention; dit_module.py:1032-1043, 1111-1122)
  flash_attn_func        (flash-attn;    dit_module.py:1062, 1090-1095)
  flash_attn_varlen_func (flash-attn;    dit_module.py:1124-1133)
  apply_rotary_emb       (flash-attn;    dit_module.py:961, 978)

plus the fused prologue and the cache-aware range attention this library adds.  PyTorch is
used for device memory and the current stream only.
"""
from __future__ import annotations

import ctypes as C
import math
from typing import Optional, Tuple

import torch

from . import _lib as L


def _stream() -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _check_thd(t: torch.Tensor, name: str) -> None:
    if t.dim() != 3:
        raise ValueError(f"{name} must be [tokens, heads, head_dim], got {tuple(t.shape)}")
    if not t.is_cuda:
        raise ValueError(f"{name} must be a CUDA (ROCm) tensor")
    if t.stride(2) != 1:
        raise ValueError(f"{name}: head_dim must be contiguous")


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return L.MAGI_DTYPE_BF16
    if t.dtype == torch.float8_e4m3fn:
        return L.MAGI_DTYPE_FP8_E4M3
    raise TypeError(f"unsupported dtype {t.dtype}: bf16 or float8_e4m3fn")


def range_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    q_ranges: torch.Tensor,
    k_ranges: torch.Tensor,
    max_seqlen_q: int,
    max_seqlen_k: int = 0,
    softmax_scale: Optional[float] = None,
    *,
    ranges_mode: int = L.MAGI_RANGES_PAIRS,
    k2: Optional[torch.Tensor] = None,
    v2: Optional[torch.Tensor] = None,
    k_split: Optional[int] = None,
    q_scale: Optional[torch.Tensor] = None,
    k_scale: Optional[torch.Tensor] = None,
    v_scale: Optional[torch.Tensor] = None,
    k2_scale: Optional[torch.Tensor] = None,
    v2_scale: Optional[torch.Tensor] = None,
    scale_chunk_tokens: int = 0,
    fp8_pow2_prescaled: bool = False,
    fp8_fast_exp2: bool = False,
    q_prescaled: bool = False,
    score_bound: float = 0.0,
    q_tile_rows: int = 0,
    bounded_mfma32: bool = False,
    auto_bound: bool = False,
    static_scratch: bool = False,
    q_norm: Optional[tuple] = None,
    out: Optional[torch.Tensor] = None,
    return_lse: bool = True,
    zero_init: bool = True,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """out[q_range_i] = softmax(q k^T * scale) v over k[k_range_i]; see magi_attn_fwd.

    k and v may be strided views (e.g. the two halves of an interleaved KV cache); with
    k2 / v2 the key axis is the concatenation [k[:k_split] | k2] without copying.

    k2_scale / v2_scale (fp8, with k2 / v2): the side segment's scale rows in tables of their own, row 0 = the chunk
    that starts at k_split; without them k_scale / v_scale are indexed across k_split as one table.

    fp8_fast_exp2 (with fp8_pow2_prescaled): piecewise-linear exp2 for the probabilities, MAGI_ATTN_FP8_FAST_EXP2.

    q_prescaled (bf16): q already carries softmax_scale * log2(e) (qk_prologue(..., q_premul=that)), so q . k is the
    exp2 exponent: the kernel skips its per-score multiply; softmax_scale is ignored.

    score_bound: promise that |q . k| * softmax_scale * log2(e) <= score_bound for every pair (with q_prescaled the
    factor is already in q); see magi_attn_args.score_bound.  Without q_prescaled the kernel applies the scale while
    it loads q.
    q_tile_rows: force a workgroup shape (0 = the library's choice); see magi_attn_args.q_tile_rows.
    bounded_mfma32 (with q_prescaled and score_bound): the 32x32x16 form of the bounded kernel, MAGI_ATTN_BOUNDED_MFMA32.
    auto_bound (bf16, instead of score_bound): the library measures max|q| and max|k| in two streaming passes and
    picks the bounded-score kernel on the device when their product allows it, MAGI_ATTN_AUTO_BOUND.  Its 16-byte
    workspace is a fresh tensor, or with static_scratch the library's own device array (magi_attn_fwd_static_scratch:
    no allocation at all when `out` is given and return_lse is False; such calls must not overlap on one GPU).
    q_norm: (gamma, beta or None, eps[, norm_kind]): q is the raw projection, normalised per (token, head) row inside
    the kernel (fp32, zero-centred gamma) and scaled by softmax_scale * log2(e); needs score_bound.
    """
    _check_thd(q, "q")
    _check_thd(k, "k")
    _check_thd(v, "v")
    Tq, Hq, D = q.shape
    Hkv = k.shape[1]
    total_k = k.shape[0] if k2 is None else int(k_split) + k2.shape[0]
    if k2 is not None:
        _check_thd(k2, "k2")
        _check_thd(v2, "v2")
        if k2.stride() != k.stride() or v2.stride() != v.stride():
            raise ValueError("k2 / v2 must have the strides of k / v")
        if k_split is None or not (0 <= k_split <= k.shape[0]):
            raise ValueError("k_split must lie inside k")
    if q_ranges.dtype != torch.int32 or k_ranges.dtype != torch.int32:
        raise TypeError("q_ranges / k_ranges must be int32")
    if not (q_ranges.is_cuda and k_ranges.is_cuda):
        raise ValueError("q_ranges / k_ranges must live on the device")
    q_ranges = q_ranges.contiguous()
    k_ranges = k_ranges.contiguous()
    if ranges_mode == L.MAGI_RANGES_PAIRS:
        n = q_ranges.shape[0]
        if q_ranges.shape != k_ranges.shape or q_ranges.dim() != 2 or q_ranges.shape[1] != 2:
            raise ValueError("q_ranges / k_ranges must both be [n, 2]")
    else:
        n = q_ranges.numel() - 1
        if q_ranges.numel() != k_ranges.numel():
            raise ValueError("cu_seqlens_q / cu_seqlens_k must have the same length")
    if out is None:
        out = (torch.zeros if zero_init else torch.empty)((Tq, Hq, D), dtype=torch.bfloat16, device=q.device)
    lse = None
    if return_lse:
        lse = torch.full((Hq, Tq), float("-inf"), dtype=torch.float32, device=q.device)
    a = L.AttnArgs()
    a.q, a.k, a.v, a.k2, a.v2 = _ptr(q), _ptr(k), _ptr(v), _ptr(k2), _ptr(v2)
    a.out, a.lse = _ptr(out), _ptr(lse)
    a.q_ranges, a.k_ranges = _ptr(q_ranges), _ptr(k_ranges)
    a.q_scale, a.k_scale, a.v_scale = _ptr(q_scale), _ptr(k_scale), _ptr(v_scale)
    for name, t in (("q_scale", q_scale), ("k_scale", k_scale), ("v_scale", v_scale), ("k2_scale", k2_scale),
                    ("v2_scale", v2_scale)):
        if t is not None and (t.dtype != torch.float32 or not t.is_contiguous() or t.device != q.device):
            raise ValueError(f"{name} must be a contiguous fp32 tensor on q's device")
    a.k2_scale, a.v2_scale = _ptr(k2_scale), _ptr(v2_scale)
    if q.dtype == torch.float8_e4m3fn and scale_chunk_tokens > 0:
        # the kernel indexes the tables by token / scale_chunk_tokens without a bound of its own
        C_ = int(scale_chunk_tokens)
        rows_of = lambda n: (n + C_ - 1) // C_
        first = total_k if (k2 is None or k2_scale is None) else int(k_split)
        need = [("q_scale", q_scale, rows_of(Tq), Hq), ("k_scale", k_scale, rows_of(first), Hkv),
                ("v_scale", v_scale, rows_of(first), Hkv)]
        if k2_scale is not None:
            need += [("k2_scale", k2_scale, rows_of(total_k - int(k_split)), Hkv),
                     ("v2_scale", v2_scale, rows_of(total_k - int(k_split)), Hkv)]
        for name, t, rows, heads in need:
            if t is not None and (t.dim() != 2 or t.shape[0] < rows or t.shape[1] != heads):
                raise ValueError(f"{name} must be [>= {rows} chunks, {heads} heads], got {tuple(t.shape)}")
    a.q_stride_t, a.q_stride_h = q.stride(0), q.stride(1)
    a.k_stride_t, a.k_stride_h = k.stride(0), k.stride(1)
    a.v_stride_t, a.v_stride_h = v.stride(0), v.stride(1)
    if out.dim() == 4:  # [Tq, groups, heads per group, D]: two-level head addressing
        if out.shape[0] != Tq or out.shape[1] * out.shape[2] != Hq or out.shape[3] != D or out.stride(3) != 1:
            raise ValueError("a 4-D out must be [Tq, groups, Hq / groups, D] with contiguous rows")
        a.o_stride_t, a.o_stride_g, a.o_stride_h, a.out_group_heads = out.stride(0), out.stride(1), out.stride(2), out.shape[2]
    else:
        a.o_stride_t, a.o_stride_h = out.stride(0), out.stride(1)
    a.total_q, a.total_k = Tq, total_k
    a.k_split = total_k if k2 is None else int(k_split)
    a.n_ranges, a.ranges_mode = max(n, 0), ranges_mode
    a.max_seqlen_q, a.max_seqlen_k = int(max_seqlen_q), int(max_seqlen_k)
    a.Hq, a.Hkv, a.D = Hq, Hkv, D
    a.dtype = _dtype_code(q)
    a.scale_chunk_tokens = int(scale_chunk_tokens)
    a.softmax_scale = 0.0 if softmax_scale is None else float(softmax_scale)
    a.flags = ((L.MAGI_ATTN_FP8_POW2_PRESCALED if fp8_pow2_prescaled else 0) | (L.MAGI_ATTN_Q_PRESCALED if q_prescaled else 0)
               | (L.MAGI_ATTN_FP8_FAST_EXP2 if fp8_fast_exp2 else 0) | (L.MAGI_ATTN_BOUNDED_MFMA32 if bounded_mfma32 else 0)
               | (L.MAGI_ATTN_AUTO_BOUND if auto_bound else 0))
    workspace = None
    if auto_bound and not static_scratch:
        workspace = torch.empty(4, dtype=torch.float32, device=q.device)  # (alive until the launches are enqueued)
        a.workspace = _ptr(workspace)
    a.score_bound = float(score_bound)
    a.q_tile_rows = int(q_tile_rows)
    keep = None
    if q_norm is not None:
        g_ = q_norm[0].to(torch.float32).contiguous()
        b_ = None if q_norm[1] is None else q_norm[1].to(torch.float32).contiguous()
        keep = (g_, b_)  # (alive until the launch is enqueued)
        a.q_norm_gamma, a.q_norm_beta = _ptr(g_), _ptr(b_)
        a.q_norm_eps = float(q_norm[2])
        a.q_norm_kind = int(q_norm[3]) if len(q_norm) > 3 else L.MAGI_NORM_LAYERNORM_1P
    with torch.cuda.device(q.device):
        entry = L.lib().magi_attn_fwd_static_scratch if static_scratch else L.lib().magi_attn_fwd
        L.check(entry(C.byref(a), _stream()))
    return out, lse


def qk_norm_score_bound(q_norm_bound: float, k_norm_bound: float, head_dim: int = 128,
                        softmax_scale: Optional[float] = None) -> float:
    """score_bound for QK-normed attention from the lengths the two norms can produce (each at most
    sqrt(head_dim) max|gamma + 1| + |beta|, which a rotary embedding preserves): Cauchy-Schwarz, in exp2-exponent
    units, plus 1 % for the roundings to bf16."""
    scale = head_dim ** -0.5 if softmax_scale is None else softmax_scale
    return 1.01 * scale * math.log2(math.e) * q_norm_bound * k_norm_bound


def _measuring_a_bound_pays(q, k, n_ranges: int, max_seqlen_q: int, max_seqlen_k: int) -> bool:
    """A bf16 call without a score_bound: are the two passes of MAGI_ATTN_AUTO_BOUND (one over q, one over k) small
    beside what the bounded-score kernel saves?  Decided from sizes the host knows, generously on the side of the
    plain online-softmax launch: the saving is put at 12 % of the attention time, the passes at twice their HBM time
    plus three launches."""
    if q.dtype != torch.bfloat16 or q.dim() != 3 or q.shape[-1] != 128:
        return False
    Tq, Hq, D = q.shape
    keys = max_seqlen_k if max_seqlen_k > 0 else k.shape[0]
    attention_s = 4.0 * D * Hq * min(Tq, max(n_ranges, 0) * max_seqlen_q) * keys / 1.2e15
    passes_s = (Tq * Hq + k.shape[0] * k.shape[1]) * 2 * D / 4e12 + 3e-5
    return 0.12 * attention_s > 2 * passes_s


def flex_flash_attn_func(q, k, v, q_ranges, k_ranges, max_seqlen_q, max_seqlen_k, softmax_scale=None,
                         deterministic=False, disable_fwd_atomic_reduction=True, score_bound: float = 0.0,
                         auto_bound: Optional[bool] = None, **_unused):
    """(out [Tq,Hq,D], lse [Hq,Tq]) for disjoint q ranges.  The forward has one writer per output
    row, so it is deterministic and needs no atomic reduction whatever the two flags say.

    score_bound (no counterpart in the reference's call, optional): the caller's promise that
    |q . k| * softmax_scale * log2(e) <= score_bound for every pair, with q unscaled as the reference passes it
    (qk_norm_score_bound derives it from the norm parameters).  Up to MAGI_SCORE_BOUND_MAX it selects the kernel
    without a running maximum, which applies the scale while it loads q.

    auto_bound: without a score_bound the library can measure one (range_attention's auto_bound).  None (default):
    it does where the two passes over q and k are small beside the attention itself, which is how the reference's
    own call, unchanged, reaches the bounded-score kernel on its QK-normed q and k."""
    if auto_bound is None:
        auto_bound = score_bound == 0.0 and _measuring_a_bound_pays(q, k, q_ranges.shape[0], max_seqlen_q, max_seqlen_k)
    return range_attention(q, k, v, q_ranges, k_ranges, max_seqlen_q, max_seqlen_k, softmax_scale,
                           score_bound=score_bound, auto_bound=bool(auto_bound) and score_bound == 0.0)


def flash_attn_func(q, k, v, dropout_p=0.0, softmax_scale=None, causal=False, deterministic=False,
                    score_bound: float = 0.0, auto_bound: Optional[bool] = None, **_unused):
    """q [B,Sq,Hq,D], k/v [B,Sk,Hkv,D] -> [B,Sq,Hq,D]; non-causal, no dropout (what the reference uses).
    score_bound, auto_bound: as in flex_flash_attn_func."""
    if dropout_p != 0.0 or causal:
        raise NotImplementedError("dropout / causal are not part of the MAGI-1 attention path")
    B, Sq, Hq, D = q.shape
    Sk = k.shape[1]
    q3 = q.reshape(B * Sq, Hq, D)
    k3 = k.reshape(B * Sk, k.shape[2], D)
    v3 = v.reshape(B * Sk, v.shape[2], D)
    cu_q = torch.arange(0, (B + 1) * Sq, Sq, dtype=torch.int32, device=q.device)
    cu_k = torch.arange(0, (B + 1) * Sk, Sk, dtype=torch.int32, device=q.device)
    if auto_bound is None:
        auto_bound = score_bound == 0.0 and _measuring_a_bound_pays(q3, k3, B, Sq, Sk)
    out, _ = range_attention(q3, k3, v3, cu_q, cu_k, Sq, Sk, softmax_scale, ranges_mode=L.MAGI_RANGES_CU,
                             return_lse=False, zero_init=False, score_bound=score_bound,
                             auto_bound=bool(auto_bound) and score_bound == 0.0)
    return out.view(B, Sq, Hq, D)


def flash_attn_varlen_func(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, dropout_p=0.0,
                           softmax_scale=None, causal=False, deterministic=False, score_bound: float = 0.0,
                           auto_bound: Optional[bool] = None, **_unused):
    """Packed varlen attention; segment s pairs q[cu_q[s]:cu_q[s+1]] with k[cu_k[s]:cu_k[s+1]].
    A segment without keys yields zero rows.  score_bound, auto_bound: as in flex_flash_attn_func."""
    if dropout_p != 0.0 or causal:
        raise NotImplementedError("dropout / causal are not part of the MAGI-1 attention path")
    if auto_bound is None:
        auto_bound = score_bound == 0.0 and _measuring_a_bound_pays(q, k, cu_seqlens_q.numel() - 1, max_seqlen_q, max_seqlen_k)
    out, _ = range_attention(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, softmax_scale,
                             ranges_mode=L.MAGI_RANGES_CU, return_lse=False, zero_init=True, score_bound=score_bound,
                             auto_bound=bool(auto_bound) and score_bound == 0.0)
    return out


def apply_rotary_emb(x, cos, sin, interleaved=False, inplace=False, **_unused):
    """x [B,S,H,D] (fp32 or bf16), cos / sin [S, R/2]: rotate the first R features, non-interleaved."""
    if interleaved:
        raise NotImplementedError("the DiT path uses the non-interleaved convention only")
    if x.dim() != 4:
        raise ValueError("x must be [batch, seqlen, heads, head_dim]")
    if x.dtype not in (torch.float32, torch.bfloat16):
        raise TypeError("x must be fp32 or bf16")
    B, S, H, D = x.shape
    R2 = cos.shape[-1]
    if cos.shape != (S, R2) or sin.shape != (S, R2):
        raise ValueError("cos / sin must be [seqlen, rotary_dim / 2]")
    if inplace and not x.is_contiguous():
        raise ValueError("inplace=True needs a contiguous x (a copy would be rotated instead of x)")
    xc = x.contiguous()
    y = xc if inplace else torch.empty_like(xc)
    cosf = cos.to(torch.float32).contiguous()
    sinf = sin.to(torch.float32).contiguous()
    with torch.cuda.device(x.device):
        L.check(L.lib().magi_apply_rotary(xc.data_ptr(), cosf.data_ptr(), sinf.data_ptr(), y.data_ptr(), B, S, H, D, R2,
                                          int(x.dtype == torch.bfloat16), _stream()))
    return y


def qk_prologue(q_raw, k_raw, v_raw, rope, gq, bq, gk, bk, *, Hq: int, Hkv: int, eps: float = 1e-6,
                norm_kind: int = L.MAGI_NORM_LAYERNORM_1P, kv_out: Optional[torch.Tensor] = None,
                n_cache_rows: Optional[int] = None, kv_tail: Optional[torch.Tensor] = None,
                q_out: Optional[torch.Tensor] = None, batch: int = 1, q_premul: float = 1.0):
    """Fused norm + rotary + cast + KV write.  q_raw [S, Hq*D], k_raw / v_raw [S, Hkv*D] bf16 (row
    strided views allowed); rope [S, 2*R2] fp32 (sin | cos) or None.

    q_premul multiplies q after norm and rotary, before the one rounding to bf16 (softmax_scale * log2(e) for
    range_attention(..., q_prescaled=True)).

    kv_out is the destination of the first n_cache_rows tokens (a view of the cache starting
    at the write position, [>= n_cache_rows, Hkv, 2D]); kv_tail takes the rest.  With neither,
    a fresh [S, Hkv, 2D] tensor is written.  Returns (q [S,Hq,D], kv_out, kv_tail)."""
    S = q_raw.shape[0]
    D = 128
    dev = q_raw.device
    if q_out is None:
        q_out = torch.empty((S, Hq, D), dtype=torch.bfloat16, device=dev)
    if kv_out is None and kv_tail is None:
        kv_out = torch.empty((S, Hkv, 2 * D), dtype=torch.bfloat16, device=dev)
        n_cache_rows = S
    if n_cache_rows is None:
        n_cache_rows = S if kv_tail is None else 0
    for name, t in (("q_raw", q_raw), ("k_raw", k_raw), ("v_raw", v_raw)):
        if t.dtype != torch.bfloat16 or t.stride(-1) != 1 or t.dim() != 2:
            raise ValueError(f"{name} must be a 2-D bf16 tensor with contiguous rows")
    for name, t in (("kv_out", kv_out), ("kv_tail", kv_tail)):
        if t is not None and (t.dtype != torch.bfloat16 or t.dim() != 3 or t.shape[1:] != (Hkv, 2 * D)
                              or t.stride(2) != 1 or t.stride(1) != 2 * D):
            raise ValueError(f"{name} must be bf16 [rows, Hkv, 2*D] with contiguous heads")
    if kv_out is not None and kv_out.shape[0] < n_cache_rows:
        raise ValueError("kv_out is shorter than n_cache_rows")
    if kv_tail is not None and kv_tail.shape[0] < S - n_cache_rows:
        raise ValueError("kv_tail is shorter than S - n_cache_rows")
    f32 = lambda t: None if t is None else t.to(torch.float32).contiguous()
    gq, bq, gk, bk = f32(gq), f32(bq), f32(gk), f32(bk)
    a = L.PrologueArgs()
    R2 = 0
    if rope is not None:
        if rope.dtype != torch.float32 or rope.dim() != 2 or rope.shape[0] * max(batch, 1) != S or not rope.is_contiguous():
            raise ValueError("rope must be a contiguous fp32 [S / batch, 2*R2] tensor")
        R2 = rope.shape[1] // 2
    a.q_raw, a.k_raw, a.v_raw, a.rope = _ptr(q_raw), _ptr(k_raw), _ptr(v_raw), _ptr(rope)
    a.gq, a.bq, a.gk, a.bk = _ptr(gq), _ptr(bq), _ptr(gk), _ptr(bk)
    a.q_out, a.kv_out, a.kv_tail = _ptr(q_out), _ptr(kv_out), _ptr(kv_tail)
    a.q_raw_stride_t, a.k_raw_stride_t, a.v_raw_stride_t = q_raw.stride(0), k_raw.stride(0), v_raw.stride(0)
    a.kv_stride_t = 0 if kv_out is None else kv_out.stride(0)
    a.kv_tail_stride_t = 0 if kv_tail is None else kv_tail.stride(0)
    a.S, a.n_cache_rows = S, int(n_cache_rows)
    a.Hq, a.Hkv, a.D, a.R2 = Hq, Hkv, D, R2
    a.norm_kind, a.eps, a.batch = int(norm_kind), float(eps), int(batch)
    a.q_premul = float(q_premul)
    with torch.cuda.device(dev):
        L.check(L.lib().magi_qk_prologue(C.byref(a), _stream()))
    return q_out, kv_out, kv_tail


def qk_prologue_fp8(q_raw, k_raw, rope, gq, bq, gk, bk, *, Hq: int, Hkv: int, q_scale: float, k_scale: float,
                    eps: float = 1e-6, norm_kind: int = L.MAGI_NORM_LAYERNORM_1P, k_out: Optional[torch.Tensor] = None,
                    n_cache_rows: Optional[int] = None, k_tail: Optional[torch.Tensor] = None,
                    q_out: Optional[torch.Tensor] = None, batch: int = 1, q_premul: float = 1.0):
    """qk_prologue with e4m3 outputs (magi_prologue_args.out_dtype): q [S, Hq, D] = sat_e4m3(q * q_premul / q_scale)
    and K rows [*, Hkv, D] = sat_e4m3(k / k_scale) straight from the norm + rotary pass, with the two constant
    scales of the call (powers of two; see pow2_scale_for).  k_out takes the first n_cache_rows tokens (a view of
    an fp8 cache's K rows at the write position), k_tail the rest; with neither a fresh [S, Hkv, D] tensor.
    V is not part of this pass (quantize_fp8_split takes it from the raw projection).
    Returns (q8, k_out, k_tail)."""
    S = q_raw.shape[0]
    D = 128
    dev = q_raw.device
    f8 = torch.float8_e4m3fn
    if q_out is None:
        q_out = torch.empty((S, Hq, D), dtype=f8, device=dev)
    if q_out.dtype != f8 or tuple(q_out.shape) != (S, Hq, D) or not q_out.is_contiguous():
        raise ValueError("q_out must be a contiguous float8_e4m3fn [S, Hq, 128] tensor")
    if k_out is None and k_tail is None:
        k_out = torch.empty((S, Hkv, D), dtype=f8, device=dev)
        n_cache_rows = S
    if n_cache_rows is None:
        n_cache_rows = S if k_tail is None else 0
    for name, t in (("q_raw", q_raw), ("k_raw", k_raw)):
        if t.dtype != torch.bfloat16 or t.stride(-1) != 1 or t.dim() != 2:
            raise ValueError(f"{name} must be a 2-D bf16 tensor with contiguous rows")
    for name, t in (("k_out", k_out), ("k_tail", k_tail)):
        if t is not None and (t.dtype != f8 or t.dim() != 3 or t.shape[1:] != (Hkv, D) or t.stride(2) != 1
                              or t.stride(1) != D):
            raise ValueError(f"{name} must be float8_e4m3fn [rows, Hkv, D] with contiguous heads")
    if k_out is not None and k_out.shape[0] < n_cache_rows:
        raise ValueError("k_out is shorter than n_cache_rows")
    if k_tail is not None and k_tail.shape[0] < S - n_cache_rows:
        raise ValueError("k_tail is shorter than S - n_cache_rows")
    f32 = lambda t: None if t is None else t.to(torch.float32).contiguous()
    gq, bq, gk, bk = f32(gq), f32(bq), f32(gk), f32(bk)
    a = L.PrologueArgs()
    R2 = 0
    if rope is not None:
        if rope.dtype != torch.float32 or rope.dim() != 2 or rope.shape[0] * max(batch, 1) != S or not rope.is_contiguous():
            raise ValueError("rope must be a contiguous fp32 [S / batch, 2*R2] tensor")
        R2 = rope.shape[1] // 2
    a.q_raw, a.k_raw, a.v_raw, a.rope = _ptr(q_raw), _ptr(k_raw), None, _ptr(rope)
    a.gq, a.bq, a.gk, a.bk = _ptr(gq), _ptr(bq), _ptr(gk), _ptr(bk)
    a.q_out, a.kv_out, a.kv_tail = _ptr(q_out), _ptr(k_out), _ptr(k_tail)
    a.q_raw_stride_t, a.k_raw_stride_t = q_raw.stride(0), k_raw.stride(0)
    a.kv_stride_t = 0 if k_out is None else k_out.stride(0)
    a.kv_tail_stride_t = 0 if k_tail is None else k_tail.stride(0)
    a.S, a.n_cache_rows = S, int(n_cache_rows)
    a.Hq, a.Hkv, a.D, a.R2 = Hq, Hkv, D, R2
    a.norm_kind, a.eps, a.batch = int(norm_kind), float(eps), int(batch)
    a.q_premul = float(q_premul)
    a.out_dtype = L.MAGI_DTYPE_FP8_E4M3
    a.q_quant_scale, a.k_quant_scale = float(q_scale), float(k_scale)
    with torch.cuda.device(dev):
        L.check(L.lib().magi_qk_prologue(C.byref(a), _stream()))
    return q_out, k_out, k_tail


def qkv_proj_prologue(x: torch.Tensor, w: torch.Tensor, rope, gq, bq, gk, bk, *, Hq: int, Hkv: int, Hqx: int = 0,
                      eps: float = 1e-6, norm_kind: int = L.MAGI_NORM_LAYERNORM_1P, kv_out: Optional[torch.Tensor] = None,
                      n_cache_rows: Optional[int] = None, kv_tail: Optional[torch.Tensor] = None,
                      q_out: Optional[torch.Tensor] = None, qx_out: Optional[torch.Tensor] = None, batch: int = 1,
                      q_premul: float = 1.0):
    """The four projections and the prologue in one launch (magi_qkv_proj_prologue): x [S, K] bf16 (the normalised
    hidden states), w [(Hq + 2 Hkv + Hqx) * 128, K] bf16 with rows ordered q | k | v | qx heads.  Destinations as in
    qk_prologue; qx_out [S, Hqx, 128] receives the cross-attention q projection unnormalised.
    Returns (q [S, Hq, 128], kv_out, kv_tail, qx_out)."""
    D = 128
    if x.dim() != 2 or w.dim() != 2 or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise ValueError("x and w must be 2-D bf16 tensors")
    if x.stride(1) != 1 or w.stride(1) != 1 or x.shape[1] != w.shape[1] or w.shape[0] != (Hq + 2 * Hkv + Hqx) * D:
        raise ValueError("x [S, K] and w [(Hq + 2 Hkv + Hqx) * 128, K] must have contiguous rows of the same length")
    if not x.is_cuda or w.device != x.device:
        raise ValueError("x and w must live on the same device (there is no CPU path)")
    S, K = x.shape
    dev = x.device
    if q_out is None:
        q_out = torch.empty((S, Hq, D), dtype=torch.bfloat16, device=dev)
    if qx_out is None and Hqx:
        qx_out = torch.empty((S, Hqx, D), dtype=torch.bfloat16, device=dev)
    if kv_out is None and kv_tail is None:
        kv_out = torch.empty((S, Hkv, 2 * D), dtype=torch.bfloat16, device=dev)
        n_cache_rows = S
    if n_cache_rows is None:
        n_cache_rows = S if kv_tail is None else 0
    for name, t, H in (("q_out", q_out, Hq), ("qx_out", qx_out, Hqx)):
        if t is not None and (t.dtype != torch.bfloat16 or tuple(t.shape) != (S, H, D) or not t.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous bf16 [S, heads, 128] tensor")
    for name, t in (("kv_out", kv_out), ("kv_tail", kv_tail)):
        if t is not None and (t.dtype != torch.bfloat16 or t.dim() != 3 or t.shape[1:] != (Hkv, 2 * D)
                              or t.stride(2) != 1 or t.stride(1) != 2 * D):
            raise ValueError(f"{name} must be bf16 [rows, Hkv, 2*D] with contiguous heads")
    if kv_out is not None and kv_out.shape[0] < n_cache_rows:
        raise ValueError("kv_out is shorter than n_cache_rows")
    if kv_tail is not None and kv_tail.shape[0] < S - n_cache_rows:
        raise ValueError("kv_tail is shorter than S - n_cache_rows")
    f32 = lambda t: None if t is None else t.to(torch.float32).contiguous()
    gq, bq, gk, bk = f32(gq), f32(bq), f32(gk), f32(bk)
    a = L.QkvProjArgs()
    R2 = 0
    if rope is not None:
        if rope.dtype != torch.float32 or rope.dim() != 2 or rope.shape[0] * max(batch, 1) != S or not rope.is_contiguous():
            raise ValueError("rope must be a contiguous fp32 [S / batch, 2*R2] tensor")
        R2 = rope.shape[1] // 2
    a.x, a.w, a.x_stride, a.w_stride = _ptr(x), _ptr(w), x.stride(0), w.stride(0)
    a.S, a.K = S, K
    a.Hq, a.Hkv, a.Hqx, a.D = Hq, Hkv, Hqx, D
    a.rope, a.R2 = _ptr(rope), R2
    a.gq, a.bq, a.gk, a.bk = _ptr(gq), _ptr(bq), _ptr(gk), _ptr(bk)
    a.norm_kind, a.eps, a.batch, a.q_premul = int(norm_kind), float(eps), int(batch), float(q_premul)
    a.q_out, a.kv_out, a.kv_tail, a.qx_out = _ptr(q_out), _ptr(kv_out), _ptr(kv_tail), _ptr(qx_out)
    a.kv_stride_t = 0 if kv_out is None else kv_out.stride(0)
    a.kv_tail_stride_t = 0 if kv_tail is None else kv_tail.stride(0)
    a.n_cache_rows = int(n_cache_rows)
    with torch.cuda.device(dev):
        L.check(L.lib().magi_qkv_proj_prologue(C.byref(a), _stream()))
    return q_out, kv_out, kv_tail, qx_out


def pow2_scale_for(bound: float) -> float:
    """Smallest power of two s with bound / s <= 448 (the largest e4m3 value): the scale to quantise values of
    magnitude <= bound with.  e4m3 being a floating-point format, a bound that is a few times too large costs
    no precision."""
    if not (bound > 0.0) or bound == float("inf"):
        raise ValueError("bound must be positive and finite")
    m, e = math.frexp(bound / 448.0)  # bound / 448 = m * 2^e, 0.5 <= m < 1
    return math.ldexp(1.0, e - 1 if m == 0.5 else e)


def layer_norm(x: torch.Tensor, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor], eps: float = 1e-5,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """LayerNorm over the last axis of a bf16 tensor with fp32 statistics: the layer input norm of
    CustomLayerNormLinear.forward_ln (dit_module.py:401, 412-413).  weight / bias: bf16 or fp32 [cols] or None.
    Rows may be strided (last axis contiguous, leading axes collapsible to one row stride)."""
    if x.dtype != torch.bfloat16:
        raise TypeError("x must be bf16")
    if not x.is_cuda:
        raise ValueError("x must be a device tensor (there is no CPU path)")
    cols = x.shape[-1]
    x2 = x if x.dim() == 2 else x.reshape(-1, cols)  # a view when the leading axes collapse, else a copy
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    y = torch.empty(x.shape, dtype=torch.bfloat16, device=x.device) if out is None else out
    if y.shape != x.shape or y.dtype != torch.bfloat16 or y.device != x.device or not y.is_contiguous():
        raise ValueError("out must be a contiguous bf16 tensor of x's shape on x's device")
    fp32 = None
    for name, p in (("weight", weight), ("bias", bias)):
        if p is None:
            continue
        if p.shape != (cols,) or not p.is_contiguous() or p.device != x.device:
            raise ValueError(f"{name} must be a contiguous [{cols}] tensor on x's device")
        if p.dtype not in (torch.bfloat16, torch.float32):
            raise TypeError(f"{name} must be bf16 or fp32")
        if fp32 is not None and fp32 != (p.dtype == torch.float32):
            raise TypeError("weight and bias must share a dtype")
        fp32 = p.dtype == torch.float32
    rows = x2.shape[0]
    with torch.cuda.device(x.device):
        L.check(L.lib().magi_layer_norm(x2.data_ptr(), x2.stride(0) if rows > 1 else cols, _ptr(weight), _ptr(bias),
                                        int(bool(fp32)), y.data_ptr(), cols, rows, cols, float(eps), _stream()))
    return y


def div_clamp_to(x: torch.Tensor, scale: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """e4m3fn(bf16(clamp(x.float() / scale.float(), -448, 448))): the input quantiser of the reference's fp8 linears
    (dit_module.py:364-384), double rounding included.  x: bf16, last axis contiguous (leading axes collapsible to one
    row stride); scale: fp32 with one element or one per element of the last axis.  -> float8_e4m3fn, x's shape."""
    if x.dtype != torch.bfloat16:
        raise TypeError("x must be bf16")
    if not x.is_cuda:
        raise ValueError("x must be a device tensor (there is no CPU path)")
    cols = x.shape[-1]
    x2 = x if x.dim() == 2 else x.reshape(-1, cols)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    sc = scale.detach().to(device=x.device, dtype=torch.float32).reshape(-1).contiguous()
    if sc.numel() not in (1, cols):
        raise ValueError("scale must have one element, or one per element of x's last axis")
    y = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device) if out is None else out
    if y.shape != x.shape or y.dtype != torch.float8_e4m3fn or y.device != x.device or not y.is_contiguous():
        raise ValueError("out must be a contiguous float8_e4m3fn tensor of x's shape on x's device")
    rows = x2.shape[0]
    with torch.cuda.device(x.device):
        L.check(L.lib().magi_div_clamp_to_e4m3(x2.data_ptr(), x2.stride(0) if rows > 1 else cols, sc.data_ptr(), sc.numel(),
                                               y.data_ptr(), cols, rows, cols, _stream()))
    return y


def head_norm(x: torch.Tensor, gamma, beta, eps: float = 1e-6, norm_kind: int = L.MAGI_NORM_LAYERNORM_1P):
    """x [S, H, 128] bf16 (strided heads allowed) -> contiguous normalised copy."""
    _check_thd(x, "x")
    if x.dtype != torch.bfloat16:
        raise TypeError("x must be bf16")
    S, H, D = x.shape
    y = torch.empty((S, H, D), dtype=torch.bfloat16, device=x.device)
    g = None if gamma is None else gamma.to(torch.float32).contiguous()
    b = None if beta is None else beta.to(torch.float32).contiguous()
    with torch.cuda.device(x.device):
        L.check(L.lib().magi_head_norm(x.data_ptr(), x.stride(0), x.stride(1), _ptr(g), _ptr(b), y.data_ptr(), S, H, D,
                                       int(norm_kind), float(eps), _stream()))
    return y


def quantize_fp8(x: torch.Tensor, chunk_tokens: int, premul: float = 1.0, pow2_scales: bool = False,
                 out: Optional[torch.Tensor] = None, scales_out: Optional[torch.Tensor] = None):
    """x [T, H, 128] bf16 (strided heads allowed) -> (y [T, H, 128] float8_e4m3fn, scales [ceil(T/chunk), H] fp32)
    with x * premul ~= y * scales[t // chunk_tokens, h]: per-(chunk, head) absmax * |premul| / 448 (rounded up to a
    power of two with pow2_scales), saturating OCP e4m3fn.

    out / scales_out: contiguous destinations (e.g. the rows of an fp8 KV cache at the write position and the
    matching rows of its scale table) instead of fresh tensors.

    For the fast attention mode quantise q with premul = softmax_scale * log2(e) and q, k, v with pow2_scales,
    then pass fp8_pow2_prescaled=True to range_attention."""
    _check_thd(x, "x")
    if x.dtype != torch.bfloat16:
        raise TypeError("x must be bf16")
    T, H, D = x.shape
    n_chunks = (T + chunk_tokens - 1) // chunk_tokens
    y = torch.empty((T, H, D), dtype=torch.float8_e4m3fn, device=x.device) if out is None else out
    scales = torch.empty((n_chunks, H), dtype=torch.float32, device=x.device) if scales_out is None else scales_out
    if y.dtype != torch.float8_e4m3fn or tuple(y.shape) != (T, H, D) or not y.is_contiguous() or y.device != x.device:
        raise ValueError("out must be a contiguous float8_e4m3fn [T, H, 128] tensor on x's device")
    if (scales.dtype != torch.float32 or tuple(scales.shape) != (n_chunks, H) or not scales.is_contiguous()
            or scales.device != x.device):
        raise ValueError("scales_out must be a contiguous fp32 [ceil(T / chunk_tokens), H] tensor on x's device")
    with torch.cuda.device(x.device):
        L.check(L.lib().magi_quantize_fp8(x.data_ptr(), x.stride(0), x.stride(1), y.data_ptr(), scales.data_ptr(), T, H, D,
                                          int(chunk_tokens), float(premul), int(pow2_scales), _stream()))
    return y, scales


def quantize_fp8_split(x: torch.Tensor, chunk_tokens: int, n_rows_first: int, out: Optional[torch.Tensor],
                       scales_out: Optional[torch.Tensor], out2: Optional[torch.Tensor],
                       scales2_out: Optional[torch.Tensor], premul: float = 1.0, pow2_scales: bool = False) -> None:
    """quantize_fp8 in ONE launch with two destinations (magi_quantize_fp8_split): tokens below n_rows_first (a
    multiple of chunk_tokens unless it is T) go to out / scales_out, e.g. the rows of an fp8 KV cache at the write
    position and the matching rows of its scale table; the others to out2 / scales2_out, indexed from
    n_rows_first.  Destinations are contiguous and at least as long as their share; a share of zero rows may
    pass None."""
    _check_thd(x, "x")
    if x.dtype != torch.bfloat16:
        raise TypeError("x must be bf16")
    T, H, D = x.shape
    n1 = int(n_rows_first)
    if not (0 <= n1 <= T) or (n1 < T and n1 % chunk_tokens):
        raise ValueError("n_rows_first must lie in [0, T] and, below T, be a multiple of chunk_tokens")
    for name, y, sc, rows in (("out", out, scales_out, n1), ("out2", out2, scales2_out, T - n1)):
        if rows == 0:
            continue
        chunks = (rows + chunk_tokens - 1) // chunk_tokens
        if (y is None or y.dtype != torch.float8_e4m3fn or y.dim() != 3 or y.shape[0] < rows or tuple(y.shape[1:]) != (H, D)
                or not y.is_contiguous() or y.device != x.device):
            raise ValueError(f"{name} must be a contiguous float8_e4m3fn [>= {rows}, H, 128] tensor on x's device")
        if (sc is None or sc.dtype != torch.float32 or sc.dim() != 2 or sc.shape[0] < chunks or sc.shape[1] != H
                or not sc.is_contiguous() or sc.device != x.device):
            raise ValueError(f"the scales of {name} must be a contiguous fp32 [>= {chunks}, H] tensor on x's device")
    a = L.QuantizeArgs()
    a.x, a.x_stride_t, a.x_stride_h = _ptr(x), x.stride(0), x.stride(1)
    a.T, a.H, a.D, a.chunk_tokens = T, H, D, int(chunk_tokens)
    a.premul, a.pow2_scales = float(premul), int(pow2_scales)
    a.y, a.scales, a.n_rows_first = _ptr(out), _ptr(scales_out), n1
    a.y2, a.scales2 = _ptr(out2), _ptr(scales2_out)
    with torch.cuda.device(x.device):
        L.check(L.lib().magi_quantize_fp8_split(C.byref(a), _stream()))
