"""CPU oracle for the MAGI-1 DiT attention hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU with plain torch / numpy, the arithmetic the
reference performs on its attention path.  Nothing here is part of the product:
only tests, the smoke check and the benchmark's CPU-baseline leg may import it.
The product path (HIP kernels behind the C-ABI library) never routes through it.

Every function cites the reference lines it follows (paths relative to the
reference checkout).  The arithmetic of the attention kernels themselves lives in
third-party packages absent from the reference tree (flash-attn 2.4.2,
MagiAttention); for those the published algorithm (softmax(QK^T/sqrt(d))V with the
GQA head mapping h_kv = h_q // (Hq/Hkv), non-interleaved rotary) is restated and
anchored on the reference's call sites.

Pin status (what besides "same formula" checks each function; see tests/test_oracle.py):
  freq_bands, rope_table            closed-form spot values, axis-separability, symmetry,
                                    identity rescale for H*W == 256, slice == offset-table
  qk_layernorm / rmsnorm            torch.nn.functional.layer_norm with weight+1; fp64 brute force
  input_layer_norm                  torch.nn.LayerNorm module (CPU, fp32), shift / scale invariances
  apply_rope_neox_partial           transformers' rotate_half convention, pair-norm invariance,
                                    pass-through dims, relative-position property
  range_attention                   fp64 brute force, block-mask SDPA, V=1 => O=1, permutation
                                    invariance, range independence, GQA == repeat_interleave MHA
  varlen_cross_attention            per-segment brute force, empty segment => zeros
  kv cache model                    list-of-chunks model, randomised state-machine sequences
  generate_sequences                the four worked examples the reference keeps in comments
  kv-range generators               hand-derived expected tables
  fp8 quantiser / fp8 attention     PARITY UNPINNED by the reference (it has no fp8 attention);
                                    pinned by quantiser properties and the fp32 oracle + tolerance
  prologue(q_premul != 1)           no counterpart in the reference (1.0 reproduces it); pinned end to end: the
                                    pre-scaled q through attention with softmax_scale = ln 2 must equal the
                                    unscaled prologue + default-scale attention (tests/test_oracle.py)
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn.functional as F

FP8_MAX = 448.0  # torch.finfo(torch.float8_e4m3fn).max


# --------------------------------------------------------------------------------------
# A1: rotary table  (inference/model/dit/dit_module.py:591-596, 599-667, 670-717, 757-770;
#                    inference/model/dit/dit_model.py:163-166)
# --------------------------------------------------------------------------------------
def freq_bands(num_bands: int = 16, temperature: float = 10000.0, step: int = 1) -> torch.Tensor:
    """bands_j = temperature ** -(j / num_bands), j = 0, step, ...  (dit_module.py:591-596)."""
    exp = torch.arange(0, num_bands, step, dtype=torch.int64).to(torch.float32) / num_bands
    return 1.0 / (temperature**exp)


def rope_table(
    T_total: int,
    H: int,
    W: int,
    bands: Optional[torch.Tensor] = None,
    ref_feat_shape: Optional[Sequence[float]] = None,
) -> torch.Tensor:
    """[T_total*H*W, 96] fp32 = [sin(48) | cos(48)], band order [t(16) | h(16) | w(16)].

    Follows build_fourier_pos_embed with in_pixels=False (dit_module.py:643-667): integer
    positions on t, centred positions on h and w (:644-647), per-axis rescale
    x / (f - 1) * (r - 1) when a reference shape is given (:648-659), grid * bands, sin and
    cos, then reshape to [S, 48] each (:715-716) and cat sin first (:770).
    """
    if bands is None:
        bands = freq_bands(16)
    feat = [T_total, H, W]
    t = [torch.arange(s, dtype=torch.int64).to(torch.float32) for s in feat]
    t[1] = t[1] - (feat[1] - 1) / 2
    t[2] = t[2] - (feat[2] - 1) / 2
    if ref_feat_shape is not None:
        resc = []
        for x, f, r in zip(t, feat, ref_feat_shape):
            if f == 1:
                assert r == 1
                resc.append(x)
            else:
                resc.append(x / (f - 1) * (r - 1))
        t = resc
    grid = torch.stack(torch.meshgrid(*t, indexing="ij"), dim=-1).unsqueeze(-1)  # [T,H,W,3,1]
    pos = grid * bands  # [T,H,W,3,nb]
    S = T_total * H * W
    sin = pos.sin().reshape(S, -1)
    cos = pos.cos().reshape(S, -1)
    return torch.cat([sin, cos], dim=-1)


def rope_for_forward(T: int, H: int, W: int, slice_point: int, denoising_range_num: int,
                     bands: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The table slice one forward uses (dit_model.py:151-166): the table is built for the
    cached prefix frames plus the T new frames, rescaled with ref shape
    [T_total, H/s, W/s], s = sqrt(H*W/256), and the last T*H*W rows are kept."""
    frame_in_range = T // denoising_range_num
    T_total = T + frame_in_range * slice_point
    s = math.sqrt((H * W) / (16 * 16))
    full = rope_table(T_total, H, W, bands, ref_feat_shape=[T_total, H / s, W / s])
    return full[-(T * H * W):]


# --------------------------------------------------------------------------------------
# A2: QK norm  (dit_module.py:323-357, used :959, :976, :1008, :1020)
# --------------------------------------------------------------------------------------
def qk_layernorm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float = 1e-6,
                 zero_centered_gamma: bool = True) -> torch.Tensor:
    """LayerNorm over the last (head_dim) axis with gamma stored zero-centred (:356-357)."""
    w = weight + 1 if zero_centered_gamma else weight
    return F.layer_norm(x, (x.shape[-1],), w, bias, eps)


def input_layer_norm(x: torch.Tensor, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor],
                     eps: float = 1e-5) -> torch.Tensor:
    """LayerNorm of the layer input over the hidden axis (torch.nn.LayerNorm in CustomLayerNormLinear,
    dit_module.py:401, applied at :412-413 / :1153): biased variance, plain (not zero-centred) weight.
    Evaluated in float64 from the definition; the caller rounds to the dtype under test."""
    xd = x.double()
    mu = xd.mean(-1, keepdim=True)
    var = ((xd - mu) ** 2).mean(-1, keepdim=True)
    y = (xd - mu) / torch.sqrt(var + eps)
    if weight is not None:
        y = y * weight.double()
    if bias is not None:
        y = y + bias.double()
    return y


def rmsnorm(x: torch.Tensor, weight: Optional[torch.Tensor] = None, eps: float = 1e-6) -> torch.Tensor:
    """Per-head RMSNorm: the variant the benchmark configuration words its inputs with.
    Not in the reference (which uses the LayerNorm above)."""
    y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


# --------------------------------------------------------------------------------------
# A3: partial non-interleaved rotary  (call sites dit_module.py:961, :978; the callee is
# flash-attn 2.4.2 flash_attn.layers.rotary.apply_rotary_emb with interleaved=False:
# rotary_dim = 2 * cos.shape[-1]; o1 = x1*cos - x2*sin; o2 = x1*sin + x2*cos on the two
# halves of the first rotary_dim features; the remaining features pass through.)
# --------------------------------------------------------------------------------------
def apply_rope_neox_partial(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [..., S, H, D]; cos, sin [S, R/2]."""
    r2 = cos.shape[-1]
    x1, x2, rest = x[..., :r2], x[..., r2:2 * r2], x[..., 2 * r2:]
    c = cos[:, None, :]
    s = sin[:, None, :]
    return torch.cat([x1 * c - x2 * s, x1 * s + x2 * c, rest], dim=-1)


# --------------------------------------------------------------------------------------
# A4: get_q / get_k / get_v / get_kv after the linear layers (dit_module.py:953-996)
# --------------------------------------------------------------------------------------
def prologue(q_raw: torch.Tensor, k_raw: torch.Tensor, v_raw: torch.Tensor, rope: torch.Tensor,
             gq: torch.Tensor, bq: torch.Tensor, gk: torch.Tensor, bk: torch.Tensor,
             eps: float = 1e-6, norm: str = "layernorm_1p", q_premul: float = 1.0,
             downcast: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    """q_raw [S, Hq, D], k_raw / v_raw [S, Hkv, D] in bf16 (the projections' outputs, batch 1).

    q_premul (no counterpart in the reference; 1.0 reproduces it): factor applied to q in fp32 ahead of the
    downcast, for kernels that want softmax_scale * log2(e) folded into q.

    Returns (q [S, Hq, D] bf16, kv [S, Hkv, 2D] bf16) as get_q (:953-963) and get_kv (:991-996)
    do: upcast to fp32, norm, rotary in fp32, downcast to the input dtype; V is only
    re-laid-out; kv = cat([k, v], -1).  sin is the first half of the table (:1147).

    downcast=False (no counterpart in the reference) stops ahead of the downcast and returns (q, k) in fp32: what
    a quantiser that reads the norm + rotary result without a bf16 intermediate sees.
    """
    sin, cos = rope.tensor_split(2, -1)

    def one(x, g, b, premul=1.0):
        xf = x.float()
        if norm == "layernorm_1p":
            xf = qk_layernorm(xf, g.float(), b.float(), eps, True)
        elif norm == "rmsnorm":
            xf = rmsnorm(xf, g.float() + 1, eps)
        else:
            raise ValueError(norm)
        xf = apply_rope_neox_partial(xf, cos.float(), sin.float())
        if premul != 1.0:
            xf = xf * premul
        return xf.to(x.dtype) if downcast else xf

    q = one(q_raw, gq, bq, q_premul)
    k = one(k_raw, gk, bk)
    if not downcast:
        return q, k
    return q, torch.cat([k, v_raw], dim=-1)


# --------------------------------------------------------------------------------------
# A5: KV cache  (dit_module.py:800-819, 891-946; inference/common/dataclass.py:62-71)
# --------------------------------------------------------------------------------------
class KVCacheModel:
    """One layer's cache as the reference keeps it: [max_seq * max_bs, Hkv, 2D]."""

    def __init__(self, max_sequence_length: int, Hkv: int, D: int, dtype=torch.bfloat16, max_batch_size: int = 1):
        self.mem = torch.zeros(max_sequence_length * max_batch_size, Hkv, 2 * D, dtype=dtype)
        self.max_batch_size = max_batch_size

    def adjust(self, kv: torch.Tensor, *, has_inference_params: bool, update_kv_cache: bool, slice_point: int,
               clip_token_nums: int, extract_prefix_video_feature: bool = False, fwd_extra_1st_chunk: bool = False,
               distill_nearly_clean_chunk: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
        """adjust_key_and_value_for_inference (:933-946) + _full_adjust_key_and_value (:891-931)."""
        if not has_inference_params:
            k, v = torch.chunk(kv, 2, dim=-1)
            return k, v
        if extract_prefix_video_feature or fwd_extra_1st_chunk or slice_point > 0:
            start = slice_point * clip_token_nums * self.max_batch_size
            prefix = self.mem[:start].clone()
            if update_kv_cache:
                clip = kv.size(0) - clip_token_nums * self.max_batch_size if distill_nearly_clean_chunk else kv.size(0)
                end = start + clip
                assert end <= self.mem.size(0)
                self.mem[start:end] = kv[:clip]
            kv = torch.cat([prefix, kv], dim=0)
        k, v = torch.chunk(kv, 2, dim=-1)
        return k.contiguous(), v.contiguous()


# --------------------------------------------------------------------------------------
# A6: core attention over (q_range, k_range) rectangles  (dit_module.py:1023-1066)
# --------------------------------------------------------------------------------------
def _sdpa_gqa(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: Optional[float]) -> torch.Tensor:
    """q [Tq,Hq,D], k/v [Tk,Hkv,D] -> [Tq,Hq,D]; q head h reads kv head h // (Hq/Hkv)."""
    Hq, Hkv = q.shape[1], k.shape[1]
    g = Hq // Hkv
    kk = k.repeat_interleave(g, dim=1) if g > 1 else k
    vv = v.repeat_interleave(g, dim=1) if g > 1 else v
    o = F.scaled_dot_product_attention(q.transpose(0, 1)[None], kk.transpose(0, 1)[None], vv.transpose(0, 1)[None],
                                       scale=scale)
    return o[0].transpose(0, 1)


def range_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_ranges, k_ranges,
                    softmax_scale: Optional[float] = None, dtype=torch.float32) -> torch.Tensor:
    """For each i: O[q_ranges[i]] = softmax(Q K^T * scale) V over K[k_ranges[i]], no mask inside
    the rectangle, scale = D**-0.5 by default.  Same loop as dit_module.py:1052-1065 (one
    flash_attn_func call per range).  Rows no range covers stay 0; an empty k range gives 0."""
    q_ranges = np.asarray(q_ranges).reshape(-1, 2)
    k_ranges = np.asarray(k_ranges).reshape(-1, 2)
    out = torch.zeros(q.shape, dtype=dtype)
    qf, kf, vf = q.to(dtype), k.to(dtype), v.to(dtype)
    for (qs, qe), (ks, ke) in zip(q_ranges, k_ranges):
        if qe <= qs or ke <= ks:
            continue
        out[qs:qe] = _sdpa_gqa(qf[qs:qe], kf[ks:ke], vf[ks:ke], softmax_scale)
    return out


def range_attention_lse(q, k, v, q_ranges, k_ranges, softmax_scale=None) -> torch.Tensor:
    """log-sum-exp of the scaled scores per (head, q row): [Hq, Tq] fp32 (-inf where no keys)."""
    q_ranges = np.asarray(q_ranges).reshape(-1, 2)
    k_ranges = np.asarray(k_ranges).reshape(-1, 2)
    Tq, Hq, D = q.shape
    g = Hq // k.shape[1]
    scale = D ** -0.5 if softmax_scale is None else softmax_scale
    lse = torch.full((Hq, Tq), float("-inf"), dtype=torch.float32)
    for (qs, qe), (ks, ke) in zip(q_ranges, k_ranges):
        if qe <= qs or ke <= ks:
            continue
        kk = k[ks:ke].float().repeat_interleave(g, dim=1)
        s = torch.einsum("qhd,khd->hqk", q[qs:qe].float(), kk) * scale
        lse[:, qs:qe] = torch.logsumexp(s, dim=-1)
    return lse


def brute_attention_fp64(q, k, v, q_ranges, k_ranges, softmax_scale=None) -> torch.Tensor:
    """Definition-level fp64 evaluation (explicit exp / sum), for small shapes only."""
    q_ranges = np.asarray(q_ranges).reshape(-1, 2)
    k_ranges = np.asarray(k_ranges).reshape(-1, 2)
    Tq, Hq, D = q.shape
    g = Hq // k.shape[1]
    scale = D ** -0.5 if softmax_scale is None else softmax_scale
    out = torch.zeros(Tq, Hq, v.shape[-1], dtype=torch.float64)
    qd, kd, vd = q.double(), k.double(), v.double()
    for (qs, qe), (ks, ke) in zip(q_ranges, k_ranges):
        if qe <= qs or ke <= ks:
            continue
        for h in range(Hq):
            s = qd[qs:qe, h] @ kd[ks:ke, h // g].T * scale
            p = torch.exp(s - s.max(dim=-1, keepdim=True).values)
            out[qs:qe, h] = (p / p.sum(-1, keepdim=True)) @ vd[ks:ke, h // g]
    return out


def block_mask_attention(q, k, v, q_ranges, k_ranges, softmax_scale=None) -> torch.Tensor:
    """Single SDPA call with a boolean mask built from the rectangles (the benchmark
    configuration's wording of the same semantics)."""
    q_ranges = np.asarray(q_ranges).reshape(-1, 2)
    k_ranges = np.asarray(k_ranges).reshape(-1, 2)
    Tq, Hq, _ = q.shape
    Tk = k.shape[0]
    g = Hq // k.shape[1]
    mask = torch.zeros(Tq, Tk, dtype=torch.bool)
    for (qs, qe), (ks, ke) in zip(q_ranges, k_ranges):
        mask[qs:qe, ks:ke] = True
    kk = k.float().repeat_interleave(g, dim=1).transpose(0, 1)[None]
    vv = v.float().repeat_interleave(g, dim=1).transpose(0, 1)[None]
    o = F.scaled_dot_product_attention(q.float().transpose(0, 1)[None], kk, vv, attn_mask=mask, scale=softmax_scale)
    o = o[0].transpose(0, 1)
    live = mask.any(dim=1)
    return torch.where(live[:, None, None], o, torch.zeros_like(o))


# --------------------------------------------------------------------------------------
# A8: varlen cross attention  (dit_module.py:1098-1136; flash_attn_varlen_func semantics:
# segment s attends q[cu_q[s]:cu_q[s+1]] to k[cu_k[s]:cu_k[s+1]], non-causal; a segment
# with no keys yields zero rows)
# --------------------------------------------------------------------------------------
def varlen_cross_attention(q, k, v, cu_seqlens_q, cu_seqlens_k, softmax_scale=None, dtype=torch.float32) -> torch.Tensor:
    cq = np.asarray(cu_seqlens_q).astype(np.int64)
    ck = np.asarray(cu_seqlens_k).astype(np.int64)
    assert cq.shape == ck.shape
    qr = np.stack([cq[:-1], cq[1:]], 1)
    kr = np.stack([ck[:-1], ck[1:]], 1)
    return range_attention(q, k, v, qr, kr, softmax_scale, dtype)


def attn_linear_proj_input(core_attn_out: torch.Tensor, cross_attn_out: torch.Tensor, hn: int = 8) -> torch.Tensor:
    """Input of linear_proj as attn_linear_proj builds it (dit_module.py:1336-1339):
    cat([core, cross], dim=2) viewed "(n hn hd)" with n = 2 and re-ordered to "(hn n hd)".
    core / cross [sq, b, Hq*D] -> [sq, b, 2*Hq*D]."""
    sq, b, width = core_attn_out.shape
    cat = torch.cat([core_attn_out, cross_attn_out], dim=2)      # (n hn hd)
    return cat.view(sq, b, 2, hn, width // hn).permute(0, 1, 3, 2, 4).reshape(sq, b, 2 * width)


def cross_attn_params_from_mask(xattn_mask: torch.Tensor, clip_token_nums: int):
    """cu_seqlens / ranges as dit_model.py:213-241 builds them.  xattn_mask [n_seg, L] of 0/1."""
    y_index = xattn_mask.reshape(xattn_mask.shape[0], -1).sum(-1).to(torch.int64)
    n = xattn_mask.shape[0]
    cu_q = torch.tensor([0] + [clip_token_nums] * n, dtype=torch.int64).cumsum(-1).to(torch.int32)
    cu_k = torch.cat([y_index.new_zeros(1), y_index]).cumsum(-1).to(torch.int32)
    q_ranges = torch.stack([cu_q[:-1], cu_q[1:]], 1)
    k_ranges = torch.stack([cu_k[:-1], cu_k[1:]], 1)
    return cu_q, cu_k, q_ranges, k_ranges


# --------------------------------------------------------------------------------------
# A11: chunk-window arithmetic  (inference/pipeline/video_generate.py:164-180, 371-387,
# 454-508; inference/model/dit/dit_model.py:92-101)
# --------------------------------------------------------------------------------------
def generate_sequences(chunk_num: int, window_size: int, chunk_offset: int):
    """video_generate.py:164-180."""
    lo, hi = chunk_offset, chunk_num + window_size - 1
    clip_start = [max(chunk_offset, i - window_size + 1) for i in range(lo, hi)]
    clip_end = [min(chunk_num, i + 1) for i in range(lo, hi)]
    t_start = [max(0, i - chunk_num + 1) for i in range(lo, hi)]
    t_end = [min(window_size, i - chunk_offset + 1) if i - chunk_offset < window_size else window_size
             for i in range(lo, hi)]
    return clip_start, clip_end, t_start, t_end


def default_kvrange(slice_point: int, denoising_range_num: int, chunk_token_nums: int) -> np.ndarray:
    """video_generate.py:454-465, batch 1: chunk j sees [0, (slice_point + j + 1) * L)."""
    return np.array([[0, (slice_point + j + 1) * chunk_token_nums] for j in range(denoising_range_num)], dtype=np.int32)


def noise2clean_kvrange(slice_point: int, denoising_range_num: int, chunk_token_nums: int,
                        noise2clean: Sequence[int], clean_chunk_kvrange: int,
                        denoise_step_of_each_chunk: Sequence[int], num_steps: int) -> np.ndarray:
    """video_generate.py:467-508, batch 1."""
    assert len(denoise_step_of_each_chunk) == denoising_range_num and len(noise2clean) > 0
    if clean_chunk_kvrange == -1:
        clean_chunk_kvrange = noise2clean[-1]
    assert num_steps % len(noise2clean) == 0
    per_stage = num_steps // len(noise2clean)
    width = [clean_chunk_kvrange if s == num_steps else noise2clean[s // per_stage] for s in denoise_step_of_each_chunk]
    out = []
    for j in range(denoising_range_num):
        end = slice_point + j + 1
        out.append([max(0, end - width[j]) * chunk_token_nums, end * chunk_token_nums])
    return np.array(out, dtype=np.int32)


def prefix_video_kvrange(range_num: int, chunk_token_nums: int, clean_chunk_kvrange: int = -1,
                         noise2clean: Sequence[int] = ()) -> np.ndarray:
    """video_generate.py:371-387, batch 1."""
    if clean_chunk_kvrange != -1:
        prev = clean_chunk_kvrange
    elif len(noise2clean) > 0:
        prev = noise2clean[-1]
    else:
        prev = 8
    return np.array([[max(0, e - prev) * chunk_token_nums, e * chunk_token_nums] for e in range(1, range_num + 1)],
                    dtype=np.int32)


def uncondition_kvrange(B: int, chunk_token_nums: int) -> np.ndarray:
    """dit_model.py:92-101: in the unconditional pass chunks become batch rows, each sees itself."""
    return np.array([[i * chunk_token_nums, (i + 1) * chunk_token_nums] for i in range(B)], dtype=np.int32)


def q_ranges_for(denoising_range_num: int, chunk_token_nums: int) -> np.ndarray:
    """dit_model.py:220-222, 246: q_range[i] = [i*L, (i+1)*L)."""
    return np.array([[i * chunk_token_nums, (i + 1) * chunk_token_nums] for i in range(denoising_range_num)], dtype=np.int32)


def attention_flops(q_ranges, k_ranges, Hq: int, D: int) -> float:
    """4 * D * Hq * sum_i |q_i| * |k_i| (QK^T and PV, live rectangles only)."""
    qr = np.asarray(q_ranges, dtype=np.int64).reshape(-1, 2)
    kr = np.asarray(k_ranges, dtype=np.int64).reshape(-1, 2)
    return float(4 * D * Hq * int(((qr[:, 1] - qr[:, 0]).clip(0) * (kr[:, 1] - kr[:, 0]).clip(0)).sum()))


# --------------------------------------------------------------------------------------
# A9: fp8 e4m3 path.  The reference has no fp8 attention; its only fp8 convention is the
# linears' quantiser div_clamp_to (dit_module.py:364-384): clamp(x / scale, -448, 448),
# round to bf16, then to float8_e4m3fn.  PARITY UNPINNED by the reference.
# --------------------------------------------------------------------------------------
def quantize_e4m3(x: torch.Tensor, scale: torch.Tensor, via_bf16: bool = False) -> torch.Tensor:
    """Saturating OCP e4m3fn quantisation of x / scale, returned as float8_e4m3fn.
    via_bf16=True reproduces the reference linears' double rounding (:376-381)."""
    y = torch.clamp(x.float() / scale.float(), -FP8_MAX, FP8_MAX)
    if via_bf16:
        y = y.bfloat16()
    return y.to(torch.float8_e4m3fn)


def per_head_chunk_scales(x: torch.Tensor, chunk_token_nums: int, premul: float = 1.0, pow2: bool = False) -> torch.Tensor:
    """absmax over (chunk tokens, D) per head * |premul| / 448 -> [n_chunks, H] fp32 (>= tiny); with pow2 the
    scale is rounded up to the next power of two."""
    T, H, D = x.shape
    n = (T + chunk_token_nums - 1) // chunk_token_nums
    out = torch.empty(n, H, dtype=torch.float32)
    for c in range(n):
        blk = x[c * chunk_token_nums:(c + 1) * chunk_token_nums].float()
        out[c] = blk.abs().amax(dim=(0, 2)) * torch.tensor(abs(premul), dtype=torch.float32) / FP8_MAX
    out = out.clamp_min(1e-12)
    if pow2:
        out = torch.exp2(torch.ceil(torch.log2(out.double()))).float()
    return out


def quantize_per_head_chunk(x: torch.Tensor, chunk_token_nums: int, premul: float = 1.0, pow2: bool = False):
    """-> (x_fp8 [T,H,D] float8_e4m3fn, scales [n_chunks,H] fp32) with x * premul ~= x_fp8 * scale."""
    scales = per_head_chunk_scales(x, chunk_token_nums, premul, pow2)
    T = x.shape[0]
    idx = torch.arange(T) // chunk_token_nums
    s = scales[idx][:, :, None]
    return quantize_e4m3(x.float() * torch.tensor(premul, dtype=torch.float32), s), scales


def dequantize_per_head_chunk(x8: torch.Tensor, scales: torch.Tensor, chunk_token_nums: int) -> torch.Tensor:
    idx = torch.arange(x8.shape[0]) // chunk_token_nums
    return x8.float() * scales[idx][:, :, None]


def fp8_range_attention(q8, k8, v8, q_scales, k_scales, v_scales, chunk_token_nums, q_ranges, k_ranges,
                        softmax_scale=None, p_scale: float = 1.0) -> torch.Tensor:
    """fp32 model of the fp8 kernel: exact products of the e4m3 values with fp32 accumulation,
    fp32 softmax, P quantised to e4m3 (P / max in [0, 1], times p_scale) before P*V.
    This evaluates the *dequantised* attention, i.e. what an ideal fp8 kernel computes."""
    q = dequantize_per_head_chunk(q8, q_scales, chunk_token_nums)
    k = dequantize_per_head_chunk(k8, k_scales, chunk_token_nums)
    v = dequantize_per_head_chunk(v8, v_scales, chunk_token_nums)
    return range_attention(q, k, v, q_ranges, k_ranges, softmax_scale)


# --------------------------------------------------------------------------------------
# seeded synthetic inputs shared by tests and the benchmark's checker
# --------------------------------------------------------------------------------------
def synthetic_qkv(Tq: int, Tk: int, Hq: int, Hkv: int, D: int, seed: int, normed: bool = True, dtype=torch.bfloat16):
    """q [Tq,Hq,D], k/v [Tk,Hkv,D]; N(0,1), Q and K per-head RMS-normalised when normed."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(Tq, Hq, D, generator=g)
    k = torch.randn(Tk, Hkv, D, generator=g)
    v = torch.randn(Tk, Hkv, D, generator=g)
    if normed:
        q, k = rmsnorm(q), rmsnorm(k)
    return q.to(dtype), k.to(dtype), v.to(dtype)
