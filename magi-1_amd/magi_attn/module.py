"""The DiT attention layer over libmagi_attn, with the interface of the reference's
FullyParallelAttention for cp_strategy == "none"
(inference/model/dit/dit_module.py:776-1173).

Method names, argument meaning and returned layouts follow the reference so that
TransformerLayer-level code can call it unchanged:

  forward(hidden_states [S,b,h], key_value_states [Ty,h*ratio], inference_params,
          rotary_pos_emb [S,96], meta_args) -> (core_attn_out [S,b,Hq*D], xattn_out [S,b,Hq*D])

What differs is what happens underneath:
  * get_q / get_k / get_v / get_kv: the upcast, LayerNorm, transpose, rotary, downcast and
    re-layout passes are one fused kernel launch;
  * the KV cache is appended to in place by that same launch and READ in place by the
    attention kernel (strided K / V views of the interleaved cache), so the prefix slice,
    the cat and the contiguous copies of _full_adjust_key_and_value / core_attention vanish;
  * when the cache must not be updated (update_kv_cache False, or the last chunk under
    distill_nearly_clean_chunk) the new KV goes to a side buffer and the kernel walks
    [cache prefix | side buffer] as one key axis.

The linear projections and the input LayerNorm are plain library GEMMs / ops (torch on
rocBLAS / hipBLASLt); they are not part of this library.  forward() runs the four projections
q, k, v, qx as ONE GEMM over a shared weight buffer (CustomLayerNormLinear.forward_qkvx).
"""
from __future__ import annotations

from typing import Callable, Optional, Tuple

import torch

import math

from . import _lib as L
from .cache import Fp8KVCache, OffloadedKVCache
from .functional import _measuring_a_bound_pays
from .functional import (div_clamp_to, head_norm, layer_norm, pow2_scale_for, qk_prologue, qk_prologue_fp8, qkv_proj_prologue,
                         quantize_fp8_split,
                         range_attention)
from .params import InferenceParams, ModelMetaArgs, PackedCrossAttnParams


PROJ_GROUPS = 8  # head groups of the linear_proj input (hard-coded "hn=8", dit_module.py:1338)


def attn_linear_proj_input(core_attn_out: torch.Tensor, cross_attn_out: torch.Tensor) -> torch.Tensor:
    """[sq, b, Hq*D] x 2 -> [sq, b, 2*Hq*D] in "(hn n hd)" order: the concat + rearrange that precedes linear_proj
    in attn_linear_proj (dit_module.py:1336-1339), done with torch copies."""
    sq, b, hd = core_attn_out.shape
    both = torch.stack([core_attn_out.reshape(sq, b, PROJ_GROUPS, hd // PROJ_GROUPS),
                        cross_attn_out.reshape(sq, b, PROJ_GROUPS, hd // PROJ_GROUPS)], dim=3)
    return both.reshape(sq, b, 2 * hd)


class FusedLayerNorm(torch.nn.Module):
    """Parameter holder of a per-head LayerNorm with zero-centred gamma (dit_module.py:323-357).
    The arithmetic runs inside the fused kernels; forward() is the stand-alone form."""

    def __init__(self, hidden_size: int, eps: float = 1e-6, zero_centered_gamma: bool = True,
                 dtype=torch.bfloat16, device=None):
        super().__init__()
        self.eps = eps
        self.zero_centered_gamma = zero_centered_gamma
        self.weight = torch.nn.Parameter(torch.zeros(hidden_size, dtype=dtype, device=device))
        self.bias = torch.nn.Parameter(torch.zeros(hidden_size, dtype=dtype, device=device))

    def gamma_beta_fp32(self) -> Tuple[torch.Tensor, torch.Tensor]:
        """(gamma - 1 form, beta) as the kernels take them.  weight + 1 is formed in the parameter
        dtype first, as the reference does, so a bf16 parameter rounds the same way.  Converted once per set of
        parameter values (no launches on later calls) and kept until a parameter is modified or replaced."""
        # (a write through `.data` does not advance _version: callers that patch parameters that way call
        # invalidate_cached_parameters())
        key = tuple(x for t in (self.weight, self.bias) for x in (id(t), t._version, t.data_ptr(), t.dtype, t.device))
        if self.__dict__.get("_gb_key") != key:
            w = self.weight.detach()
            g = ((w + 1).float() - 1.0) if self.zero_centered_gamma else (w.float() - 1.0)
            self.__dict__["_gb"] = (g.contiguous(), self.bias.detach().float().contiguous())
            self.__dict__["_gb_key"] = key
            self.__dict__["_gb_epoch"] = self.__dict__.get("_gb_epoch", 0) + 1
        return self.__dict__["_gb"]

    def parameter_epoch(self) -> int:
        """A counter that advances whenever gamma_beta_fp32() had to convert the parameters anew: what values derived
        from the parameters (score bounds, quantisation scales) key their own caches on."""
        self.gamma_beta_fp32()
        return self.__dict__["_gb_epoch"]

    def invalidate_cached_parameters(self) -> None:
        self.__dict__.pop("_gb_key", None)

    def output_norm_bound(self) -> float:
        """Upper bound of the Euclidean norm of any output row: the normalised row has norm <= sqrt(n) (exactly
        sqrt(n) up to eps), so |y| <= sqrt(n) max|gamma + 1| + |beta|.  One host read of the parameters."""
        g, b = self.gamma_beta_fp32()
        n = g.numel()
        return float(math.sqrt(n) * (g + 1.0).abs().max().item() + b.norm().item())

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        g, b = self.gamma_beta_fp32()
        shape = x.shape
        y = head_norm(x.reshape(-1, shape[-2], shape[-1]).to(torch.bfloat16), g, b, self.eps)
        return y.reshape(shape).to(x.dtype)


def qk_score_bound(q_norm: FusedLayerNorm, k_norm: FusedLayerNorm, rotary_half: int = 0) -> float:
    """Upper bound of |q . k| over all rows the two norms can produce, with a rotary embedding of 2 * rotary_half
    features (pairs (i, i + rotary_half); 0 = none) applied to both.

    A normed row is n * (gamma + 1) + beta with |n|^2 <= D.  The rotation acts inside each pair and preserves the
    pair's length, so with groups p = the rotary pairs and the unpaired features one by one,
    G_p = max over the group of |gamma + 1| and B_p = the length of beta inside the group:

        |q . k| <= sum_p (Gq_p |nq_p| + Bq_p) (Gk_p |nk_p| + Bk_p)
                <= D max_p(Gq_p Gk_p) + sqrt(D) (|Gq * Bk| + |Gk * Bq|) + Bq . Bk          (Cauchy-Schwarz)

    which is never above the product of the two rows' lengths (sqrt(D) max|gamma + 1| + |beta|)^2 and is tighter
    when the large gains of the two norms sit on different features.  One host read of the parameters."""
    gq, bq = q_norm.gamma_beta_fp32()
    gk, bk = k_norm.gamma_beta_fp32()
    D = gq.numel()
    r = int(rotary_half)
    if not 0 <= 2 * r <= D:
        raise ValueError("rotary_half must satisfy 0 <= 2 * rotary_half <= head_dim")

    def groups(g, b):
        G, B2 = (g.double() + 1.0).abs(), b.double() ** 2
        if r:
            Gp, Bp = torch.maximum(G[:r], G[r:2 * r]), B2[:r] + B2[r:2 * r]
            G, B2 = torch.cat([Gp, G[2 * r:]]), torch.cat([Bp, B2[2 * r:]])
        return G, B2.sqrt()

    Gq, Bq = groups(gq, bq)
    Gk, Bk = groups(gk, bk)
    bound = (D * (Gq * Gk).max() + math.sqrt(D) * ((Gq * Bk).norm() + (Gk * Bq).norm()) + (Bq * Bk).sum())
    return float(bound.item())


class PerTensorQuantizedFp8Linear(torch.nn.Module):
    """The reference's fp8 linear layer (dit_module.py:431-456) with its parameter names and shapes, so that its
    checkpoints load: `weight` [1, out, in] float8_e4m3fn, `weight_scale` [1] fp32, `input_scale` [in] fp32.

    forward: x8 = div_clamp_to(x, input_scale) (magi_div_clamp_to_e4m3: the reference's quantiser, bf16 intermediate
    included), then the library's fp8 GEMM with fp32 accumulation, de-quantised by input_scale * weight_scale, bf16
    out (the reference calls flashinfer's bmm_fp8, which reads ONE value behind each scale pointer: with the
    per-channel shape the reference gives input_scale, that is its first element, as here).  The GEMM itself is
    a library routine (hipBLASLt through torch._scaled_mm), like the bf16 projections'."""

    def __init__(self, in_features: int, out_features: int, bias=False, dtype=torch.bfloat16, device=None) -> None:
        super().__init__()
        self.in_features, self.out_features, self.output_dtype = in_features, out_features, dtype
        P_ = torch.nn.Parameter
        self.weight = P_(torch.zeros((1, out_features, in_features), device=device).to(torch.float8_e4m3fn), requires_grad=False)
        self.weight_scale = P_(torch.ones(1, dtype=torch.float32, device=device), requires_grad=False)
        self.input_scale = P_(torch.ones(in_features, dtype=torch.float32, device=device), requires_grad=False)

    @classmethod
    def from_linear(cls, lin: torch.nn.Linear, input_absmax: float) -> "PerTensorQuantizedFp8Linear":
        """Per-tensor quantisation of a bf16 linear layer (for tests and calibration scripts): weight scale from the
        weight's absmax, input scale from the given absmax of the inputs, both so that the maximum maps to 448."""
        w = lin.weight.detach().float()
        q = cls(lin.in_features, lin.out_features, dtype=lin.weight.dtype, device=w.device)
        ws = (w.abs().max() / 448.0).clamp_min(1e-12)
        q.weight.data = (w / ws).clamp(-448, 448).to(torch.float8_e4m3fn)[None]
        q.weight_scale.data = ws.reshape(1).float()
        q.input_scale.data = torch.full((lin.in_features,), float(input_absmax) / 448.0, dtype=torch.float32, device=w.device)
        return q

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        x8 = div_clamp_to(input, self.input_scale)
        prefix = input.shape[:-1]
        y = torch._scaled_mm(x8.reshape(-1, self.in_features), self.weight[0].t(), scale_a=self.input_scale.reshape(-1)[:1],
                             scale_b=self.weight_scale.reshape(-1)[:1], out_dtype=self.output_dtype)
        return y.reshape(prefix + (self.out_features,))


class CustomLayerNormLinear(torch.nn.Module):
    """Input LayerNorm + the four projections q, qx, k, v (dit_module.py:390-425).

    fp8_quant=True builds the four projections as PerTensorQuantizedFp8Linear, as the reference does for every
    layer but the first and the last under EngineConfig.fp8_quant (:405-409): each quantises the normalised input
    with its own input scale and runs the library's fp8 GEMM; there is no shared weight buffer then.

    The four weights keep the reference's parameter names (q.weight, qx.weight, k.weight, v.weight) but live
    side by side in ONE buffer, rows ordered [q | k | v | qx], so forward_qkvx() is a single GEMM over the
    normalised input instead of four (the input, 1 GB at the 720p shape, is read once, and the fused prologue
    takes q / k / v as row-strided views of the one result).  Loading a state dict copies into the shared buffer
    in place; after anything that re-allocates the parameters (.to(), .bfloat16()) the buffer is rebuilt on the
    next call."""

    def __init__(self, input_size: int, output_size_q: int, output_size_kv: int, eps: float = 1e-6,
                 dtype=torch.bfloat16, device=None, fp8_quant: bool = False):
        super().__init__()
        self.fp8_quant = bool(fp8_quant)
        self.layer_norm = torch.nn.LayerNorm(input_size, eps=eps, dtype=dtype, device=device)
        mk = (lambda n: PerTensorQuantizedFp8Linear(input_size, n, dtype=dtype, device=device)) if self.fp8_quant else \
            (lambda n: torch.nn.Linear(input_size, n, bias=False, dtype=dtype, device=device))
        self.q, self.qx, self.k, self.v = mk(output_size_q), mk(output_size_q), mk(output_size_kv), mk(output_size_kv)
        if not self.fp8_quant:
            self._fuse_weights()

    def _projections(self):
        return (self.q, self.k, self.v, self.qx)  # row order of the shared buffer

    def _fuse_weights(self) -> torch.Tensor:
        """Move the four weights into one [2*out_q + 2*out_kv, in] buffer and make each parameter a view of it."""
        ws = [m.weight.data for m in self._projections()]
        fused = torch.cat(ws, dim=0)
        row = 0
        for m, w in zip(self._projections(), ws):
            m.weight.data = fused[row:row + w.shape[0]]
            row += w.shape[0]
        return fused

    def fused_weight(self) -> torch.Tensor:
        """The [q | k | v | qx] weight as one tensor (rebuilt first if the parameters no longer share a buffer)."""
        ws = [m.weight.data for m in self._projections()]
        base = ws[0]
        ptr = base.data_ptr()
        shared = True
        for w in ws:
            shared &= (w.data_ptr() == ptr and w.is_contiguous() and w.dtype == base.dtype and w.device == base.device
                       and w.untyped_storage().data_ptr() == base.untyped_storage().data_ptr())
            ptr += w.numel() * w.element_size()
        if not shared:
            return self._fuse_weights()
        rows = sum(w.shape[0] for w in ws)
        return base.as_strided((rows, base.shape[1]), (base.shape[1], 1))

    def forward_qkvx(self, hidden_states):
        """One GEMM for all four projections of the (already normalised) input -> views (q, k, v, qx) of one
        [..., 2*out_q + 2*out_kv] result.  (fp8_quant: four quantise + fp8 GEMM pairs, each with its own scales.)"""
        if self.fp8_quant:
            return self.q(hidden_states), self.k(hidden_states), self.v(hidden_states), self.qx(hidden_states)
        y = torch.nn.functional.linear(hidden_states, self.fused_weight())
        oq, okv = self.q.weight.shape[0], self.k.weight.shape[0]
        return y[..., :oq], y[..., oq:oq + okv], y[..., oq + okv:oq + 2 * okv], y[..., oq + 2 * okv:]

    def forward_ln(self, hidden_states):
        """LayerNorm of the layer input (dit_module.py:412-413) as one HIP launch; the parameters stay on the
        torch.nn.LayerNorm sub-module under the reference's names."""
        ln = self.layer_norm
        return layer_norm(hidden_states, ln.weight.detach(), ln.bias.detach(), ln.eps)

    def forward_q(self, hidden_states):
        return self.q(hidden_states)

    def forward_qx(self, hidden_states):
        return self.qx(hidden_states)

    def forward_k(self, hidden_states):
        return self.k(hidden_states)

    def forward_v(self, hidden_states):
        return self.v(hidden_states)


class FullyParallelAttention(torch.nn.Module):
    def __init__(self, hidden_size: int, num_attention_heads: int, num_query_groups: int, kv_channels: int = 128,
                 layer_number: int = 0, layernorm_epsilon: float = 1e-6, apply_layernorm_1p: bool = True,
                 xattn_cond_hidden_ratio: float = 1.0, params_dtype=torch.bfloat16, device=None,
                 attention_dtype: str = "bf16", fp8_fast_exp2: bool = False, fused_projection: bool = False,
                 fp8_quant: bool = False):
        """attention_dtype "fp8" (not in the reference, which has no fp8 attention) runs the self-attention on
        e4m3 operands with per-(video chunk, head) power-of-two scales and keeps the KV cache in that form
        (Fp8KVCache); the cross attention and everything else stay in bf16.
        fp8_fast_exp2: False (default) = the exact exponential, "softmax in fp32"; True opts into the fp8 kernel's
        piecewise-linear exp2 (MAGI_ATTN_FP8_FAST_EXP2: about 15 % faster, probabilities up to 6.2 % off each, the
        output inside a looser accuracy bar; see include/magi_attn.h).
        fp8_quant: the q / qx / k / v projections as PerTensorQuantizedFp8Linear (the reference's fp8_quant layers).
        fused_projection: run the four projections and the prologue as ONE launch (magi_qkv_proj_prologue, the
        hand-written GEMM whose epilogue is the prologue) instead of a library GEMM followed by the prologue kernel;
        bf16 attention at batch 1 only.  Off by default: at the 720p shape the library GEMM + prologue take
        10.9 ms, the fused launch 14.9 ms."""
        super().__init__()
        if kv_channels != 128:
            raise NotImplementedError("head_dim 128 only")
        if attention_dtype not in ("bf16", "fp8"):
            raise ValueError("attention_dtype must be 'bf16' or 'fp8'")
        self.attention_dtype = attention_dtype
        self.fp8_fast_exp2 = bool(fp8_fast_exp2)
        self.fused_projection = bool(fused_projection) and not fp8_quant
        # When the bound that follows from the norm parameters exceeds MAGI_SCORE_BOUND_MAX (it takes the largest gain
        # on both sides for every element), the core attention has the library MEASURE max|q| max|k| on the actual
        # rows (MAGI_ATTN_AUTO_BOUND), which is far smaller for gains that vary across features.  None: where the two
        # passes are small beside the attention; True / False: always / never.
        self.measure_bound_above_limit: Optional[bool] = None
        # forward() has the prologue fold softmax_scale * log2(e) into q ahead of q's one rounding to bf16 and tells
        # the attention kernel so (no per-score multiply there); get_q / get_qkv return q unscaled, as the reference
        self._q_premul = kv_channels ** -0.5 * math.log2(math.e)
        self.layer_number = layer_number
        self.hidden_size_per_attention_head = kv_channels
        self.num_attention_heads = num_attention_heads
        self.num_query_groups_per_partition = num_query_groups
        self.query_projection_size = kv_channels * num_attention_heads
        self.kv_projection_size = kv_channels * num_query_groups
        self.eps = layernorm_epsilon
        self.linear_qkv = CustomLayerNormLinear(hidden_size, self.query_projection_size, self.kv_projection_size,
                                                eps=layernorm_epsilon, dtype=params_dtype, device=device, fp8_quant=fp8_quant)
        self.linear_kv_xattn = torch.nn.Linear(int(hidden_size * xattn_cond_hidden_ratio), 2 * self.kv_projection_size,
                                               bias=False, dtype=params_dtype, device=device)
        mk = lambda dt: FusedLayerNorm(kv_channels, layernorm_epsilon, apply_layernorm_1p, dtype=dt, device=device)
        # the self-attention norms run in fp32 in the reference (promoted after load,
        # inference/model/dit/dit_model.py:628-633); the cross-attention norms stay in bf16
        self.q_layernorm = mk(torch.float32)
        self.k_layernorm = mk(torch.float32)
        self.q_layernorm_xattn = mk(params_dtype)
        self.k_layernorm_xattn = mk(params_dtype)

    # ------------------------------------------------------------------ score bounds
    def score_bounds(self, rotary_half: int = 48) -> Tuple[float, float]:
        """(self attention, cross attention) upper bounds of |q . k| in exp2-exponent units (q carrying
        softmax_scale * log2(e)), from the norm parameters (qk_score_bound: QK-normed rows have a known length, and
        the rotary embedding of 2 * rotary_half features preserves it), plus 1 % for the roundings to bf16.  Within
        MAGI_SCORE_BOUND_MAX the attention kernels then need no running maximum (magi_attn_args.score_bound);
        larger values make them fall back to it.  Computed once per set of parameter values (it reads them on the
        host) and cached until a parameter is modified or replaced (see invalidate_cached_parameters)."""
        lns = (self.q_layernorm, self.k_layernorm, self.q_layernorm_xattn, self.k_layernorm_xattn)
        key = tuple(ln.parameter_epoch() for ln in lns)
        if getattr(self, "_bounds_key", None) != key:
            self._bounds, self._bounds_key = {}, key
        r = int(rotary_half)
        if r not in self._bounds:  # (the cross-attention half does not depend on r)
            cross = next(iter(self._bounds.values()))[1] if self._bounds else \
                1.01 * self._q_premul * qk_score_bound(lns[2], lns[3], 0)
            self._bounds[r] = (1.01 * self._q_premul * qk_score_bound(lns[0], lns[1], r), cross)
        return self._bounds[r]

    def invalidate_cached_parameters(self) -> None:
        """Forget everything derived from the norm parameters (their fp32 forms, the score bounds, the e4m3 operand
        scales).  Needed only after a parameter was written through `.data`, which advances no version counter;
        in-place writes (`copy_`, `load_state_dict`) and replaced parameters (`load_state_dict(assign=True)`, `.to()`)
        are noticed by themselves."""
        for ln in (self.q_layernorm, self.k_layernorm, self.q_layernorm_xattn, self.k_layernorm_xattn):
            ln.invalidate_cached_parameters()
        self._bounds_key = self._fp8_scales_key = None

    # ------------------------------------------------------------------ cache
    def _allocate_key_and_value_memory(self, sequence_length: int, batch_size: int, dtype) -> torch.Tensor:
        """[max_seq * max_bs, Hkv, 2D] in HBM (dit_module.py:800-819).  The pinned-host variant is not made here: a
        KVCacheArena(kv_offload=True) attached to the InferenceParams supplies it for all layers."""
        return torch.empty(sequence_length * batch_size, self.num_query_groups_per_partition,
                           2 * self.hidden_size_per_attention_head, dtype=dtype,
                           device=self.linear_qkv.q.weight.device)

    def _cache(self, inference_params: InferenceParams, dtype) -> torch.Tensor:
        d = inference_params.key_value_memory_dict
        if self.layer_number not in d:
            d[self.layer_number] = self._allocate_key_and_value_memory(
                inference_params.max_sequence_length, inference_params.max_batch_size, dtype)
        return d[self.layer_number]

    def _cache_fp8(self, inference_params: InferenceParams, chunk_tokens: int) -> Fp8KVCache:
        d = inference_params.key_value_memory_dict
        if self.layer_number not in d:
            d[self.layer_number] = Fp8KVCache(inference_params.max_sequence_length * inference_params.max_batch_size,
                                              self.num_query_groups_per_partition, chunk_tokens,
                                              self.hidden_size_per_attention_head,
                                              device=self.linear_qkv.q.weight.device)
        cache = d[self.layer_number]
        if not isinstance(cache, Fp8KVCache) or cache.chunk_tokens != chunk_tokens:
            raise ValueError("this layer's cache entry is not an Fp8KVCache with chunk_tokens == clip_token_nums")
        return cache

    def fp8_operand_scales(self) -> Tuple[float, float]:
        """Constant power-of-two scales for the e4m3 forms of q (carrying softmax_scale * log2(e)) and k: no
        element of a QK-normed row can exceed the row's length, which the norm parameters bound
        (FusedLayerNorm.output_norm_bound) and the rotary embedding preserves, so these scales never saturate and
        the prologue can quantise without an absmax pass.  Cached like score_bounds()."""
        lns = (self.q_layernorm, self.k_layernorm)
        key = tuple(ln.parameter_epoch() for ln in lns)
        if getattr(self, "_fp8_scales_key", None) != key:
            nq, nk = (ln.output_norm_bound() for ln in lns)
            self._fp8_scales = (pow2_scale_for(self._q_premul * nq), pow2_scale_for(nk))
            self._fp8_scales_key = key
        return self._fp8_scales

    def _const_scale_table(self, value: float, rows: int, heads: int, device) -> torch.Tensor:
        """[rows, heads] fp32 filled with `value`, kept between calls (a launch only when it has to grow)."""
        tabs = self.__dict__.setdefault("_const_tabs", {})
        key = (value, heads, str(device))
        t = tabs.get(key)
        if t is None or t.shape[0] < rows:
            if len(tabs) > 8:
                tabs.clear()
            t = torch.full((max(rows, 16), heads), value, dtype=torch.float32, device=device)
            tabs[key] = t
        return t[:rows]

    def _side_buffer(self, name: str, shape, dtype, device) -> torch.Tensor:
        """A per-layer buffer for rows that must not be persisted, kept between calls."""
        t = getattr(self, name, None)
        if t is None or t.shape[0] < shape[0] or t.shape[1:] != tuple(shape[1:]) or t.dtype != dtype or t.device != device:
            t = torch.empty(shape, dtype=dtype, device=device)
            setattr(self, name, t)
        return t[:shape[0]]

    def _core_attention_fp8(self, raw, rope: torch.Tensor, inference_params: Optional[InferenceParams],
                            meta_args: ModelMetaArgs, use_cache: bool, out: Optional[torch.Tensor]) -> torch.Tensor:
        """Self-attention on e4m3 operands, three launches from the raw projections (q_raw, k_raw, v_raw) on: the
        prologue writes q and k as e4m3 with the constant scales of fp8_operand_scales(), k straight into the
        cache rows; one quantiser launch takes v's per-(chunk, head) absmax scales and writes v; the attention.
        Scale chunks are video chunks (clip_token_nums tokens), so the cache rules of the bf16 path
        (dit_module.py:905-931: append at slice_point, keep nothing when update_kv_cache is False, keep all but
        the last chunk under distill_nearly_clean_chunk) carry over chunk by chunk."""
        D = self.hidden_size_per_attention_head
        Hq, Hkv = self.num_attention_heads, self.num_query_groups_per_partition
        Lc = meta_args.clip_token_nums
        p = meta_args.core_attn_params
        q_raw, k_raw, v_raw = (t.reshape(t.shape[0] * t.shape[1], -1) for t in raw)
        S = q_raw.shape[0]
        dev = q_raw.device
        n_chunks = (S + Lc - 1) // Lc
        v3 = v_raw.view(S, Hkv, D)
        qs_c, ks_c = self.fp8_operand_scales()
        gq, bq = self.q_layernorm.gamma_beta_fp32()
        gk, bk = self.k_layernorm.gamma_beta_fp32()
        pro = dict(Hq=Hq, Hkv=Hkv, q_scale=qs_c, k_scale=ks_c, eps=self.eps, q_premul=self._q_premul)
        kw = dict(q_scale=self._const_scale_table(qs_c, n_chunks, Hq, dev), scale_chunk_tokens=Lc,
                  fp8_pow2_prescaled=True, fp8_fast_exp2=self.fp8_fast_exp2, out=out, return_lse=False)
        f8 = torch.float8_e4m3fn
        if not use_cache:
            q8, k8, _ = qk_prologue_fp8(q_raw, k_raw, rope, gq, bq, gk, bk, **pro)
            v8 = torch.empty((S, Hkv, D), dtype=f8, device=dev)
            vs = torch.empty((n_chunks, Hkv), dtype=torch.float32, device=dev)
            quantize_fp8_split(v3, Lc, S, v8, vs, None, None, pow2_scales=True)
            o, _ = range_attention(q8, k8, v8, p.q_range, p.k_range, p.max_seqlen_q, p.max_seqlen_k,
                                   k_scale=self._const_scale_table(ks_c, n_chunks, Hkv, dev), v_scale=vs, **kw)
            return o
        cache = self._cache_fp8(inference_params, Lc)
        start = meta_args.slice_point * Lc
        if inference_params.update_kv_cache:
            n_keep = S - Lc if meta_args.distill_nearly_clean_chunk else S
        else:
            n_keep = 0
        if S % Lc or n_keep < 0:
            raise ValueError("the fp8 path works on whole video chunks")
        if start + n_keep > cache.max_sequence_length:
            raise ValueError("KV cache overflow")
        c0 = start // Lc
        n_side = S - n_keep
        k_side = v_side = vs_side = None
        if n_side:
            k_side = self._side_buffer("_k8_side", (n_side, Hkv, D), f8, dev)
            v_side = self._side_buffer("_v8_side", (n_side, Hkv, D), f8, dev)
            vs_side = self._side_buffer("_v8_side_scale", (n_side // Lc, Hkv), torch.float32, dev)
        if n_keep:
            cache.note_constant_k_scale(ks_c, c0, n_keep // Lc)
        q8, _, _ = qk_prologue_fp8(q_raw, k_raw, rope, gq, bq, gk, bk, k_out=cache.k[start:], n_cache_rows=n_keep,
                                   k_tail=k_side, **pro)
        quantize_fp8_split(v3, Lc, n_keep, cache.v[start:], cache.v_scale[c0:], v_side, vs_side, pow2_scales=True)
        split = start + n_keep
        if not n_side:
            o, _ = range_attention(q8, cache.k[:split], cache.v[:split], p.q_range, p.k_range, p.max_seqlen_q,
                                   p.max_seqlen_k, k_scale=cache.k_scale, v_scale=cache.v_scale, **kw)
            return o
        # rows that must not be persisted: side buffers behind the cached prefix, with scale tables of their own
        o, _ = range_attention(q8, cache.k[:split], cache.v[:split], p.q_range, p.k_range, p.max_seqlen_q, p.max_seqlen_k,
                               k2=k_side, v2=v_side, k_split=split, k_scale=cache.k_scale, v_scale=cache.v_scale,
                               k2_scale=self._const_scale_table(ks_c, n_side // Lc, Hkv, dev), v2_scale=vs_side, **kw)
        return o

    # --------------------------------------------------- reference-shaped pieces
    def _prologue_single(self, raw: torch.Tensor, which: str, cos_emb, sin_emb) -> torch.Tensor:
        """raw [sq, b, H*D] -> [(sq b), H, D] through the fused kernel (one of q / k)."""
        sq, b = raw.shape[0], raw.shape[1]
        D = self.hidden_size_per_attention_head
        flat = raw.reshape(sq * b, -1)
        H = flat.shape[1] // D
        rope = torch.cat([sin_emb, cos_emb], dim=-1).float().contiguous()
        ln = self.q_layernorm if which == "q" else self.k_layernorm
        g, be = ln.gamma_beta_fp32()
        if which == "q":
            q, _, _ = qk_prologue(flat, flat[:, :0], flat[:, :0], rope, g, be, None, None, Hq=H, Hkv=0, eps=self.eps,
                                  batch=b)
            return q
        # K alone: run it through the Q slot (same arithmetic, contiguous output)
        k, _, _ = qk_prologue(flat, flat[:, :0], flat[:, :0], rope, g, be, None, None, Hq=H, Hkv=0, eps=self.eps,
                              batch=b)
        return k

    def get_q(self, mixed_qqkv: torch.Tensor, cos_emb: torch.Tensor, sin_emb: torch.Tensor) -> torch.Tensor:
        """[sq, b, h] -> [(sq b), Hq, D]; dit_module.py:953-963."""
        return self._prologue_single(self.linear_qkv.forward_q(mixed_qqkv), "q", cos_emb, sin_emb)

    def get_k(self, mixed_qqkv: torch.Tensor, cos_emb: torch.Tensor, sin_emb: torch.Tensor) -> torch.Tensor:
        """dit_module.py:970-980."""
        return self._prologue_single(self.linear_qkv.forward_k(mixed_qqkv), "k", cos_emb, sin_emb)

    def get_v(self, mixed_qqkv: torch.Tensor) -> torch.Tensor:
        """dit_module.py:987-989."""
        v = self.linear_qkv.forward_v(mixed_qqkv)
        return v.reshape(v.shape[0] * v.shape[1], -1, self.hidden_size_per_attention_head)

    def get_kv(self, mixed_qqkv: torch.Tensor, cos_emb: torch.Tensor, sin_emb: torch.Tensor) -> torch.Tensor:
        """[(sq b), Hkv, 2D] with K | V interleaved per head; dit_module.py:991-996."""
        _, kv = self._fused_qkv(mixed_qqkv, cos_emb, sin_emb, want_q=False)
        return kv

    def get_qkv(self, mixed_qqkv, cos_emb, sin_emb):
        """dit_module.py:998-1003."""
        q, kv = self._fused_qkv(mixed_qqkv, cos_emb, sin_emb, want_q=True)
        D = self.hidden_size_per_attention_head
        return q, kv[..., :D].contiguous(), kv[..., D:].contiguous()

    def _fused_qkv(self, mixed_qqkv, cos_emb, sin_emb, want_q=True, kv_out=None, n_cache_rows=None, kv_tail=None,
                   raw=None, q_premul=1.0, rope=None):
        """raw: (q_raw, k_raw, v_raw) already projected (views of forward_qkvx's result), else projected here.
        q_premul: factor folded into q ahead of its rounding to bf16 (see qk_prologue).
        rope: the [S, 2*R2] sin | cos table when the caller has it in one piece (else built from the two halves)."""
        sq, b = mixed_qqkv.shape[0], mixed_qqkv.shape[1]
        S = sq * b
        Hq, Hkv = self.num_attention_heads, self.num_query_groups_per_partition
        if raw is not None:
            q_raw, k_raw, v_raw = (t.reshape(S, -1) for t in raw)  # [sq, b, n] row-strided: still a view
        else:
            k_raw = self.linear_qkv.forward_k(mixed_qqkv).reshape(S, -1)
            v_raw = self.linear_qkv.forward_v(mixed_qqkv).reshape(S, -1)
            if want_q:
                q_raw = self.linear_qkv.forward_q(mixed_qqkv).reshape(S, -1)
            else:
                q_raw = k_raw[:, :0]
        if rope is None:
            rope = torch.cat([sin_emb, cos_emb], dim=-1).float().contiguous()
        gq, bq = self.q_layernorm.gamma_beta_fp32()
        gk, bk = self.k_layernorm.gamma_beta_fp32()
        q, kv, tail = qk_prologue(q_raw, k_raw, v_raw, rope, gq, bq, gk, bk, Hq=Hq if want_q else 0, Hkv=Hkv,
                                  eps=self.eps, kv_out=kv_out, n_cache_rows=n_cache_rows, kv_tail=kv_tail, batch=b,
                                  q_premul=q_premul)
        return (q if want_q else None), (kv if tail is None else (kv, tail))

    def get_xqkv(self, mixed_qqkv: torch.Tensor, key_value_states: torch.Tensor, qx_raw: Optional[torch.Tensor] = None):
        """Cross-attention q (normed) and k (normed) / v from the text states; dit_module.py:1005-1021.
        qx_raw: the qx projection when the caller already has it (forward_qkvx), else projected here."""
        D = self.hidden_size_per_attention_head
        qx = self.linear_qkv.forward_qx(mixed_qqkv) if qx_raw is None else qx_raw  # [sq, b, Hq*D]
        qx = qx.transpose(0, 1).reshape(qx.shape[0] * qx.shape[1], -1, D)  # "(b sq) hn hd"
        gq, bq = self.q_layernorm_xattn.gamma_beta_fp32()
        qx = head_norm(qx, gq, bq, self.eps)
        kv = torch.nn.functional.linear(key_value_states, self.linear_kv_xattn.weight)  # [Ty, 2*Hkv*D]
        kv = kv.view(key_value_states.shape[0], -1, 2 * D)
        gk, bk = self.k_layernorm_xattn.gamma_beta_fp32()
        kx = head_norm(kv[..., :D], gk, bk, self.eps)  # strided read, contiguous result
        return qx, kx, kv[..., D:]

    def _full_adjust_key_and_value(self, inference_params: InferenceParams, key_and_value: torch.Tensor,
                                   meta_args: ModelMetaArgs) -> torch.Tensor:
        """Appends key_and_value's persistent rows to this layer's cache and returns [cached prefix | key_and_value]
        (dit_module.py:891-931).  With an offloaded cache the prefix comes through the staging buffer and the appended
        rows go back to the host."""
        cache = self._cache(inference_params, key_and_value.dtype)
        start = meta_args.slice_point * meta_args.clip_token_nums * inference_params.max_batch_size
        offloaded = cache if isinstance(cache, OffloadedKVCache) else None
        if offloaded is not None:
            cache = offloaded.stage(start)
        clip = 0
        try:
            prefix = cache[:start]
            if inference_params.update_kv_cache:
                total = key_and_value.size(0)
                clip = (total - meta_args.clip_token_nums * inference_params.max_batch_size
                        if meta_args.distill_nearly_clean_chunk else total)
                if start + clip > cache.shape[0]:
                    clip = 0
                    raise ValueError("KV cache overflow")
                cache[start:start + clip] = key_and_value[:clip]
            return torch.cat([prefix, key_and_value], dim=0)
        finally:
            if offloaded is not None:
                offloaded.release(start, clip)

    def adjust_key_and_value_for_inference(self, key_and_value: torch.Tensor, inference_params: Optional[InferenceParams],
                                           meta_args: ModelMetaArgs):
        """Copying form with the reference's exact semantics (dit_module.py:933-946), for callers
        that hold a materialised key_and_value.  forward() does not use it: it appends in place."""
        D = self.hidden_size_per_attention_head
        if inference_params is None:
            return key_and_value[..., :D], key_and_value[..., D:]
        if meta_args.extract_prefix_video_feature or meta_args.fwd_extra_1st_chunk or meta_args.slice_point > 0:
            key_and_value = self._full_adjust_key_and_value(inference_params, key_and_value, meta_args)
        return key_and_value[..., :D].contiguous(), key_and_value[..., D:].contiguous()

    def core_attention(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, bs: int,
                       meta_args: ModelMetaArgs, out: Optional[torch.Tensor] = None,
                       q_prescaled: bool = False, score_bound: float = 0.0, auto_bound: bool = False) -> torch.Tensor:
        """query [(sq b), Hq, D], key / value [(sk b), Hkv, D] -> [(sq b), Hq, D]; dit_module.py:1023-1066.
        bs > 1 only occurs with one range per batch row (asserted there too).  `out` (bs == 1 only) is a
        destination view, possibly in the grouped layout of range_attention.  q_prescaled: query carries
        softmax_scale * log2(e); score_bound, auto_bound: see range_attention."""
        p = meta_args.core_attn_params
        if bs == 1:
            out, _ = range_attention(query, key, value, p.q_range, p.k_range, p.max_seqlen_q, p.max_seqlen_k,
                                     out=out, return_lse=False, q_prescaled=q_prescaled, score_bound=score_bound,
                                     auto_bound=auto_bound)
            return out
        if meta_args.denoising_range_num > 1:
            raise ValueError("bs > 1 with several denoising ranges is not a layout the pipeline produces")
        # Batch rows attend to themselves over the whole sequence (dit_module.py:1046-1050): with the token axis
        # ordered (position, batch) that is ONE range over positions with bs * Hq heads, since head b * Hq + h of
        # the [(sq), (b Hq), D] view uses kv head (b * Hq + h) / (Hq / Hkv) = b * Hkv + h / (Hq / Hkv).
        sq, sk = query.shape[0] // bs, key.shape[0] // bs
        Hq, Hkv, D = query.shape[1], key.shape[1], query.shape[2]
        if not (query.is_contiguous() and key.stride(0) == Hkv * key.stride(1) and value.stride(0) == Hkv * value.stride(1)):
            raise ValueError("bs > 1 needs the (position, batch, head) axes of q / k / v evenly strided")
        dev = query.device
        ranges = getattr(self, "_one_range", None)
        if ranges is None or ranges[0] != (sq, sk, dev):
            ranges = ((sq, sk, dev), torch.tensor([[0, sq]], dtype=torch.int32, device=dev),
                      torch.tensor([[0, sk]], dtype=torch.int32, device=dev))
            self._one_range = ranges
        o, _ = range_attention(query.view(sq, bs * Hq, D), key.as_strided((sk, bs * Hkv, D), (bs * key.stride(0), key.stride(1), 1)),
                               value.as_strided((sk, bs * Hkv, D), (bs * value.stride(0), value.stride(1), 1)),
                               ranges[1], ranges[2], sq, sk, return_lse=False, q_prescaled=q_prescaled,
                               score_bound=score_bound)
        return o.view(sq * bs, Hq, D)

    def full_attention(self, bs: int, meta_args: ModelMetaArgs, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, i: int,
                       score_bound: float = 0.0) -> torch.Tensor:
        """The rectangle of denoising range i alone: q [rows of range i, Hq, D] against the keys k_range[i] of the
        whole key axis k / v [(sk), Hkv, D] -> [rows, Hq, D]; dit_module.py:1068-1096 (what the reference's
        cp_shuffle_overlap strategy calls chunk by chunk, batch 1 only as there).  The range tensors are sliced on the
        device, so the call does not synchronise."""
        if bs != 1:
            raise ValueError("full_attention is defined for batch 1 (as in the reference)")
        p = meta_args.core_attn_params
        q_range = (p.q_range[i:i + 1] - p.q_range[i, 0]).contiguous()
        out, _ = range_attention(q, k, v, q_range, p.k_range[i:i + 1].contiguous(), p.max_seqlen_q, p.max_seqlen_k,
                                 return_lse=False, score_bound=score_bound)
        return out

    def cross_attention(self, mixed_qqkv: torch.Tensor, key_value_states: torch.Tensor,
                        cross_attn_params: PackedCrossAttnParams, get_xqkv_func: Callable,
                        out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """-> [sq, b, Hq*D]; dit_module.py:1098-1136.  With `out` (b == 1 only: a destination view, possibly in
        the grouped layout of range_attention) the result is written there (segments without text get zero rows
        from the kernel) and `out` is returned."""
        qx, kx, vx = get_xqkv_func(mixed_qqkv, key_value_states)
        b = mixed_qqkv.shape[1]
        sq = mixed_qqkv.shape[0]
        if out is not None:
            if b != 1:
                raise ValueError("a destination view for the cross attention needs batch 1")
            range_attention(qx, kx, vx, cross_attn_params.cu_seqlens_q, cross_attn_params.cu_seqlens_kv,
                            cross_attn_params.max_seqlen_q, cross_attn_params.max_seqlen_kv,
                            ranges_mode=L.MAGI_RANGES_CU, out=out, return_lse=False)
            return out
        out, _ = range_attention(qx, kx, vx, cross_attn_params.cu_seqlens_q, cross_attn_params.cu_seqlens_kv,
                                 cross_attn_params.max_seqlen_q, cross_attn_params.max_seqlen_kv,
                                 ranges_mode=L.MAGI_RANGES_CU, return_lse=False, zero_init=True)
        out = out.view(b, sq, -1)
        return out.transpose(0, 1).contiguous() if b > 1 else out.view(sq, 1, -1)

    def _cross_attention_fused(self, qx_raw: torch.Tensor, key_value_states: torch.Tensor,
                               cross_attn_params: PackedCrossAttnParams, out: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
        """Batch-1 cross attention on the RAW qx projection [sq, 1, Hq*D]: the attention kernel applies
        q_layernorm_xattn while it loads q (no normalised copy of q in memory) and, the scores of normed q and k
        being bounded, runs without a running maximum.  Returns None when that path does not apply (then the
        caller takes get_xqkv + cross_attention); else the [sq, Hq, D]-shaped result (`out` if given)."""
        bound = self.score_bounds()[1]
        if qx_raw.shape[1] != 1 or not (0.0 < bound <= L.MAGI_SCORE_BOUND_MAX):
            return None
        D = self.hidden_size_per_attention_head
        sq = qx_raw.shape[0]
        q = qx_raw.reshape(sq, -1, D)  # row-strided view of the projection
        kv = torch.nn.functional.linear(key_value_states, self.linear_kv_xattn.weight)
        kv = kv.view(key_value_states.shape[0], -1, 2 * D)
        gk, bk = self.k_layernorm_xattn.gamma_beta_fp32()
        kx = head_norm(kv[..., :D], gk, bk, self.eps)
        gq, bq = self.q_layernorm_xattn.gamma_beta_fp32()
        o, _ = range_attention(q, kx, kv[..., D:], cross_attn_params.cu_seqlens_q, cross_attn_params.cu_seqlens_kv,
                               cross_attn_params.max_seqlen_q, cross_attn_params.max_seqlen_kv,
                               ranges_mode=L.MAGI_RANGES_CU, out=out, return_lse=False, zero_init=True,
                               score_bound=bound, q_norm=(gq, bq, self.eps))
        return o

    # ------------------------------------------------------------------ forward
    def forward(self, hidden_states: torch.Tensor, key_value_states: torch.Tensor,
                inference_params: Optional[InferenceParams], rotary_pos_emb: torch.Tensor, meta_args: ModelMetaArgs,
                proj_layout: bool = False):
        """-> (core_attn_out, xattn_out), each [sq, b, Hq*D], as the reference (dit_module.py:1138-1173).

        With proj_layout=True the return value is ONE tensor [sq, b, 2*Hq*D] already in the "(hn n hd)" order
        that linear_proj consumes (what attn_linear_proj builds with concat + rearrange, dit_module.py:1332-1340):
        at batch 1 both attention launches write straight into it."""
        if rotary_pos_emb is None:
            raise ValueError("FullyParallelAttention needs rotary_pos_emb")
        sin_emb, cos_emb = rotary_pos_emb.tensor_split(2, -1)
        # the incoming table already is the [sin | cos] layout the prologue takes
        rope = rotary_pos_emb if (rotary_pos_emb.dtype == torch.float32 and rotary_pos_emb.is_contiguous()) else None
        bound_core = self.score_bounds(rotary_pos_emb.shape[-1] // 2)[0]
        core_bound_kw = {"score_bound": bound_core}  # (above the limit: the online-softmax kernel, unless measured)
        measured = False
        if not (0.0 < bound_core <= L.MAGI_SCORE_BOUND_MAX) and self.attention_dtype == "bf16" and hidden_states.shape[1] == 1:
            p_ = meta_args.core_attn_params
            n_q = hidden_states.shape[0]
            measured = self.measure_bound_above_limit
            if measured is None:
                shape_q = torch.empty(n_q, self.num_attention_heads, 128, dtype=torch.bfloat16, device="meta")
                shape_k = torch.empty(max(int(p_.max_seqlen_k), n_q), self.num_query_groups_per_partition, 128,
                                      dtype=torch.bfloat16, device="meta")
                measured = _measuring_a_bound_pays(shape_q, shape_k, p_.q_range.shape[0], p_.max_seqlen_q, p_.max_seqlen_k)
            if measured:
                core_bound_kw = {"auto_bound": True}
        # which attention kernels this forward selects (diagnostics; the choice follows from the norm parameters)
        bounded = lambda b: "bounded-score, 64 rows per wavefront" if 0.0 < b <= L.MAGI_SCORE_BOUND_MAX \
            else "online softmax, 32 rows per wavefront"
        self.last_forward_kernels = {
            "core": "fp8" if self.attention_dtype == "fp8" else
            ("measured bound: bounded-score or online softmax, chosen on the device" if measured else bounded(bound_core)),
            "core_score_bound": bound_core,
            "cross": bounded(self.score_bounds()[1] if hidden_states.shape[1] == 1 else float("inf")),
            "cross_score_bound": self.score_bounds()[1]}
        bs = hidden_states.shape[1]
        sq = hidden_states.shape[0]
        D = self.hidden_size_per_attention_head
        mixed_qqkv = self.linear_qkv.forward_ln(hidden_states)
        one_launch = (self.fused_projection and self.attention_dtype == "bf16" and bs == 1 and rope is not None
                      and rope.shape[-1] == 96 and mixed_qqkv.shape[-1] % 64 == 0)
        if one_launch:
            # projections + prologue in one launch: nothing raw reaches memory (qx leaves unnormalised, as the
            # cross-attention kernel takes it)
            raw = qx_raw = None
        else:
            # all four projections in one GEMM; q / k / v feed the fused prologue as row-strided views of its result
            q_raw, k_raw, v_raw, qx_raw = self.linear_qkv.forward_qkvx(mixed_qqkv)
            raw = (q_raw, k_raw, v_raw)

        def project(kv_out=None, n_cache_rows=None, kv_tail=None):
            """-> (q [S, Hq, D] carrying the softmax scale, kv destination(s), qx_raw [sq, 1, Hq*D])"""
            if not one_launch:
                q_, kv_ = self._fused_qkv(mixed_qqkv, cos_emb, sin_emb, kv_out=kv_out, n_cache_rows=n_cache_rows,
                                          kv_tail=kv_tail, raw=raw, q_premul=self._q_premul, rope=rope)
                return q_, kv_, qx_raw
            gq_, bq_ = self.q_layernorm.gamma_beta_fp32()
            gk_, bk_ = self.k_layernorm.gamma_beta_fp32()
            q_, kv_, tail_, qx_ = qkv_proj_prologue(
                mixed_qqkv.view(sq, -1), self.linear_qkv.fused_weight(), rope, gq_, bq_, gk_, bk_,
                Hq=self.num_attention_heads, Hkv=self.num_query_groups_per_partition, Hqx=self.num_attention_heads,
                eps=self.eps, kv_out=kv_out, n_cache_rows=n_cache_rows, kv_tail=kv_tail, q_premul=self._q_premul)
            return q_, (kv_ if tail_ is None else (kv_, tail_)), qx_.view(sq, 1, -1)

        get_xqkv = lambda m, y: self.get_xqkv(m, y, qx_raw=qx_raw)
        p = meta_args.core_attn_params
        Hq = self.num_attention_heads
        fused = None
        core_dst = cross_dst = None
        if proj_layout and bs == 1 and Hq % PROJ_GROUPS == 0:
            # (rows that no q range / cu_seqlens segment covers are left as allocated: the pipeline's ranges cover
            # every row, dit_model.py:220-222, 246)
            fused = torch.empty(sq, 1, 2 * Hq * D, dtype=hidden_states.dtype, device=hidden_states.device)
            grouped = fused.view(sq, PROJ_GROUPS, 2, Hq // PROJ_GROUPS, D)
            core_dst, cross_dst = grouped[:, :, 0], grouped[:, :, 1]

        use_cache = inference_params is not None and (
            meta_args.extract_prefix_video_feature or meta_args.fwd_extra_1st_chunk or meta_args.slice_point > 0)
        if self.attention_dtype == "fp8":
            if bs != 1 or (use_cache and inference_params.max_batch_size != 1):
                raise ValueError("the fp8 self-attention runs at batch 1")
            rope8 = rope if rope is not None else torch.cat([sin_emb, cos_emb], dim=-1).float().contiguous()
            core = self._core_attention_fp8(raw, rope8, inference_params, meta_args, use_cache, core_dst)
        elif not use_cache:
            q, kv, qx_raw = project()
            core = self.core_attention(q, kv[..., :D], kv[..., D:], bs, meta_args, out=core_dst, q_prescaled=True,
                                       **core_bound_kw)
        else:
            if bs != 1 or inference_params.max_batch_size != 1:
                raise ValueError("the cached path runs at batch 1 (as the reference pipeline does)")
            cache = self._cache(inference_params, hidden_states.dtype)
            start = meta_args.slice_point * meta_args.clip_token_nums
            S = sq
            offloaded = cache if isinstance(cache, OffloadedKVCache) else None
            if offloaded is not None:  # kv_offload: the prefix comes through a device staging buffer
                cache = offloaded.stage(start)
            if inference_params.update_kv_cache:
                n_keep = S - meta_args.clip_token_nums if meta_args.distill_nearly_clean_chunk else S
            else:
                n_keep = 0
            if start + n_keep > cache.shape[0]:
                if offloaded is not None:
                    offloaded.release()
                raise ValueError("KV cache overflow")
            tail = None
            if n_keep < S:  # side buffer for the rows that must not be persisted, kept between calls
                tail = getattr(self, "_kv_tail", None)
                if (tail is None or tail.shape[0] < S - n_keep or tail.shape[1:] != cache.shape[1:]
                        or tail.dtype != cache.dtype or tail.device != cache.device):
                    tail = torch.empty(S - n_keep, cache.shape[1], cache.shape[2], dtype=cache.dtype, device=cache.device)
                    self._kv_tail = tail
                tail = tail[:S - n_keep]
            persisted = 0
            try:
                q, _, qx_raw = project(kv_out=cache[start:], n_cache_rows=n_keep, kv_tail=tail)
                split = start + n_keep
                kc, vc = cache[:split, :, :D], cache[:split, :, D:]
                if tail is None:
                    core, _ = range_attention(q, kc, vc, p.q_range, p.k_range, p.max_seqlen_q, p.max_seqlen_k,
                                              out=core_dst, return_lse=False, q_prescaled=True, **core_bound_kw)
                else:
                    core, _ = range_attention(q, kc, vc, p.q_range, p.k_range, p.max_seqlen_q, p.max_seqlen_k,
                                              k2=tail[:, :, :D], v2=tail[:, :, D:], k_split=split, out=core_dst,
                                              return_lse=False, q_prescaled=True, **core_bound_kw)
                persisted = n_keep
            finally:
                if offloaded is not None:  # the persisted rows go back to the host behind the attention launch
                    offloaded.release(start, persisted)
        if fused is not None:
            if self._cross_attention_fused(qx_raw, key_value_states, meta_args.cross_attn_params, cross_dst) is None:
                self.cross_attention(mixed_qqkv, key_value_states, meta_args.cross_attn_params, get_xqkv, out=cross_dst)
            return fused
        core_attn_out = core.view(sq, bs, -1)
        xo = self._cross_attention_fused(qx_raw, key_value_states, meta_args.cross_attn_params, None)
        if xo is not None:
            xattn_out = xo.view(sq, 1, -1)
        else:
            xattn_out = self.cross_attention(mixed_qqkv, key_value_states, meta_args.cross_attn_params, get_xqkv)
        if proj_layout:
            return attn_linear_proj_input(core_attn_out, xattn_out)
        return core_attn_out, xattn_out
