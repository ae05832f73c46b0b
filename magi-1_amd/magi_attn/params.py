"""Metadata containers of the attention path, field-for-field as the reference's
inference/common/dataclass.py:22-83 so that pipeline code can hand them over unchanged."""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional

import numpy as np
import torch


@dataclass(frozen=True)
class PackedCoreAttnParams:
    q_range: torch.Tensor
    k_range: torch.Tensor
    np_q_range: np.ndarray
    np_k_range: np.ndarray
    max_seqlen_q: int
    max_seqlen_k: int


@dataclass(frozen=True)
class PackedCrossAttnParams:
    q_ranges: Optional[torch.Tensor] = None
    kv_ranges: Optional[torch.Tensor] = None
    cu_seqlens_q: Optional[torch.Tensor] = None
    cu_seqlens_kv: Optional[torch.Tensor] = None
    max_seqlen_q: Optional[int] = None
    max_seqlen_kv: Optional[int] = None


@dataclass(frozen=True)
class ModelMetaArgs:
    H: int
    W: int
    cp_pad_size: Optional[int]
    cp_split_sizes: Optional[List[int]]
    slice_point: int
    denoising_range_num: int
    range_num: int
    extract_prefix_video_feature: bool
    fwd_extra_1st_chunk: bool
    distill_nearly_clean_chunk: bool
    clip_token_nums: int
    enable_cuda_graph: bool
    core_attn_params: PackedCoreAttnParams
    cross_attn_params: PackedCrossAttnParams


class InferenceParams:
    """Run-time state of one generation: the per-layer KV cache (dataclass.py:62-71).

    key_value_memory_dict[layer_number] is a [max_sequence_length * max_batch_size, Hkv, 2*D]
    tensor, K in [..., :D] and V in [..., D:].  On MI355X it normally lives in HBM (288 GB hold
    every layer of the 24B model at 720p); a KVCacheArena(kv_offload=True) puts OffloadedKVCache
    objects here instead (pinned host memory behind device staging buffers)."""

    def __init__(self, max_batch_size: int, max_sequence_length: int):
        self.max_sequence_length = max_sequence_length
        self.max_batch_size = max_batch_size
        self.sequence_len_offset = 0
        self.key_value_memory_dict = {}
        self.update_kv_cache = False

    def swap_key_value_dict(self, batch_idx):
        """Re-order the batch rows of every layer's cache (dataclass.py:72-83).  The reference's method is written
        for a (key, value) tuple of [seq, batch, ...] tensors, a layout its DiT never stores (its caches are the
        single [max_seq * max_bs, Hkv, 2D] tensors of dit_module.py:800-819, tokens ordered (position, batch)), and
        the shipped pipeline never calls it; this one does the same thing on the layout that is actually used.
        Raises on an empty dict like the reference."""
        if len(self.key_value_memory_dict) == 0:
            raise ValueError("should not swap when dict in empty")
        idx = torch.as_tensor(batch_idx, dtype=torch.long)
        if idx.numel() != self.max_batch_size:
            raise ValueError("batch_idx must name every batch row once")
        for layer_number, cache in self.key_value_memory_dict.items():
            if not isinstance(cache, torch.Tensor):
                raise TypeError("swap_key_value_dict works on tensor caches (not on an Fp8KVCache or an offloaded cache)")
            rows = cache.view(self.max_sequence_length, self.max_batch_size, *cache.shape[1:])
            self.key_value_memory_dict[layer_number] = rows[:, idx.to(cache.device)].reshape(cache.shape)


def build_core_attn_params(q_range: torch.Tensor, k_range: torch.Tensor, max_seqlen_q: int,
                           max_seqlen_k: Optional[int] = None) -> PackedCoreAttnParams:
    """As inference/model/dit/dit_model.py:246-259, 301-308.  max_seqlen_k defaults to
    max(k_range) - min(k_range) like the reference (:247-248), computed from the host copy."""
    np_q = q_range.detach().cpu().numpy()
    np_k = k_range.detach().cpu().numpy()
    if max_seqlen_k is None:
        max_seqlen_k = int(np_k.max() - np_k.min()) if np_k.size else 0
    return PackedCoreAttnParams(q_range=q_range, k_range=k_range, np_q_range=np_q, np_k_range=np_k,
                                max_seqlen_q=int(max_seqlen_q), max_seqlen_k=int(max_seqlen_k))


def build_cross_attn_params(xattn_mask: torch.Tensor, clip_token_nums: int, caption_max_length: int = 800
                            ) -> PackedCrossAttnParams:
    """As inference/model/dit/dit_model.py:213-241: one segment per (batch x chunk) with
    clip_token_nums queries and sum(mask) text tokens."""
    m = xattn_mask.reshape(xattn_mask.shape[0], -1)
    y_index = m.sum(dim=-1).to(torch.int64)
    n = m.shape[0]
    dev = m.device
    cu_q = (torch.arange(n + 1, dtype=torch.int64, device=dev) * clip_token_nums).to(torch.int32)
    cu_k = torch.cat([y_index.new_zeros(1), y_index]).cumsum(-1).to(torch.int32)
    return PackedCrossAttnParams(
        q_ranges=torch.stack([cu_q[:-1], cu_q[1:]], dim=1), kv_ranges=torch.stack([cu_k[:-1], cu_k[1:]], dim=1),
        cu_seqlens_q=cu_q, cu_seqlens_kv=cu_k, max_seqlen_q=int(clip_token_nums), max_seqlen_kv=int(caption_max_length))
