"""One HBM arena for the KV caches of all layers.

The reference allocates each layer's cache lazily on first use (`_allocate_key_and_value_memory`,
inference/model/dit/dit_module.py:800-819, keyed by layer number in
`InferenceParams.key_value_memory_dict`, :905-912) and ships `kv_offload: true` for the 24B model
(example/24B/24B_base_config.json:83), which keeps the caches in pinned host memory and copies the prefix to the
GPU in every layer (:915).  A 720p 24B generation needs 48 layers x 1.06 GB = 51 GB; an MI355X has 288 GB, so the
caches stay resident: one allocation made up front, one view per layer, no host staging, no allocator traffic
inside the denoising loop.  The attention kernels read the views in place."""
from __future__ import annotations

from typing import Dict, Iterable, Optional

import torch

from .params import InferenceParams


class KVCacheArena:
    """[num_layers, max_sequence_length * max_batch_size, Hkv, 2*D]; layer i's cache is `arena[i]`, K in
    [..., :D] and V in [..., D:], the layout of the reference's per-layer tensor."""

    def __init__(self, num_layers: int, max_sequence_length: int, num_query_groups: int, head_dim: int = 128,
                 max_batch_size: int = 1, dtype: torch.dtype = torch.bfloat16, device=None,
                 memory_budget_bytes: Optional[int] = None, kv_offload: bool = False):
        if kv_offload:
            raise ValueError("kv_offload is not offered: the caches of every layer fit in HBM (see the module docstring)")
        if min(num_layers, max_sequence_length, num_query_groups, head_dim, max_batch_size) <= 0:
            raise ValueError("all sizes must be positive")
        self.num_layers = num_layers
        self.max_sequence_length = max_sequence_length
        self.max_batch_size = max_batch_size
        rows = max_sequence_length * max_batch_size
        need = self.bytes_needed(num_layers, max_sequence_length, num_query_groups, head_dim, max_batch_size, dtype)
        if memory_budget_bytes is not None and need > memory_budget_bytes:
            raise MemoryError(f"KV caches need {need / 2**30:.1f} GiB, budget is {memory_budget_bytes / 2**30:.1f} GiB")
        self.buffer = torch.empty(num_layers, rows, num_query_groups, 2 * head_dim, dtype=dtype, device=device)

    @staticmethod
    def bytes_needed(num_layers: int, max_sequence_length: int, num_query_groups: int, head_dim: int = 128,
                     max_batch_size: int = 1, dtype: torch.dtype = torch.bfloat16) -> int:
        return (num_layers * max_sequence_length * max_batch_size * num_query_groups * 2 * head_dim
                * torch.empty((), dtype=dtype).element_size())

    def layer(self, index: int) -> torch.Tensor:
        return self.buffer[index]

    def attach(self, inference_params: InferenceParams, layer_numbers: Optional[Iterable[int]] = None
               ) -> Dict[int, torch.Tensor]:
        """Hands the layer views to `inference_params.key_value_memory_dict` (what the attention module looks
        up by layer number); `layer_numbers` defaults to 0 .. num_layers-1 in arena order."""
        if (inference_params.max_sequence_length != self.max_sequence_length
                or inference_params.max_batch_size != self.max_batch_size):
            raise ValueError("arena and InferenceParams disagree on max_sequence_length / max_batch_size")
        numbers = list(range(self.num_layers)) if layer_numbers is None else list(layer_numbers)
        if len(numbers) != self.num_layers or len(set(numbers)) != len(numbers):
            raise ValueError("need one distinct layer number per arena layer")
        for i, n in enumerate(numbers):
            inference_params.key_value_memory_dict[n] = self.buffer[i]
        return inference_params.key_value_memory_dict


class Fp8KVCache:
    """One layer's KV cache for the fp8 attention path: K and V as e4m3 bytes [max_sequence_length, Hkv, D] each,
    plus one power-of-two fp32 scale per (chunk of `chunk_tokens` tokens, KV head).  A chunk of the cache is a
    video chunk (`clip_token_nums` tokens, the unit in which the pipeline appends and re-reads KV,
    inference/model/dit/dit_module.py:905-929), so appending a chunk never re-scales rows already stored.
    Half the bytes of the bf16 cache: 0.53 GB per layer at the 24B / 720p shape.

    The reference has no fp8 attention; this object takes the place of the tensor it keeps in
    `InferenceParams.key_value_memory_dict[layer_number]` when the layer runs with attention_dtype="fp8"."""

    def __init__(self, max_sequence_length: int, num_query_groups: int, chunk_tokens: int, head_dim: int = 128,
                 device=None):
        if min(max_sequence_length, num_query_groups, chunk_tokens) <= 0:
            raise ValueError("all sizes must be positive")
        self.chunk_tokens = chunk_tokens
        n_chunks = (max_sequence_length + chunk_tokens - 1) // chunk_tokens
        self.k = torch.zeros(max_sequence_length, num_query_groups, head_dim, dtype=torch.float8_e4m3fn, device=device)
        self.v = torch.zeros_like(self.k)
        self.k_scale = torch.ones(n_chunks, num_query_groups, dtype=torch.float32, device=device)
        self.v_scale = torch.ones_like(self.k_scale)
        self._k_const = None  # the value every row of k_scale holds, once a writer with constant K scales said so

    def note_constant_k_scale(self, value: float, first_chunk: int, n_chunks: int) -> None:
        """A writer whose K scale is one constant (the prologue with e4m3 outputs) is about to store chunks
        [first_chunk, first_chunk + n_chunks).  While every writer uses the same constant the table is filled
        once and never touched again; a different constant (the norm parameters changed while rows quantised
        with the old one are still cached) only rewrites the rows of the chunks being stored."""
        if self._k_const is None:
            self.k_scale.fill_(value)
            self._k_const = value
        elif self._k_const != value:
            self.k_scale[first_chunk:first_chunk + n_chunks].fill_(value)
            self._k_const = float("nan")  # mixed from now on: every later store writes its rows

    @property
    def max_sequence_length(self) -> int:
        return self.k.shape[0]
