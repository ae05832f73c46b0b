"""One HBM arena for the KV caches of all layers.

The reference allocates each layer's cache lazily on first use (`_allocate_key_and_value_memory`,
inference/model/dit/dit_module.py:800-819, keyed by layer number in
`InferenceParams.key_value_memory_dict`, :905-912) and ships `kv_offload: true` for the 24B model
(example/24B/24B_base_config.json:83), which keeps the caches in pinned host memory and copies the prefix to the
GPU in every layer (:915).  A 720p 24B generation needs 48 layers x 1.06 GB = 51 GB; an MI355X has 288 GB, so the
caches stay resident: one allocation made up front, one view per layer, no host staging, no allocator traffic
inside the denoising loop.  The attention kernels read the views in place.

`kv_offload=True` is there as an option for generations whose caches do not fit (longer videos, several side
passes): the layers' caches live in pinned host memory and pass through a small ring of device staging buffers,
the next layer's prefix on its way over a copy stream while the current layer computes (OffloadedKVCache)."""
from __future__ import annotations

from typing import Dict, Iterable, Optional

import torch

from .params import InferenceParams


class KVCacheArena:
    """[num_layers, max_sequence_length * max_batch_size, Hkv, 2*D]; layer i's cache is `arena[i]`, K in
    [..., :D] and V in [..., D:], the layout of the reference's per-layer tensor."""

    def __init__(self, num_layers: int, max_sequence_length: int, num_query_groups: int, head_dim: int = 128,
                 max_batch_size: int = 1, dtype: torch.dtype = torch.bfloat16, device=None,
                 memory_budget_bytes: Optional[int] = None, kv_offload: bool = False, staging_buffers: int = 2):
        if min(num_layers, max_sequence_length, num_query_groups, head_dim, max_batch_size) <= 0:
            raise ValueError("all sizes must be positive")
        self.num_layers = num_layers
        self.max_sequence_length = max_sequence_length
        self.max_batch_size = max_batch_size
        self.kv_offload = bool(kv_offload)
        rows = max_sequence_length * max_batch_size
        # (with kv_offload the budget is for the device side: the staging ring)
        need = self.bytes_needed(min(num_layers, staging_buffers) if kv_offload else num_layers, max_sequence_length,
                                 num_query_groups, head_dim, max_batch_size, dtype)
        if memory_budget_bytes is not None and need > memory_budget_bytes:
            raise MemoryError(f"KV caches need {need / 2**30:.1f} GiB, budget is {memory_budget_bytes / 2**30:.1f} GiB")
        if not kv_offload:
            self.buffer = torch.empty(num_layers, rows, num_query_groups, 2 * head_dim, dtype=dtype, device=device)
            return
        if max_batch_size != 1:
            raise ValueError("kv_offload runs at batch 1 (as the cached path of the layer does)")
        if staging_buffers < 1:
            raise ValueError("kv_offload needs at least one staging buffer")
        dev = torch.device("cuda" if device is None else device)
        if dev.type != "cuda":
            raise ValueError("kv_offload stages pinned host memory through a GPU: the arena's device must be one")
        self.buffer = None
        # pinned memory is allocated as such (registering existing memory is not available everywhere)
        self.host = torch.empty(num_layers, rows, num_query_groups, 2 * head_dim, dtype=dtype, pin_memory=True)
        n_stage = min(num_layers, staging_buffers)
        self.stages = [torch.empty(rows, num_query_groups, 2 * head_dim, dtype=dtype, device=dev) for _ in range(n_stage)]
        self.stage_holds = [None] * n_stage  # (layer index, rows valid) of the copy issued into each stage
        self.stage_ready = [torch.cuda.Event() for _ in range(n_stage)]
        self.copy_stream = torch.cuda.Stream(device=dev)  # default priority
        self.layers = [OffloadedKVCache(self, i) for i in range(num_layers)]

    @staticmethod
    def bytes_needed(num_layers: int, max_sequence_length: int, num_query_groups: int, head_dim: int = 128,
                     max_batch_size: int = 1, dtype: torch.dtype = torch.bfloat16) -> int:
        return (num_layers * max_sequence_length * max_batch_size * num_query_groups * 2 * head_dim
                * torch.empty((), dtype=dtype).element_size())

    def layer(self, index: int):
        """Layer `index`'s cache: a view of the arena, or the OffloadedKVCache that stands for it."""
        return self.layers[index] if self.kv_offload else self.buffer[index]

    def synchronize(self) -> None:
        """kv_offload: waits until every copy issued so far has landed (before the host copies are read)."""
        if self.kv_offload:
            self.copy_stream.synchronize()

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
            inference_params.key_value_memory_dict[n] = self.layer(i)
        return inference_params.key_value_memory_dict


class OffloadedKVCache:
    """What `key_value_memory_dict[layer_number]` holds under kv_offload (the reference keeps a pinned host tensor
    there and copies its prefix to the GPU in every layer forward, inference/model/dit/dit_module.py:803-811, 915,
    923-929).  Same data flow, arranged for overlap: the cached prefix is copied into a device staging buffer on the
    arena's copy stream, the layer appends its new rows there and attends in place exactly as with a resident cache,
    and the rows to be persisted go back to the host behind the attention launch.  When the arena has a second staging
    buffer, staging layer i also starts the copy for layer i + 1 (the layers of one denoising step read the same
    prefix length), so that only the first layer of a step waits for PCIe.

    All copies run in order on one stream: a staging buffer is handed to its next layer only behind the copy-out of
    its previous one, which in turn waits for that layer's attention launch."""

    def __init__(self, arena: KVCacheArena, index: int):
        self.arena, self.index = arena, index
        self._stage = None  # staging buffer in use between stage() and release()

    @property
    def host(self) -> torch.Tensor:
        return self.arena.host[self.index]

    @property
    def shape(self):
        return self.host.shape

    def _issue(self, stage: int, rows: int) -> None:
        a = self.arena
        with torch.cuda.stream(a.copy_stream):
            if rows:
                a.stages[stage][:rows].copy_(self.host[:rows], non_blocking=True)
            a.stage_ready[stage].record(a.copy_stream)
        a.stage_holds[stage] = (self.index, rows)

    def stage(self, prefix_rows: int) -> torch.Tensor:
        """-> the device buffer [rows, Hkv, 2D] whose first `prefix_rows` rows are this layer's cached prefix; the
        current stream waits for the copy.  Starts the same copy for the next layer into the next staging buffer."""
        a = self.arena
        if self._stage is not None:
            raise RuntimeError("stage() twice without release()")
        if not 0 <= prefix_rows <= self.host.shape[0]:
            raise ValueError("prefix_rows outside the cache")
        n = len(a.stages)
        s = self.index % n
        if a.stage_holds[s] != (self.index, prefix_rows):
            self._issue(s, prefix_rows)
        torch.cuda.current_stream(a.stages[s].device).wait_event(a.stage_ready[s])
        a.stage_holds[s] = None  # the layer is about to append: the buffer no longer equals a host prefix
        self._stage = s
        nxt = self.index + 1
        if (n > 1 and nxt < a.num_layers and a.stage_holds[nxt % n] != (nxt, prefix_rows)
                and all(layer._stage != nxt % n for layer in a.layers)):
            a.layers[nxt]._issue(nxt % n, prefix_rows)
        return a.stages[s]

    def release(self, start: int = 0, n_keep: int = 0) -> None:
        """Call behind the launches that read the staging buffer: rows [start, start + n_keep) (the chunks this
        forward persists) go back to the host, and the buffer becomes available to the next layer that maps to it."""
        a = self.arena
        if self._stage is None:
            raise RuntimeError("release() without stage()")
        s, self._stage = self._stage, None
        done = torch.cuda.Event()
        done.record(torch.cuda.current_stream(a.stages[s].device))
        a.copy_stream.wait_event(done)
        if n_keep:
            with torch.cuda.stream(a.copy_stream):
                self.host[start:start + n_keep].copy_(a.stages[s][start:start + n_keep], non_blocking=True)
            # a prefix of this layer copied ahead of time no longer equals the host rows
            a.stage_holds = [None if h is not None and h[0] == self.index else h for h in a.stage_holds]


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
