"""Writes the fixtures in this directory.  Run from the repository root: python tests/golden/make_fixtures.py

generate_sequences_examples.json  the four worked examples the reference keeps in comments next to
                                  generate_sequences (inference/pipeline/video_generate.py:139-161): the only
                                  input/output vectors the reference holds for the attention path.  Typed in by
                                  hand from those comments, not produced by running anything.
layer_small.npz                   one small seeded layer pass (prefix chunk in the cache + 2 denoising chunks):
                                  inputs as bf16 bit patterns and the CPU oracle's outputs.  The reference ships no
                                  tensors for this path, so this fixture is the oracle's own output frozen at a
                                  point where all its pinning tests passed; it guards the oracle against drift
                                  and gives the HIP path a fixed, machine-independent target.
"""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))
from oracle import magi_oracle as O  # noqa: E402

EXAMPLES = [
    {"chunk_num": 8, "window_size": 8, "chunk_offset": 0,
     "clip_start": [0, 0, 0, 0, 0, 0, 0, 0, 1, 2, 3, 4, 5, 6, 7], "clip_end": [1, 2, 3, 4, 5, 6, 7, 8, 8, 8, 8, 8, 8, 8, 8],
     "t_start": [0, 0, 0, 0, 0, 0, 0, 0, 1, 2, 3, 4, 5, 6, 7], "t_end": [1, 2, 3, 4, 5, 6, 7, 8, 8, 8, 8, 8, 8, 8, 8]},
    {"chunk_num": 8, "window_size": 4, "chunk_offset": 0,
     "clip_start": [0, 0, 0, 0, 1, 2, 3, 4, 5, 6, 7], "clip_end": [1, 2, 3, 4, 5, 6, 7, 8, 8, 8, 8],
     "t_start": [0, 0, 0, 0, 0, 0, 0, 0, 1, 2, 3], "t_end": [1, 2, 3, 4, 4, 4, 4, 4, 4, 4, 4]},
    {"chunk_num": 8, "window_size": 4, "chunk_offset": 2,
     "clip_start": [2, 2, 2, 2, 3, 4, 5, 6, 7], "clip_end": [3, 4, 5, 6, 7, 8, 8, 8, 8],
     "t_start": [0, 0, 0, 0, 0, 0, 1, 2, 3], "t_end": [1, 2, 3, 4, 4, 4, 4, 4, 4]},
    {"chunk_num": 8, "window_size": 1, "chunk_offset": 0,
     "clip_start": [0, 1, 2, 3, 4, 5, 6, 7], "clip_end": [1, 2, 3, 4, 5, 6, 7, 8],
     "t_start": [0] * 8, "t_end": [1] * 8},
]

# layer_small: latent chunk 1 x 5 x 8 = 40 tokens, 1 cached chunk + 2 denoising chunks
T_CHUNK, H, W, PREFIX, DENOISE, HQ, HKV, D, SEED = 1, 5, 8, 1, 2, 4, 2, 128, 20240
XLENS = [7, 0]  # cross-attention text lengths per denoising chunk (the second one is empty)


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def layer_small():
    L = T_CHUNK * H * W
    S = DENOISE * L
    g = torch.Generator().manual_seed(SEED)
    rn = lambda *s: torch.randn(*s, generator=g)
    q_raw, k_raw, v_raw = rn(S, HQ, D).bfloat16(), rn(S, HKV, D).bfloat16(), rn(S, HKV, D).bfloat16()
    gq, bq, gk, bk = (rn(D) * 0.2 for _ in range(4))
    prefix_kv = rn(PREFIX * L, HKV, 2 * D).bfloat16()
    xk, xv = rn(sum(XLENS), HKV, D).bfloat16(), rn(sum(XLENS), HKV, D).bfloat16()
    rope = O.rope_for_forward(DENOISE * T_CHUNK, H, W, PREFIX, DENOISE)
    q, kv = O.prologue(q_raw, k_raw, v_raw, rope, gq, bq, gk, bk)
    cache = torch.cat([prefix_kv, kv], 0)
    q_ranges = O.q_ranges_for(DENOISE, L)
    k_ranges = O.default_kvrange(PREFIX, DENOISE, L)
    out = O.range_attention(q, cache[..., :D], cache[..., D:], q_ranges, k_ranges)
    lse = O.range_attention_lse(q, cache[..., :D], cache[..., D:], q_ranges, k_ranges)
    cu_q = np.array([0, L, 2 * L], dtype=np.int32)
    cu_k = np.concatenate([[0], np.cumsum(XLENS)]).astype(np.int32)
    xout = O.varlen_cross_attention(q, xk, xv, cu_q, cu_k)
    return dict(
        q_raw=bits(q_raw), k_raw=bits(k_raw), v_raw=bits(v_raw), prefix_kv=bits(prefix_kv), xk=bits(xk), xv=bits(xv),
        gq=gq.numpy(), bq=bq.numpy(), gk=gk.numpy(), bk=bk.numpy(), rope=rope.numpy(),
        q_ranges=np.asarray(q_ranges, dtype=np.int32), k_ranges=np.asarray(k_ranges, dtype=np.int32), cu_q=cu_q, cu_k=cu_k,
        q=bits(q), kv=bits(kv), out=out.float().numpy(), lse=lse.float().numpy(), xout=xout.float().numpy(),
        dims=np.array([T_CHUNK, H, W, PREFIX, DENOISE, HQ, HKV, D], dtype=np.int32))


if __name__ == "__main__":
    with open(os.path.join(HERE, "generate_sequences_examples.json"), "w") as f:
        json.dump(EXAMPLES, f, indent=1)
    np.savez_compressed(os.path.join(HERE, "layer_small.npz"), **layer_small())
    print("wrote", sorted(os.listdir(HERE)))
