"""Chunk-window arithmetic that produces the (q_range, k_range) chunk map the attention
kernel walks.  Integer host logic; mirrors the scheduler of the reference
(inference/pipeline/video_generate.py) so the same maps can be produced without it."""
from __future__ import annotations

from typing import List, Sequence, Tuple

import torch


def generate_sequences(chunk_num: int, window_size: int, chunk_offset: int) -> Tuple[List[int], ...]:
    """Per denoising stage (clip_start, clip_end, t_start, t_end); video_generate.py:164-180."""
    clip_start, clip_end, t_start, t_end = [], [], [], []
    for i in range(chunk_offset, chunk_num + window_size - 1):
        clip_start.append(max(chunk_offset, i - window_size + 1))
        clip_end.append(min(chunk_num, i + 1))
        t_start.append(max(0, i - chunk_num + 1))
        rel = i - chunk_offset
        t_end.append(min(window_size, rel + 1) if rel < window_size else window_size)
    return clip_start, clip_end, t_start, t_end


def _to_tensor(rows, device) -> torch.Tensor:
    return torch.tensor(rows, dtype=torch.int32, device=device).reshape(-1, 2)


def generate_default_kvrange(slice_point: int, denoising_range_num: int, chunk_token_nums: int, batch_size: int = 1,
                             device="cpu") -> torch.Tensor:
    """Chunk j of batch b sees every chunk up to itself (video_generate.py:454-465)."""
    range_num = slice_point + denoising_range_num
    rows = []
    for b in range(batch_size):
        for j in range(denoising_range_num):
            rows.append([b * range_num * chunk_token_nums, (b * range_num + slice_point + j + 1) * chunk_token_nums])
    return _to_tensor(rows, device)


def generate_noise2clean_kvrange(slice_point: int, denoising_range_num: int, chunk_token_nums: int,
                                 noise2clean_kvrange: Sequence[int], clean_chunk_kvrange: int,
                                 denoise_step_of_each_chunk: Sequence[int], num_steps: int, batch_size: int = 1,
                                 device="cpu") -> torch.Tensor:
    """Sliding window whose width depends on how far each chunk is denoised (video_generate.py:467-508)."""
    if len(denoise_step_of_each_chunk) != denoising_range_num:
        raise ValueError("one denoise step per chunk is required")
    if len(noise2clean_kvrange) == 0:
        raise ValueError("noise2clean_kvrange is empty")
    if clean_chunk_kvrange == -1:
        clean_chunk_kvrange = noise2clean_kvrange[-1]
    if num_steps % len(noise2clean_kvrange) != 0:
        raise ValueError("num_steps must be a multiple of len(noise2clean_kvrange)")
    per_stage = num_steps // len(noise2clean_kvrange)
    width = []
    for step in denoise_step_of_each_chunk:
        width.append(clean_chunk_kvrange if step == num_steps else noise2clean_kvrange[step // per_stage])
    range_num = slice_point + denoising_range_num
    rows = []
    for b in range(batch_size):
        base = b * range_num
        for j in range(denoising_range_num):
            end = slice_point + j + 1
            rows.append([(base + max(0, end - width[j])) * chunk_token_nums, (base + end) * chunk_token_nums])
    return _to_tensor(rows, device)


def generate_kvrange_for_denoising_video(slice_point, denoising_range_num, chunk_token_nums, noise2clean_kvrange,
                                         clean_chunk_kvrange, denoise_step_of_each_chunk, num_steps, batch_size=1,
                                         device="cpu") -> torch.Tensor:
    """Dispatch of video_generate.py:510-527."""
    if len(noise2clean_kvrange) == 0:
        return generate_default_kvrange(slice_point, denoising_range_num, chunk_token_nums, batch_size, device)
    return generate_noise2clean_kvrange(slice_point, denoising_range_num, chunk_token_nums, noise2clean_kvrange,
                                        clean_chunk_kvrange, denoise_step_of_each_chunk, num_steps, batch_size, device)


def generate_kvrange_for_prefix_video(range_num: int, chunk_token_nums: int, clean_chunk_kvrange: int = -1,
                                      noise2clean_kvrange: Sequence[int] = (), batch_size: int = 1,
                                      device="cpu") -> torch.Tensor:
    """Clean prefix chunks see a fixed number of trailing chunks (video_generate.py:371-387)."""
    if clean_chunk_kvrange != -1:
        prev = clean_chunk_kvrange
    elif len(noise2clean_kvrange) > 0:
        prev = noise2clean_kvrange[-1]
    else:
        prev = 8
    rows = []
    for b in range(batch_size):
        for end in range(1, range_num + 1):
            rows.append([(b * range_num + max(0, end - prev)) * chunk_token_nums, (b * range_num + end) * chunk_token_nums])
    return _to_tensor(rows, device)


def generate_kv_range_for_uncondition(batch: int, chunk_token_nums: int, device="cpu") -> torch.Tensor:
    """Unconditional pass: chunks are batch rows and each sees only itself (dit_model.py:92-101)."""
    return _to_tensor([[i * chunk_token_nums, (i + 1) * chunk_token_nums] for i in range(batch)], device)


def q_ranges_from_chunks(n_chunks: int, chunk_token_nums: int, device="cpu") -> torch.Tensor:
    """q_range[i] = [i*L, (i+1)*L) (dit_model.py:220-222, 246)."""
    return _to_tensor([[i * chunk_token_nums, (i + 1) * chunk_token_nums] for i in range(n_chunks)], device)
