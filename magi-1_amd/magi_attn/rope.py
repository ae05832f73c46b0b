"""3-D (t, h, w) rotary table of the DiT, built on the device the caller names.

Restates LearnableRotaryEmbeddingCat of the reference (inference/model/dit/dit_module.py:591-596,
599-667, 670-717, 720-770) for its in_pixels=False use: one [S, 96] fp32 table per forward,
[sin(48) | cos(48)], bands ordered [t(16) | h(16) | w(16)]."""
from __future__ import annotations

import math
from typing import List, Optional, Sequence

import torch


def freq_bands(num_bands: int, temperature: float = 10000.0, step: int = 1, device=None) -> torch.Tensor:
    exp = torch.arange(0, num_bands, step, dtype=torch.int64, device=device).to(torch.float32) / num_bands
    return 1.0 / (temperature**exp)


def build_rotary_table(feat_shape: Sequence[int], bands: torch.Tensor,
                       ref_feat_shape: Optional[Sequence[float]] = None) -> torch.Tensor:
    device = bands.device
    axes: List[torch.Tensor] = [torch.arange(s, device=device, dtype=torch.int64).to(torch.float32) for s in feat_shape]
    axes[1] = axes[1] - (feat_shape[1] - 1) / 2
    axes[2] = axes[2] - (feat_shape[2] - 1) / 2
    if ref_feat_shape is not None:
        scaled = []
        for x, f, r in zip(axes, feat_shape, ref_feat_shape):
            if f == 1:
                if r != 1:
                    raise ValueError("ref_feat_shape must be 1 where feat_shape is 1")
                scaled.append(x)
            else:
                scaled.append(x / (f - 1) * (r - 1))
        axes = scaled
    grid = torch.stack(torch.meshgrid(*axes, indexing="ij"), dim=-1).unsqueeze(-1)
    pos = grid * bands
    n = 1
    for s in feat_shape:
        n *= s
    return torch.cat([pos.sin().reshape(n, -1), pos.cos().reshape(n, -1)], dim=-1)


def build_fourier_pos_embed(feat_shape: Sequence[int], bands: Optional[torch.Tensor] = None, num_bands: int = 64,
                            temperature: float = 10000.0, include_grid: bool = False, in_pixels: bool = False,
                            ref_feat_shape: Optional[Sequence[float]] = None, dtype: torch.dtype = torch.float32,
                            device=None, **_unused) -> List[torch.Tensor]:
    """[pos_sin, pos_cos], each feat_shape + [3, num_bands]: the reference's function of this name
    (dit_module.py:599-667) for the token-index positions the DiT uses (in_pixels=False, dit_model.py:76-78); the
    pixel-frequency mode is not part of this path."""
    if in_pixels:
        raise NotImplementedError("the DiT builds its table with in_pixels=False")
    if include_grid:
        raise NotImplementedError("include_grid is not used on this path")
    if bands is None:
        bands = freq_bands(num_bands, temperature=temperature, step=1, device=device)
    table = build_rotary_table(feat_shape, bands, ref_feat_shape)  # [N, 2 * 3 * num_bands] = sin | cos
    half = table.shape[-1] // 2
    shape = list(feat_shape) + [len(feat_shape), bands.numel()]
    return [table[:, :half].reshape(shape).to(dtype), table[:, half:].reshape(shape).to(dtype)]


def build_rotary_pos_embed(feat_shape: Sequence[int], bands: Optional[torch.Tensor] = None, dim: int = 64,
                           temperature: float = 10000.0, in_pixels: bool = False,
                           ref_feat_shape: Optional[Sequence[float]] = None, dtype: torch.dtype = torch.float32,
                           device=None, **_unused):
    """(sin_emb, cos_emb), each [prod(feat_shape), 3 * dim / 8]: dit_module.py:670-717."""
    sin, cos = build_fourier_pos_embed(feat_shape, bands=bands, num_bands=dim // 8, temperature=temperature,
                                       in_pixels=in_pixels, ref_feat_shape=ref_feat_shape, dtype=dtype, device=device)
    n = 1
    for s in feat_shape:
        n *= s
    return sin.reshape(n, -1), cos.reshape(n, -1)


class LearnableRotaryEmbeddingCat(torch.nn.Module):
    """Holds the (learnable) bands and builds the table for a [T, H, W] token grid."""

    def __init__(self, dim: int, temperature: float = 10000.0, device=None, in_pixels: bool = False, **_unused):
        super().__init__()
        if in_pixels:
            raise NotImplementedError("the DiT builds its table with in_pixels=False (dit_model.py:76-78)")
        self.dim = dim
        self.temperature = temperature
        self.bands = torch.nn.Parameter(freq_bands(dim // 8, temperature=temperature, step=1, device=device))

    def get_embed(self, shape: Sequence[int], ref_feat_shape: Optional[Sequence[float]] = None) -> torch.Tensor:
        return build_rotary_table(shape, self.bands.detach(), ref_feat_shape)

    def get_embed_for_forward(self, T: int, H: int, W: int, slice_point: int, denoising_range_num: int) -> torch.Tensor:
        """The slice one forward consumes (inference/model/dit/dit_model.py:151-166): positions are
        absolute in time, so the table covers the cached prefix frames too and the last T*H*W rows
        are returned."""
        frame_in_range = T // denoising_range_num
        T_total = T + frame_in_range * slice_point
        rescale = math.sqrt((H * W) / (16 * 16))
        rope = self.get_embed([T_total, H, W], [T_total, H / rescale, W / rescale])
        return rope[-(T * H * W):].contiguous()
