"""Synthetic inputs of the benchmark configurations: spatially coherent q/k/v on a Z-ordered
pixel grid, so that block similarity has the structure the selection is designed for."""
from __future__ import annotations

import math

import torch

from .zorder import zorder_perm


def smooth_field(seed: int, B: int, H: int, N: int, D: int, dtype=torch.bfloat16, length_scale: float = 8.0,
                 mix=(0.7, 0.3), zorder: bool = True) -> torch.Tensor:
    """mix[0] * (Gaussian random field with the given length scale in pixels, unit variance per
    (b,h,channel), periodic) + mix[1] * N(0,1) on a sqrt(N) x sqrt(N) grid, permuted raster ->
    Z-order (left in raster order with zorder=False).  CPU, deterministic in `seed`.  Returns (B,H,N,D)."""
    W = math.isqrt(N)
    if W * W != N:
        raise ValueError("N must be a square")
    gen = torch.Generator().manual_seed(seed)
    white = torch.randn(B, H, D, W, W, generator=gen)
    d = torch.minimum(torch.arange(W), W - torch.arange(W)).float()
    kern = torch.exp(-(d[:, None] ** 2 + d[None, :] ** 2) / (2 * length_scale ** 2))
    field = torch.fft.irfft2(torch.fft.rfft2(white) * torch.fft.rfft2(kern), s=(W, W))
    field = field / field.std(dim=(-2, -1), keepdim=True)
    x = mix[0] * field + mix[1] * torch.randn(B, H, D, W, W, generator=gen)
    x = x.reshape(B, H, D, N).transpose(-1, -2)
    if zorder:
        x = x[:, :, zorder_perm(W)[1], :]
    return x.to(dtype).contiguous()
