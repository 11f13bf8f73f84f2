"""2-D RoPE tables in the layout my_rope_fn reads.  Mirrors gen_rope_freq / rope /
RopeEmbedding and RopeAttnProcessor.register_rope_emb of the reference
(models/rope_dit_transformer_2d.py:71-109, 153-173)."""
from __future__ import annotations

from typing import Sequence

import torch

from .zorder import zorder_perm


def gen_rope_freq(dim: int, theta: float) -> torch.Tensor:
    """omega_j = theta^(-2j/dim), j = 0 .. dim/2-1, fp64 (:71-74)."""
    return 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float64) / dim))


def rope(pos: torch.Tensor, dim: int, theta: float) -> torch.Tensor:
    """[sin(pos*w0), cos(pos*w0), sin(pos*w1), ...] per position (:77-90)."""
    assert dim % 2 == 0, "The dimension must be even."
    ang = pos.double()[..., None] * gen_rope_freq(dim, theta).to(pos.device)
    return torch.stack([torch.sin(ang), torch.cos(ang)], dim=-1).reshape(-1, dim)


class RopeEmbedding(torch.nn.Module):
    """(:93-109) ids (..., n, n_axes) -> (n, sum(axes_dim)) table."""

    def __init__(self, dim: int, theta: int, axes_dim: Sequence[int]):
        super().__init__()
        self.dim, self.theta, self.axes_dim = dim, theta, list(axes_dim)

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        if ids.dim() == 3:
            ids = ids[0]
        return torch.cat([rope(ids[..., i], self.axes_dim[i], self.theta) for i in range(ids.shape[-1])], dim=-1)


def rope_table(side: int, axes_dim: Sequence[int] = (32, 32), theta: float = 10000.0,
               dtype: torch.dtype = torch.bfloat16, zorder: bool = True) -> torch.Tensor:
    """The table register_rope_emb builds for a side x side pixel grid at patch_size 1 (:153-173):
    axis 0 = row id, axis 1 = column id, rows of the table in Z-order when `zorder`."""
    pos = torch.arange(side, dtype=torch.float32)
    ids = torch.stack([pos[:, None].expand(side, side), pos[None, :].expand(side, side)], dim=-1).reshape(side * side, 2)
    if zorder:
        ids = ids[zorder_perm(side)[1]]
    return RopeEmbedding(sum(axes_dim), theta, axes_dim)(ids).to(dtype)
