"""Z-order (Morton) token permutation.  Mirrors gen_permuatations of the reference
(models/rope_dit_transformer_2d.py:714-732): `gen_permutations(log_num_tokens)` returns
(perm, inv_perm) for a grid of side 2^(1+log_num_tokens); tokens are put in Z-order with
x[:, inv_perm] and restored with x[:, perm] (:963-965, :1028-1030)."""
from __future__ import annotations

import torch


def morton_codes(side: int) -> torch.Tensor:
    """(side, side) table of Z-order positions: bit l of the row lands on bit 2l+1, bit l of the
    column on bit 2l, so the order inside every 2x2 cell is [[0, 1], [2, 3]]."""
    if side < 1 or side & (side - 1):
        raise ValueError("side must be a power of two")

    def spread(v: torch.Tensor) -> torch.Tensor:     # abcd -> 0a0b0c0d
        v = v.clone()
        v = (v | (v << 8)) & 0x00FF00FF
        v = (v | (v << 4)) & 0x0F0F0F0F
        v = (v | (v << 2)) & 0x33333333
        v = (v | (v << 1)) & 0x55555555
        return v

    i = torch.arange(side, dtype=torch.int64)
    return (spread(i)[:, None] << 1) | spread(i)[None, :]


def zorder_perm(side: int):
    """perm[r*side + c] = z, inv_perm[z] = r*side + c."""
    perm = morton_codes(side).flatten()
    inv_perm = torch.empty_like(perm)
    inv_perm[perm] = torch.arange(side * side)
    return perm, inv_perm


def gen_permutations(log_num_tokens: int):
    """Same arguments and results as the reference's gen_permuatations (sic)."""
    return zorder_perm(2 ** (1 + log_num_tokens))


gen_permuatations = gen_permutations      # the reference's spelling


# Host-side helpers for preparing inputs and tables (plain indexing on whatever device x lives on).
# Inside a model the permutation of (B, N, C) activations is llsa_amd.permute_tokens, a HIP kernel.
def to_zorder(x: torch.Tensor, side: int, dim: int = 1) -> torch.Tensor:
    _, inv_perm = zorder_perm(side)
    return x.index_select(dim, inv_perm.to(x.device))


def from_zorder(x: torch.Tensor, side: int, dim: int = 1) -> torch.Tensor:
    perm, _ = zorder_perm(side)
    return x.index_select(dim, perm.to(x.device))
