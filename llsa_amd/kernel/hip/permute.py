"""Token permutation of a (B, N, C) tensor, the form in which the model puts its tokens into
Z-order and back (models/rope_dit_transformer_2d.py:963-965 `hidden_states[:, fwd_perm, :]`,
:1028-1030 `hidden_states[:, bwd_perm, :]`, :1020 after the REPA pooling)."""
from __future__ import annotations

import torch

from ._common import lib_for, ptr, stream_of


def gather_tokens(x: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
    """y[:, i, :] = x[:, index[i], :].  x is (B, N, C) with contiguous rows of a multiple of 16
    bytes; index is an integer tensor on x's device (int32 is used as it is)."""
    if x.dim() != 3:
        raise ValueError("gather_tokens expects (B, N, C)")
    lib = lib_for(x, index)
    B, N, Cc = x.shape
    row_bytes = Cc * x.element_size()
    if row_bytes % 16:
        raise NotImplementedError(f"rows of {row_bytes} bytes: a multiple of 16 is needed")
    if not (x.stride(2) == 1 and x.stride(1) == Cc and (x.stride(0) * x.element_size()) % 16 == 0 and x.data_ptr() % 16 == 0):
        x = x.contiguous()
    if index.dtype != torch.int32 or not index.is_contiguous():
        index = index.to(torch.int32).contiguous()
    n_out = index.numel()
    y = torch.empty(B, n_out, Cc, dtype=x.dtype, device=x.device)
    if B == 0 or n_out == 0:
        return y
    es = x.element_size()
    lib.check(lib.gather_rows(ptr(x), ptr(y), ptr(index), B, n_out, N, row_bytes, x.stride(0) * es, y.stride(0) * es,
                              stream_of(lib, x)), "gather_tokens")
    return y


class PermuteTokens(torch.autograd.Function):
    """x[:, perm, :] for a permutation `perm` whose inverse is `inv`: the gradient is dy[:, inv, :]."""

    @staticmethod
    def forward(ctx, x, perm, inv):
        ctx.save_for_backward(inv)
        return gather_tokens(x, perm)

    @staticmethod
    def backward(ctx, dy):
        inv, = ctx.saved_tensors
        return gather_tokens(dy, inv), None, None


def permute_tokens(x: torch.Tensor, perm: torch.Tensor, inv: torch.Tensor) -> torch.Tensor:
    return PermuteTokens.apply(x, perm, inv)
