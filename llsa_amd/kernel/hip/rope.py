"""RoPE rotation with a precomputed [S, D] table of interleaved (sin, cos).  Mirrors
kernel/triton/rope.py: `my_rope_fn(x, freq)`."""
from __future__ import annotations

import torch

from ._common import HEAD_DIM, as_rows, i64x, lib_for, ptr, require_bf16, stream_of


def _rope(lib, bwd, x, freq):
    require_bf16(x, freq)
    B, H, S, D = x.shape
    if D != HEAD_DIM:
        raise NotImplementedError(f"my_rope_fn needs head dim {HEAD_DIM} (got {D})")
    xr = as_rows(x)
    y = torch.empty_like(xr)
    fn = lib.rope_bwd if bwd else lib.rope_fwd
    s = lambda t: i64x((t.stride(0), t.stride(1), t.stride(2)))
    lib.check(fn(ptr(xr), s(xr), ptr(freq), ptr(y), s(y), B, H, S, stream_of(lib, x)), "my_rope_fn")
    return y


class MyRopeFunction(torch.autograd.Function):
    """rope.py:100-145."""

    @staticmethod
    def forward(ctx, x, freq):
        assert x.dim() == 4 and freq.dim() == 2, "x:[B,H,S,D], freq:[S,D]"
        B, H, S, D = x.shape
        assert D % 2 == 0, "D must be even (pairs of cos/sin)."
        assert freq.shape[0] == S and freq.shape[1] == D
        lib = lib_for(x, freq)
        freq = freq.contiguous()
        ctx.save_for_backward(freq)
        return _rope(lib, False, x, freq)

    @staticmethod
    def backward(ctx, grad_output):
        freq, = ctx.saved_tensors
        lib = lib_for(grad_output)
        return _rope(lib, True, grad_output, freq), None


my_rope_fn = MyRopeFunction.apply
