"""Mean pooling over consecutive tokens.  Mirrors the reference module
kernel/triton/mean_pool.py: `mean_pool1d(x, k, format)` is an autograd function with the
same rounding (accumulator in the tensor dtype, token order).  `pool_pyramid` is the fused
launcher the operators use: several tensors, two levels, optional RoPE and the
block-transposed copies in one pass."""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from ..._lib import PoolItem
from ._common import BLOCK, HEAD_DIM, as_rows, i64x, lib_for, ptr, require_bf16, stream_of

_DTYPES = {torch.bfloat16: 0, torch.float32: 1}


def _pool_launch(lib, bwd, a, o, B, H, S_out, C, K):
    if a.dtype not in _DTYPES:
        raise NotImplementedError(f"mean_pool1d supports bf16 and fp32 (got {a.dtype})")
    fn = lib.mean_pool_bwd if bwd else lib.mean_pool_fwd
    n = S_out if bwd else S_out * K
    lib.check(fn(ptr(a), i64x(a.stride()), ptr(o), i64x(o.stride()), B, H, n, C, K, _DTYPES[a.dtype],
                 stream_of(lib, a)), "mean_pool1d")


class MeanPool1dFunction_BHSC(torch.autograd.Function):
    """mean_pool.py:129-165."""

    @staticmethod
    def forward(ctx, x, kernel_size: int):
        B, H, S, C = x.shape
        assert S % kernel_size == 0
        lib = lib_for(x)
        y = torch.empty((B, H, S // kernel_size, C), device=x.device, dtype=x.dtype)
        _pool_launch(lib, False, x, y, B, H, S // kernel_size, C, kernel_size)
        ctx.kernel_size = kernel_size
        return y

    @staticmethod
    def backward(ctx, dy):
        K = ctx.kernel_size
        B, H, S_out, C = dy.shape
        lib = lib_for(dy)
        dx = torch.empty((B, H, S_out * K, C), device=dy.device, dtype=dy.dtype)
        _pool_launch(lib, True, dy, dx, B, H, S_out, C, K)
        return dx, None


class MeanPool1dFunction_BSC(torch.autograd.Function):
    """mean_pool.py:168-206: the (B,S,C) layout is the (B,1,S,C) case of the same kernel."""

    @staticmethod
    def forward(ctx, x, kernel_size: int):
        B, S, C = x.shape
        assert S % kernel_size == 0
        lib = lib_for(x)
        y = torch.empty((B, S // kernel_size, C), device=x.device, dtype=x.dtype)
        _pool_launch(lib, False, x.unsqueeze(1), y.unsqueeze(1), B, 1, S // kernel_size, C, kernel_size)
        ctx.kernel_size = kernel_size
        return y

    @staticmethod
    def backward(ctx, dy):
        K = ctx.kernel_size
        B, S_out, C = dy.shape
        lib = lib_for(dy)
        dx = torch.empty((B, S_out * K, C), device=dy.device, dtype=dy.dtype)
        _pool_launch(lib, True, dy.unsqueeze(1), dx.unsqueeze(1), B, 1, S_out, C, K)
        return dx, None


def mean_pool1d(x: torch.Tensor, k: int, format='bhsc'):
    """mean_pool.py:209-216."""
    if format == 'bhsc':
        return MeanPool1dFunction_BHSC.apply(x, k)
    elif format == 'bsc':
        return MeanPool1dFunction_BSC.apply(x, k)
    else:
        raise NotImplementedError(f'Format {format} is not implemented for mean_pool1d')


class PoolSpec:
    """What to produce from one (B,H,n,64) bf16 tensor in a pool_pyramid launch: y1 / y2 pooled
    rows, xr / xt operand tiles of the (rotated) tensor, y1r / y1t operand tiles of y1, xrot a
    row-major copy of the rows as transformed (normalised with `gamma` (64) fp32 and `eps` first, then
    rotated)."""

    def __init__(self, x, y1=False, y2=False, xr=False, xt=False, y1r=False, y1t=False, rope=False, xrot=False,
                 gamma=None, eps=0.0, y2r=False, y2t=False):
        self.x, self.y1, self.y2, self.xr, self.xt, self.y1r, self.y1t = x, y1, y2, xr, xt, y1r, y1t
        self.y2r, self.y2t = y2r, y2t              # operand tiles of y2 (n a multiple of 4096)
        self.rope, self.xrot, self.gamma, self.eps = rope, xrot, gamma, eps


def pool_pyramid(specs: Sequence[PoolSpec], freq: Optional[torch.Tensor] = None):
    """One launch of llsa_pool_pyramid_fwd.  Returns, per spec, a dict with the requested
    outputs: y1 (B,H,n/16,64), y2 (B,H,n/256,64), xr / xt (B,H,n/16,1024), y1r / y1t
    (B,H,n/256,1024), y2r / y2t (B,H,n/4096,1024), xrot (B,H,n,64).  The tile layouts are described in include/llsa_hip.h."""
    assert 1 <= len(specs) <= 4
    x0 = specs[0].x
    lib = lib_for(*[s.x for s in specs], freq)
    B, H = x0.shape[0], x0.shape[1]
    items, outs, keep = [], [], []
    for s in specs:
        x = s.x
        require_bf16(x)
        if x.shape[-1] != HEAD_DIM or x.shape[0] != B or x.shape[1] != H:
            raise ValueError("pool_pyramid: all tensors must be (B,H,n,64)")
        x = as_rows(x)
        keep.append(x)
        n = x.shape[2]
        if n % BLOCK != 0:
            raise ValueError(f"token count {n} is not a multiple of {BLOCK}")
        if (s.y2 or s.y1t or s.y1r) and n % (BLOCK * BLOCK) != 0:
            raise ValueError(f"token count {n} is not a multiple of {BLOCK * BLOCK}")
        e = lambda *shape: torch.empty(shape, device=x.device, dtype=x.dtype)
        o = {}
        if s.y1:
            o["y1"] = e(B, H, n // 16, 64)
        if s.y2:
            o["y2"] = e(B, H, n // 256, 64)
        if s.xr:
            o["xr"] = e(B, H, n // 16, 1024)
        if s.xt:
            o["xt"] = e(B, H, n // 16, 1024)
        if s.y1r:
            o["y1r"] = e(B, H, n // 256, 1024)
        if s.y1t:
            o["y1t"] = e(B, H, n // 256, 1024)
        if (s.y2r or s.y2t) and n % 4096 != 0:
            raise ValueError(f"token count {n} is not a multiple of 4096")
        if s.y2r:
            o["y2r"] = e(B, H, n // 4096, 1024)
        if s.y2t:
            o["y2t"] = e(B, H, n // 4096, 1024)
        if s.rope and freq is None:
            raise ValueError("rope requested without a table")
        if s.xrot:
            o["xrot"] = e(B, H, n, 64)
        outs.append(o)
        gamma = None
        if s.gamma is not None:
            gamma = s.gamma.to(device=x.device, dtype=torch.float32).contiguous()
            if gamma.numel() != HEAD_DIM:
                raise ValueError("gamma must have 64 entries")
            keep.append(gamma)
        items.append(PoolItem(x.data_ptr(), x.stride(0), x.stride(1), x.stride(2), n, 1 if s.rope else 0,
                              *(o[k].data_ptr() if k in o else None for k in ("y1", "y2", "xr", "xt", "y1r", "y1t", "xrot")),
                              None if gamma is None else gamma.data_ptr(), float(s.eps), 0,
                              o["y2r"].data_ptr() if "y2r" in o else None, o["y2t"].data_ptr() if "y2t" in o else None))
    if freq is not None:
        require_bf16(freq)
        freq = freq.contiguous()
        if any(s.rope and freq.shape != (s.x.shape[2], HEAD_DIM) for s in specs):
            raise ValueError("rope table must be (n, 64)")
    arr = (PoolItem * len(items))(*items)
    lib.check(lib.pool_pyramid_fwd(arr, len(items), ptr(freq), B, H, stream_of(lib, x0)), "pool_pyramid")
    return outs


def operand_tiles(*specs):
    """specs: (tensor, 'r' | 't' | 'rt').  Up to 4 tensors in one launch; returns a flat list of the
    requested tile tensors in order (R before T for 'rt')."""
    outs = pool_pyramid([PoolSpec(t, xr='r' in k, xt='t' in k) for t, k in specs])
    res = []
    for o, (_, k) in zip(outs, specs):
        if 'r' in k:
            res.append(o["xr"])
        if 't' in k:
            res.append(o["xt"])
    return res


def pool_bwd_accum(dx, dy1, dy2=None, freq=None, out=None):
    """out = rn(dx + rn(g1/16)) per token, g1 = dy1 or rn(dy1 + rn(dy2/16)); with freq the result is
    rotated back.  The fused equivalent of mean_pool backward + autograd's accumulation."""
    lib = lib_for(dx, dy1, dy2, freq)
    require_bf16(dx, dy1, dy2, freq)
    B, H, N, D = dx.shape
    dxr = as_rows(dx)
    if out is None:
        out = torch.empty_like(dxr)
    s = lambda t: i64x((t.stride(0), t.stride(1), t.stride(2)))
    lib.check(lib.pool_bwd_accum(ptr(dxr), s(dxr), ptr(dy1.contiguous()), ptr(None if dy2 is None else dy2.contiguous()),
                                 ptr(out), s(out), ptr(None if freq is None else freq.contiguous()), B, H, N,
                                 stream_of(lib, dx)), "pool_bwd_accum")
    return out
