"""qk RMS norm: the normalisation the reference's attention processor applies to q and k
before the RoPE (models/rope_dit_transformer_2d.py:215-219, diffusers' RMSNorm with an fp32
weight).  The forward is fused into the pooling pass (PoolSpec(gamma=, eps=)); this module
has the stand-alone forms."""
from __future__ import annotations

import torch
from torch.autograd import Function

from ._common import HEAD_DIM, as_rows, i64x, lib_for, ptr, require_bf16, require_head_dim, s3, stream_of
from .mean_pool import PoolSpec, pool_pyramid


def rms_norm_fwd(x, gamma, eps):
    """bf16(x * rsqrt(mean(x^2) + eps) * gamma) for x (B,H,N,64) bf16, N a multiple of 16."""
    return pool_pyramid([PoolSpec(x, xrot=True, gamma=gamma, eps=eps)])[0]["xrot"]


def rms_norm_bwd(dy, x, gamma, eps, out=None):
    """(dx, dgamma) for the normalisation above; dx has x's dtype and may be written over dy (out=dy)."""
    lib = lib_for(dy, x)
    require_bf16(dy, x)
    require_head_dim(x)
    B, H, N, _ = x.shape
    dy, x = as_rows(dy), as_rows(x)
    gamma = gamma.to(device=x.device, dtype=torch.float32).contiguous()
    dx = out if out is not None else torch.empty_like(dy)
    dgamma = torch.empty(HEAD_DIM, device=x.device, dtype=torch.float32)
    partials = torch.empty(lib.rmsnorm_bwd_partials(B, H, N), device=x.device, dtype=torch.float32)
    lib.check(lib.rmsnorm_bwd(ptr(dy), i64x(s3(dy)), ptr(x), i64x(s3(x)), ptr(gamma), float(eps), ptr(dx), i64x(s3(dx)), ptr(dgamma),
                              ptr(partials), B, H, N, stream_of(lib, x)), "rmsnorm_bwd")
    return dx, dgamma


class MyRmsNormFunction(Function):
    @staticmethod
    def forward(ctx, x, gamma, eps):
        ctx.save_for_backward(x, gamma)
        ctx.eps = eps
        return rms_norm_fwd(x, gamma, eps)

    @staticmethod
    def backward(ctx, dy):
        x, gamma = ctx.saved_tensors
        dx, dgamma = rms_norm_bwd(dy, x, gamma, ctx.eps)
        return dx, dgamma.to(gamma.dtype), None


def my_rms_norm_fn(x, gamma, eps=1e-5):
    return MyRmsNormFunction.apply(x, gamma, eps)
