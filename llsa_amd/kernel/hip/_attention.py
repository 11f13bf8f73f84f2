"""Launchers of the forward / backward attention kernels shared by the l1 and l2 modules."""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from ..._lib import CHUNK_COARSE, CHUNK_FINE, AttnBwdArgs, AttnFwdArgs
from ._common import BLOCK, as_rows, lib_for, ptr, require_bf16, require_head_dim, s3, stream_of
from .indices_transpose import transpose_indices
from .mean_pool import block_transpose


def _check_shapes(q, k, v, pk, pv, pk2, pv2, levels):
    B, H, N, D = q.shape
    if k.shape != q.shape or v.shape != q.shape:
        raise ValueError("self-attention only: q, k, v must have the same shape")
    n1 = N // BLOCK
    if pk.shape != (B, H, n1, D) or pv.shape != (B, H, n1, D):
        raise ValueError(f"pooled k/v must be {(B, H, n1, D)}")
    if levels == 2 and (pk2.shape != (B, H, n1 // BLOCK, D) or pv2.shape != (B, H, n1 // BLOCK, D)):
        raise ValueError(f"level-2 pooled k/v must be {(B, H, n1 // BLOCK, D)}")
    mult = 1024 if levels == 1 else 16384
    if N % mult != 0:
        raise ValueError(f"llsa_l{levels} needs a token count that is a multiple of {mult} (got {N})")


def attn_fwd(q, k, v, pk, pv, indices, token_weight, pk2=None, pv2=None, p_indices=None, token_weight_2=1.0,
             vt=None, pvt=None, pv2t=None):
    """Forward.  vt / pvt / pv2t are the block-transposed copies of v / pv / pv2; computed here
    when the caller does not have them.  Returns (o, lse)."""
    levels = 1 if pk2 is None else 2
    lib = lib_for(q, k, v, pk, pv, pk2, pv2)
    require_bf16(q, k, v, pk, pv, pk2, pv2)
    require_head_dim(q)
    _check_shapes(q, k, v, pk, pv, pk2, pv2, levels)
    B, H, N, D = q.shape
    T = indices.shape[-1]
    T2 = p_indices.shape[-1] if levels == 2 else 0
    q, k = as_rows(q), as_rows(k)
    pk = pk.contiguous()
    if vt is None or pvt is None or (levels == 2 and pv2t is None):
        if levels == 2:
            vt, pvt, pv2t = block_transpose(v, pv, pv2)
        else:
            vt, pvt = block_transpose(v, pv)
    idx = indices.to(torch.int32).contiguous()
    pidx = p_indices.to(torch.int32).contiguous() if levels == 2 else None
    o = torch.empty_like(q)
    lse = torch.empty(B, H, N, device=q.device, dtype=torch.float32)
    a = AttnFwdArgs()
    a.q, (a.sqb, a.sqh, a.sqn) = q.data_ptr(), s3(q)
    a.k, (a.skb, a.skh, a.skn) = k.data_ptr(), s3(k)
    a.vt, a.pk, a.pvt = vt.data_ptr(), pk.data_ptr(), pvt.data_ptr()
    if levels == 2:
        pk2 = pk2.contiguous()
        a.pk2, a.pv2t, a.pidx = pk2.data_ptr(), pv2t.data_ptr(), pidx.data_ptr()
    a.idx = idx.data_ptr()
    a.o, (a.sob, a.soh, a.son) = o.data_ptr(), s3(o)
    a.lse = lse.data_ptr()
    a.B, a.H, a.N, a.T, a.T2, a.levels = B, H, N, T, T2, levels
    a.w1, a.w2 = float(token_weight), float(token_weight_2)
    lib.check(lib.attn_fwd(C.byref(a), stream_of(lib, q)), "attn_fwd")
    return o, lse


def attn_bwd(do, q, k, v, pk, pv, o, lse, indices, token_weight, coarse_grad_weight, pk2=None, pv2=None,
             p_indices=None, token_weight_2=1.0, qt=None, kt=None, pkt=None, pk2t=None,
             freq_dq: Optional[torch.Tensor] = None, stages: int = 0, csr=None):
    """Backward.  Returns (dq, dk, dv, dpk, dpv[, dpk2, dpv2]) with the reference's conventions:
    every gradient is `empty_like` of its primal; the pooled gradients are NOT yet folded
    into dk / dv (autograd, or pool_bwd_accum, does that).  `stages` (a mask of the LLSA_BWD_*
    bits of include/llsa_hip.h) launches only some of the kernels, for profiling."""
    levels = 1 if pk2 is None else 2
    lib = lib_for(do, q, k, v, pk, pv, pk2, pv2, o, lse)
    require_bf16(do, q, k, v, pk, pv, pk2, pv2, o)
    require_head_dim(q)
    _check_shapes(q, k, v, pk, pv, pk2, pv2, levels)
    B, H, N, D = q.shape
    T = indices.shape[-1]
    T2 = p_indices.shape[-1] if levels == 2 else 0
    do, q, k, v, o = as_rows(do), as_rows(q), as_rows(k), as_rows(v), as_rows(o)
    pk, pv = pk.contiguous(), pv.contiguous()
    if levels == 2:
        pk2, pv2 = pk2.contiguous(), pv2.contiguous()
    need = [t for t, have in ((q, qt), (k, kt), (pk, pkt)) if have is None]
    if levels == 2 and pk2t is None:
        need.append(pk2)
    if need:
        got = iter(block_transpose(*need))
        qt = qt if qt is not None else next(got)
        kt = kt if kt is not None else next(got)
        pkt = pkt if pkt is not None else next(got)
        if levels == 2 and pk2t is None:
            pk2t = next(got)
    idx = indices.to(torch.int32).contiguous()
    if levels == 2:
        pidx = p_indices.to(torch.int32).contiguous()
    if csr is not None:                       # (off, flat, work[, poff, pflat, pwork]) from transpose_indices
        off, flat, work = csr[:3]
        if levels == 2:
            poff, pflat, pwork = csr[3:6]
    else:
        off, flat, work = transpose_indices(idx, N // BLOCK, CHUNK_FINE)
        if levels == 2:
            poff, pflat, pwork = transpose_indices(pidx, N // (BLOCK * BLOCK), CHUNK_COARSE)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dpk, dpv = torch.empty_like(pk), torch.empty_like(pv)
    ws_bytes = lib.attn_bwd_workspace_bytes(B, H, N, T, T2, levels)
    ws = torch.empty(ws_bytes, device=q.device, dtype=torch.uint8)
    a = AttnBwdArgs()
    a.dout, (a.sdob, a.sdoh, a.sdon) = do.data_ptr(), s3(do)
    a.q, (a.sqb, a.sqh, a.sqn) = q.data_ptr(), s3(q)
    a.k, (a.skb, a.skh, a.skn) = k.data_ptr(), s3(k)
    a.v, (a.svb, a.svh, a.svn) = v.data_ptr(), s3(v)
    a.o, (a.sob, a.soh, a.son) = o.data_ptr(), s3(o)
    lse = lse.contiguous()
    a.lse, a.pk, a.pv = lse.data_ptr(), pk.data_ptr(), pv.data_ptr()
    a.qt, a.kt, a.pkt = qt.data_ptr(), kt.data_ptr(), pkt.data_ptr()
    a.idx, a.off, a.flat, a.work = idx.data_ptr(), off.data_ptr(), flat.data_ptr(), work.data_ptr()
    a.dq, (a.sdqb, a.sdqh, a.sdqn) = dq.data_ptr(), s3(dq)
    a.dk, (a.sdkb, a.sdkh, a.sdkn) = dk.data_ptr(), s3(dk)
    a.dv, (a.sdvb, a.sdvh, a.sdvn) = dv.data_ptr(), s3(dv)
    a.dpk, a.dpv = dpk.data_ptr(), dpv.data_ptr()
    outs = [dq, dk, dv, dpk, dpv]
    if levels == 2:
        dpk2, dpv2 = torch.empty_like(pk2), torch.empty_like(pv2)
        a.pk2, a.pv2, a.pk2t = pk2.data_ptr(), pv2.data_ptr(), pk2t.data_ptr()
        a.pidx, a.poff, a.pflat, a.pwork = pidx.data_ptr(), poff.data_ptr(), pflat.data_ptr(), pwork.data_ptr()
        a.dpk2, a.dpv2 = dpk2.data_ptr(), dpv2.data_ptr()
        outs += [dpk2, dpv2]
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws_bytes
    if freq_dq is not None:
        require_bf16(freq_dq)
        freq_dq = freq_dq.contiguous()
        a.freq_dq = freq_dq.data_ptr()
    a.B, a.H, a.N, a.T, a.T2, a.levels = B, H, N, T, T2, levels
    a.w1, a.w2, a.cgw1 = float(token_weight), float(token_weight_2), float(coarse_grad_weight)
    a.stages = stages
    lib.check(lib.attn_bwd(C.byref(a), stream_of(lib, q)), "attn_bwd")
    return tuple(outs)
