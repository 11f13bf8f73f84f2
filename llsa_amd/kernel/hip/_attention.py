"""Launchers of the forward / backward attention kernels shared by the l1 and l2 modules."""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from ..._lib import AttnBwdArgs, AttnFwdArgs
from ._common import BLOCK, as_rows, lib_for, ptr, require_bf16, require_head_dim, s3, stream_of
from .indices_transpose import transpose_indices


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


def _tiles(tiles, need):
    """tiles: dict name -> tensor or None; need: dict name -> (source tensor, kind).  Computes the
    missing ones with as few launches as possible and returns the completed dict."""
    from .mean_pool import operand_tiles
    tiles = dict(tiles or {})
    by_src = {}
    for name, (src, kind) in need.items():
        if tiles.get(name) is None:
            by_src.setdefault(id(src), [src, "", []])
            by_src[id(src)][1] += kind
            by_src[id(src)][2].append(name)
    jobs = list(by_src.values())
    for i in range(0, len(jobs), 4):
        chunk = jobs[i:i + 4]
        specs = [(src, "".join(k for k in "rt" if k in kinds)) for src, kinds, _ in chunk]
        got = iter(operand_tiles(*specs))
        for (src, kinds, names), (_, kk) in zip(chunk, specs):
            made = {k: next(got) for k in kk}
            for name in names:
                tiles[name] = made[need[name][1]]
    return tiles


def attn_fwd(q, k, v, pk, pv, indices, token_weight, pk2=None, pv2=None, p_indices=None, token_weight_2=1.0,
             tiles=None):
    """Forward.  `tiles` may carry operand tiles the caller already has (keys qr, kr, vt, pkr, pvt,
    pk2r, pv2t); the rest are computed here.  Returns (o, lse)."""
    levels = 1 if pk2 is None else 2
    lib = lib_for(q, k, v, pk, pv, pk2, pv2)
    require_bf16(q, k, v, pk, pv, pk2, pv2)
    require_head_dim(q)
    _check_shapes(q, k, v, pk, pv, pk2, pv2, levels)
    B, H, N, D = q.shape
    T = indices.shape[-1]
    T2 = p_indices.shape[-1] if levels == 2 else 0
    need = dict(qr=(q, "r"), kr=(k, "r"), vt=(v, "t"), pkr=(pk, "r"), pvt=(pv, "t"))
    if levels == 2:
        need.update(pk2r=(pk2, "r"), pv2t=(pv2, "t"))
    tl = _tiles(tiles, need)
    idx = indices.to(torch.int32).contiguous()
    pidx = p_indices.to(torch.int32).contiguous() if levels == 2 else None
    o = torch.empty_like(q) if rows_ok8(q) else torch.empty(q.shape, device=q.device, dtype=q.dtype)
    lse = torch.empty(B, H, N, device=q.device, dtype=torch.float32)
    a = AttnFwdArgs()
    a.qr, a.kr, a.vt = (tl[n].data_ptr() for n in ("qr", "kr", "vt"))
    a.idx = idx.data_ptr()
    a.o, (a.sob, a.soh, a.son) = o.data_ptr(), s3(o)
    a.lse = lse.data_ptr()
    a.B, a.H, a.N, a.T, a.levels = B, H, N, T, levels
    a.lvl[0].kr, a.lvl[0].vt, a.lvl[0].w = tl["pkr"].data_ptr(), tl["pvt"].data_ptr(), float(token_weight)
    if levels == 2:
        a.lvl[0].sel, a.lvl[0].T = pidx.data_ptr(), T2
        a.lvl[1].kr, a.lvl[1].vt, a.lvl[1].w = tl["pk2r"].data_ptr(), tl["pv2t"].data_ptr(), float(token_weight_2)
    lib.check(lib.attn_fwd(C.byref(a), stream_of(lib, q)), "attn_fwd")
    return o, lse


def rows_ok8(t):
    """Rows start 8-byte aligned with unit channel stride (what the 8-byte output stores need)."""
    return t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(s % 4 == 0 for s in t.stride()[:-1])


def attn_bwd(do, q, k, v, pk, pv, o, lse, indices, token_weight, coarse_grad_weight, pk2=None, pv2=None,
             p_indices=None, token_weight_2=1.0, tiles=None, freq_dq: Optional[torch.Tensor] = None, stages: int = 0,
             csr=None, fold_pooled: bool = False, freq_dk: Optional[torch.Tensor] = None):
    """Backward.  Returns (dq, dk, dv, dpk, dpv[, dpk2, dpv2]) with the reference's conventions:
    every gradient is `empty_like` of its primal; the pooled gradients are NOT yet folded
    into dk / dv (autograd, or pool_bwd_accum, does that) unless `fold_pooled` is set, in which case
    the fine pass adds them on its way out (same roundings) and rotates dk back with `freq_dk`.  `tiles` may carry operand tiles the
    caller already has (qr, kr, vr, pkr, pvr, pk2r, pv2r).  `stages` (a mask of
    the LLSA_BWD_* bits of include/llsa_hip.h) launches only some of the kernels, for profiling."""
    levels = 1 if pk2 is None else 2
    lib = lib_for(do, q, k, v, pk, pv, pk2, pv2, o, lse)
    require_bf16(do, q, k, v, pk, pv, pk2, pv2, o)
    require_head_dim(q)
    _check_shapes(q, k, v, pk, pv, pk2, pv2, levels)
    B, H, N, D = q.shape
    T = indices.shape[-1]
    T2 = p_indices.shape[-1] if levels == 2 else 0
    do, o = as_rows(do), as_rows(o)
    need = dict(qr=(q, "r"), kr=(k, "r"), vr=(v, "r"), pkr=(pk, "r"), pvr=(pv, "r"))
    if levels == 2:
        need.update(pk2r=(pk2, "r"), pv2r=(pv2, "r"))
    tl = _tiles(tiles, need)
    idx = indices.to(torch.int32).contiguous()
    if levels == 2:
        pidx = p_indices.to(torch.int32).contiguous()
    if csr is not None:                       # (off, flat, work[, poff, pflat, pinv]) from transpose_indices
        off, flat, work = csr[:3]
        if levels == 2:
            poff, _, pinv = csr[3:6]
    else:
        off, flat, work = transpose_indices(idx, N // BLOCK, lib.fine_chunk(N))
        if levels == 2:
            # A row that names a block twice would give both entries one inverse position and leave another slot of the
            # segment unwritten (the kernels assume what a top-k guarantees): a caller's own p_indices are checked.
            if T2 > 1 and bool((pidx.sort(-1).values.diff(dim=-1) == 0).any()):
                raise ValueError("p_indices: a row names a block twice")
            poff, _, pinv = transpose_indices(pidx, N // (BLOCK * BLOCK), inverse=True)
    mk = lambda t: torch.empty_like(t) if rows_ok8(t) else torch.empty(t.shape, device=t.device, dtype=t.dtype)
    dq, dk, dv = mk(q), mk(k), mk(v)
    dpk, dpv = torch.empty_like(pk, memory_format=torch.contiguous_format), torch.empty_like(pv, memory_format=torch.contiguous_format)
    ws_bytes = lib.attn_bwd_workspace_bytes(B, H, N, (C.c_int32 * levels)(*([T, T2][:levels])), levels)
    ws = torch.empty(ws_bytes, device=q.device, dtype=torch.uint8)
    a = AttnBwdArgs()
    a.dout, (a.sdob, a.sdoh, a.sdon) = do.data_ptr(), s3(do)
    a.o, (a.sob, a.soh, a.son) = o.data_ptr(), s3(o)
    lse = lse.contiguous()
    a.lse = lse.data_ptr()
    for n in ("qr", "kr", "vr"):
        setattr(a, n, tl[n].data_ptr())
    a.idx, a.off, a.flat, a.work = idx.data_ptr(), off.data_ptr(), flat.data_ptr(), work.data_ptr()
    a.dq, (a.sdqb, a.sdqh, a.sdqn) = dq.data_ptr(), s3(dq)
    a.dk, (a.sdkb, a.sdkh, a.sdkn) = dk.data_ptr(), s3(dk)
    a.dv, (a.sdvb, a.sdvh, a.sdvn) = dv.data_ptr(), s3(dv)
    l1 = a.lvl[0]
    l1.kr, l1.vr, l1.dk, l1.dv = tl["pkr"].data_ptr(), tl["pvr"].data_ptr(), dpk.data_ptr(), dpv.data_ptr()
    l1.w, l1.gw = float(token_weight), float(coarse_grad_weight)
    outs = [dq, dk, dv, dpk, dpv]
    if levels == 2:
        dpk2 = torch.empty_like(pk2, memory_format=torch.contiguous_format)
        dpv2 = torch.empty_like(pv2, memory_format=torch.contiguous_format)
        l1.sel, l1.off, l1.inv, l1.T = pidx.data_ptr(), poff.data_ptr(), pinv.data_ptr(), T2
        l2 = a.lvl[1]
        l2.kr, l2.vr, l2.dk, l2.dv = tl["pk2r"].data_ptr(), tl["pv2r"].data_ptr(), dpk2.data_ptr(), dpv2.data_ptr()
        l2.w = l2.gw = float(token_weight_2)
        outs += [dpk2, dpv2]
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws_bytes
    if freq_dq is not None:
        require_bf16(freq_dq)
        freq_dq = freq_dq.contiguous()
        a.freq_dq = freq_dq.data_ptr()
    a.B, a.H, a.N, a.T, a.levels = B, H, N, T, levels
    if freq_dk is not None:
        require_bf16(freq_dk)
        freq_dk = freq_dk.contiguous()
        a.freq_dk = freq_dk.data_ptr()
    a.stages = stages
    a.fold_pooled = int(bool(fold_pooled))
    lib.check(lib.attn_bwd(C.byref(a), stream_of(lib, q)), "attn_bwd")
    return tuple(outs)
