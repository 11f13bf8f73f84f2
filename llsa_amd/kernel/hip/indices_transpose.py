"""Query-major top-k lists -> key-major CSR.  Mirrors kernel/triton/indices_transpose.py."""
from __future__ import annotations

import torch

from ..._lib import TransposeJob
from ._common import lib_for, ptr, stream_of


def transpose_indices(q_topk_indices, k_ntx=None, chunk=0, stream=None, inverse=False):
    """indices_transpose.py:104-109.  Returns (offsets (B,H,1+Kb), flat (B,H,Mb*T)), int32; the
    entries of each segment are in ascending query-block order.  With chunk > 0 a third tensor
    is returned: the work list the backward kernels use to walk every segment in pieces of at
    most `chunk` entries (layout in include/llsa_hip.h).  With inverse=True the last tensor returned is
    inv (B,H,Mb,T): the position in flat of every entry of the input (the backward needs it for the
    selections of the pooled levels).  `stream`: raw handle of the stream to launch on (default: the current one)."""
    lib = lib_for(q_topk_indices)
    B, H, Mb, T = q_topk_indices.shape
    if k_ntx is None:
        k_ntx = Mb
    idx = q_topk_indices.to(torch.int32).contiguous()
    offsets = torch.empty(B, H, 1 + k_ntx, device=idx.device, dtype=torch.int32)
    flat = torch.empty(B, H, Mb * T, device=idx.device, dtype=torch.int32)
    work = None
    if chunk > 0:
        work = torch.empty(B, H, lib.work_list_len(Mb, k_ntx, T, chunk), device=idx.device, dtype=torch.int32)
    inv = torch.empty(B, H, Mb, T, device=idx.device, dtype=torch.int32) if inverse else None
    lib.check(lib.transpose_indices(ptr(idx), ptr(offsets), ptr(flat), ptr(work), ptr(inv), B, H, Mb, k_ntx, T, max(chunk, 1),
                                    stream_of(lib, idx) if stream is None else stream), "transpose_indices")
    return (offsets, flat) + (() if work is None else (work,)) + (() if inv is None else (inv,))



def transpose_indices_levels(selections, chunk, stream=None):
    """The selections of all levels of one operator call, finest first, with one call of the library
    (llsa_transpose_indices_multi: one launch for every level whose (key block, query block) bitmaps fit LDS).
    selections[0] (B,H,Mb,T) gets a work list with pieces of `chunk` entries, the pooled levels get inverse
    positions, as the backward wants them.  Returns [(offsets, flat, work), (offsets, flat, inv), ...]."""
    lib = lib_for(selections[0])
    B, H = selections[0].shape[:2]
    jobs = (TransposeJob * len(selections))()
    out = []
    for l, sel in enumerate(selections):
        Mb, T = sel.shape[2:]
        idx = sel.to(torch.int32).contiguous()
        offsets = torch.empty(B, H, 1 + Mb, device=idx.device, dtype=torch.int32)
        flat = torch.empty(B, H, Mb * T, device=idx.device, dtype=torch.int32)
        if l == 0:
            extra = torch.empty(B, H, lib.work_list_len(Mb, Mb, T, chunk), device=idx.device, dtype=torch.int32)
            jobs[l] = TransposeJob(ptr(idx), ptr(offsets), ptr(flat), ptr(extra), None, Mb, Mb, T, chunk)
        else:
            extra = torch.empty(B, H, Mb, T, device=idx.device, dtype=torch.int32)
            jobs[l] = TransposeJob(ptr(idx), ptr(offsets), ptr(flat), None, ptr(extra), Mb, Mb, T, 1)
        out.append((offsets, flat, extra, idx))       # (idx is kept alive until the launch is issued)
    lib.check(lib.transpose_indices_multi(jobs, len(selections), B, H, stream_of(lib, selections[0]) if stream is None else stream),
              "transpose_indices")
    return [t[:3] for t in out]
