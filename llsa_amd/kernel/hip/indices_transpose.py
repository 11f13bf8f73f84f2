"""Query-major top-k lists -> key-major CSR.  Mirrors kernel/triton/indices_transpose.py."""
from __future__ import annotations

import torch

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

