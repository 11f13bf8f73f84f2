"""Query-major top-k lists -> key-major CSR.  Mirrors kernel/triton/indices_transpose.py."""
from __future__ import annotations

import torch

from ._common import lib_for, ptr, stream_of


def transpose_indices(q_topk_indices, k_ntx=None):
    """indices_transpose.py:104-109.  Returns (offsets (B,H,1+Kb), flat (B,H,Mb*T)), int32; the
    entries of each segment are in ascending query-block order."""
    lib = lib_for(q_topk_indices)
    B, H, Mb, T = q_topk_indices.shape
    if k_ntx is None:
        k_ntx = Mb
    idx = q_topk_indices.to(torch.int32).contiguous()
    offsets = torch.empty(B, H, 1 + k_ntx, device=idx.device, dtype=torch.int32)
    flat = torch.empty(B, H, Mb * T, device=idx.device, dtype=torch.int32)
    lib.check(lib.transpose_indices(ptr(idx), ptr(offsets), ptr(flat), B, H, Mb, k_ntx, T, stream_of(lib, idx)),
              "transpose_indices")
    return offsets, flat
