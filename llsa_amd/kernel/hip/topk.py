"""Block selection.  Mirrors kernel/triton/topk.py."""
from __future__ import annotations

import torch

from ._common import BLOCK, lib_for, ptr, require_bf16, require_head_dim, stream_of


def gen_sparse_indices(pq, pk, topk, round_scores=True):
    """topk.py:6-9: top-k of pq.pk^T per row.  Scores are rounded to the input dtype as the
    reference's matmul does; equal scores are ordered by smaller index.  Returns int32
    (B,H,n,min(topk,n)) -- the reference returns int64, nothing outside the operator sees it."""
    lib = lib_for(pq, pk)
    require_bf16(pq, pk)
    require_head_dim(pq)
    B, H, n, D = pq.shape
    if pk.shape != pq.shape:
        raise ValueError("self-attention only: pq and pk must have the same shape")
    topk = min(topk, n)
    out = torch.empty(B, H, n, topk, device=pq.device, dtype=torch.int32)
    lib.check(lib.topk_dense(ptr(pq.contiguous()), ptr(pk.contiguous()), ptr(out), B, H, n, topk,
                             1 if round_scores else 0, stream_of(lib, pq)), "gen_sparse_indices")
    return out


def compute_topk_indices_sparse(pq, pk, p_indices, topk=8, p_topk=8, block_size=16):
    """topk.py:172-197."""
    lib = lib_for(pq, pk, p_indices)
    require_bf16(pq, pk)
    require_head_dim(pq)
    if block_size != BLOCK:
        raise NotImplementedError("block_size must be 16")
    B, H, M, D = pq.shape
    if p_indices.shape != (B, H, M // BLOCK, p_topk):
        raise ValueError(f"p_indices must be {(B, H, M // BLOCK, p_topk)}, got {tuple(p_indices.shape)}")
    pi = p_indices.to(torch.int32).contiguous()
    out = torch.empty(B, H, M, topk, device=pq.device, dtype=torch.int32)
    lib.check(lib.topk_sparse(ptr(pq.contiguous()), ptr(pk.contiguous()), ptr(pi), ptr(out), B, H, M, topk, p_topk,
                              stream_of(lib, pq)), "compute_topk_indices_sparse")
    return out


def topk_cascade(pq_parent, pk_parent, pq, pk, topk=8, p_topk=8):
    """gen_sparse_indices on the parent level and compute_topk_indices_sparse under its result in one launch
    (topk.py:6-9, :172-197): returns (p_indices, indices) exactly as the two calls would.  The parent level may
    have at most llsa_topk_cascade_max_parents() tokens."""
    lib = lib_for(pq, pk, pq_parent, pk_parent)
    require_bf16(pq, pk, pq_parent, pk_parent)
    require_head_dim(pq)
    B, H, M, D = pq.shape
    if pq_parent.shape != (B, H, M // BLOCK, D) or pk_parent.shape != pq_parent.shape or pk.shape != pq.shape:
        raise ValueError("the parent level must be (B, H, M/16, 64) for (B, H, M, 64) rows")
    p_topk = min(p_topk, M // BLOCK)
    p_out = torch.empty(B, H, M // BLOCK, p_topk, device=pq.device, dtype=torch.int32)
    out = torch.empty(B, H, M, topk, device=pq.device, dtype=torch.int32)
    lib.check(lib.topk_cascade(ptr(pq_parent.contiguous()), ptr(pk_parent.contiguous()), ptr(p_out), ptr(pq.contiguous()),
                               ptr(pk.contiguous()), ptr(out), B, H, M, topk, p_topk, stream_of(lib, pq)), "topk_cascade")
    return p_out, out
