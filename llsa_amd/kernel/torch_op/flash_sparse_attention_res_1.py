"""llsa_l1: one pooled level.  Mirrors torch_op/flash_sparse_attention_res_1.py of the
reference: `FlashSparseResidualAttentionL1`, `flash_sparse_residual_attention_l1_op`,
`llsa_l1(q, k, v, topk=8, block_size=16)` with the same positional arguments.

`llsa_l1` additionally accepts `rope=freq` (an (N, 64) table of interleaved sin/cos): then
q and k are rotated inside the pooling pass and the gradients are rotated back inside the
backward kernels, which is the same function as
`llsa_l1(my_rope_fn(q, freq), my_rope_fn(k, freq), v, ...)`.

`qk_norm=(gamma_q, gamma_k, eps)` (two fp32 vectors of 64 weights and the epsilon) moves the
attention processor's RMS norms of q and k (rope_dit_transformer_2d.py:215-218) into the same
pass: rows are normalised before the rotation, the gradients come back through the norm, and
gamma_q / gamma_k receive theirs.  Same function as
`llsa_l1(my_rms_norm_fn(q, gamma_q, eps), my_rms_norm_fn(k, gamma_k, eps), v, ...)`.
"""
from __future__ import annotations

import torch
from torch.autograd import Function

from ..hip.mean_pool import mean_pool1d
from ._fused import LlsaFused
from ..hip.sparse_attention_res_1 import sparse_indices_attn_res_fwd, sparse_indices_attn_res_scatter_bwd_v2
from ..hip.topk import gen_sparse_indices


class FlashSparseResidualAttentionL1(Function):
    """flash_sparse_attention_res_1.py:10-35."""

    @staticmethod
    def forward(ctx, q, k, v, pq, pk, pv, topk, token_weight=1, block_size=16):
        indices = gen_sparse_indices(pq, pk, topk)
        output, m = sparse_indices_attn_res_fwd(q, k, v, pk, pv, indices, indices.shape[-1], token_weight,
                                                int(block_size ** 0.5))
        ctx.save_for_backward(q, k, v, pk, pv, output, m, indices)
        ctx.topk = indices.shape[-1]
        ctx.block_size = block_size
        ctx.token_weight = token_weight
        return output

    @staticmethod
    def backward(ctx, do):
        q, k, v, pk, pv, o, m, indices = ctx.saved_tensors
        return *sparse_indices_attn_res_scatter_bwd_v2(do, q, k, v, pk, pv, o, m, indices, ctx.topk,
                                                       ctx.block_size, ctx.token_weight), None, None, None


flash_sparse_residual_attention_l1_op = FlashSparseResidualAttentionL1.apply


def llsa_l1(q, k, v, topk=8, block_size=16, rope=None, qk_norm=None):
    """flash_sparse_attention_res_1.py:41-47."""
    gq, gk, eps = qk_norm if qk_norm is not None else (None, None, 0.0)
    return LlsaFused.apply(q, k, v, (topk,), block_size, rope, gq, gk, eps)


def llsa_l1_unfused(q, k, v, topk=8, block_size=16):
    """The reference's own composition, kernel for kernel: three mean_pool1d calls, then the op
    (gradients reach k and v through mean_pool1d's backward and autograd's accumulation)."""
    pq = mean_pool1d(q, block_size)
    pk = mean_pool1d(k, block_size)
    pv = mean_pool1d(v, block_size)
    return flash_sparse_residual_attention_l1_op(q, k, v, pq, pk, pv, topk, block_size, block_size)
