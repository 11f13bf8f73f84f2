"""One-level sparse attention with the dense pooled residual.  Mirrors
kernel/triton/sparse_attention_res_1.py (same function names and argument order)."""
from __future__ import annotations

from ._attention import attn_bwd, attn_fwd


def _block_size_from_down_scale(down_scale):
    if down_scale * down_scale != 16:
        raise NotImplementedError("block_size must be 16 (down_scale 4)")


def sparse_indices_attn_res_fwd(q, k, v, pk, pv, indices, topk, token_weight=1, down_scale=4, tiles=None):
    """sparse_attention_res_1.py:123-150.  Returns (o, m): o like q, m = logsumexp (B,H,N) fp32."""
    _block_size_from_down_scale(down_scale)
    assert indices.shape[-1] == topk
    return attn_fwd(q, k, v, pk, pv, indices, token_weight, tiles=tiles)


def sparse_indices_attn_res_scatter_bwd_v2(do, q, k, v, pk, pv, o, m, indices, topk, block_size, token_weight,
                                           tiles=None, freq_dq=None, **bwd_opts):
    """sparse_attention_res_1.py:403-471.  Returns (dq, dk, dv, None, dpk, dpv).  As in the
    reference the dpk/dpv path uses weight 1 where the forward used token_weight (:388-389)."""
    if block_size != 16:
        raise NotImplementedError("block_size must be 16")
    dq, dk, dv, dpk, dpv = attn_bwd(do, q, k, v, pk, pv, o, m, indices, token_weight, 1.0, tiles=tiles, freq_dq=freq_dq, **bwd_opts)
    return dq, dk, dv, None, dpk, dpv
