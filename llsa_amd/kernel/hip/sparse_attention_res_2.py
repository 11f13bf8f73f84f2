"""Two-level sparse attention with pooled residuals.  Mirrors
kernel/triton/sparse_attention_res_2.py (same function names and argument order)."""
from __future__ import annotations

from ._attention import attn_bwd, attn_fwd


def sparse_indices_attn_res_2_2_fwd(q, k, v, pk, pv, pk2, pv2, indices, p_indices, topk, topk_p, token_weight=1,
                                    token_weight_2=1, down_scale=4, tiles=None):
    """sparse_attention_res_2.py:166-199."""
    if down_scale * down_scale != 16:
        raise NotImplementedError("block_size must be 16 (down_scale 4)")
    assert indices.shape[-1] == topk and p_indices.shape[-1] == topk_p
    return attn_fwd(q, k, v, pk, pv, indices, token_weight, pk2=pk2, pv2=pv2, p_indices=p_indices,
                    token_weight_2=token_weight_2, tiles=tiles)


def sparse_indices_attn_res_scatter_2_2_bwd_v2(do, q, k, v, pk, pv, pk2, pv2, o, m, indices, prev_indices, topk, topk_p,
                                               block_size, token_weight, token_weight_2, tiles=None, freq_dq=None, **bwd_opts):
    """sparse_attention_res_2.py:578-681.  Returns (dq, dk, dv, None, dpk, dpv, None, dpk2, dpv2)."""
    if block_size != 16:
        raise NotImplementedError("block_size must be 16")
    dq, dk, dv, dpk, dpv, dpk2, dpv2 = attn_bwd(do, q, k, v, pk, pv, o, m, indices, token_weight, token_weight, pk2=pk2,
                                                pv2=pv2, p_indices=prev_indices, token_weight_2=token_weight_2,
                                                tiles=tiles, freq_dq=freq_dq, **bwd_opts)
    return dq, dk, dv, None, dpk, dpv, None, dpk2, dpv2
