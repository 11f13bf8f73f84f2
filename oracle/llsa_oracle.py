"""CPU oracle for the llsa_l1 / llsa_l2 hot path.  TEST INFRASTRUCTURE ONLY.

This file is a plain-PyTorch (CPU) restatement of the algorithm that the
reference implements with Triton kernels.  It exists so that the HIP kernels can
be checked against something; it is never imported by the product package
(`llsa_amd`).  Only `tests/`, `__graft_entry__.smoke()` and the `cpu_baseline`
leg of `bench.py` may import it.

Every function names the reference file:line it restates (paths relative to the
reference checkout, `src/llsa/...`).  Nothing here is copied: the reference is
Triton device code, this is dense tensor algebra with the same rounding points.

Rounding model ("faithful" functions): a tensor of dtype `dt` (bf16 in the
headline configs) is rounded to `dt` wherever the reference materialises a value
in `dt`; matrix products take `dt` operands and accumulate in fp32 (tl.dot);
soft-max statistics are fp32.

Pinning status (what each function is checked against, see tests/test_oracle_*):
  zorder_perm            closed form (Morton code), brute force, inverse property
  rope_table/rope_apply  complex multiplication (library), orthogonality,
                         relative-position property.  The *order of bf16
                         roundings inside one rotation* (three roundings, no
                         FMA contraction) is read from rope.py:46-47 and cannot
                         be checked without an NVIDIA GPU: parity unpinned for
                         that detail only (it is far inside the tolerance).
  mean_pool              F.avg_pool1d (fp32); brute-force sequential bf16 loop
  gen_sparse_indices     is library code (matmul + topk) restated verbatim
  topk_sparse            brute-force python sort with the tie rule of topk.py:155-164
  transpose_indices      bincount / stable argsort brute force
  attn_fwd_*             closed form soft-max over the augmented logits (fp64),
                         special cases that reduce to F.scaled_dot_product_attention
  attn_bwd_*             torch.autograd on the fp64 closed form (+ the L1
                         dpk/dpv quirk, sparse_attention_res_1.py:388-389)
  delta rounding         the reference sums O*dO in the tensor dtype
                         (sparse_attention_res_1.py:173); which reduction tree
                         Triton uses is not observable here: parity unpinned for
                         `delta_in_dtype=True`; the default keeps fp32.
  *_l3                   three levels, no counterpart in the reference: fp64 closed form over the four
                         weighted segments and torch.autograd on it, selection cascade property
  *_lk                   any number of levels: equal to *_l1, *_l2, *_l3 bit for bit at k = 1, 2, 3; at k = 4 the key
                         sets of single queries against a direct enumeration of the definition
  rms_norm / _bwd        F.rms_norm and its autograd (fp32).  The module the model
                         calls (diffusers' RMSNorm, rope_dit_transformer_2d.py:215-218)
                         is not in the reference checkout: parity unpinned for its
                         eps and rounding points.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import torch
import torch.nn.functional as F

# --------------------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------------------


def _rn(x: torch.Tensor, dt: torch.dtype) -> torch.Tensor:
    """Round an fp32/fp64 tensor to `dt` and return it in its original dtype."""
    if dt == x.dtype:
        return x
    return x.to(dt).to(x.dtype)


def _up(x: torch.Tensor) -> torch.Tensor:
    """Working precision: fp32, or fp64 for fp64 inputs."""
    return x if x.dtype == torch.float64 else x.float()


def _mm(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """tl.dot: operands already representable in the storage dtype, fp32 accumulate."""
    return torch.matmul(a.float(), b.float())


# --------------------------------------------------------------------------------------
# Z-order (Morton) permutation  --  models/rope_dit_transformer_2d.py:714-732
# --------------------------------------------------------------------------------------


def zorder_perm(side: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Return (perm, inv_perm) for a side x side grid, side a power of two >= 2.

    perm[r*side + c] = z  with z = interleave(row bits above column bits)
    inv_perm[z]      = r*side + c
    The reference builds the same table recursively from the seed [[0,1],[2,3]]
    (rope_dit_transformer_2d.py:716-727) and inverts it (:729-731); tokens are
    put in Z-order with x[:, inv_perm] and restored with x[:, perm] (:963-965,
    :1028-1030).
    """
    assert side >= 2 and side & (side - 1) == 0
    r = torch.arange(side).view(-1, 1).expand(side, side)
    c = torch.arange(side).view(1, -1).expand(side, side)
    z = torch.zeros(side, side, dtype=torch.long)
    for bit in range(side.bit_length() - 1):
        z |= ((c >> bit) & 1) << (2 * bit)
        z |= ((r >> bit) & 1) << (2 * bit + 1)
    perm = z.flatten()
    inv_perm = torch.empty_like(perm)
    inv_perm[perm] = torch.arange(side * side)
    return perm, inv_perm


# --------------------------------------------------------------------------------------
# 2-D RoPE table and rotation  --  rope_dit_transformer_2d.py:71-109,153-173; rope.py:6-97
# --------------------------------------------------------------------------------------


def rope_table(side: int, axes_dim: Sequence[int] = (32, 32), theta: float = 10000.0,
               dtype: torch.dtype = torch.float32, zorder: bool = True) -> torch.Tensor:
    """(side*side, sum(axes_dim)) table: per axis [sin w0, cos w0, sin w1, cos w1, ...].

    axis 0 uses the row id, axis 1 the column id (register_rope_emb :160-162),
    w_j = theta^(-2j/dim) in fp64 (gen_rope_freq :71-74), sin/cos interleaved by
    torch.stack([sin, cos], -1) (:87).  ids are float32 aranges (:155-156, the
    interpolation at :158-159 is the identity when patch_size == 1).  Rows are
    reordered to Z-order with the same index the tokens use (:167-169).
    """
    pos = torch.arange(side, dtype=torch.float32)
    ids = torch.zeros(side, side, 2)
    ids[..., 0] += pos[:, None]
    ids[..., 1] += pos[None, :]
    ids = ids.reshape(side * side, 2)
    if zorder:
        _, inv_perm = zorder_perm(side)
        ids = ids[inv_perm]
    cols = []
    for a, dim in enumerate(axes_dim):
        omega = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float64) / dim))
        ang = ids[:, a].double()[:, None] * omega[None, :]  # einsum('n,d->nd') promotes to fp64
        cols.append(torch.stack([torch.sin(ang), torch.cos(ang)], dim=-1).reshape(-1, dim))
    return torch.cat(cols, dim=-1).to(dtype)


def rope_apply(x: torch.Tensor, freq: torch.Tensor) -> torch.Tensor:
    """rope.py:28-50.  freq[s, 2p] = sin, freq[s, 2p+1] = cos; arithmetic in x.dtype,
    every binary op rounded to x.dtype (two products, one subtraction/addition)."""
    dt = x.dtype
    xe, xo = _up(x[..., 0::2]), _up(x[..., 1::2])
    f = freq.to(dt)
    sin, cos = _up(f[..., 0::2]), _up(f[..., 1::2])
    ye = _rn(_rn(cos * xe, dt) - _rn(sin * xo, dt), dt)
    yo = _rn(_rn(sin * xe, dt) + _rn(cos * xo, dt), dt)
    return torch.stack([ye, yo], dim=-1).reshape(x.shape).to(dt)


def rope_apply_bwd(dy: torch.Tensor, freq: torch.Tensor) -> torch.Tensor:
    """rope.py:84-97: the transposed rotation, same rounding model."""
    dt = dy.dtype
    de, do = _up(dy[..., 0::2]), _up(dy[..., 1::2])
    f = freq.to(dt)
    sin, cos = _up(f[..., 0::2]), _up(f[..., 1::2])
    xe = _rn(_rn(cos * de, dt) + _rn(sin * do, dt), dt)
    xo = _rn(_rn(-sin * de, dt) + _rn(cos * do, dt), dt)
    return torch.stack([xe, xo], dim=-1).reshape(dy.shape).to(dt)


# --------------------------------------------------------------------------------------
# qk RMS norm  --  call site models/rope_dit_transformer_2d.py:215-219 (diffusers' RMSNorm)
# --------------------------------------------------------------------------------------


def rms_norm(x: torch.Tensor, gamma: torch.Tensor, eps: float) -> torch.Tensor:
    """The qk-norm of the attention processor (rope_dit_transformer_2d.py:215-219: attn.norm_q /
    attn.norm_k, applied to (B,H,N,D) before the RoPE, result cast back to the input dtype).
    diffusers' RMSNorm is not in the reference checkout; this is the textbook definition it
    implements, computed in fp32 with an fp32 weight: y = x * rsqrt(mean(x^2, -1) + eps) * gamma.
    PARITY UNPINNED against diffusers itself (eps, and where exactly it rounds)."""
    xf = _up(x)
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * _up(gamma)
    return y.to(x.dtype)


def rms_norm_bwd(dy: torch.Tensor, x: torch.Tensor, gamma: torch.Tensor, eps: float):
    """Backward of rms_norm in fp32: returns (dx in x.dtype, dgamma fp32/fp64 like gamma)."""
    xf, g = _up(x), _up(dy) * _up(gamma)
    rstd = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    xn = xf * rstd
    dx = rstd * (g - xn * (g * xn).mean(-1, keepdim=True))
    dgamma = (_up(dy) * xn).reshape(-1, x.shape[-1]).sum(0)
    return dx.to(x.dtype), dgamma


# --------------------------------------------------------------------------------------
# mean pooling  --  kernel/triton/mean_pool.py:6-58
# --------------------------------------------------------------------------------------


def mean_pool(x: torch.Tensor, k: int = 16) -> torch.Tensor:
    """y[..., s, :] = mean of k consecutive tokens; the accumulator has x.dtype, so a
    bf16 input is summed sequentially with a rounding after every add and after
    the division (mean_pool.py:26-30)."""
    B, H, S, C = x.shape
    assert S % k == 0
    dt = x.dtype
    xb = x.reshape(B, H, S // k, k, C).float()
    acc = torch.zeros(B, H, S // k, C)
    for t in range(k):
        acc = _rn(acc + xb[:, :, :, t], dt)
    return _rn(acc / k, dt).to(dt)


def mean_pool_bwd(dy: torch.Tensor, k: int = 16) -> torch.Tensor:
    """dx[..., s*k + t, :] = dy[..., s, :] / k in dy.dtype (mean_pool.py:54-58)."""
    dt = dy.dtype
    g = _rn(dy.float() / k, dt).to(dt)
    return g.repeat_interleave(k, dim=2)


# --------------------------------------------------------------------------------------
# selection  --  kernel/triton/topk.py
# --------------------------------------------------------------------------------------


def gen_sparse_indices(pq: torch.Tensor, pk: torch.Tensor, topk: int) -> torch.Tensor:
    """topk.py:6-9 restated: scores in the input dtype, library top-k, int64 indices.
    The order among equal scores is whatever torch.topk does on this device."""
    score = torch.matmul(pq, pk.transpose(-2, -1))
    topk = min(topk, score.shape[-1])
    return torch.topk(score, topk).indices


def dense_scores(pq: torch.Tensor, pk: torch.Tensor, round_to_input: bool = True) -> torch.Tensor:
    """The score matrix of gen_sparse_indices as fp32 values (rounded through the input
    dtype when round_to_input), for gap analysis in tests."""
    s = _mm(pq, pk.transpose(-2, -1))
    return _rn(s, pq.dtype) if round_to_input else s


def topk_lowest_index(score: torch.Tensor, topk: int, idx: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Deterministic top-k: descending score, equal scores -> smaller index first.
    This is the selection loop of topk.py:155-164 (row max, among equal maxima the
    smallest global index, mask, repeat).  `idx` gives the global index of every
    column (defaults to arange)."""
    n = score.shape[-1]
    if idx is None:
        idx = torch.arange(n).expand(score.shape)
    # sort by index ascending first, then stable-sort by score descending
    order_i = torch.argsort(idx, dim=-1, stable=True)
    s_i = torch.gather(score, -1, order_i)
    g_i = torch.gather(idx, -1, order_i)
    order_s = torch.argsort(s_i, dim=-1, descending=True, stable=True)
    return torch.gather(g_i, -1, order_s)[..., :topk]


def topk_sparse(pq: torch.Tensor, pk: torch.Tensor, p_indices: torch.Tensor, topk: int,
                block_size: int = 16, return_scores: bool = False):
    """topk.py:102-197.  For level-2 query block G the candidates are the level-1 key
    blocks p_indices[G, a]*bs + b; each of the bs level-1 query rows of G scores
    them in fp32 (tl.dot, :141-143) and keeps the `topk` best, descending, ties to
    the smaller index (:155-164).  int32 output (:175)."""
    B, H, M, D = pq.shape
    bs = block_size
    T2 = p_indices.shape[-1]
    G = M // bs
    cand = (p_indices.long()[..., None] * bs + torch.arange(bs)).reshape(B, H, G, T2 * bs)
    pkc = torch.gather(pk.float()[:, :, None].expand(B, H, G, pk.shape[2], D), 3,
                       cand[..., None].expand(B, H, G, T2 * bs, D))          # (B,H,G,C,D)
    pqg = pq.float().reshape(B, H, G, bs, D)
    score = torch.matmul(pqg, pkc.transpose(-2, -1))                          # (B,H,G,bs,C)
    gidx = cand[:, :, :, None, :].expand(B, H, G, bs, T2 * bs)
    out = topk_lowest_index(score, topk, gidx).reshape(B, H, M, topk).to(torch.int32)
    if return_scores:
        return out, score.reshape(B, H, M, T2 * bs), gidx.reshape(B, H, M, T2 * bs)
    return out


# --------------------------------------------------------------------------------------
# index transpose  --  kernel/triton/indices_transpose.py:6-109
# --------------------------------------------------------------------------------------


def transpose_indices(indices: torch.Tensor, k_ntx: Optional[int] = None):
    """Q-major (B,H,Mb,T) -> K-major CSR.  offsets (B,H,1+Kb) int64 with offsets[0]=0
    (inclusive cumsum of a histogram shifted by one, :30-45,:108); flat (B,H,Mb*T)
    lists, for key block n, the query blocks that selected it.  The reference fills
    each segment in atomic (arbitrary) order (:72-78); this restatement fixes the
    order to ascending query block, which is one of the orders the reference can
    produce."""
    B, H, Mb, T = indices.shape
    if k_ntx is None:
        k_ntx = Mb
    idx = indices.long().reshape(B, H, Mb * T)
    qid = torch.arange(Mb).repeat_interleave(T).expand(B, H, Mb * T)
    count = torch.zeros(B, H, 1 + k_ntx, dtype=torch.long)
    count.scatter_add_(-1, idx + 1, torch.ones_like(idx))
    offsets = torch.cumsum(count, -1)
    order = torch.argsort(idx * Mb + qid, dim=-1, stable=True)
    flat = torch.gather(qid, -1, order)
    return offsets, flat


# --------------------------------------------------------------------------------------
# forward  --  sparse_attention_res_1.py:9-150, sparse_attention_res_2.py:9-199
# --------------------------------------------------------------------------------------


def _gather_blocks(x: torch.Tensor, idx: torch.Tensor, bs: int) -> torch.Tensor:
    """x (B,H,n,D) viewed as blocks of bs rows; idx (B,H,G,T) block ids ->
    (B,H,G,T*bs,D)."""
    B, H, n, D = x.shape
    G, T = idx.shape[2], idx.shape[3]
    xb = x.reshape(B, H, n // bs, bs * D)
    bi = torch.arange(B)[:, None, None, None]
    hi = torch.arange(H)[None, :, None, None]
    return xb[bi, hi, idx.long()].reshape(B, H, G, T * bs, D)


def _segments_l1(q, k, v, pk, pv, indices, token_weight, bs):
    B, H, N, D = q.shape
    N1 = N // bs
    kf = _gather_blocks(k, indices, bs)                     # (B,H,N1,T*bs,D)
    vf = _gather_blocks(v, indices, bs)
    kc = pk[:, :, None].expand(B, H, N1, pk.shape[2], D)
    vc = pv[:, :, None].expand(B, H, N1, pv.shape[2], D)
    return [(kf, vf, 1.0), (kc, vc, float(token_weight))]


def _segments_l2(q, k, v, pk, pv, pk2, pv2, indices, p_indices, w1, w2, bs):
    B, H, N, D = q.shape
    N1 = N // bs
    kf = _gather_blocks(k, indices, bs)
    vf = _gather_blocks(v, indices, bs)
    # level-1 pooled tokens inside the parent's selected coarse blocks
    # (sparse_attention_res_2.py:94-112): parent of query block g is g // bs
    par = p_indices.long().repeat_interleave(bs, dim=2)     # (B,H,N1,T2)
    k1 = _gather_blocks(pk, par, bs)
    v1 = _gather_blocks(pv, par, bs)
    k2 = pk2[:, :, None].expand(B, H, N1, pk2.shape[2], D)
    v2 = pv2[:, :, None].expand(B, H, N1, pv2.shape[2], D)
    return [(kf, vf, 1.0), (k1, v1, float(w1)), (k2, v2, float(w2))]


def _segments_l3(q, k, v, pk, pv, pk2, pv2, pk3, pv3, indices, p_indices, pp_indices, w1, w2, w3, bs):
    """Three pooled levels, the two-level scheme (sparse_attention_res_2.py:94-149) continued by one step: a
    query block sees its selected fine blocks, the level-1 pooled tokens inside its parent's selected level-1
    blocks, the level-2 pooled tokens inside its grand-parent's selected level-2 blocks, and every level-3
    pooled token.  The reference stops at two levels; there is nothing of its to compare this with."""
    B, H, N, D = q.shape
    N1 = N // bs
    kf = _gather_blocks(k, indices, bs)
    vf = _gather_blocks(v, indices, bs)
    par = p_indices.long().repeat_interleave(bs, dim=2)              # (B,H,N1,T2): parent of block g is g // bs
    k1, v1 = _gather_blocks(pk, par, bs), _gather_blocks(pv, par, bs)
    gpar = pp_indices.long().repeat_interleave(bs * bs, dim=2)       # (B,H,N1,T3): grand-parent is g // bs^2
    k2, v2 = _gather_blocks(pk2, gpar, bs), _gather_blocks(pv2, gpar, bs)
    k3 = pk3[:, :, None].expand(B, H, N1, pk3.shape[2], D)
    v3 = pv3[:, :, None].expand(B, H, N1, pv3.shape[2], D)
    return [(kf, vf, 1.0), (k1, v1, float(w1)), (k2, v2, float(w2)), (k3, v3, float(w3))]


def _online_softmax(q, segments, bs, tile=64):
    """The tile loop shared by both forward kernels (sparse_attention_res_1.py:54-106):
    64-wide KV tiles in list order; P is rounded to the value dtype before P.V
    (:82); the weight multiplies the row sum and the P.V product (:103-105)."""
    B, H, N, D = q.shape
    dt = q.dtype
    scale = 1.0 / math.sqrt(D)
    qs = _rn(q.float() * scale, dt).reshape(B, H, N // bs, bs, D)   # q *= scale in q.dtype (:48)
    m = torch.full((B, H, N // bs, bs), -float("inf"))
    l = torch.zeros(B, H, N // bs, bs)
    acc = torch.zeros(B, H, N // bs, bs, D)
    for ks, vs, w in segments:
        n = ks.shape[3]
        for t0 in range(0, n - n % tile, tile):          # a tail shorter than a tile is dropped (:85)
            kt = ks[:, :, :, t0:t0 + tile].float()
            vt = vs[:, :, :, t0:t0 + tile].float()
            s = torch.matmul(qs, kt.transpose(-2, -1))
            m_new = torch.maximum(m, s.max(dim=-1).values)
            p = torch.exp(s - m_new[..., None])
            alpha = torch.exp(m - m_new)
            l = l * alpha + p.sum(-1) * w
            acc = acc * alpha[..., None] + torch.matmul(_rn(p, vs.dtype), vt) * w
            m = m_new
    o = _rn(acc / l[..., None], dt).reshape(B, H, N, D).to(dt)
    lse = (m + torch.log(l)).reshape(B, H, N)
    return o, lse


def attn_fwd_l1(q, k, v, pk, pv, indices, token_weight=16, block_size=16):
    """sparse_indices_attn_res_fwd (sparse_attention_res_1.py:123-150)."""
    return _online_softmax(q, _segments_l1(q, k, v, pk, pv, indices, token_weight, block_size), block_size)


def attn_fwd_l2(q, k, v, pk, pv, pk2, pv2, indices, p_indices, token_weight=16, token_weight_2=256,
                block_size=16):
    """sparse_indices_attn_res_2_2_fwd (sparse_attention_res_2.py:166-199)."""
    seg = _segments_l2(q, k, v, pk, pv, pk2, pv2, indices, p_indices, token_weight, token_weight_2, block_size)
    return _online_softmax(q, seg, block_size)


def attn_fwd_l3(q, k, v, pk, pv, pk2, pv2, pk3, pv3, indices, p_indices, pp_indices, w1=16, w2=256, w3=4096, block_size=16):
    """Three-level forward, same tile loop (no counterpart in the reference)."""
    seg = _segments_l3(q, k, v, pk, pv, pk2, pv2, pk3, pv3, indices, p_indices, pp_indices, w1, w2, w3, block_size)
    return _online_softmax(q, seg, block_size)


# --------------------------------------------------------------------------------------
# closed form (fp64), used to pin the faithful forward/backward above
# --------------------------------------------------------------------------------------


def attn_closed_form(q, segments_kvw, bs=16):
    """softmax over the concatenation of all segments with log(w) added to the logits of
    a segment of weight w (w * e^s = e^(s + log w)).  Differentiable, any dtype.
    segments_kvw: list of (K (B,H,N/bs,n,D), V same, w)."""
    B, H, N, D = q.shape
    scale = 1.0 / math.sqrt(D)
    qb = q.reshape(B, H, N // bs, bs, D)
    logits, vals = [], []
    for ks, vs, w in segments_kvw:
        logits.append(torch.matmul(qb, ks.transpose(-2, -1)) * scale + math.log(w))
        vals.append(vs)
    logits = torch.cat(logits, dim=-1)
    vals = torch.cat(vals, dim=-2)
    lse = torch.logsumexp(logits, dim=-1)
    o = torch.matmul(torch.softmax(logits, dim=-1), vals)
    return o.reshape(B, H, N, D), lse.reshape(B, H, N)


def closed_form_l1(q, k, v, pk, pv, indices, token_weight=16, bs=16):
    return attn_closed_form(q, _segments_l1(q, k, v, pk, pv, indices, token_weight, bs), bs)


def closed_form_l2(q, k, v, pk, pv, pk2, pv2, indices, p_indices, w1=16, w2=256, bs=16):
    return attn_closed_form(q, _segments_l2(q, k, v, pk, pv, pk2, pv2, indices, p_indices, w1, w2, bs), bs)


def closed_form_l3(q, k, v, pk, pv, pk2, pv2, pk3, pv3, indices, p_indices, pp_indices, w1=16, w2=256, w3=4096, bs=16):
    return attn_closed_form(q, _segments_l3(q, k, v, pk, pv, pk2, pv2, pk3, pv3, indices, p_indices, pp_indices,
                                            w1, w2, w3, bs), bs)


# --------------------------------------------------------------------------------------
# backward  --  sparse_attention_res_1.py:153-471, sparse_attention_res_2.py:202-681
# --------------------------------------------------------------------------------------


def attn_delta(o, do, in_dtype=False):
    """_attn_bwd_preprocess (sparse_attention_res_1.py:153-177): delta = rowsum(O * dO).
    in_dtype=True multiplies and sums in the tensor dtype, left to right."""
    if not in_dtype:
        return (o.float() * do.float()).sum(-1)
    dt = o.dtype
    prod = _rn(o.float() * do.float(), dt)
    acc = torch.zeros(prod.shape[:-1])
    for c in range(prod.shape[-1]):
        acc = _rn(acc + prod[..., c], dt)
    return acc


def _scatter_blocks(dst, src, idx, bs):
    """dst (B,H,n,D) += src (B,H,G,T*bs,D) at block ids idx (B,H,G,T)."""
    B, H, n, D = dst.shape
    G, T = idx.shape[2], idx.shape[3]
    d = dst.reshape(B, H, n // bs, bs * D)
    s = src.reshape(B, H, G * T, bs * D)
    d.scatter_add_(2, idx.long().reshape(B, H, G * T, 1).expand(B, H, G * T, bs * D), s)
    return d.reshape(B, H, n, D)


def _bwd_segment(qb, dob, lse, delta, ks, vs, w, scale, dt):
    """One KV list for every query block: the body shared by the dQ loops
    (sparse_attention_res_1.py:240-278) and the dK/dV loops (:300-322).
    qb, dob (B,H,G,bs,D) fp32 values representable in dt; ks, vs (B,H,G,n,D).
    Returns dq (B,H,G,bs,D), dk, dv (B,H,G,n,D), all fp32."""
    kt = _rn(ks.float() * scale, dt)                              # k * scale in k.dtype (:420-422)
    s = torch.matmul(qb, kt.transpose(-2, -1))
    p = torch.exp(s - lse[..., None]) * w
    dp = torch.matmul(dob, vs.float().transpose(-2, -1))
    ds = p * (dp - delta[..., None])
    ds_r = _rn(ds, dt)
    dq = torch.matmul(ds_r, kt)
    dv = torch.matmul(_rn(p, dt).transpose(-2, -1), dob)
    dk = torch.matmul(ds_r.transpose(-2, -1), qb) * scale
    return dq, dk, dv


def attn_bwd_l1(do, q, k, v, pk, pv, o, lse, indices, token_weight=16, block_size=16,
                coarse_grad_weight: Optional[float] = 1.0, delta_in_dtype=False):
    """sparse_indices_attn_res_scatter_bwd_v2 (sparse_attention_res_1.py:403-471).
    Returns dq, dk, dv, dpk, dpv in the primal dtypes.  `coarse_grad_weight` is the
    factor inside p on the dpk/dpv path: the reference omits TOKEN_WEIGHT there
    (:388-389) while the forward (:103-105) and the dq path (:272) use it, so the
    reference's dpk/dpv are the true gradients divided by token_weight; pass
    coarse_grad_weight=None to get the true gradient instead."""
    B, H, N, D = q.shape
    bs, dt = block_size, q.dtype
    G = N // bs
    scale = 1.0 / math.sqrt(D)
    cgw = float(token_weight) if coarse_grad_weight is None else float(coarse_grad_weight)
    qb = q.float().reshape(B, H, G, bs, D)
    dob = do.float().reshape(B, H, G, bs, D)
    lse_b = lse.reshape(B, H, G, bs)
    delta = attn_delta(o, do, delta_in_dtype).reshape(B, H, G, bs)
    (kf, vf, _), (kc, vc, w) = _segments_l1(q, k, v, pk, pv, indices, token_weight, bs)
    dq_f, dk_f, dv_f = _bwd_segment(qb, dob, lse_b, delta, kf, vf, 1.0, scale, dt)
    dq_c, _, _ = _bwd_segment(qb, dob, lse_b, delta, kc, vc, w, scale, dt)
    _, dk_c, dv_c = _bwd_segment(qb, dob, lse_b, delta, kc, vc, cgw, scale, dt)
    dq = (dq_f + dq_c).reshape(B, H, N, D)
    dk = _scatter_blocks(torch.zeros(B, H, N, D), dk_f, indices, bs)
    dv = _scatter_blocks(torch.zeros(B, H, N, D), dv_f, indices, bs)
    dpk, dpv = dk_c.sum(2), dv_c.sum(2)
    return tuple(_rn(x, dt).to(dt) for x in (dq, dk, dv, dpk, dpv))


def attn_bwd_l2(do, q, k, v, pk, pv, pk2, pv2, o, lse, indices, p_indices, token_weight=16,
                token_weight_2=256, block_size=16, delta_in_dtype=False):
    """sparse_indices_attn_res_scatter_2_2_bwd_v2 (sparse_attention_res_2.py:578-681).
    All three coarse paths carry their weight here (:478, :564)."""
    B, H, N, D = q.shape
    bs, dt = block_size, q.dtype
    G = N // bs
    scale = 1.0 / math.sqrt(D)
    qb = q.float().reshape(B, H, G, bs, D)
    dob = do.float().reshape(B, H, G, bs, D)
    lse_b = lse.reshape(B, H, G, bs)
    delta = attn_delta(o, do, delta_in_dtype).reshape(B, H, G, bs)
    segs = _segments_l2(q, k, v, pk, pv, pk2, pv2, indices, p_indices, token_weight, token_weight_2, bs)
    (kf, vf, _), (k1, v1, w1), (k2, v2, w2) = segs
    dq_f, dk_f, dv_f = _bwd_segment(qb, dob, lse_b, delta, kf, vf, 1.0, scale, dt)
    dq_1, dk_1, dv_1 = _bwd_segment(qb, dob, lse_b, delta, k1, v1, w1, scale, dt)
    dq_2, dk_2, dv_2 = _bwd_segment(qb, dob, lse_b, delta, k2, v2, w2, scale, dt)
    dq = (dq_f + dq_1 + dq_2).reshape(B, H, N, D)
    dk = _scatter_blocks(torch.zeros(B, H, N, D), dk_f, indices, bs)
    dv = _scatter_blocks(torch.zeros(B, H, N, D), dv_f, indices, bs)
    par = p_indices.long().repeat_interleave(bs, dim=2)
    dpk = _scatter_blocks(torch.zeros(B, H, pk.shape[2], D), dk_1, par, bs)
    dpv = _scatter_blocks(torch.zeros(B, H, pv.shape[2], D), dv_1, par, bs)
    dpk2, dpv2 = dk_2.sum(2), dv_2.sum(2)
    return tuple(_rn(x, dt).to(dt) for x in (dq, dk, dv, dpk, dpv, dpk2, dpv2))


def attn_bwd_l3(do, q, k, v, pk, pv, pk2, pv2, pk3, pv3, o, lse, indices, p_indices, pp_indices, w1=16, w2=256, w3=4096,
                block_size=16, delta_in_dtype=False):
    """Backward of the three-level forward, the two-level launcher continued by one level: every pooled path
    carries its weight.  Returns dq, dk, dv, dpk, dpv, dpk2, dpv2, dpk3, dpv3."""
    B, H, N, D = q.shape
    bs, dt = block_size, q.dtype
    G = N // bs
    scale = 1.0 / math.sqrt(D)
    qb = q.float().reshape(B, H, G, bs, D)
    dob = do.float().reshape(B, H, G, bs, D)
    lse_b = lse.reshape(B, H, G, bs)
    delta = attn_delta(o, do, delta_in_dtype).reshape(B, H, G, bs)
    segs = _segments_l3(q, k, v, pk, pv, pk2, pv2, pk3, pv3, indices, p_indices, pp_indices, w1, w2, w3, bs)
    parts = [_bwd_segment(qb, dob, lse_b, delta, ks, vs, w, scale, dt) for ks, vs, w in segs]
    dq = sum(p[0] for p in parts).reshape(B, H, N, D)
    dk = _scatter_blocks(torch.zeros(B, H, N, D), parts[0][1], indices, bs)
    dv = _scatter_blocks(torch.zeros(B, H, N, D), parts[0][2], indices, bs)
    par = p_indices.long().repeat_interleave(bs, dim=2)
    dpk = _scatter_blocks(torch.zeros(B, H, pk.shape[2], D), parts[1][1], par, bs)
    dpv = _scatter_blocks(torch.zeros(B, H, pv.shape[2], D), parts[1][2], par, bs)
    gpar = pp_indices.long().repeat_interleave(bs * bs, dim=2)
    dpk2 = _scatter_blocks(torch.zeros(B, H, pk2.shape[2], D), parts[2][1], gpar, bs)
    dpv2 = _scatter_blocks(torch.zeros(B, H, pv2.shape[2], D), parts[2][2], gpar, bs)
    dpk3, dpv3 = parts[3][1].sum(2), parts[3][2].sum(2)
    return tuple(_rn(x, dt).to(dt) for x in (dq, dk, dv, dpk, dpv, dpk2, dpv2, dpk3, dpv3))


# --------------------------------------------------------------------------------------
# whole operators  --  torch_op/flash_sparse_attention_res_{1,2}.py
# --------------------------------------------------------------------------------------


def llsa_l1_fwd(q, k, v, topk=8, block_size=16, indices=None):
    """llsa_l1 forward (flash_sparse_attention_res_1.py:41-47, :12-21).  Returns
    (o, ctx) where ctx holds everything the backward needs.  `indices` overrides
    the selection (used when comparing against a device that broke score ties
    differently)."""
    pq, pk, pv = mean_pool(q, block_size), mean_pool(k, block_size), mean_pool(v, block_size)
    if indices is None:
        indices = gen_sparse_indices(pq, pk, topk)
    o, lse = attn_fwd_l1(q, k, v, pk, pv, indices, block_size, block_size)
    return o, dict(q=q, k=k, v=v, pq=pq, pk=pk, pv=pv, o=o, lse=lse, indices=indices,
                   token_weight=block_size, block_size=block_size)


def llsa_l1_bwd(do, ctx, delta_in_dtype=False):
    """Backward of llsa_l1 including what autograd adds around the op: the pooled
    gradients flow through mean_pool's backward and are added to dk, dv in the
    tensor dtype (mean_pool.py:150-165)."""
    c = ctx
    dq, dk, dv, dpk, dpv = attn_bwd_l1(do, c["q"], c["k"], c["v"], c["pk"], c["pv"], c["o"], c["lse"],
                                       c["indices"], c["token_weight"], c["block_size"],
                                       delta_in_dtype=delta_in_dtype)
    bs = c["block_size"]
    dk = dk + mean_pool_bwd(dpk, bs)
    dv = dv + mean_pool_bwd(dpv, bs)
    return dq, dk, dv, dict(dpk=dpk, dpv=dpv)


def llsa_l2_fwd(q, k, v, topk1=8, topk2=8, block_size=16, indices=None, p_indices=None):
    """llsa_l2 forward (flash_sparse_attention_res_2.py:48-59, :12-30)."""
    bs = block_size
    pq, pk, pv = mean_pool(q, bs), mean_pool(k, bs), mean_pool(v, bs)
    pq2, pk2, pv2 = mean_pool(pq, bs), mean_pool(pk, bs), mean_pool(pv, bs)
    if p_indices is None:
        p_indices = gen_sparse_indices(pq2, pk2, topk2)
    if indices is None:
        indices = topk_sparse(pq, pk, p_indices, topk1, bs)
    o, lse = attn_fwd_l2(q, k, v, pk, pv, pk2, pv2, indices, p_indices, bs, bs * bs, bs)
    return o, dict(q=q, k=k, v=v, pq=pq, pk=pk, pv=pv, pq2=pq2, pk2=pk2, pv2=pv2, o=o, lse=lse,
                   indices=indices, p_indices=p_indices, token_weight=bs, token_weight_2=bs * bs,
                   block_size=bs)


def llsa_l2_bwd(do, ctx, delta_in_dtype=False):
    """Backward of llsa_l2 with the autograd accumulation around it: dpk2 -> pool bwd ->
    added to dpk; that sum -> pool bwd -> added to dk (same for v)."""
    c = ctx
    bs = c["block_size"]
    dq, dk, dv, dpk, dpv, dpk2, dpv2 = attn_bwd_l2(
        do, c["q"], c["k"], c["v"], c["pk"], c["pv"], c["pk2"], c["pv2"], c["o"], c["lse"], c["indices"],
        c["p_indices"], c["token_weight"], c["token_weight_2"], bs, delta_in_dtype=delta_in_dtype)
    dpk_t = dpk + mean_pool_bwd(dpk2, bs)
    dpv_t = dpv + mean_pool_bwd(dpv2, bs)
    dk = dk + mean_pool_bwd(dpk_t, bs)
    dv = dv + mean_pool_bwd(dpv_t, bs)
    return dq, dk, dv, dict(dpk=dpk, dpv=dpv, dpk2=dpk2, dpv2=dpv2)


def llsa_l3_fwd(q, k, v, topk1=8, topk2=8, topk3=8, block_size=16, indices=None, p_indices=None, pp_indices=None):
    """Three levels (no counterpart in the reference, whose deepest operator is llsa_l2): dense selection on the
    level-3 pooled tokens, then parent-guided selection twice, as llsa_l2 does once."""
    bs = block_size
    pq, pk, pv = mean_pool(q, bs), mean_pool(k, bs), mean_pool(v, bs)
    pq2, pk2, pv2 = mean_pool(pq, bs), mean_pool(pk, bs), mean_pool(pv, bs)
    pq3, pk3, pv3 = mean_pool(pq2, bs), mean_pool(pk2, bs), mean_pool(pv2, bs)
    if pp_indices is None:
        pp_indices = gen_sparse_indices(pq3, pk3, topk3)
    if p_indices is None:
        p_indices = topk_sparse(pq2, pk2, pp_indices, topk2, bs)
    if indices is None:
        indices = topk_sparse(pq, pk, p_indices, topk1, bs)
    o, lse = attn_fwd_l3(q, k, v, pk, pv, pk2, pv2, pk3, pv3, indices, p_indices, pp_indices, bs, bs * bs, bs ** 3, bs)
    return o, dict(q=q, k=k, v=v, pq=pq, pk=pk, pv=pv, pq2=pq2, pk2=pk2, pv2=pv2, pq3=pq3, pk3=pk3, pv3=pv3, o=o, lse=lse,
                   indices=indices, p_indices=p_indices, pp_indices=pp_indices, block_size=bs)


def llsa_l3_bwd(do, ctx, delta_in_dtype=False):
    """Backward of llsa_l3 with the chain of pool backwards autograd would add around it."""
    c = ctx
    bs = c["block_size"]
    dq, dk, dv, dpk, dpv, dpk2, dpv2, dpk3, dpv3 = attn_bwd_l3(
        do, c["q"], c["k"], c["v"], c["pk"], c["pv"], c["pk2"], c["pv2"], c["pk3"], c["pv3"], c["o"], c["lse"],
        c["indices"], c["p_indices"], c["pp_indices"], bs, bs * bs, bs ** 3, bs, delta_in_dtype=delta_in_dtype)
    dpk2_t = dpk2 + mean_pool_bwd(dpk3, bs)
    dpv2_t = dpv2 + mean_pool_bwd(dpv3, bs)
    dpk_t = dpk + mean_pool_bwd(dpk2_t, bs)
    dpv_t = dpv + mean_pool_bwd(dpv2_t, bs)
    dk = dk + mean_pool_bwd(dpk_t, bs)
    dv = dv + mean_pool_bwd(dpv_t, bs)
    return dq, dk, dv, dict(dpk=dpk, dpv=dpv, dpk2=dpk2, dpv2=dpv2, dpk3=dpk3, dpv3=dpv3)


# --------------------------------------------------------------------------------------
# any number of pooled levels.  The reference has one (llsa_l1) and two (llsa_l2); the functions below state the
# scheme for k levels by induction on sparse_attention_res_2.py:94-149 and reduce to the functions above for
# k = 1, 2, 3 (tests/test_oracle_pins.py checks that they do, bit for bit).
#   pks, pvs : pooled k, v of level 1 .. k        sels : [indices, p_indices, pp_indices, ...], k entries --
#   sels[l] (B,H,N/bs^(l+1),T_l) holds the blocks of level l (level 0 = the tokens) that every group of bs^(l+1)
#   queries selected; the coarsest level k is read in full.
# --------------------------------------------------------------------------------------


def _segments_lk(q, k, v, pks, pvs, sels, weights, bs):
    B, H, N, D = q.shape
    N1 = N // bs
    L = len(pks)
    segs = [(_gather_blocks(k, sels[0], bs), _gather_blocks(v, sels[0], bs), 1.0)]
    for l in range(1, L):                                     # owner of query block g at level l: g // bs^l
        own = sels[l].long().repeat_interleave(bs ** l, dim=2)
        segs.append((_gather_blocks(pks[l - 1], own, bs), _gather_blocks(pvs[l - 1], own, bs), float(weights[l - 1])))
    kc, vc = pks[L - 1], pvs[L - 1]
    segs.append((kc[:, :, None].expand(B, H, N1, kc.shape[2], D), vc[:, :, None].expand(B, H, N1, vc.shape[2], D), float(weights[L - 1])))
    return segs


def attn_fwd_lk(q, k, v, pks, pvs, sels, weights=None, block_size=16):
    weights = weights or [block_size ** (l + 1) for l in range(len(pks))]
    return _online_softmax(q, _segments_lk(q, k, v, pks, pvs, sels, weights, block_size), block_size)


def closed_form_lk(q, k, v, pks, pvs, sels, weights=None, bs=16):
    weights = weights or [bs ** (l + 1) for l in range(len(pks))]
    return attn_closed_form(q, _segments_lk(q, k, v, pks, pvs, sels, weights, bs), bs)


def attn_bwd_lk(do, q, k, v, pks, pvs, o, lse, sels, weights=None, block_size=16, coarse_grad_weight=None, delta_in_dtype=False):
    """Returns (dq, dk, dv, [dpk_1 .. dpk_k], [dpv_1 .. dpv_k]).  coarse_grad_weight replaces the weight of the coarsest
    level on the path to its own gradient (the llsa_l1 quirk, see attn_bwd_l1)."""
    B, H, N, D = q.shape
    bs, dt = block_size, q.dtype
    L = len(pks)
    weights = weights or [bs ** (l + 1) for l in range(L)]
    G = N // bs
    scale = 1.0 / math.sqrt(D)
    qb = q.float().reshape(B, H, G, bs, D)
    dob = do.float().reshape(B, H, G, bs, D)
    lse_b = lse.reshape(B, H, G, bs)
    delta = attn_delta(o, do, delta_in_dtype).reshape(B, H, G, bs)
    segs = _segments_lk(q, k, v, pks, pvs, sels, weights, bs)
    parts = [_bwd_segment(qb, dob, lse_b, delta, ks, vs, w, scale, dt) for ks, vs, w in segs]
    dq = sum(p[0] for p in parts).reshape(B, H, N, D)
    dk = _scatter_blocks(torch.zeros(B, H, N, D), parts[0][1], sels[0], bs)
    dv = _scatter_blocks(torch.zeros(B, H, N, D), parts[0][2], sels[0], bs)
    dpks, dpvs = [], []
    for l in range(1, L):
        own = sels[l].long().repeat_interleave(bs ** l, dim=2)
        dpks.append(_scatter_blocks(torch.zeros(B, H, pks[l - 1].shape[2], D), parts[l][1], own, bs))
        dpvs.append(_scatter_blocks(torch.zeros(B, H, pvs[l - 1].shape[2], D), parts[l][2], own, bs))
    last = parts[L]
    if coarse_grad_weight is not None:
        last = _bwd_segment(qb, dob, lse_b, delta, segs[L][0], segs[L][1], float(coarse_grad_weight), scale, dt)
    dpks.append(last[1].sum(2))
    dpvs.append(last[2].sum(2))
    rn = lambda x: _rn(x, dt).to(dt)
    return rn(dq), rn(dk), rn(dv), [rn(x) for x in dpks], [rn(x) for x in dpvs]


def llsa_lk_fwd(q, k, v, topks, block_size=16, sels=None):
    """k = len(topks) pooled levels: dense selection on the coarsest level's tokens (topk.py:6-9), then parent-guided
    selection level by level (topk.py:102-197) down to the fine blocks.  sels overrides the selection."""
    bs = block_size
    L = len(topks)
    pqs, pks, pvs = [], [], []
    xq, xk, xv = q, k, v
    for _ in range(L):
        xq, xk, xv = mean_pool(xq, bs), mean_pool(xk, bs), mean_pool(xv, bs)
        pqs.append(xq), pks.append(xk), pvs.append(xv)
    if sels is None:
        sels = [None] * L
        sels[L - 1] = gen_sparse_indices(pqs[L - 1], pks[L - 1], topks[L - 1])
        for l in range(L - 1, 0, -1):
            sels[l - 1] = topk_sparse(pqs[l - 1], pks[l - 1], sels[l], topks[l - 1], bs)
    o, lse = attn_fwd_lk(q, k, v, pks, pvs, sels, None, bs)
    return o, dict(q=q, k=k, v=v, pqs=pqs, pks=pks, pvs=pvs, o=o, lse=lse, sels=sels, block_size=bs)


def llsa_lk_bwd(do, ctx, delta_in_dtype=False):
    """Backward with the chain of pool backwards autograd adds around the operator (one level: the llsa_l1 quirk)."""
    c = ctx
    bs = c["block_size"]
    L = len(c["pks"])
    dq, dk, dv, dpks, dpvs = attn_bwd_lk(do, c["q"], c["k"], c["v"], c["pks"], c["pvs"], c["o"], c["lse"], c["sels"], None, bs,
                                         coarse_grad_weight=1.0 if L == 1 else None, delta_in_dtype=delta_in_dtype)
    gk, gv = dpks[L - 1], dpvs[L - 1]
    for l in range(L - 2, -1, -1):
        gk = dpks[l] + mean_pool_bwd(gk, bs)
        gv = dpvs[l] + mean_pool_bwd(gv, bs)
    dk = dk + mean_pool_bwd(gk, bs)
    dv = dv + mean_pool_bwd(gv, bs)
    return dq, dk, dv, dict(dpks=dpks, dpvs=dpvs)

