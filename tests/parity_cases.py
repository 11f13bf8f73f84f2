"""Parity checks of the HIP kernels against the CPU oracle, written once and run twice:
on the GPU through libllsa_hip.so (tests/test_gpu_parity.py, `-m gpu`) and, at tiny sizes,
on the CPU through the x86 emulation build of the same sources (tests/test_emu_parity.py).

Tolerances (bf16): outputs and gradients must satisfy
    rel-L2 error      <= 1e-2
    max-abs error     <= 2e-2             flat, on the benchmark configurations and in the smoke test (FLAT = True below:
                                          every check of the whole operator on the smooth-field inputs)
                      <= 2e-2             for every element whose reference value is below 2 in magnitude, and
                      <= 2e-2 * |ref|     for the others, on the random stress shapes only (N(0,1) inputs scaled up, hot
                                          blocks: one bf16 ulp is 1.6e-2 in [2, 4), 3.1e-2 in [4, 8), so a flat 2e-2 is
                                          below the resolution of the output format there)
Integer results (pool bit patterns, indices on rows the rounding cannot decide otherwise, CSR) must be identical.
"""
import math

import torch

from oracle import llsa_oracle as O

REL_L2 = 1e-2
MAX_ABS = 2e-2
MEASURED = {}        # name of the last check -> {tensor: (rel-L2, max-abs)}, for reports


def close(name, got, ref, rel=REL_L2, mabs=MAX_ABS, report=None, flat=False):
    """flat=True: max-abs <= mabs on every element below |ref| = 4 (the flat bound the target states; there a bf16 ulp is
    at most 1.6e-2), and at most one bf16 ulp of the reference (2^-7 |ref|: 3.1e-2 in [4, 8)) above, where two correctly
    rounded results on either side of a rounding step already differ by more than mabs."""
    g, r = got.detach().double().cpu(), ref.detach().double().cpu()
    assert g.shape == r.shape, f"{name}: shape {tuple(g.shape)} vs {tuple(r.shape)}"
    assert torch.isfinite(g).all(), f"{name}: non-finite values"
    err = (g - r).abs()
    e_rel = ((g - r).norm() / r.norm().clamp_min(1e-30)).item()
    e_abs = err.max().item()
    if flat:
        over = (err - torch.where(r.abs() < 4.0, torch.full_like(r, mabs), 2.0 ** -7 * r.abs())).max().item()
        assert over <= 0.0, f"{name}: max-abs {e_abs:.3e}; an element exceeds the flat bound ({mabs} below |ref| = 4, one bf16 ulp above) by {over:.3e}"
    bound = torch.where(r.abs() < 2.0, torch.full_like(r, mabs), mabs * r.abs())
    worst = (err - bound).max().item()
    assert e_rel <= rel, f"{name}: rel-L2 {e_rel:.3e} (<= {rel})"
    assert worst <= 0.0, f"{name}: max-abs {e_abs:.3e}; an element exceeds its bound ({mabs} below |ref| = 2, {mabs} * |ref| above) by {worst:.3e}"
    if report is not None:
        MEASURED.setdefault(report, {})[name] = (e_rel, e_abs)
    return e_rel, e_abs


def smooth_inputs(B, H, N, D, dev, seeds=(1, 2, 3, 4)):
    from llsa_amd.utils.synth import smooth_field
    q = smooth_field(seeds[0], B, H, N, D)
    k = smooth_field(seeds[1], B, H, N, D)
    v = smooth_field(seeds[2], B, H, N, D)
    do = torch.randn(B, H, N, D, generator=torch.Generator().manual_seed(seeds[3])).bfloat16()
    return tuple(t.to(dev) for t in (q, k, v, do))


def randn_inputs(B, H, N, D, dev, seed=0, strided=False):
    g = torch.Generator().manual_seed(seed)
    if strided:      # physical layout (B,N,H,D) viewed as (B,H,N,D), what the DiT attention processor passes
        mk = lambda: torch.randn(B, N, H, D, generator=g).bfloat16().to(dev).transpose(1, 2)
    else:
        mk = lambda: torch.randn(B, H, N, D, generator=g).bfloat16().to(dev)
    return mk(), mk(), mk(), mk()


# ------------------------------------------------------------------------------------------
def _r_tiles(x):
    """(B,H,n,64) -> (B,H,n/16,1024) R tiles: element (row t, channel c) at ((c>>3)*16 + t)*8 + (c&7)."""
    B, H, n, _ = x.shape
    return x.reshape(B, H, n // 16, 16, 8, 8).permute(0, 1, 2, 4, 3, 5).reshape(B, H, n // 16, 1024)


def _t_tiles(x):
    """T tiles: element (row t, channel c) at (((c>>4)*4 + (t>>2))*16 + (c&15))*4 + (t&3)."""
    B, H, n, _ = x.shape
    return x.reshape(B, H, n // 16, 4, 4, 4, 16).permute(0, 1, 2, 5, 3, 6, 4).reshape(B, H, n // 16, 1024)


def check_pool_pyramid(dev, B=1, H=2, N=512, strided=True, rope=True):
    from llsa_amd.kernel.hip.mean_pool import PoolSpec, pool_pyramid
    x, *_ = randn_inputs(B, H, N, 64, dev, seed=5, strided=strided)
    x = x * 2
    freq = torch.randn(N, 64, generator=torch.Generator().manual_seed(6)).bfloat16().to(dev) if rope else None
    lvl2 = N % 4096 == 0
    out, = pool_pyramid([PoolSpec(x, y1=True, y2=True, xr=True, xt=True, y1r=True, y1t=True, rope=rope, xrot=rope,
                                  y2r=lvl2, y2t=lvl2)], freq)
    xc = x.cpu()
    xr = O.rope_apply(xc, freq.cpu()) if rope else xc
    p1 = O.mean_pool(xr)
    p2 = O.mean_pool(p1)
    if rope:
        assert torch.equal(out["xrot"].cpu(), xr), "rotated copy differs"
    assert torch.equal(out["y1"].cpu(), p1), "level-1 pool differs"
    assert torch.equal(out["y2"].cpu(), p2), "level-2 pool differs"
    assert torch.equal(out["xr"].cpu(), _r_tiles(xr)), "R tiles differ"
    assert torch.equal(out["xt"].cpu(), _t_tiles(xr)), "T tiles differ"
    assert torch.equal(out["y1r"].cpu(), _r_tiles(p1)), "R tiles of the pooled level differ"
    assert torch.equal(out["y1t"].cpu(), _t_tiles(p1)), "T tiles of the pooled level differ"
    if lvl2:
        assert torch.equal(out["y2r"].cpu(), _r_tiles(p2)), "R tiles of the level-2 rows differ"
        assert torch.equal(out["y2t"].cpu(), _t_tiles(p2)), "T tiles of the level-2 rows differ"


def check_mean_pool1d(dev, dtype=torch.bfloat16, K=16, C=64, S=128, fmt='bhsc'):
    from llsa_amd.kernel.hip.mean_pool import mean_pool1d
    g = torch.Generator().manual_seed(7)
    shape = (2, 3, S, C) if fmt == 'bhsc' else (2, S, C)
    x = (torch.randn(*shape, generator=g) * 3).to(dtype).to(dev).requires_grad_(True)
    y = mean_pool1d(x, K, fmt)
    dy = torch.randn(*y.shape, generator=g).to(dtype).to(dev)
    y.backward(dy)
    xc = x.detach().cpu()
    x4 = xc if fmt == 'bhsc' else xc.unsqueeze(1)
    ref = O.mean_pool(x4, K)
    dref = O.mean_pool_bwd(dy.cpu() if fmt == 'bhsc' else dy.cpu().unsqueeze(1), K)
    if fmt == 'bsc':
        ref, dref = ref.squeeze(1), dref.squeeze(1)
    assert torch.equal(y.detach().cpu(), ref), "mean_pool1d forward differs"
    assert torch.equal(x.grad.cpu(), dref), "mean_pool1d backward differs"


def check_rope(dev, B=1, H=2, side=8, strided=True):
    from llsa_amd.kernel.hip.rope import my_rope_fn
    from llsa_amd.utils.rope_table import rope_table
    N = side * side
    x, dy, *_ = randn_inputs(B, H, N, 64, dev, seed=8, strided=strided)
    freq = rope_table(side, dtype=torch.bfloat16).to(dev)
    assert torch.equal(freq.cpu(), O.rope_table(side, dtype=torch.bfloat16)), "rope table differs"
    x = x.detach().requires_grad_(True)
    y = my_rope_fn(x, freq)
    y.backward(dy)
    assert torch.equal(y.detach().cpu(), O.rope_apply(x.detach().cpu(), freq.cpu())), "rope forward differs"
    assert torch.equal(x.grad.cpu(), O.rope_apply_bwd(dy.cpu(), freq.cpu())), "rope backward differs"


def _safe_rows(score, T, eps_rel):
    """Rows whose T-th / (T+1)-th scores (and, for the ordered check, all adjacent pairs among
    the best T+1) are separated by more than eps_rel * max(1, |score|)."""
    s, _ = torch.sort(score, dim=-1, descending=True)
    top = s[..., :T + 1] if s.shape[-1] > T else s
    gaps = top[..., :-1] - top[..., 1:]
    tol = eps_rel * top[..., :-1].abs().clamp_min(1.0)
    boundary_ok = (gaps[..., T - 1] > tol[..., T - 1]) if s.shape[-1] > T else torch.ones_like(gaps[..., 0], dtype=torch.bool)
    ordered_ok = (gaps > tol).all(-1)
    return boundary_ok, ordered_ok


def decided_rows_dense(pq, pk, T):
    """Rows of the bf16-rounded dense selection whose top-T SET cannot depend on how the fp32 dot products were
    summed.  Device and oracle round the same 64-term dot product to bf16 (topk.py:7), added in different orders:
    the two fp32 values differ by a few ulps, and the rounded values differ only where the fp32 value sits that close
    to the midpoint of two neighbouring bf16 numbers.  With delta = 2^-20 * sum_c |pq_c pk_c| (a bound on the
    summation error with a wide margin: 64 terms, eps = 2^-24), every score has a lowest and a highest possible
    rounded value, lo = bf16(s - delta) and hi = bf16(s + delta) (equal for an unambiguous score).  A row is decided
    when every ambiguous member of the oracle's top-T stays strictly above whatever any outsider can reach and
    every ambiguous outsider stays strictly below whatever any member can fall to; the unambiguous scores have the
    same bits on both sides, and so the same ranking with the same tie rule (smaller index first).  Returns
    (decided (.., n) bool, ordered (.., n) bool: no ambiguous score anywhere among the best T + 1, so that the order
    of the T indices is decided too)."""
    s = pq.float() @ pk.float().transpose(-1, -2)
    mag = pq.float().abs() @ pk.float().abs().transpose(-1, -2)
    delta = mag * 2.0 ** -20
    lo, hi = (s - delta).bfloat16().float(), (s + delta).bfloat16().float()
    amb = lo != hi
    ref = O.topk_lowest_index(s.bfloat16(), T)
    member = torch.zeros_like(amb).scatter_(-1, ref, True)
    inf = torch.full_like(s, float("inf"))
    min_in_lo = torch.where(member, lo, inf).amin(-1, keepdim=True)
    max_out_hi = torch.where(member, -inf, hi).amax(-1, keepdim=True)
    bad = amb & ((member & (lo <= max_out_hi)) | (~member & (hi >= min_in_lo)))
    decided = ~bad.any(-1)
    # order: the best T + 1 (by the rounded score) and everything that could tie with them must be unambiguous
    n = s.shape[-1]
    kth1 = torch.sort(s.bfloat16().float(), -1, descending=True).values[..., min(T, n - 1):min(T, n - 1) + 1]
    ordered = decided & ~(amb & (hi >= kth1)).any(-1)
    return decided, ordered


def check_topk_dense(dev, B=1, H=2, n=64, T=8, round_scores=True, min_safe=0.3):
    from llsa_amd.kernel.hip.topk import gen_sparse_indices
    g = torch.Generator().manual_seed(9)
    pq = torch.randn(B, H, n, 64, generator=g).bfloat16()
    pk = torch.randn(B, H, n, 64, generator=g).bfloat16()
    idx = gen_sparse_indices(pq.to(dev), pk.to(dev), T, round_scores=round_scores).cpu().long()
    assert idx.shape == (B, H, n, T) and idx.min() >= 0 and idx.max() < n
    assert (idx.sort(-1).values.diff(dim=-1) > 0).all(), "duplicate index in a row"
    exact = O.dense_scores(pq, pk, round_to_input=False)
    ref = O.topk_lowest_index(O.dense_scores(pq, pk, round_to_input=round_scores), T)
    if round_scores:
        b_ok, o_ok = decided_rows_dense(pq, pk, T)
        min_safe = max(min_safe, 0.85)
    else:
        b_ok, o_ok = _safe_rows(exact, T, 1e-4)
    assert b_ok.float().mean() >= min_safe, f"test input has too few decided rows ({b_ok.float().mean():.2f})"
    same_set = (idx.sort(-1).values == ref.sort(-1).values).all(-1)
    assert same_set[b_ok].all(), "selected set differs on tie-free rows"
    assert (idx == ref).all(-1)[o_ok].all(), "order differs on rows with well separated scores"
    # descending by the rounded score everywhere
    sc = torch.gather(O.dense_scores(pq, pk, round_to_input=round_scores), -1, idx)
    tol = (2.0 ** -6 if round_scores else 1e-4) * sc.abs().clamp_min(1.0)
    assert (sc[..., :-1] - sc[..., 1:] >= -tol[..., 1:]).all(), "not descending"
    return idx


def check_topk_dense_ties(dev):
    """Exact ties (duplicated key rows): the smaller index must come first."""
    from llsa_amd.kernel.hip.topk import gen_sparse_indices
    g = torch.Generator().manual_seed(10)
    pq = torch.randn(1, 1, 32, 64, generator=g).bfloat16()
    pk = torch.randn(1, 1, 32, 64, generator=g).bfloat16()
    pk[0, 0, 20] = pk[0, 0, 3]
    pk[0, 0, 9] = pk[0, 0, 3]
    idx = gen_sparse_indices(pq.to(dev), pk.to(dev), 32).cpu().long()      # full ranking
    for row in idx[0, 0]:
        pos = {int(v): i for i, v in enumerate(row)}
        assert pos[3] + 1 == pos[9] and pos[9] + 1 == pos[20], "equal scores must be ordered by index"


def check_topk_sparse(dev, B=1, H=2, N1=256, T=8, T2=4):
    from llsa_amd.kernel.hip.topk import compute_topk_indices_sparse
    g = torch.Generator().manual_seed(11)
    pq = torch.randn(B, H, N1, 64, generator=g).bfloat16()
    pk = torch.randn(B, H, N1, 64, generator=g).bfloat16()
    N2 = N1 // 16
    pidx = torch.stack([torch.randperm(N2, generator=g)[:T2] for _ in range(B * H * N2)]).reshape(B, H, N2, T2).int()
    idx = compute_topk_indices_sparse(pq.to(dev), pk.to(dev), pidx.to(dev), T, T2).cpu()
    assert idx.dtype == torch.int32 and idx.shape == (B, H, N1, T)
    ref, score, gidx = O.topk_sparse(pq, pk, pidx.long(), T, return_scores=True)
    par = pidx.long().repeat_interleave(16, dim=2)
    assert ((idx.long()[..., None] // 16) == par[:, :, :, None, :]).any(-1).all(), "index outside the parent's blocks"
    assert (idx.long().sort(-1).values.diff(dim=-1) > 0).all(), "duplicate index in a row"
    b_ok, o_ok = _safe_rows(score, T, 1e-4)
    assert b_ok.float().mean() > 0.9
    assert (idx.sort(-1).values == ref.sort(-1).values).all(-1)[b_ok].all(), "selected set differs on tie-free rows"
    assert (idx == ref).all(-1)[o_ok].all(), "order differs on rows with well separated scores"


def check_topk_cascade(dev, B=1, H=2, N1=1024, T=8, T2=4):
    """The one-launch cascade gives, bit for bit, what the dense selection followed by the parent-guided one give."""
    from llsa_amd.kernel.hip.topk import compute_topk_indices_sparse, gen_sparse_indices, topk_cascade
    g = torch.Generator().manual_seed(17)
    pq = torch.randn(B, H, N1, 64, generator=g).bfloat16()
    pk = torch.randn(B, H, N1, 64, generator=g).bfloat16()
    pq2, pk2 = O.mean_pool(pq, 16), O.mean_pool(pk, 16)
    p_ref = gen_sparse_indices(pq2.to(dev), pk2.to(dev), T2)
    ref = compute_topk_indices_sparse(pq.to(dev), pk.to(dev), p_ref, T, T2)
    p_got, got = topk_cascade(pq2.to(dev), pk2.to(dev), pq.to(dev), pk.to(dev), T, T2)
    assert torch.equal(p_got.cpu(), p_ref.cpu()), "parent selection differs from llsa_topk_dense"
    assert torch.equal(got.cpu(), ref.cpu()), "selection differs from llsa_topk_sparse under the same parents"


def check_transpose(dev, B=2, H=2, Mb=64, T=8, Kb=None, chunk=0):
    """chunk > 0 also asks for the work list, which with Mb*T >= 65536 entries switches the kernel to
    its split form (histogram and scatter over many workgroups)."""
    from llsa_amd.kernel.hip.indices_transpose import transpose_indices
    g = torch.Generator().manual_seed(12)
    kb = Kb or Mb
    if Mb <= 16384:
        idx = torch.stack([torch.randperm(kb, generator=g)[:T] for _ in range(B * H * Mb)]).reshape(B, H, Mb, T).int()
    else:            # distinct within a row: base + t * stride with T * stride <= kb, modulo kb
        base = torch.randint(0, kb, (B, H, Mb, 1), generator=g)
        stride = torch.randint(1, kb // T + 1, (B, H, Mb, 1), generator=g)
        idx = ((base + torch.arange(T) * stride) % kb).int()
    res = transpose_indices(idx.to(dev), Kb, chunk, inverse=True)
    off, flat, inv = res[0], res[1], res[-1].cpu().long()
    ro, rf = O.transpose_indices(idx.long(), Kb)
    assert torch.equal(off.cpu().long(), ro), "offsets differ"
    assert torch.equal(flat.cpu().long(), rf), "flat list differs"
    # the inverse: entry (q, t) sits at a position of the segment of key block idx[q, t], and that position holds q
    qid = torch.arange(Mb).view(1, 1, Mb, 1).expand(B, H, Mb, T)
    assert torch.equal(torch.gather(rf, -1, inv.reshape(B, H, -1)).reshape(B, H, Mb, T), qid), "inverse positions do not hold their query block"
    lo, hi = torch.gather(ro, -1, idx.long().reshape(B, H, -1)), torch.gather(ro, -1, idx.long().reshape(B, H, -1) + 1)
    assert ((inv.reshape(B, H, -1) >= lo) & (inv.reshape(B, H, -1) < hi)).all(), "inverse position outside its key block's segment"


def check_transpose_levels(dev, B=2, H=3, sizes=((1024, 16), (64, 16)), chunk=64):
    """All levels with one call of the library (one launch when the bitmaps fit) against the oracle and against
    the work list the single-level call builds."""
    from llsa_amd.kernel.hip.indices_transpose import transpose_indices, transpose_indices_levels
    g = torch.Generator().manual_seed(14)
    sels = [torch.stack([torch.randperm(Mb, generator=g)[:T] for _ in range(B * H * Mb)]).reshape(B, H, Mb, T).int() for Mb, T in sizes]
    res = transpose_indices_levels([s.to(dev) for s in sels], chunk)
    for l, (sel, (off, flat, extra)) in enumerate(zip(sels, res)):
        Mb, T = sel.shape[2:]
        ro, rf = O.transpose_indices(sel.long(), None)
        assert torch.equal(off.cpu().long(), ro), f"level {l}: offsets differ"
        assert torch.equal(flat.cpu().long(), rf), f"level {l}: flat list differs"
        if l == 0:
            work = transpose_indices(sel.to(dev), None, chunk)[2].cpu()
            got, max_items = extra.cpu(), Mb * T // chunk + Mb
            for b in range(B):              # header, items and multi-piece records (what lies beyond them is never read)
                for h in range(H):
                    a, w = got[b, h], work[b, h]
                    assert torch.equal(a[:4], w[:4]), "work list header differs from the single call's"
                    assert torch.equal(a[4:4 + 4 * int(w[0])], w[4:4 + 4 * int(w[0])]), "work items differ from the single call's"
                    m0 = 4 + 4 * max_items
                    assert torch.equal(a[m0:m0 + 4 * int(w[2])], w[m0:m0 + 4 * int(w[2])]), "multi-piece records differ"
        else:
            qid = torch.arange(Mb).view(1, 1, Mb, 1).expand(B, H, Mb, T)
            inv = extra.cpu().long().reshape(B, H, -1)
            assert torch.equal(torch.gather(rf, -1, inv).reshape(B, H, Mb, T), qid), f"level {l}: inverse positions do not hold their query block"


def check_transpose_hot_block(dev):
    """Every query block selects key block 5 (a segment as long as the query axis) plus others."""
    from llsa_amd.kernel.hip.indices_transpose import transpose_indices
    B, H, Mb, T = 1, 1, 256, 4
    g = torch.Generator().manual_seed(13)
    rest = torch.stack([(torch.randperm(Mb - 1, generator=g)[:T - 1] + 6) % Mb for _ in range(Mb)])
    rest[rest == 5] = 4
    idx = torch.cat([torch.full((Mb, 1), 5), rest], 1).reshape(B, H, Mb, T).int()
    # make rows distinct where the remap collided
    for r in range(Mb):
        while len(set(idx[0, 0, r].tolist())) < T:
            idx[0, 0, r, 1:] = (torch.randperm(Mb - 8, generator=g)[:T - 1] + 8).int()
    off, flat = transpose_indices(idx.to(dev))
    ro, rf = O.transpose_indices(idx.long())
    assert torch.equal(off.cpu().long(), ro) and torch.equal(flat.cpu().long(), rf)


# ------------------------------------------------------------------------------------------
def _selection_l1(q, k, T):
    pq, pk = O.mean_pool(q.cpu()), O.mean_pool(k.cpu())
    return O.topk_lowest_index(O.dense_scores(pq, pk), T)


def _hot_indices(B, H, Mb, Kb, T, hot, seed):
    """Every row selects block `hot` first; the rest are distinct random blocks."""
    g = torch.Generator().manual_seed(seed)
    rows = []
    for _ in range(B * H * Mb):
        rest = torch.randperm(Kb - 1, generator=g)[:T - 1]
        rest = rest + (rest >= hot).long()
        rows.append(torch.cat([torch.tensor([hot]), rest]))
    return torch.stack(rows).reshape(B, H, Mb, T)


def check_attn_l1(dev, B=1, H=2, N=1024, T=8, strided=False, smooth=False, weight=16.0, hot=None):
    """Forward and backward kernels with oracle-chosen indices (or, with `hot`, indices in which
    one key block is selected by every query block, so that its list is cut into chunks)."""
    from llsa_amd.kernel.hip._attention import attn_bwd, attn_fwd
    q, k, v, do = smooth_inputs(B, H, N, 64, dev) if smooth else randn_inputs(B, H, N, 64, dev, seed=14, strided=strided)
    qc, kc, vc, doc = (t.cpu() for t in (q, k, v, do))
    pk, pv = O.mean_pool(kc), O.mean_pool(vc)
    idx = _selection_l1(qc, kc, T) if hot is None else _hot_indices(B, H, N // 16, N // 16, T, hot, 21)
    o, lse = attn_fwd(q, k, v, pk.to(dev), pv.to(dev), idx.int().to(dev), weight)
    ro, rl = O.attn_fwd_l1(qc, kc, vc, pk, pv, idx, weight)
    assert o.stride() == q.stride(), "o must have q's strides"
    close("o", o, ro)
    assert (lse.cpu() - rl).abs().max() < 2e-3, f"lse differs by {(lse.cpu() - rl).abs().max():.3e}"
    got = attn_bwd(do, q, k, v, pk.to(dev), pv.to(dev), o, lse, idx.int().to(dev), weight, 1.0)
    ref = O.attn_bwd_l1(doc, qc, kc, vc, pk, pv, o.cpu(), lse.cpu(), idx, weight)
    for name, a, b in zip(("dq", "dk", "dv", "dpk", "dpv"), got, ref):
        close(name, a, b)
    _check_fold(dev, got, lambda **kw: attn_bwd(do, q, k, v, pk.to(dev), pv.to(dev), o, lse, idx.int().to(dev), weight, 1.0,
                                                **kw), N)


def check_attn_fwd_repeated_block(dev, B=1, H=2, N=1024, T=8):
    """The forward kernel with rows that name a block twice (a caller's indices may; a top-k output does not): such
    a row counts the block twice, like the reference's gather, and the sibling row that shares a wave with it must
    not be affected.  Every fourth query block repeats its first entry in its last."""
    from llsa_amd.kernel.hip._attention import attn_fwd
    q, k, v, _ = randn_inputs(B, H, N, 64, dev, seed=31)
    qc, kc, vc = (t.cpu() for t in (q, k, v))
    pk, pv = O.mean_pool(kc), O.mean_pool(vc)
    idx = _selection_l1(qc, kc, T).clone()
    idx[:, :, ::4, T - 1] = idx[:, :, ::4, 0]
    idx[:, :, 1::8, 1] = idx[:, :, 0::8, 0]              # and some siblings that share blocks with the repeating row
    o, lse = attn_fwd(q, k, v, pk.to(dev), pv.to(dev), idx.int().to(dev), 16.0)
    ro, rl = O.attn_fwd_l1(qc, kc, vc, pk, pv, idx, 16.0)
    close("o", o, ro)
    assert (lse.cpu() - rl).abs().max() < 2e-3, f"lse differs by {(lse.cpu() - rl).abs().max():.3e}"


def check_attn_l2(dev, B=1, H=1, N=16384, T=8, T2=4, smooth=False, hot=None):
    from llsa_amd.kernel.hip._attention import attn_bwd, attn_fwd
    q, k, v, do = smooth_inputs(B, H, N, 64, dev) if smooth else randn_inputs(B, H, N, 64, dev, seed=15)
    qc, kc, vc, doc = (t.cpu() for t in (q, k, v, do))
    pq, pk, pv = O.mean_pool(qc), O.mean_pool(kc), O.mean_pool(vc)
    pq2, pk2, pv2 = O.mean_pool(pq), O.mean_pool(pk), O.mean_pool(pv)
    if hot is None:
        pidx = O.topk_lowest_index(O.dense_scores(pq2, pk2), T2)
    else:                     # every parent selects coarse block `hot`: its parent list is cut into chunks
        pidx = _hot_indices(B, H, N // 256, N // 256, T2, hot, 22)
    idx = O.topk_sparse(pq, pk, pidx, T)
    d = lambda t: t.to(dev)
    o, lse = attn_fwd(q, k, v, d(pk), d(pv), d(idx), 16.0, pk2=d(pk2), pv2=d(pv2), p_indices=d(pidx.int()),
                      token_weight_2=256.0)
    ro, rl = O.attn_fwd_l2(qc, kc, vc, pk, pv, pk2, pv2, idx, pidx)
    close("o", o, ro)
    assert (lse.cpu() - rl).abs().max() < 2e-3
    got = attn_bwd(do, q, k, v, d(pk), d(pv), o, lse, d(idx), 16.0, 16.0, pk2=d(pk2), pv2=d(pv2),
                   p_indices=d(pidx.int()), token_weight_2=256.0)
    ref = O.attn_bwd_l2(doc, qc, kc, vc, pk, pv, pk2, pv2, o.cpu(), lse.cpu(), idx, pidx)
    for name, a, b in zip(("dq", "dk", "dv", "dpk", "dpv", "dpk2", "dpv2"), got, ref):
        close(name, a, b)
    _check_fold(dev, got, lambda **kw: attn_bwd(do, q, k, v, d(pk), d(pv), o, lse, d(idx), 16.0, 16.0, pk2=d(pk2), pv2=d(pv2),
                                                p_indices=d(pidx.int()), token_weight_2=256.0, **kw), N)


def _check_fold(dev, plain, run, N):
    """fold_pooled=True must give, bit for bit, what pool_bwd_accum makes of the unfolded outputs
    (with the same RoPE rotate-back of dk), and leave the other outputs unchanged."""
    import math
    from llsa_amd.kernel.hip.mean_pool import pool_bwd_accum
    side = 1 << math.ceil(math.log2(N) / 2)                   # any (N, 64) sin/cos table will do here
    freq = O.rope_table(side, dtype=torch.bfloat16)[:N].contiguous().to(dev)
    folded = run(fold_pooled=True, freq_dk=freq)
    dpk2, dpv2 = (plain[5], plain[6]) if len(plain) > 5 else (None, None)
    want_dk = pool_bwd_accum(plain[1], plain[3], dpk2, freq)
    want_dv = pool_bwd_accum(plain[2], plain[4], dpv2, None)
    assert torch.equal(folded[1].cpu(), want_dk.cpu()), "folded dk differs from pool_bwd_accum"
    assert torch.equal(folded[2].cpu(), want_dv.cpu()), "folded dv differs from pool_bwd_accum"
    for i in (0,) + tuple(range(3, len(plain))):
        assert torch.equal(folded[i].cpu(), plain[i].cpu()), f"output {i} changed with fold_pooled"


def check_attn_reduces_to_sdpa(dev, B=1, H=2, N=1024):
    """All blocks selected and a vanishing pooled weight: the kernel must equal dense attention."""
    import torch.nn.functional as F
    from llsa_amd.kernel.hip._attention import attn_fwd
    q, k, v, _ = randn_inputs(B, H, N, 64, dev, seed=16)
    N1 = N // 16
    g = torch.Generator().manual_seed(17)
    idx = torch.stack([torch.randperm(N1, generator=g) for _ in range(B * H * N1)]).reshape(B, H, N1, N1).int()
    pk, pv = O.mean_pool(k.cpu()).to(dev), O.mean_pool(v.cpu()).to(dev)
    o, lse = attn_fwd(q, k, v, pk, pv, idx.to(dev), 2.0 ** -60)
    ref = F.scaled_dot_product_attention(q.cpu().float(), k.cpu().float(), v.cpu().float())
    close("o vs sdpa", o, ref)
    rl = torch.logsumexp(q.cpu().float() @ k.cpu().float().transpose(-1, -2) / 8.0, -1)
    assert (lse.cpu() - rl).abs().max() < 2e-3


def check_constant_v(dev, N=1024):
    from llsa_amd.kernel.hip._attention import attn_fwd
    q, k, _, _ = randn_inputs(1, 1, N, 64, dev, seed=18)
    v = torch.full((1, 1, N, 64), 0.75, dtype=torch.bfloat16, device=dev)
    idx = _selection_l1(q, k, 4)
    o, _ = attn_fwd(q, k, v, O.mean_pool(k.cpu()).to(dev), O.mean_pool(v.cpu()).to(dev), idx.int().to(dev), 16.0)
    assert (o.float() - 0.75).abs().max() < 4e-3


# ------------------------------------------------------------------------------------------
def selection_dense_vs_oracle(what, pq, pk, got, T, strict=True):
    """The device's coarsest selection `got` (.., n, T) against the oracle's own: torch.matmul's bf16-rounded
    scores (topk.py:6-9) ranked with ties to the smaller index.  Index sets must be identical on every row that
    the summation order of the dot products cannot decide otherwise (decided_rows_dense: exact ties included, they
    go to the smaller index on both sides), and everywhere the selection must be a legal top-k of the rounded
    scores.  Returns (fraction of rows with identical sets, fraction of rows under the strict check)."""
    got = got.long()
    rounded = O.dense_scores(pq, pk)
    ref = O.topk_lowest_index(rounded, T)
    b_ok, _ = decided_rows_dense(pq, pk, T)
    same = (got.sort(-1).values == ref.sort(-1).values).all(-1)
    assert (got.sort(-1).values.diff(dim=-1) > 0).all(), f"{what}: duplicate index in a row"
    if strict:
        assert same[b_ok].all(), f"{what}: {int((~same[b_ok]).sum())} tie-free rows select another set than the oracle"
    else:
        assert same[b_ok].float().mean() > 0.95, f"{what}: only {same[b_ok].float().mean():.3f} of the tie-free rows agree"
    kth = torch.sort(rounded, -1, descending=True).values[..., T - 1:T]
    picked = torch.gather(rounded, -1, got)
    assert (picked >= kth - 2.0 ** -6 * kth.abs().clamp_min(1.0)).all(), f"{what}: selected a block below the top-k threshold"
    return same.float().mean().item(), b_ok.float().mean().item()


def selection_sparse_vs_oracle(what, pq, pk, pidx, got, T, strict=True):
    """The device's parent-guided selection `got` (.., N1, T) against the oracle's (fp32 scores over the blocks
    under the parents in `pidx`, ties to the smaller index, topk.py:102-197), given the same parents."""
    got = got.long()
    ref, score, gidx = O.topk_sparse(pq, pk, pidx.long(), T, return_scores=True)
    par = pidx.long().repeat_interleave(16, dim=2)
    assert ((got[..., None] // 16) == par[:, :, :, None, :]).any(-1).all(), f"{what}: index outside the parent's blocks"
    assert (got.sort(-1).values.diff(dim=-1) > 0).all(), f"{what}: duplicate index in a row"
    b_ok, _ = _safe_rows(score, T, 1e-4)
    same = (got.sort(-1).values == ref.long().sort(-1).values).all(-1)
    if strict:
        assert same[b_ok].all(), f"{what}: {int((~same[b_ok]).sum())} tie-free rows select another set than the oracle"
    else:
        assert same[b_ok].float().mean() > 0.95, f"{what}: only {same[b_ok].float().mean():.3f} of the tie-free rows agree"
    # legal top-k: every picked score reaches the T-th best score of its row
    kth = torch.sort(score, -1, descending=True).values[..., T - 1:T]
    pos = (gidx[..., None, :] == got[..., :, None]).float().argmax(-1)
    picked = torch.gather(score, -1, pos)
    assert (picked >= kth - 1e-4 * kth.abs().clamp_min(1.0)).all(), f"{what}: selected a block below the top-k threshold"
    return same.float().mean().item(), b_ok.float().mean().item()


def _grads(fn, q, k, v, do):
    q, k, v = (t.detach().requires_grad_(True) for t in (q, k, v))
    o = fn(q, k, v)
    o.backward(do)
    return o.detach(), q.grad, k.grad, v.grad


def check_permute(dev, B=2, side=32, C=96, dtype=torch.bfloat16):
    """gather_tokens / permute_tokens against plain indexing: bit for bit, gradients included."""
    from llsa_amd.kernel.hip.permute import gather_tokens, permute_tokens
    perm, inv = O.zorder_perm(side)
    N = side * side
    g = torch.Generator().manual_seed(5)
    x = torch.randn(B, N, C, generator=g).to(dtype)
    xd = x.clone().to(dev).requires_grad_(True)
    y = permute_tokens(xd, inv.to(dev), perm.to(dev))
    assert torch.equal(y.detach().cpu(), x[:, inv])
    dy = torch.randn(B, N, C, generator=g).to(dtype)
    y.backward(dy.to(dev))
    ref = x.clone().requires_grad_(True)
    ref[:, inv].backward(dy)
    assert torch.equal(xd.grad.cpu(), ref.grad)
    assert torch.equal(gather_tokens(y.detach(), perm.to(dev)).cpu(), x), "entry then exit is not the identity"
    # a shorter index list (a pooled grid), a view with padded batches, and an index out of range
    idx = torch.tensor([3, N - 1, 0, N, -1, 7], dtype=torch.int64)
    wide = torch.randn(B, N + 5, C, generator=g).to(dtype).to(dev)
    got = gather_tokens(wide[:, :N], idx.to(dev)).cpu()
    want = wide.cpu()[:, idx.clamp(0, N - 1)]
    want[:, 3:5] = 0
    assert torch.equal(got, want)


def _norm_weights(dev):
    """(gamma_q, gamma_k, eps) of a qk RMS norm, as the fused operators take them."""
    g = torch.Generator().manual_seed(31)
    return ((torch.rand(64, generator=g) + 0.5).to(dev), (torch.rand(64, generator=g) + 0.5).to(dev), 1e-5)


def _apply_norm(qc, kc, norm):
    if norm is None:
        return qc, kc
    return O.rms_norm(qc, norm[0].cpu(), norm[2]), O.rms_norm(kc, norm[1].cpu(), norm[2])


def _norm_backward(rq, rk, qc, kc, norm):
    if norm is None:
        return rq, rk
    return (O.rms_norm_bwd(rq.to(qc.dtype), qc, norm[0].cpu(), norm[2])[0], O.rms_norm_bwd(rk.to(kc.dtype), kc, norm[1].cpu(), norm[2])[0])


def check_rms_norm(dev, B=2, H=3, N=512, strided=True):
    """Stand-alone forms against the oracle: forward bit for bit up to one bf16 ulp of rounding-order
    freedom (the row's sum of squares is added in another order), backward within the operator's
    tolerance, dgamma in fp32."""
    from llsa_amd.kernel.hip.rms_norm import rms_norm_bwd, rms_norm_fwd
    x, _, _, dy = randn_inputs(B, H, N, 64, dev, seed=23, strided=strided)
    gq, _, eps = _norm_weights(dev)
    y = rms_norm_fwd(x, gq, eps)
    ry = O.rms_norm(x.cpu(), gq.cpu(), eps)
    assert (y.cpu().float() - ry.float()).abs().max() <= 2.0 ** -7 * ry.float().abs().max()
    assert (y.cpu() != ry).float().mean() < 0.02, "more than 2 % of the normalised values differ from the oracle's"
    dx, dg = rms_norm_bwd(dy, x, gq, eps)
    rdx, rdg = O.rms_norm_bwd(dy.cpu(), x.cpu(), gq.cpu(), eps)
    close("dx", dx, rdx)
    assert torch.allclose(dg.cpu(), rdg, rtol=2e-3, atol=2e-2), f"dgamma differs by {(dg.cpu() - rdg).abs().max():.3e}"


def check_op_l1(dev, B=1, H=2, N=1024, T=8, fused=True, rope=False, strided=False, smooth=False, qk_norm=False):
    """The whole operator through autograd, against the oracle's composition fed with the
    indices the device selected (selection itself is checked separately)."""
    from llsa_amd.kernel.hip.rope import my_rope_fn
    from llsa_amd.kernel.torch_op import flash_sparse_attention_res_1 as M
    from llsa_amd.kernel.torch_op._fused import selection
    from llsa_amd.utils.rope_table import rope_table
    q, k, v, do = smooth_inputs(B, H, N, 64, dev) if smooth else randn_inputs(B, H, N, 64, dev, seed=19, strided=strided)
    freq = rope_table(int(math.isqrt(N)), dtype=torch.bfloat16).to(dev) if rope else None
    captured = {}
    norm = _norm_weights(dev) if qk_norm else None

    def run(q_, k_, v_):
        if fused:
            out = M.llsa_l1(q_, k_, v_, T, 16, rope=freq, qk_norm=norm)
            captured["idx"] = selection(out)[0]
            return out
        if rope:
            q_, k_ = my_rope_fn(q_, freq), my_rope_fn(k_, freq)
        out = M.llsa_l1_unfused(q_, k_, v_, T, 16)
        captured["idx"] = out.grad_fn.saved_tensors[7]
        return out

    o, dq, dk, dv = _grads(run, q, k, v, do)
    qc, kc, vc, doc = (t.cpu() for t in (q, k, v, do))
    fc = freq.cpu() if rope else None
    qn, kn = _apply_norm(qc, kc, norm)
    qr, kr = (O.rope_apply(qn, fc), O.rope_apply(kn, fc)) if rope else (qn, kn)
    idx = captured["idx"].cpu().long()
    ro, ctx = O.llsa_l1_fwd(qr, kr, vc, T, 16, indices=idx)
    rq, rk, rv, _ = O.llsa_l1_bwd(doc, ctx)
    if rope:
        rq, rk = O.rope_apply_bwd(rq, fc), O.rope_apply_bwd(rk, fc)
    rq, rk = _norm_backward(rq, rk, qc, kc, norm)
    tag = f"l1 B={B} H={H} N={N} T={T}" + (" rope" if rope else "") + (" qk_norm" if qk_norm else "") + ("" if fused else " unfused")
    for name, a, b in (("o", o, ro), ("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
        close(name, a, b, report=tag, flat=smooth)
    # the selection against the oracle's own (the oracle pooled the same rows: ctx) -- identical index sets on
    # tie-free rows, a legal top-k everywhere
    MEASURED[tag]["selection (same, tie-free)"] = selection_dense_vs_oracle("indices", ctx["pq"], ctx["pk"], idx, T, strict=not qk_norm)


def check_op_l2(dev, B=1, H=1, N=16384, T=8, T2=4, fused=True, rope=False, smooth=False, qk_norm=False, slices=None):
    """slices: the (b, h) pairs the oracle is run on, one at a time (no (b,h) sees another); None = all at once."""
    from llsa_amd.kernel.hip.rope import my_rope_fn
    from llsa_amd.kernel.torch_op import flash_sparse_attention_res_2 as M
    from llsa_amd.kernel.torch_op._fused import selection
    from llsa_amd.utils.rope_table import rope_table
    q, k, v, do = smooth_inputs(B, H, N, 64, dev) if smooth else randn_inputs(B, H, N, 64, dev, seed=20)
    freq = rope_table(int(math.isqrt(N)), dtype=torch.bfloat16).to(dev) if rope else None
    captured = {}
    norm = _norm_weights(dev) if qk_norm else None

    def run(q_, k_, v_):
        if fused:
            out = M.llsa_l2(q_, k_, v_, T, T2, 16, rope=freq, qk_norm=norm)
            captured["idx"], captured["pidx"] = selection(out)
            return out
        if rope:
            q_, k_ = my_rope_fn(q_, freq), my_rope_fn(k_, freq)
        out = M.llsa_l2_unfused(q_, k_, v_, T, T2, 16)
        captured["idx"], captured["pidx"] = out.grad_fn.saved_tensors[9], out.grad_fn.saved_tensors[10]
        return out

    o, dq, dk, dv = _grads(run, q, k, v, do)
    if slices is not None:
        for b, h in slices:
            cut = lambda t: t[b:b + 1, h:h + 1]
            _compare_op_l2(f"l2 B={B} H={H} N={N} T={T}/{T2} slice ({b},{h})", *(cut(t) for t in (q, k, v, do, o, dq, dk, dv)),
                           cut(captured["idx"]), cut(captured["pidx"]), T, T2, freq, norm, flat=smooth)
        return
    _compare_op_l2(f"l2 B={B} H={H} N={N} T={T}/{T2}" + (" rope" if rope else "") + (" qk_norm" if qk_norm else "")
                   + ("" if fused else " unfused"), q, k, v, do, o, dq, dk, dv, captured["idx"], captured["pidx"], T, T2, freq, norm,
                   flat=smooth)


def _compare_op_l2(tag, q, k, v, do, o, dq, dk, dv, dev_idx, dev_pidx, T, T2, freq, norm, flat=False):
    rope, qk_norm = freq is not None, norm is not None
    qc, kc, vc, doc = (t.cpu().contiguous() for t in (q, k, v, do))
    fc = freq.cpu() if rope else None
    qn, kn = _apply_norm(qc, kc, norm)
    qr, kr = (O.rope_apply(qn, fc), O.rope_apply(kn, fc)) if rope else (qn, kn)
    ro, ctx = O.llsa_l2_fwd(qr, kr, vc, T, T2, 16, indices=dev_idx.cpu(), p_indices=dev_pidx.cpu().long())
    rq, rk, rv, _ = O.llsa_l2_bwd(doc, ctx)
    if rope:
        rq, rk = O.rope_apply_bwd(rq, fc), O.rope_apply_bwd(rk, fc)
    rq, rk = _norm_backward(rq, rk, qc, kc, norm)
    for name, a, b in (("o", o, ro), ("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
        close(name, a, b, report=tag, flat=flat)
    # both levels of the selection against the oracle's own: the coarse one on the level-2 pooled rows, the fine
    # one under the parents the device chose (wherever those equal the oracle's this is the whole cascade)
    pidx, idx = dev_pidx.cpu().long(), dev_idx.cpu().long()
    MEASURED[tag]["p_indices (same, tie-free)"] = selection_dense_vs_oracle("p_indices", ctx["pq2"], ctx["pk2"], pidx, T2, strict=not qk_norm)
    MEASURED[tag]["indices (same, tie-free)"] = selection_sparse_vs_oracle("indices", ctx["pq"], ctx["pk"], pidx, idx, T, strict=not qk_norm)


def check_op_l3(dev, B=1, H=1, N=262144, T=16, T2=16, T3=16, rope=True, qk_norm=False):
    """llsa_l3 through autograd against the oracle's three-level composition fed with the device's own
    selection; the selection itself must be a legal cascade (every block under a block its parent chose) and,
    on these smooth inputs, equal to the oracle's at the two coarse levels wherever the bf16 scores do not tie."""
    import llsa_amd
    from llsa_amd.kernel.torch_op._fused import selection
    from llsa_amd.utils.rope_table import rope_table
    q, k, v, do = smooth_inputs(B, H, N, 64, dev)
    freq = rope_table(int(math.isqrt(N)), dtype=torch.bfloat16).to(dev) if rope else None
    norm = _norm_weights(dev) if qk_norm else None
    captured = {}

    def run(q_, k_, v_):
        out = llsa_amd.llsa_l3(q_, k_, v_, T, T2, T3, 16, rope=freq, qk_norm=norm)
        captured["sel"] = [t.cpu().long() for t in selection(out)]
        return out

    o, dq, dk, dv = _grads(run, q, k, v, do)
    idx, pidx, ppidx = captured["sel"]
    assert idx.shape == (B, H, N // 16, T) and pidx.shape == (B, H, N // 256, T2) and ppidx.shape == (B, H, N // 4096, T3)
    par = pidx.repeat_interleave(16, dim=2)
    assert ((idx[..., :, None] // 16) == par[..., None, :]).any(-1).all(), "a fine block outside its parent's selection"
    gpar = ppidx.repeat_interleave(16, dim=2)
    assert ((pidx[..., :, None] // 16) == gpar[..., None, :]).any(-1).all(), "a level-1 block outside its grand-parent's selection"
    qc, kc, vc, doc = (t.cpu() for t in (q, k, v, do))
    fc = freq.cpu() if rope else None
    qn, kn = _apply_norm(qc, kc, norm)
    qr, kr = (O.rope_apply(qn, fc), O.rope_apply(kn, fc)) if rope else (qn, kn)
    ro, ctx = O.llsa_l3_fwd(qr, kr, vc, T, T2, T3, 16, indices=idx, p_indices=pidx, pp_indices=ppidx)
    rq, rk, rv, _ = O.llsa_l3_bwd(doc, ctx)
    if rope:
        rq, rk = O.rope_apply_bwd(rq, fc), O.rope_apply_bwd(rk, fc)
    rq, rk = _norm_backward(rq, rk, qc, kc, norm)
    close("o", o, ro, flat=True)
    close("dq", dq, rq, flat=True)
    close("dk", dk, rk, flat=True)
    close("dv", dv, rv, flat=True)
    _, own = O.llsa_l3_fwd(qr, kr, vc, T, T2, T3, 16)
    same = lambda a, b: (a.sort(-1).values == b.long().sort(-1).values).all(-1).float().mean().item()
    assert same(ppidx, own["pp_indices"]) > 0.9 and same(pidx, own["p_indices"]) > 0.9 and same(idx, own["indices"]) > 0.9



def check_op_lk_sparse_dout(dev, N=4194304, topks=(16, 16, 16, 16), H=1, query_blocks=(0, 7777, -1), rope=True):
    """dK and dV of llsa_lk, every element, at sizes the whole-tensor oracle cannot hold.  dO is zero outside a few
    query blocks: a query with dO = 0 has dP = 0 and delta = 0, so it adds exact zeros to dK and dV, and the whole of
    dK / dV follows from those few queries -- enumerated here in fp64 (torch.autograd over each query's key set, taken
    from the device's own selection: its fine blocks, the pooled blocks of every level, the dense coarsest level) and
    pushed down the chain of mean pools (a pooled token's gradient goes to its 16 children, divided by 16) and back
    through the rotation.  This pins what the single-query checks of o and dq cannot: the group-major pass of every
    level (its list owners 16, 256, ... groups wide), the partial sums placed by inverse positions, their reduction,
    the dense coarsest level, and the fold of the whole chain into the fine dK / dV."""
    import llsa_amd
    from llsa_amd.kernel.torch_op._fused import selection
    from llsa_amd.utils.rope_table import rope_table
    L = len(topks)
    assert L >= 2, "one level keeps the reference's weight-1 pooled gradient (sparse_attention_res_1.py:388-389): not enumerated here"
    q, k, v, _ = smooth_inputs(1, H, N, 64, dev)
    freq = rope_table(int(math.isqrt(N)), dtype=torch.bfloat16).to(dev) if rope else None
    g = torch.Generator().manual_seed(31)
    blocks = [b % (N // 16) for b in query_blocks]
    do = torch.zeros(1, H, N, 64, dtype=torch.bfloat16)
    for b in blocks:
        do[0, :, b * 16:b * 16 + 16] = torch.randn(H, 16, 64, generator=g).bfloat16()
    captured = {}

    def run(q_, k_, v_):
        out = llsa_amd.llsa_lk(q_, k_, v_, topks, 16, rope=freq)
        captured["sel"] = [t.cpu().long() for t in selection(out)]
        return out

    _, _, dk, dv = _grads(run, q, k, v, do.to(dev))
    sels = captured["sel"]
    qc, kc, vc = (t.cpu() for t in (q, k, v))
    fc = freq.cpu() if rope else None
    qr, kr = (O.rope_apply(qc, fc), O.rope_apply(kc, fc)) if rope else (qc, kc)
    ks, vs = [kr], [vc]                                       # level 0 .. L: what the attention multiplies (bf16 rows)
    for _ in range(L):
        ks.append(O.mean_pool(ks[-1], 16)), vs.append(O.mean_pool(vs[-1], 16))
    for h in range(H):
        gk = [torch.zeros(N // 16 ** l, 64, dtype=torch.float64) for l in range(L + 1)]
        gv = [torch.zeros(N // 16 ** l, 64, dtype=torch.float64) for l in range(L + 1)]
        for b in blocks:
            rows, lvls = [], []                               # the key set of this query block: (level, token) lists
            for l in range(L):
                for blk in sels[l][0, h, b // 16 ** l].tolist():
                    rows.append(torch.arange(blk * 16, blk * 16 + 16)), lvls.append(l)
            rows.append(torch.arange(N // 16 ** L)), lvls.append(L)
            kk = [ks[l][0, h, r].double().requires_grad_(True) for r, l in zip(rows, lvls)]
            vv = [vs[l][0, h, r].double().requires_grad_(True) for r, l in zip(rows, lvls)]
            logw = torch.cat([torch.full((len(r),), math.log(16.0 ** l), dtype=torch.float64) for r, l in zip(rows, lvls)])
            qq = qr[0, h, b * 16:b * 16 + 16].double()
            p = torch.softmax(qq @ torch.cat(kk).T / 8.0 + logw, -1)
            loss = ((p @ torch.cat(vv)) * do[0, h, b * 16:b * 16 + 16].double()).sum()
            grads = torch.autograd.grad(loss, kk + vv)
            for i, (r, l) in enumerate(zip(rows, lvls)):
                gk[l].index_add_(0, r, grads[i])
                gv[l].index_add_(0, r, grads[len(rows) + i])
        for l in range(L, 0, -1):                             # down the chain of mean pools
            gk[l - 1] += gk[l].repeat_interleave(16, 0) / 16.0
            gv[l - 1] += gv[l].repeat_interleave(16, 0) / 16.0
        rk = gk[0].float().view(1, 1, N, 64)
        if rope:
            rk = O.rope_apply_bwd(rk.bfloat16(), fc).float()
        tag = f"l{L} N={N} sparse dO"
        close(f"dk[{h}]", dk[:, h:h + 1], rk, report=tag)
        close(f"dv[{h}]", dv[:, h:h + 1], gv[0].float().view(1, 1, N, 64), report=tag)


def check_op_lk_samples(dev, N=4194304, topks=(16, 16, 16, 16), H=1, queries=(0, 1234567, -1), rows=16384):
    """llsa_lk with k = len(topks) levels at a size the whole-tensor oracle cannot hold: the selection must be a legal
    cascade at every level and equal to the oracle's at the coarsest level and (on the first `rows` groups) below it;
    the output and dq rows of single queries are compared with the soft-max over the key set the scheme defines,
    enumerated on the CPU in fp64 from the device's own selection (torch.autograd for dq)."""
    import llsa_amd
    from llsa_amd.kernel.torch_op._fused import selection
    L = len(topks)
    q, k, v, do = smooth_inputs(1, H, N, 64, dev)
    captured = {}

    def run(q_, k_, v_):
        out = llsa_amd.llsa_lk(q_, k_, v_, topks, 16)
        captured["sel"] = [t.cpu().long() for t in selection(out)]
        return out

    o, dq, dk, dv = _grads(run, q, k, v, do)
    sels = captured["sel"]
    assert [tuple(s.shape) for s in sels] == [(1, H, N // 16 ** (l + 1), topks[l]) for l in range(L)]
    for l in range(L - 1):
        par = sels[l + 1].repeat_interleave(16, dim=2)
        assert ((sels[l][..., :, None] // 16) == par[..., None, :]).any(-1).all(), f"level {l}: a block outside its parent's selection"
    qc, kc, vc, doc = (t.cpu() for t in (q, k, v, do))
    pqs, pks, pvs, xq, xk, xv = [], [], [], qc, kc, vc
    for _ in range(L):
        xq, xk, xv = O.mean_pool(xq, 16), O.mean_pool(xk, 16), O.mean_pool(xv, 16)
        pqs.append(xq), pks.append(xk), pvs.append(xv)
    rep = MEASURED.setdefault(f"op_l{L}_N{N}", {})
    rep[f"level {L} selection (same, tie-free)"] = selection_dense_vs_oracle(f"level {L}", pqs[L - 1], pks[L - 1], sels[L - 1], topks[L - 1])
    for l in range(L - 1, 0, -1):                            # sels[l-1] chosen under the parents sels[l]
        r = min(rows, sels[l - 1].shape[2])
        rep[f"level {l} selection (same, tie-free)"] = selection_sparse_vs_oracle(
            f"level {l}", pqs[l - 1][:, :, :r], pks[l - 1], sels[l][:, :, :max(r // 16, 1)], sels[l - 1][:, :, :r], topks[l - 1])
    for h in range(H):
        for n in queries:
            n = n % N
            keys, vals, wts = [], [], []
            for l in range(L):
                src_k, src_v = (kc, vc) if l == 0 else (pks[l - 1], pvs[l - 1])
                for blk in sels[l][0, h, n // 16 ** (l + 1)].tolist():
                    keys.append(src_k[0, h, blk * 16:blk * 16 + 16]), vals.append(src_v[0, h, blk * 16:blk * 16 + 16])
                    wts += [16.0 ** l] * 16
            keys.append(pks[L - 1][0, h]), vals.append(pvs[L - 1][0, h])
            wts += [16.0 ** L] * pks[L - 1].shape[2]
            kk, vv, ww = torch.cat(keys).double(), torch.cat(vals).double(), torch.tensor(wts, dtype=torch.float64)
            qq = qc[0, h, n].double().requires_grad_(True)
            want = torch.softmax((kk @ qq) / 8.0 + ww.log(), 0) @ vv
            gq, = torch.autograd.grad(want, qq, doc[0, h, n].double())
            close(f"o[{h},{n}]", o[0, h, n], want.detach())
            close(f"dq[{h},{n}]", dq[0, h, n], gq, rel=2e-2)
    assert all(torch.isfinite(t).all() for t in (dk, dv))
