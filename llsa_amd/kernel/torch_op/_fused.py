"""llsa_l1 / llsa_l2 as ONE autograd node with a lean host side.

The reference composes the operator from nine Python launchers (six mean pools, two selections,
the attention) and autograd adds the pooled gradients afterwards.  The kernels of this package
fuse most of that work, and at the sizes of interest they finish a whole forward + backward in
a few hundred microseconds -- less than it costs Python to allocate ~40 tensors and to fill the
argument structures through the general-purpose wrappers.  This module is the same sequence of
C-ABI calls as those wrappers make, with one arena per data type instead of a tensor per
intermediate and raw pointer arithmetic instead of views:

    forward   pool_pyramid_fwd (q, k, v: pooled rows, RoPE, operand tiles) [+ level-2 tiles]
              topk_dense [+ topk_sparse]
              transpose_indices x levels  (second stream, beside the attention kernel)
              attn_fwd
    backward  attn_bwd with fold_pooled = 1  (dq, dk, dv complete, rotated back)
"""
from __future__ import annotations

import ctypes as C

import torch
from torch.autograd import Function

from ..._lib import MAX_LEVELS, AttnBwdArgs, AttnFwdArgs, PoolItem, TransposeJob, current_lib

_side = {}          # device -> second stream
_SIDE_STREAM_MIN_TOKENS = 1 << 17
_BITMAP_MAX_PAIRS = 1 << 20          # query blocks x key blocks up to which llsa_transpose_indices_multi is one small launch


def _rows_ok(t):
    return t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in t.stride()[:-1])


def _align(n, a):
    return (n + a - 1) // a * a


class _Layout:
    """Offsets (in elements) of everything the forward produces, inside one bf16 arena and one
    int32 arena; every section is contiguous (B*H, ...) and starts 256-byte aligned.  Level 0 is the
    tokens themselves, level l = 1..L the pooled levels (n[l] = N / 16^l tokens each)."""

    def __init__(self, lib, B, H, N, topks, grad):
        BH = B * H
        L = len(topks)
        n = [N // 16 ** l for l in range(L + 2)]
        self.n, self.L = n, L
        o = 0

        def take(rows_per_bh, width, on=True):
            nonlocal o
            if not on:
                return None
            at = o
            o = _align(o + BH * rows_per_bh * width, 128)
            return at

        # pooled rows of q, k, v per level (index l - 1), then operand tiles: level 0 (the tokens) and the pooled levels
        self.pq = [take(n[l], 64) for l in range(1, L + 1)]
        self.pk = [take(n[l], 64) for l in range(1, L + 1)]
        self.pv = [take(n[l], 64) for l in range(1, L + 1)]
        self.qr, self.kr, self.vr, self.vt = take(n[1], 1024), take(n[1], 1024), take(n[1], 1024, grad), take(n[1], 1024)
        self.pkr = [take(n[l + 1], 1024) for l in range(1, L + 1)]
        self.pvr = [take(n[l + 1], 1024, grad) for l in range(1, L + 1)]
        self.pvt = [take(n[l + 1], 1024) for l in range(1, L + 1)]
        self.n_bf16 = o

        o = 0

        def take_i(per_bh, on=True):
            nonlocal o
            if not on:
                return None
            at = o
            o = _align(o + BH * per_bh, 64)
            return at

        self.chunk = lib.fine_chunk(N)          # entries per work item of the fine level
        self.wl_f = lib.work_list_len(n[1], n[1], topks[0], self.chunk)
        # sel[0] = idx (fine blocks per query block), sel[l] = blocks of level l per group of 16^(l+1) queries
        self.sel = [take_i(n[l + 1] * topks[l]) for l in range(L)]
        self.off = [take_i(n[l + 1] + 1, grad) for l in range(L)]
        self.flat = [take_i(n[l + 1] * topks[l], grad) for l in range(L)]
        self.work = take_i(self.wl_f, grad)
        self.inv = [None] + [take_i(n[l + 1] * topks[l], grad) for l in range(1, L)]
        self.n_i32 = o
        # backward arena (bytes): pooled gradients, then the kernels' workspace
        self.ws_bytes = lib.attn_bwd_workspace_bytes(B, H, N, (C.c_int32 * L)(*topks), L)
        o = 0
        self.dpk, self.dpv = [], []
        for l in range(1, L + 1):
            self.dpk.append(o)
            o += _align(BH * n[l] * 128, 256)
            self.dpv.append(o)
            o += _align(BH * n[l] * 128, 256)
        self.ws = o
        self.n_bwd = self.ws + self.ws_bytes


_layouts = {}


def _layout(lib, B, H, N, topks, grad):
    key = (lib.path, B, H, N, topks, grad)
    lay = _layouts.get(key)
    if lay is None:
        if len(_layouts) > 64:
            _layouts.clear()
        lay = _layouts[key] = _Layout(lib, B, H, N, topks, grad)
    return lay


def _stream(lib, t):
    if not lib.device_library:
        return None
    idx = t.device.index
    return C.c_void_p(torch._C._cuda_getCurrentRawStream(torch.cuda.current_device() if idx is None else idx))


def _check(lib, rc, what):
    if rc != 0:
        lib.check(rc, what)


class LlsaFused(Function):
    """forward(q, k, v, topks, block_size, freq, gamma_q, gamma_k, eps) -> o

    topks: one entry per pooled level, (topk1, topk2, ...): the fine blocks a query block keeps, then the blocks of
    pooled level 1, 2, ... its ancestor groups keep; len(topks) = 1 is llsa_l1, 2 is llsa_l2.
    gamma_q / gamma_k ((64,) fp32 or None): RMS-normalise q / k over the head dimension first (the
    qk-norm of the reference's attention processor), inside the pooling pass; they receive gradients."""

    @staticmethod
    def forward(ctx, q, k, v, topks, block_size, freq, gamma_q=None, gamma_k=None, eps=1e-5):
        lib = current_lib()
        if block_size != 16:
            raise NotImplementedError("block_size must be 16")
        for t in (q, k, v):
            if lib.device_library and not t.is_cuda:
                raise RuntimeError("llsa_amd runs on an AMD GPU only (got a CPU tensor); there is no CPU implementation")
            if t.dtype != torch.bfloat16:
                raise NotImplementedError(f"llsa_amd attention kernels are bf16 only (got {t.dtype})")
        if q.dim() != 4 or q.shape[-1] != 64:
            raise NotImplementedError(f"llsa_amd attention kernels need (B,H,N,64) tensors (got {tuple(q.shape)})")
        if k.shape != q.shape or v.shape != q.shape:
            raise ValueError("self-attention only: q, k, v must have the same shape")
        B, H, N, _ = q.shape
        L = len(topks)
        if not 1 <= L <= MAX_LEVELS:
            raise ValueError(f"1 to {MAX_LEVELS} pooled levels (got {L})")
        mult = 64 * 16 ** L
        if N % mult != 0:
            raise ValueError(f"llsa_l{L} needs a token count that is a multiple of {mult} (got {N})")
        topks = tuple(min(int(t), N // 16 ** (l + 1)) for l, t in enumerate(topks))
        rope = freq is not None
        if rope:
            if freq.dtype != torch.bfloat16 or tuple(freq.shape) != (N, 64):
                raise ValueError("rope table must be bf16 (N, 64)")
            freq = freq.contiguous()
        grad = any(ctx.needs_input_grad[:3]) or ctx.needs_input_grad[6] or ctx.needs_input_grad[7]
        q, k, v = (t if _rows_ok(t) else t.contiguous() for t in (q, k, v))
        gq = gk = None
        if gamma_q is not None:
            gq = gamma_q.detach().to(device=q.device, dtype=torch.float32).contiguous()
        if gamma_k is not None:
            gk = gamma_k.detach().to(device=q.device, dtype=torch.float32).contiguous()
        if any(g is not None and g.numel() != 64 for g in (gq, gk)):
            raise ValueError("qk-norm weights must have 64 entries")
        lay = _layout(lib, B, H, N, topks, grad)
        n = lay.n
        dev = q.device
        A = torch.empty(lay.n_bf16, device=dev, dtype=torch.bfloat16)
        I = torch.empty(lay.n_i32, device=dev, dtype=torch.int32)
        o = torch.empty_like(q) if all(s % 4 == 0 for s in q.stride()[:-1]) else torch.empty(q.shape, device=dev, dtype=q.dtype)
        lse = torch.empty(B, H, N, device=dev, dtype=torch.float32)
        a0, i0 = A.data_ptr(), I.data_ptr()
        pa = lambda off: None if off is None else a0 + 2 * off
        pi = lambda off: None if off is None else i0 + 4 * off
        stream = _stream(lib, q)
        at = lambda lst, l: pa(lst[l - 1]) if l <= L else None      # section of pooled level l (None beyond the last)

        # The pyramid.  One pass over q, k, v gives the rows of levels 1 and 2 and the tiles of levels 0, 1, 2; every
        # further pass starts from the rows of level 2p and gives rows and tiles of levels 2p + 1 and 2p + 2.
        items = (PoolItem * 3)(
            PoolItem(q.data_ptr(), q.stride(0), q.stride(1), q.stride(2), N, int(rope), at(lay.pq, 1), at(lay.pq, 2), pa(lay.qr),
                     None, None, None, None, None if gq is None else gq.data_ptr(), float(eps), 0, None, None),
            PoolItem(k.data_ptr(), k.stride(0), k.stride(1), k.stride(2), N, int(rope), at(lay.pk, 1), at(lay.pk, 2), pa(lay.kr),
                     None, at(lay.pkr, 1), None, None, None if gk is None else gk.data_ptr(), float(eps), 0, at(lay.pkr, 2), None),
            PoolItem(v.data_ptr(), v.stride(0), v.stride(1), v.stride(2), N, 0, at(lay.pv, 1), at(lay.pv, 2), pa(lay.vr),
                     pa(lay.vt), at(lay.pvr, 1), at(lay.pvt, 1), None, None, 0.0, 0, at(lay.pvr, 2), at(lay.pvt, 2)))
        _check(lib, lib.pool_pyramid_fwd(items, 3, freq.data_ptr() if rope else None, B, H, stream), "pool_pyramid")
        for l0 in range(2, L, 2):               # rows of level l0 -> levels l0 + 1, l0 + 2
            s = (H * n[l0] * 64, n[l0] * 64, 64)
            more = (PoolItem * 3)(
                PoolItem(at(lay.pk, l0), *s, n[l0], 0, at(lay.pk, l0 + 1), at(lay.pk, l0 + 2), None, None, at(lay.pkr, l0 + 1), None,
                         None, None, 0.0, 0, at(lay.pkr, l0 + 2), None),
                PoolItem(at(lay.pv, l0), *s, n[l0], 0, at(lay.pv, l0 + 1), at(lay.pv, l0 + 2), None, None, at(lay.pvr, l0 + 1),
                         at(lay.pvt, l0 + 1), None, None, 0.0, 0, at(lay.pvr, l0 + 2), at(lay.pvt, l0 + 2)),
                PoolItem(at(lay.pq, l0), *s, n[l0], 0, at(lay.pq, l0 + 1), at(lay.pq, l0 + 2), None, None, None, None, None))
            _check(lib, lib.pool_pyramid_fwd(more, 3, None, B, H, stream), "pool_pyramid (deeper levels)")

        # Selection, coarse to fine: a dense top-k over the coarsest level's tokens (each of them is a block of the level
        # below), then level by level among the blocks under the parent's selection.
        first = L - 1               # the first parent-guided selection still to do
        if L >= 2 and n[L] <= lib.topk_cascade_max_parents():
            # the dense selection rides in the workgroups of the first parent-guided one: one launch less
            _check(lib, lib.topk_cascade(at(lay.pq, L), at(lay.pk, L), pi(lay.sel[L - 1]), at(lay.pq, L - 1), at(lay.pk, L - 1),
                                         pi(lay.sel[L - 2]), B, H, n[L - 1], topks[L - 2], topks[L - 1], stream), "topk_cascade")
            first = L - 2
        else:
            _check(lib, lib.topk_dense(at(lay.pq, L), at(lay.pk, L), pi(lay.sel[L - 1]), B, H, n[L], topks[L - 1], 1, stream),
                   "gen_sparse_indices")
        for l in range(first, 0, -1):
            _check(lib, lib.topk_sparse(at(lay.pq, l), at(lay.pk, l), pi(lay.sel[l]), pi(lay.sel[l - 1]), B, H, n[l], topks[l - 1],
                                        topks[l], stream), "compute_topk_indices_sparse")

        # The lists of the backward (the transposed selections of all levels).  Up to 2^14 tokens a (b,h)'s bitmap of
        # (key block, query block) fits LDS and one launch of one workgroup per (b,h) and level does everything, sorted as
        # it goes, behind the attention kernel on the same stream (on a second stream, beside the backward's dQ kernel, the
        # two event edges cost more than the overlap saves: 0.373 against 0.358 ms a step at B=2, H=6, N=16384).  Beyond
        # that the lists take several kernels per level, which run on a second stream beside the attention kernel: the
        # attention kernel is issued first (the GPU is waiting for it), and an event recorded before it lets the second
        # stream start as soon as the selection is done.  With few tokens over all heads the step is bound by the host,
        # which the event calls cost more than the GPU saves: everything then goes to the one stream.
        jobs = (TransposeJob * L)()
        if grad:
            jobs[0] = TransposeJob(pi(lay.sel[0]), pi(lay.off[0]), pi(lay.flat[0]), pi(lay.work), None, n[1], n[1], topks[0], lay.chunk)
            for l in range(1, L):
                jobs[l] = TransposeJob(pi(lay.sel[l]), pi(lay.off[l]), pi(lay.flat[l]), None, pi(lay.inv[l]), n[l + 1], n[l + 1], topks[l], 1)
        cur = side = None
        if grad and lib.device_library and n[1] * n[1] > _BITMAP_MAX_PAIRS and B * H * N >= _SIDE_STREAM_MIN_TOKENS:
            cur = torch.cuda.current_stream(dev)
            side = _side.get(dev)
            if side is None:
                side = _side[dev] = torch.cuda.Stream(device=dev)
            ev_idx = torch.cuda.Event()
            ev_idx.record(cur)

        f = AttnFwdArgs()
        f.qr, f.kr, f.vt, f.idx = pa(lay.qr), pa(lay.kr), pa(lay.vt), pi(lay.sel[0])
        f.o, f.sob, f.soh, f.son = o.data_ptr(), o.stride(0), o.stride(1), o.stride(2)
        f.lse = lse.data_ptr()
        f.B, f.H, f.N, f.T, f.levels = B, H, N, topks[0], L
        for l in range(1, L + 1):
            lv = f.lvl[l - 1]
            lv.kr, lv.vt, lv.w = at(lay.pkr, l), at(lay.pvt, l), float(16 ** l)
            if l < L:
                lv.sel, lv.T = pi(lay.sel[l]), topks[l]
        _check(lib, lib.attn_fwd(C.byref(f), stream), "attn_fwd")

        if grad:
            s_lists = stream
            if side is not None:
                side.wait_event(ev_idx)         # (the arena is older than the selection, so this covers it too)
                s_lists = C.c_void_p(side.cuda_stream)
            _check(lib, lib.transpose_indices_multi(jobs, L, B, H, s_lists), "transpose_indices")
            if side is not None:
                ev_lists = torch.cuda.Event()
                ev_lists.record(side)
                cur.wait_event(ev_lists)        # (and the arena is not handed out again before the second stream is done)

        if grad:
            # (q and k themselves are needed again only by the backward of the qk-norm)
            ctx.save_for_backward(A, I, o, lse, freq, gq, gk, q if gq is not None else None, k if gk is not None else None)
            ctx.meta = (lib, lay, B, H, N, topks, q.shape, q.stride(), k.stride(), v.stride())
            ctx.eps = float(eps)
            ctx.gamma_dtypes = (None if gamma_q is None else gamma_q.dtype, None if gamma_k is None else gamma_k.dtype)
        return o

    @staticmethod
    def backward(ctx, do):
        A, I, o, lse, freq, gq, gk, q_in, k_in = ctx.saved_tensors
        lib, lay, B, H, N, topks, shape, sq, sk, sv = ctx.meta
        L = len(topks)
        dev = o.device
        if not _rows_ok(do):
            do = do.contiguous()

        def like(strides):      # gradients have the layout of their primals when the 8-byte stores allow it
            if all(s % 4 == 0 for s in strides[:-1]) and strides[-1] == 1:
                return torch.empty_strided(shape, strides, device=dev, dtype=torch.bfloat16)
            return torch.empty(shape, device=dev, dtype=torch.bfloat16)

        dq, dk, dv = like(sq), like(sk), like(sv)
        W = torch.empty(lay.n_bwd, device=dev, dtype=torch.uint8)
        a0, i0, w0 = A.data_ptr(), I.data_ptr(), W.data_ptr()
        pa = lambda off: None if off is None else a0 + 2 * off
        pi = lambda off: None if off is None else i0 + 4 * off
        a = AttnBwdArgs()
        a.dout, a.sdob, a.sdoh, a.sdon = do.data_ptr(), do.stride(0), do.stride(1), do.stride(2)
        a.o, a.sob, a.soh, a.son = o.data_ptr(), o.stride(0), o.stride(1), o.stride(2)
        a.lse = lse.data_ptr()
        a.qr, a.kr, a.vr = pa(lay.qr), pa(lay.kr), pa(lay.vr)
        a.idx, a.off, a.flat, a.work = pi(lay.sel[0]), pi(lay.off[0]), pi(lay.flat[0]), pi(lay.work)
        a.dq, a.sdqb, a.sdqh, a.sdqn = dq.data_ptr(), dq.stride(0), dq.stride(1), dq.stride(2)
        a.dk, a.sdkb, a.sdkh, a.sdkn = dk.data_ptr(), dk.stride(0), dk.stride(1), dk.stride(2)
        a.dv, a.sdvb, a.sdvh, a.sdvn = dv.data_ptr(), dv.stride(0), dv.stride(1), dv.stride(2)
        for l in range(1, L + 1):
            lv = a.lvl[l - 1]
            lv.kr, lv.vr = pa(lay.pkr[l - 1]), pa(lay.pvr[l - 1])
            lv.dk, lv.dv = w0 + lay.dpk[l - 1], w0 + lay.dpv[l - 1]
            # llsa_l1 keeps the reference's quirk: its pooled path is differentiated with weight 1
            # (sparse_attention_res_1.py:388-389) although the forward uses token_weight
            lv.w, lv.gw = float(16 ** l), (1.0 if L == 1 else float(16 ** l))
            if l < L:
                lv.sel, lv.off, lv.inv, lv.T = pi(lay.sel[l]), pi(lay.off[l]), pi(lay.inv[l]), topks[l]
        a.workspace, a.workspace_bytes = w0 + lay.ws, lay.ws_bytes
        if freq is not None:
            a.freq_dq = a.freq_dk = freq.data_ptr()
        a.B, a.H, a.N, a.T, a.levels = B, H, N, topks[0], L
        a.stages, a.fold_pooled = 0, 1
        stream = _stream(lib, o)
        _check(lib, lib.attn_bwd(C.byref(a), stream), "attn_bwd")
        dgq = dgk = None
        if gq is not None or gk is not None:      # back through the qk-norm, in place on dq / dk
            P = torch.empty(lib.rmsnorm_bwd_partials(B, H, N), device=dev, dtype=torch.float32)
            i3 = lambda t: (C.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2))
            for g, x, d, which in ((gq, q_in, dq, 0), (gk, k_in, dk, 1)):
                if g is None:
                    continue
                dg = torch.empty(64, device=dev, dtype=torch.float32)
                _check(lib, lib.rmsnorm_bwd(d.data_ptr(), i3(d), x.data_ptr(), i3(x), g.data_ptr(), ctx.eps, d.data_ptr(), i3(d),
                                            dg.data_ptr(), P.data_ptr(), B, H, N, stream), "rmsnorm_bwd")
                dg = dg.to(ctx.gamma_dtypes[which])
                if which == 0:
                    dgq = dg
                else:
                    dgk = dg
        return dq, dk, dv, None, None, None, dgq, dgk, None


def selection(out):
    """The blocks the forward that produced `out` chose, finest first: (indices (B,H,N/16,T), p_indices
    (B,H,N/256,T2) or None for one level, then one more tensor per further level), int32 views of the arena its
    autograd node holds."""
    node = out.grad_fn
    I = node.saved_tensors[1]
    _, lay, B, H, N, topks = node.meta[:6]
    L = len(topks)
    views = [I[lay.sel[l]:lay.sel[l] + B * H * lay.n[l + 1] * topks[l]].view(B, H, lay.n[l + 1], topks[l]) for l in range(L)]
    return tuple(views) if L >= 2 else (views[0], None)
