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

from ..._lib import CHUNK_FINE, AttnBwdArgs, AttnFwdArgs, PoolItem, current_lib

_side = {}          # device -> (second stream, two events)
_SIDE_STREAM_MIN_TOKENS = 1 << 17


def _rows_ok(t):
    return t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in t.stride()[:-1])


def _align(n, a):
    return (n + a - 1) // a * a


class _Layout:
    """Offsets (in elements) of everything the forward produces, inside one bf16 arena and one
    int32 arena; every section is contiguous (B*H, ...) and starts 256-byte aligned."""

    def __init__(self, lib, B, H, N, levels, T, T2, grad, T3=0):
        BH = B * H
        n1, n2 = N // 16, N // 256
        self.n1, self.n2 = n1, n2
        o = 0

        def take(rows_per_bh, width, on=True):
            nonlocal o
            if not on:
                return None
            at = o
            o = _align(o + BH * rows_per_bh * width, 128)
            return at

        l2, l3 = levels >= 2, levels == 3
        self.pq, self.pk, self.pv = take(n1, 64), take(n1, 64), take(n1, 64)
        self.pq2, self.pk2, self.pv2 = take(n2, 64, l2), take(n2, 64, l2), take(n2, 64, l2)
        self.qr, self.kr, self.vr, self.vt = take(n1, 1024), take(n1, 1024), take(n1, 1024, grad), take(n1, 1024)
        self.pkr, self.pvr, self.pvt = take(n2, 1024), take(n2, 1024, grad), take(n2, 1024)
        n3 = max(n2 // 16, 1)
        self.pk2r, self.pv2r, self.pv2t = take(n3, 1024, l2), take(n3, 1024, l2 and grad), take(n3, 1024, l2)
        n4 = max(n3 // 16, 1)
        self.n3 = n3
        self.pq3, self.pk3, self.pv3 = take(n3, 64, l3), take(n3, 64, l3), take(n3, 64, l3)
        self.pk3r, self.pv3r, self.pv3t = take(n4, 1024, l3), take(n4, 1024, l3 and grad), take(n4, 1024, l3)
        self.n_bf16 = o

        o = 0

        def take_i(per_bh, on=True):
            nonlocal o
            if not on:
                return None
            at = o
            o = _align(o + BH * per_bh, 64)
            return at

        self.wl_f = lib.work_list_len(n1, n1, T, CHUNK_FINE)
        self.idx, self.pidx, self.ppidx = take_i(n1 * T), take_i(n2 * T2, l2), take_i(n3 * T3, l3)
        self.off, self.flat, self.work = take_i(n1 + 1, grad), take_i(n1 * T, grad), take_i(self.wl_f, grad)
        self.poff, self.pflat, self.pinv = (take_i(n2 + 1, grad and l2), take_i(n2 * T2, grad and l2),
                                            take_i(n2 * T2, grad and l2))
        self.ppoff, self.ppflat, self.ppinv = (take_i(n3 + 1, grad and l3), take_i(n3 * T3, grad and l3),
                                               take_i(n3 * T3, grad and l3))
        self.n_i32 = o
        # backward arena (bytes): pooled gradients, then the kernels' workspace
        self.ws_bytes = lib.attn_bwd_workspace_bytes(B, H, N, T, T2, T3, levels)
        self.dpk = 0
        self.dpv = _align(BH * n1 * 128, 256)
        self.dpk2 = self.dpv + _align(BH * n1 * 128, 256)
        self.dpv2 = self.dpk2 + _align(BH * n2 * 128, 256)
        self.dpk3 = self.dpv2 + _align(BH * n2 * 128, 256)
        self.dpv3 = self.dpk3 + _align(BH * n3 * 128, 256)
        self.ws = self.dpv3 + _align(BH * n3 * 128, 256)
        self.n_bwd = self.ws + self.ws_bytes


_layouts = {}


def _layout(lib, B, H, N, levels, T, T2, grad, T3=0):
    key = (lib.path, B, H, N, levels, T, T2, grad, T3)
    lay = _layouts.get(key)
    if lay is None:
        if len(_layouts) > 64:
            _layouts.clear()
        lay = _layouts[key] = _Layout(lib, B, H, N, levels, T, T2, grad, T3)
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
    """forward(q, k, v, levels, topk1, topk2, block_size, freq, gamma_q, gamma_k, eps) -> o

    gamma_q / gamma_k ((64,) fp32 or None): RMS-normalise q / k over the head dimension first (the
    qk-norm of the reference's attention processor), inside the pooling pass; they receive gradients."""

    @staticmethod
    def forward(ctx, q, k, v, levels, topk1, topk2, block_size, freq, gamma_q=None, gamma_k=None, eps=1e-5, topk3=0):
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
        mult = {1: 1024, 2: 16384, 3: 262144}[levels]
        if N % mult != 0:
            raise ValueError(f"llsa_l{levels} needs a token count that is a multiple of {mult} (got {N})")
        n1, n2, n3 = N // 16, N // 256, N // 4096
        T = min(topk1, n1)
        T2 = min(topk2, n2) if levels >= 2 else 0
        T3 = min(topk3, n3) if levels == 3 else 0
        rope = freq is not None
        if rope:
            if freq.dtype != torch.bfloat16 or tuple(freq.shape) != (N, 64):
                raise ValueError("rope table must be bf16 (N, 64)")
            freq = freq.contiguous()
        grad = any(ctx.needs_input_grad[:3]) or ctx.needs_input_grad[8] or ctx.needs_input_grad[9]
        q, k, v = (t if _rows_ok(t) else t.contiguous() for t in (q, k, v))
        gq = gk = None
        if gamma_q is not None:
            gq = gamma_q.detach().to(device=q.device, dtype=torch.float32).contiguous()
        if gamma_k is not None:
            gk = gamma_k.detach().to(device=q.device, dtype=torch.float32).contiguous()
        if any(g is not None and g.numel() != 64 for g in (gq, gk)):
            raise ValueError("qk-norm weights must have 64 entries")
        lay = _layout(lib, B, H, N, levels, T, T2, grad, T3)
        dev = q.device
        A = torch.empty(lay.n_bf16, device=dev, dtype=torch.bfloat16)
        I = torch.empty(lay.n_i32, device=dev, dtype=torch.int32)
        o = torch.empty_like(q) if all(s % 4 == 0 for s in q.stride()[:-1]) else torch.empty(q.shape, device=dev, dtype=q.dtype)
        lse = torch.empty(B, H, N, device=dev, dtype=torch.float32)
        a0, i0 = A.data_ptr(), I.data_ptr()
        pa = lambda off: None if off is None else a0 + 2 * off
        pi = lambda off: None if off is None else i0 + 4 * off
        stream = _stream(lib, q)
        l2, l3 = levels >= 2, levels == 3

        two = l2 and not l3     # two levels: the tiles of the level-2 rows come out of the same pass (with three, a second one makes them)
        items = (PoolItem * 3)(
            PoolItem(q.data_ptr(), q.stride(0), q.stride(1), q.stride(2), N, int(rope), pa(lay.pq), pa(lay.pq2), pa(lay.qr),
                     None, None, None, None, None if gq is None else gq.data_ptr(), float(eps), 0, None, None),
            PoolItem(k.data_ptr(), k.stride(0), k.stride(1), k.stride(2), N, int(rope), pa(lay.pk), pa(lay.pk2), pa(lay.kr),
                     None, pa(lay.pkr), None, None, None if gk is None else gk.data_ptr(), float(eps), 0,
                     pa(lay.pk2r) if two else None, None),
            PoolItem(v.data_ptr(), v.stride(0), v.stride(1), v.stride(2), N, 0, pa(lay.pv), pa(lay.pv2), pa(lay.vr),
                     pa(lay.vt), pa(lay.pvr), pa(lay.pvt), None, None, 0.0, 0,
                     pa(lay.pv2r) if two else None, pa(lay.pv2t) if two else None))
        _check(lib, lib.pool_pyramid_fwd(items, 3, freq.data_ptr() if rope else None, B, H, stream), "pool_pyramid")
        if two:
            _check(lib, lib.topk_dense(pa(lay.pq2), pa(lay.pk2), pi(lay.pidx), B, H, n2, T2, 1, stream), "gen_sparse_indices")
            _check(lib, lib.topk_sparse(pa(lay.pq), pa(lay.pk), pi(lay.pidx), pi(lay.idx), B, H, n1, T, T2, stream),
                   "compute_topk_indices_sparse")
        elif l2:
            s2 = (H * n2 * 64, n2 * 64, 64)
            # the level-2 rows again: their tiles and (three levels) the level-3 rows with theirs
            items2 = (PoolItem * 3)(
                PoolItem(pa(lay.pk2), *s2, n2, 0, pa(lay.pk3), None, pa(lay.pk2r), None, pa(lay.pk3r), None, None),
                PoolItem(pa(lay.pv2), *s2, n2, 0, pa(lay.pv3), None, pa(lay.pv2r), pa(lay.pv2t), pa(lay.pv3r), pa(lay.pv3t), None),
                PoolItem(pa(lay.pq2), *s2, n2, 0, pa(lay.pq3), None, None, None, None, None, None))
            _check(lib, lib.pool_pyramid_fwd(items2, 3 if l3 else 2, None, B, H, stream), "pool_pyramid (level-2 tiles)")
            if l3:
                _check(lib, lib.topk_dense(pa(lay.pq3), pa(lay.pk3), pi(lay.ppidx), B, H, n3, T3, 1, stream), "gen_sparse_indices")
                _check(lib, lib.topk_sparse(pa(lay.pq2), pa(lay.pk2), pi(lay.ppidx), pi(lay.pidx), B, H, n2, T2, T3, stream),
                       "compute_topk_indices_sparse (level 2)")
            else:
                _check(lib, lib.topk_dense(pa(lay.pq2), pa(lay.pk2), pi(lay.pidx), B, H, n2, T2, 1, stream), "gen_sparse_indices")
            _check(lib, lib.topk_sparse(pa(lay.pq), pa(lay.pk), pi(lay.pidx), pi(lay.idx), B, H, n1, T, T2, stream),
                   "compute_topk_indices_sparse")
        else:
            _check(lib, lib.topk_dense(pa(lay.pq), pa(lay.pk), pi(lay.idx), B, H, n1, T, 1, stream), "gen_sparse_indices")

        # The lists of the backward go to a second stream, beside the attention kernel.  The attention
        # kernel is issued first (the GPU is waiting for it); an event recorded before it lets the
        # second stream start as soon as the selection is done.
        # (Below _SIDE_STREAM_MIN_TOKENS tokens over all heads the step is bound by the host, which the two
        # event waits cost 30 us; the GPU then has the time to build the lists on the one stream.)
        cur = side = None
        if grad and lib.device_library and B * H * N >= _SIDE_STREAM_MIN_TOKENS:
            cur = torch.cuda.current_stream(dev)
            pack = _side.get(dev)
            if pack is None:
                pack = _side[dev] = (torch.cuda.Stream(device=dev), torch.cuda.Event(), torch.cuda.Event())
            side, ev_idx, ev_lists = pack
            ev_idx.record(cur)

        f = AttnFwdArgs()
        f.qr, f.kr, f.vt, f.pkr, f.pvt = pa(lay.qr), pa(lay.kr), pa(lay.vt), pa(lay.pkr), pa(lay.pvt)
        f.pk2r, f.pv2t, f.pidx = pa(lay.pk2r), pa(lay.pv2t), pi(lay.pidx)
        f.idx = pi(lay.idx)
        f.o, f.sob, f.soh, f.son = o.data_ptr(), o.stride(0), o.stride(1), o.stride(2)
        f.lse = lse.data_ptr()
        f.B, f.H, f.N, f.T, f.T2, f.levels = B, H, N, T, T2, levels
        f.w1, f.w2 = 16.0, 256.0
        if l3:
            f.pk3r, f.pv3t, f.ppidx, f.T3, f.w3 = pa(lay.pk3r), pa(lay.pv3t), pi(lay.ppidx), T3, 4096.0
        _check(lib, lib.attn_fwd(C.byref(f), stream), "attn_fwd")

        if grad:
            s_lists = stream
            if side is not None:
                side.wait_event(ev_idx)         # (the arena is older than the selection, so this covers it too)
                s_lists = C.c_void_p(side.cuda_stream)
            _check(lib, lib.transpose_indices(pi(lay.idx), pi(lay.off), pi(lay.flat), pi(lay.work), None, B, H, n1, n1, T, CHUNK_FINE,
                                              s_lists), "transpose_indices")
            if l2:
                _check(lib, lib.transpose_indices(pi(lay.pidx), pi(lay.poff), pi(lay.pflat), None, pi(lay.pinv), B, H, n2, n2, T2,
                                                  1, s_lists), "transpose_indices (coarse)")
            if l3:
                _check(lib, lib.transpose_indices(pi(lay.ppidx), pi(lay.ppoff), pi(lay.ppflat), None, pi(lay.ppinv), B, H, n3, n3, T3,
                                                  1, s_lists), "transpose_indices (level 3)")
            if side is not None:
                ev_lists.record(side)
                cur.wait_event(ev_lists)

        if grad:
            # (q and k themselves are needed again only by the backward of the qk-norm)
            ctx.save_for_backward(A, I, o, lse, freq, gq, gk, q if gq is not None else None, k if gk is not None else None)
            ctx.meta = (lib, lay, B, H, N, T, T2, levels, q.shape, q.stride(), k.stride(), v.stride(), T3)
            ctx.eps = float(eps)
            ctx.gamma_dtypes = (None if gamma_q is None else gamma_q.dtype, None if gamma_k is None else gamma_k.dtype)
        return o

    @staticmethod
    def backward(ctx, do):
        A, I, o, lse, freq, gq, gk, q_in, k_in = ctx.saved_tensors
        lib, lay, B, H, N, T, T2, levels, shape, sq, sk, sv, T3 = ctx.meta
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
        a.qr, a.kr, a.vr, a.pkr, a.pvr = pa(lay.qr), pa(lay.kr), pa(lay.vr), pa(lay.pkr), pa(lay.pvr)
        a.pk2r, a.pv2r = pa(lay.pk2r), pa(lay.pv2r)
        a.idx, a.pidx = pi(lay.idx), pi(lay.pidx)
        a.off, a.flat, a.work = pi(lay.off), pi(lay.flat), pi(lay.work)
        a.poff, a.pinv = pi(lay.poff), pi(lay.pinv)
        a.dq, a.sdqb, a.sdqh, a.sdqn = dq.data_ptr(), dq.stride(0), dq.stride(1), dq.stride(2)
        a.dk, a.sdkb, a.sdkh, a.sdkn = dk.data_ptr(), dk.stride(0), dk.stride(1), dk.stride(2)
        a.dv, a.sdvb, a.sdvh, a.sdvn = dv.data_ptr(), dv.stride(0), dv.stride(1), dv.stride(2)
        a.dpk, a.dpv = w0 + lay.dpk, w0 + lay.dpv
        if levels >= 2:
            a.dpk2, a.dpv2 = w0 + lay.dpk2, w0 + lay.dpv2
        if levels == 3:
            a.pk3r, a.pv3r, a.ppidx = pa(lay.pk3r), pa(lay.pv3r), pi(lay.ppidx)
            a.ppoff, a.ppinv = pi(lay.ppoff), pi(lay.ppinv)
            a.dpk3, a.dpv3, a.T3, a.w3 = w0 + lay.dpk3, w0 + lay.dpv3, T3, 4096.0
        a.workspace, a.workspace_bytes = w0 + lay.ws, lay.ws_bytes
        if freq is not None:
            a.freq_dq = a.freq_dk = freq.data_ptr()
        a.B, a.H, a.N, a.T, a.T2, a.levels = B, H, N, T, T2, levels
        # llsa_l1 keeps the reference's quirk: its pooled path is differentiated with weight 1
        # (sparse_attention_res_1.py:388-389) although the forward uses token_weight
        a.w1, a.w2, a.cgw1 = 16.0, 256.0, (16.0 if levels >= 2 else 1.0)
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
        return dq, dk, dv, None, None, None, None, None, dgq, dgk, None, None


def selection(out):
    """The blocks the forward that produced `out` chose: (indices (B,H,N/16,T), p_indices
    (B,H,N/256,T2) or None), int32 views of the arena its autograd node holds."""
    node = out.grad_fn
    I = node.saved_tensors[1]
    _, lay, B, H, N, T, T2, levels = node.meta[:8]
    idx = I[lay.idx:lay.idx + B * H * lay.n1 * T].view(B, H, lay.n1, T)
    pidx = I[lay.pidx:lay.pidx + B * H * lay.n2 * T2].view(B, H, lay.n2, T2) if levels >= 2 else None
    if levels == 3:
        T3 = node.meta[12]
        return idx, pidx, I[lay.ppidx:lay.ppidx + B * H * lay.n3 * T3].view(B, H, lay.n3, T3)
    return idx, pidx
