"""Query-major top-k lists -> key-major CSR.  Mirrors kernel/triton/indices_transpose.py."""
from __future__ import annotations

import ctypes as C

import torch

from ..._lib import CHUNK_COARSE, CHUNK_FINE
from ._common import BLOCK, lib_for, ptr, stream_of


def transpose_indices(q_topk_indices, k_ntx=None, chunk=0, stream=None):
    """indices_transpose.py:104-109.  Returns (offsets (B,H,1+Kb), flat (B,H,Mb*T)), int32; the
    entries of each segment are in ascending query-block order.  With chunk > 0 a third tensor
    is returned: the work list the backward kernels use to walk every segment in pieces of at
    most `chunk` entries (layout in include/llsa_hip.h).  `stream`: raw handle of the stream to launch on
    (default: the current one)."""
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
    lib.check(lib.transpose_indices(ptr(idx), ptr(offsets), ptr(flat), ptr(work), B, H, Mb, k_ntx, T, max(chunk, 1),
                                    stream_of(lib, idx) if stream is None else stream), "transpose_indices")
    return (offsets, flat) if work is None else (offsets, flat, work)


_side_streams = {}


class BackwardLists:
    """The key-major lists the backward needs -- (offsets, flat, work) of `indices` and, for two
    levels, of `p_indices` -- built on a second stream while the caller's stream goes on with
    the forward attention kernel, which does not need them.  `join()` makes the caller's
    stream wait for them; `csr` is what attn_bwd takes."""

    def __init__(self, indices, p_indices=None):
        n_fine = indices.shape[2]
        self._event = None
        stream = None
        if indices.is_cuda:                      # (the CPU emulation used by the tests has no streams)
            dev = indices.device
            cur = torch.cuda.current_stream(dev)
            side, self._event = _side_streams.get(dev, (None, None))
            if side is None:
                side, self._event = _side_streams[dev] = (torch.cuda.Stream(device=dev), torch.cuda.Event())
            side.wait_stream(cur)                # the indices are produced on the caller's stream
            stream = C.c_void_p(side.cuda_stream)
        # The lists are allocated on the caller's stream (only the kernels run on the other one), so the
        # allocator needs no word about the second stream: join() orders every later use and the eventual
        # release after the kernels that fill them.
        self.csr = transpose_indices(indices, n_fine, CHUNK_FINE, stream=stream)
        if p_indices is not None:
            self.csr += transpose_indices(p_indices, n_fine // BLOCK, CHUNK_COARSE, stream=stream)
        if self._event is not None:
            self._event.record(side)

    def join(self):
        if self._event is not None:
            torch.cuda.current_stream(self.csr[0].device).wait_event(self._event)
        return self.csr
