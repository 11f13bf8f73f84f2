"""Shared plumbing of the launchers: argument checks, pointers, stream."""
from __future__ import annotations

import ctypes as C

import torch

from ..._lib import Lib, current_lib

HEAD_DIM = 64
BLOCK = 16


def lib_for(*tensors: torch.Tensor) -> Lib:
    lib = current_lib()
    for t in tensors:
        if t is None:
            continue
        if lib.device_library and not t.is_cuda:
            raise RuntimeError("llsa_amd runs on an AMD GPU only (got a CPU tensor); there is no CPU implementation")
    return lib


def stream_of(lib: Lib, t: torch.Tensor):
    """The raw handle of the current stream of t's device (None for the CPU emulation of the tests)."""
    if not lib.device_library:
        return None
    idx = t.device.index
    return C.c_void_p(torch._C._cuda_getCurrentRawStream(torch.cuda.current_device() if idx is None else idx))


def ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def require_bf16(*tensors):
    for t in tensors:
        if t is not None and t.dtype != torch.bfloat16:
            raise NotImplementedError(f"llsa_amd attention kernels are bf16 only (got {t.dtype})")


def require_head_dim(t):
    if t.shape[-1] != HEAD_DIM:
        raise NotImplementedError(f"llsa_amd attention kernels need head dim {HEAD_DIM} (got {t.shape[-1]})")


def rows_ok(t: torch.Tensor) -> bool:
    """Last stride 1 and every row start 16-byte aligned (what the 16-byte loads need)."""
    return (t.stride(-1) == 1 and t.data_ptr() % 16 == 0
            and all(s % 8 == 0 for s in t.stride()[:-1]))


def as_rows(t: torch.Tensor) -> torch.Tensor:
    """Return t if the kernels can read it in place, else a contiguous copy."""
    return t if rows_ok(t) else t.contiguous()


def s3(t: torch.Tensor):
    return t.stride(0), t.stride(1), t.stride(2)


def i64x(vals):
    return (C.c_int64 * len(vals))(*vals)
