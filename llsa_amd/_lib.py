"""ctypes binding of libllsa_hip.so (the C ABI declared in include/llsa_hip.h).

The product path loads llsa_amd/lib/libllsa_hip.so and nothing else; if it is missing the
import of any operator fails with an error that says how to build it.  There is no CPU
implementation in this package.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libllsa_hip.so")

c_void_p, c_int, c_int32, c_int64, c_float = C.c_void_p, C.c_int, C.c_int32, C.c_int64, C.c_float


class PoolItem(C.Structure):
    _fields_ = [("x", c_void_p), ("sxb", c_int64), ("sxh", c_int64), ("sxn", c_int64),
                ("n", c_int32), ("rope", c_int32),
                ("y1", c_void_p), ("y2", c_void_p), ("xr", c_void_p), ("xt", c_void_p), ("y1r", c_void_p),
                ("y1t", c_void_p), ("xrot", c_void_p),
                ("gamma", c_void_p), ("eps", c_float), ("reserved", c_int32), ("y2r", c_void_p), ("y2t", c_void_p)]


MAX_LEVELS = 4                                              # LLSA_MAX_LEVELS


class FwdLevel(C.Structure):
    _fields_ = [("kr", c_void_p), ("vt", c_void_p), ("sel", c_void_p), ("T", c_int32), ("w", c_float)]


class AttnFwdArgs(C.Structure):
    _fields_ = [("qr", c_void_p), ("kr", c_void_p), ("vt", c_void_p), ("idx", c_void_p),
                ("o", c_void_p), ("sob", c_int64), ("soh", c_int64), ("son", c_int64),
                ("lse", c_void_p),
                ("B", c_int32), ("H", c_int32), ("N", c_int32), ("T", c_int32), ("levels", c_int32), ("reserved", c_int32),
                ("lvl", FwdLevel * MAX_LEVELS)]


def _t3(name):
    return [(name, c_void_p), ("s" + name + "b", c_int64), ("s" + name + "h", c_int64), ("s" + name + "n", c_int64)]


class BwdLevel(C.Structure):
    _fields_ = [("kr", c_void_p), ("vr", c_void_p), ("sel", c_void_p), ("off", c_void_p), ("inv", c_void_p),
                ("dk", c_void_p), ("dv", c_void_p), ("T", c_int32), ("w", c_float), ("gw", c_float), ("reserved", c_int32)]


class AttnBwdArgs(C.Structure):
    _fields_ = (
        [("dout", c_void_p), ("sdob", c_int64), ("sdoh", c_int64), ("sdon", c_int64)]
        + _t3("o")
        + [("lse", c_void_p), ("qr", c_void_p), ("kr", c_void_p), ("vr", c_void_p),
           ("idx", c_void_p), ("off", c_void_p), ("flat", c_void_p), ("work", c_void_p)]
        + [("dq", c_void_p), ("sdqb", c_int64), ("sdqh", c_int64), ("sdqn", c_int64),
           ("dk", c_void_p), ("sdkb", c_int64), ("sdkh", c_int64), ("sdkn", c_int64),
           ("dv", c_void_p), ("sdvb", c_int64), ("sdvh", c_int64), ("sdvn", c_int64)]
        + [("workspace", c_void_p), ("workspace_bytes", c_int64), ("freq_dq", c_void_p), ("freq_dk", c_void_p),
           ("B", c_int32), ("H", c_int32), ("N", c_int32), ("T", c_int32), ("levels", c_int32),
           ("stages", c_int32), ("fold_pooled", c_int32), ("reserved", c_int32),
           ("lvl", BwdLevel * MAX_LEVELS)])


P64 = C.POINTER(c_int64)


class TransposeJob(C.Structure):
    _fields_ = [("idx", c_void_p), ("offsets", c_void_p), ("flat", c_void_p), ("work", c_void_p), ("inv", c_void_p),
                ("Mb", c_int32), ("Kb", c_int32), ("T", c_int32), ("chunk", c_int32)]


_SIGNATURES = {
    "llsa_version": (c_int, []),
    "llsa_last_error_string": (C.c_char_p, []),
    "llsa_pool_pyramid_fwd": (c_int, [C.POINTER(PoolItem), c_int, c_void_p, c_int, c_int, c_void_p]),
    "llsa_mean_pool_fwd": (c_int, [c_void_p, P64, c_void_p, P64, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "llsa_mean_pool_bwd": (c_int, [c_void_p, P64, c_void_p, P64, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "llsa_pool_bwd_accum": (c_int, [c_void_p, P64, c_void_p, c_void_p, c_void_p, P64, c_void_p, c_int, c_int, c_int, c_void_p]),
    "llsa_rmsnorm_bwd_partials": (c_int64, [c_int, c_int, c_int]),
    "llsa_rmsnorm_bwd": (c_int, [c_void_p, P64, c_void_p, P64, c_void_p, c_float, c_void_p, P64, c_void_p, c_void_p,
                                 c_int, c_int, c_int, c_void_p]),
    "llsa_rmsnorm_bwd_static": (c_int, [c_void_p, P64, c_void_p, P64, c_void_p, c_float, c_void_p, P64, c_void_p,
                                        c_int, c_int, c_int, c_void_p]),
    "llsa_gather_rows": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int64, c_int64, c_void_p]),
    "llsa_rope_fwd": (c_int, [c_void_p, P64, c_void_p, c_void_p, P64, c_int, c_int, c_int, c_void_p]),
    "llsa_rope_bwd": (c_int, [c_void_p, P64, c_void_p, c_void_p, P64, c_int, c_int, c_int, c_void_p]),
    "llsa_topk_dense": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "llsa_topk_sparse": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "llsa_topk_cascade": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "llsa_topk_cascade_max_parents": (c_int, []),
    "llsa_attn_fwd": (c_int, [C.POINTER(AttnFwdArgs), c_void_p]),
    "llsa_transpose_indices": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "llsa_transpose_indices_multi": (c_int, [C.POINTER(TransposeJob), c_int, c_int, c_int, c_void_p]),
    "llsa_work_list_len": (c_int64, [c_int, c_int, c_int, c_int]),
    "llsa_fine_chunk": (c_int, [c_int]),
    "llsa_attn_bwd_workspace_bytes": (c_int64, [c_int, c_int, c_int, C.POINTER(c_int32), c_int]),
    "llsa_attn_bwd": (c_int, [C.POINTER(AttnBwdArgs), c_void_p]),
}

EXPORTS = tuple(_SIGNATURES)
CHUNK_FINE_MAX = 256                                        # LLSA_CHUNK_FINE_MAX of include/llsa_hip.h
ABI_VERSION = 203                                           # LLSA_ABI_VERSION
STATIC_PARTIALS_MAX = 262144                                # LLSA_STATIC_PARTIALS_MAX


class LlsaError(RuntimeError):
    pass


class Lib:
    """A loaded libllsa shared object with typed entry points."""

    def __init__(self, path: str, device_library: bool = True):
        if not os.path.exists(path):
            raise ImportError(
                f"{path} not found: build the HIP extension first (python -m llsa_amd.build, needs hipcc); "
                "llsa_amd has no CPU implementation")
        self.path = path
        self.device_library = device_library
        self.cdll = C.CDLL(path)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(self.cdll, name)          # AttributeError if the library lacks an export
            fn.restype = res
            fn.argtypes = args
            setattr(self, name[len("llsa_"):], fn)
        if self.version() != ABI_VERSION:      # a library built from other sources than this binding describes
            raise ImportError(f"{path} has ABI version {self.version()}, this package needs {ABI_VERSION}: rebuild it "
                              "(python -m llsa_amd.build)")

    def check(self, rc: int, what: str):
        if rc != 0:
            raise LlsaError(f"{what} failed ({rc}): {self.last_error_string().decode()}")


_LIB: Optional[Lib] = None


def get_lib() -> Lib:
    global _LIB
    if _LIB is None:
        _LIB = Lib(LIB_PATH)
    return _LIB


# --------------------------------------------------------------------------------------
# Test hook.  tests/cpu_emu builds the same HIP sources for x86 (one fiber per GPU thread) so
# that kernels and the Python glue can be exercised at tiny sizes without a GPU.  That
# library is only ever used when a test installs it explicitly with this context manager;
# nothing in the package selects it on its own, and with the real library CPU tensors are
# rejected.
# --------------------------------------------------------------------------------------
import contextlib

_OVERRIDE: Optional[Lib] = None


@contextlib.contextmanager
def override_library_for_tests(lib: Lib):
    global _OVERRIDE
    prev, _OVERRIDE = _OVERRIDE, lib
    try:
        yield lib
    finally:
        _OVERRIDE = prev


def current_lib() -> Lib:
    return _OVERRIDE if _OVERRIDE is not None else get_lib()
