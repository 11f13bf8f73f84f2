"""Loads the x86 build of the HIP sources (tests/cpu_emu) for CPU-side kernel tests."""
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "cpu_emu"))

_EMU = None


def emu_lib():
    """Build (when sources are newer than the library) and load libllsa_emu.so."""
    global _EMU
    if _EMU is not None:
        return _EMU
    import build_emu
    from llsa_amd._lib import Lib
    out = os.path.join(build_emu.OUT, "libllsa_emu.so")
    csrc = os.path.join(ROOT, "llsa_amd", "csrc")
    srcs = [os.path.join(csrc, f) for f in os.listdir(csrc)]
    srcs += [os.path.join(ROOT, "include", "llsa_hip.h")]
    emu_dir = os.path.join(ROOT, "tests", "cpu_emu")
    srcs += [os.path.join(emu_dir, "emu_runtime.cpp"), os.path.join(emu_dir, "include", "hip", "hip_runtime.h")]
    if not os.path.exists(out) or os.path.getmtime(out) < max(os.path.getmtime(s) for s in srcs):
        if not os.path.exists(build_emu.CLANG):   # no host clang: these tests cannot run
            pytest.skip(f"cannot build the CPU emulation library: {build_emu.CLANG} is missing")
        build_emu.build(verbose=False)            # a compile error is a failure of the suite, not a skip
    _EMU = Lib(out, device_library=False)
    return _EMU
