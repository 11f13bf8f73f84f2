"""Builds tests/cpu_emu/_build/libllsa_emu.so: the HIP sources of llsa_amd/csrc compiled for
x86 against the fiber-based stand-in for the HIP runtime in tests/cpu_emu/include.  Test
infrastructure only -- lets the kernels run on the CPU (tiny sizes) under gdb / ASan."""
from __future__ import annotations

import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "llsa_amd", "csrc")
OUT = os.path.join(HERE, "_build")
CLANG = os.environ.get("EMU_CXX", "/opt/rocm/llvm/bin/clang++")


def build(asan: bool = False, verbose: bool = True) -> str:
    os.makedirs(OUT, exist_ok=True)
    flags = ["-x", "c++", "-std=c++17", "-O1", "-g", "-fPIC", "-I", os.path.join(HERE, "include"),
             "-Wno-unknown-attributes", "-Wno-unused-value", "-ffp-contract=off", "-DLLSA_CPU_EMU_BUILD"]
    if asan:
        flags += ["-fsanitize=address", "-fno-omit-frame-pointer"]
    srcs = [os.path.join(CSRC, f) for f in sorted(os.listdir(CSRC)) if f.endswith(".hip")]
    srcs.append(os.path.join(HERE, "emu_runtime.cpp"))

    def comp(src):
        obj = os.path.join(OUT, os.path.basename(src) + (".asan.o" if asan else ".o"))
        r = subprocess.run([CLANG, *flags, "-c", src, "-o", obj], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"emu compile failed on {src}:\n{r.stderr}")
        return obj

    with cf.ThreadPoolExecutor(max_workers=8) as ex:
        objs = list(ex.map(comp, srcs))
    name = "libllsa_emu_asan.so" if asan else "libllsa_emu.so"
    out = os.path.join(OUT, name)
    link = [CLANG, "-shared", "-fPIC", "-o", out, *objs]
    if asan:
        link += ["-fsanitize=address", "-shared-libasan"]
    r = subprocess.run(link, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("emu link failed:\n" + r.stderr)
    if verbose:
        print("built", out)
    return out


if __name__ == "__main__":
    build(asan="--asan" in sys.argv)
