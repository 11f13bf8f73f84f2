"""Builds llsa_amd/lib/libllsa_hip.so from llsa_amd/csrc/*.hip with hipcc for gfx950.

    python -m llsa_amd.build            # compile every source (parallel), link the shared library

hipcc cross-compiles without a GPU.  The library is kept in-tree (git-ignored) so that a
checkout that was built once can be used on a machine without recompiling.
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "lib", "obj")
LIBNAME = "libllsa_hip.so"

HIPCC = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",     # no packed-fp32 VALU ops
    "-mllvm", "-amdgpu-mfma-vgpr-form",      # MFMA results straight into VGPRs: no v_accvgpr copies around the soft-max
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src: str) -> str:
    obj = os.path.join(OBJDIR, src.replace(".hip", ".o"))
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        print(err, file=sys.stderr)
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = sources()
    with cf.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    out = os.path.join(LIBDIR, LIBNAME)
    tmp = out + ".tmp"
    r = subprocess.run([HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    os.replace(tmp, out)
    if verbose:
        print(f"built {out} from {len(srcs)} sources")
    return out


if __name__ == "__main__":
    build()
