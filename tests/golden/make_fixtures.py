"""Writes the fixtures of this directory.

The reference ships no golden vectors, known-answer tests or fixture files for this path, and
its kernels cannot run here (Triton on an NVIDIA GPU), so there is nothing of the reference's
to record.  These files are regression anchors of the CPU oracle instead: the oracle is pinned
against independent formulations in tests/test_oracle_pins.py, and the fixtures freeze what it
returned at that point, so that a later edit of the oracle (or of the kernels) that changes a
result is noticed.  Inputs are regenerated from seeds; outputs are stored for every 16th token.

    python tests/golden/make_fixtures.py        # rewrites l1_small.npz and l2_small.npz
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import llsa_oracle as O  # noqa: E402

STEP = 16        # token stride of the stored rows


def inputs(B, H, N, seed):
    """bf16-representable inputs as fp32 tensors (what both the oracle and the kernels are fed)."""
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(B, H, N, 64, generator=g).bfloat16().float() for _ in range(4))


def l1_case():
    B, H, N, T = 1, 2, 1024, 8
    q, k, v, do = inputs(B, H, N, 101)
    o, ctx = O.llsa_l1_fwd(q.bfloat16(), k.bfloat16(), v.bfloat16(), T, 16)
    dq, dk, dv, _ = O.llsa_l1_bwd(do.bfloat16(), ctx)
    return dict(B=B, H=H, N=N, T=T, seed=101, indices=ctx["indices"].numpy().astype(np.int32),
                lse=ctx["lse"].float().numpy()[..., ::STEP], **_sub(o=o, dq=dq, dk=dk, dv=dv))


def l2_case():
    B, H, N, T, T2 = 1, 1, 16384, 8, 4
    q, k, v, do = inputs(B, H, N, 202)
    o, ctx = O.llsa_l2_fwd(q.bfloat16(), k.bfloat16(), v.bfloat16(), T, T2, 16)
    dq, dk, dv, _ = O.llsa_l2_bwd(do.bfloat16(), ctx)
    return dict(B=B, H=H, N=N, T=T, T2=T2, seed=202, indices=ctx["indices"].numpy().astype(np.int32),
                p_indices=ctx["p_indices"].numpy().astype(np.int32), lse=ctx["lse"].float().numpy()[..., ::STEP],
                **_sub(o=o, dq=dq, dk=dk, dv=dv))


def _sub(**tensors):
    out = {}
    for name, t in tensors.items():
        t = t.float()
        out[name] = t[:, :, ::STEP].numpy().astype(np.float32)
        out[name + "_sum"] = np.float64(t.double().sum().item())
        out[name + "_abs"] = np.float64(t.double().abs().sum().item())
    return out


if __name__ == "__main__":
    np.savez_compressed(os.path.join(HERE, "l1_small.npz"), **l1_case())
    np.savez_compressed(os.path.join(HERE, "l2_small.npz"), **l2_case())
    for f in ("l1_small.npz", "l2_small.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
