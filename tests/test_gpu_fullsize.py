"""The benchmark configurations at their full sizes.

C2 and C3 are small enough for the CPU oracle, slice by slice.  At N = 65536, 262144, (three levels) 1048576 and
(four levels) 4194304 the oracle would take minutes, so the operator is checked through properties that do not depend on
the size (the selection depends on q and k only, so it is the same on both sides of each):
  * constant V            -> O is that constant (the weights of fine and pooled tokens sum to 1)
  * linearity in V        -> O(a V1 + b V2) = a O(V1) + b O(V2)
  * column sums           -> sum over tokens of dV = sum over tokens of dO, channel by channel
                             (every query's weights sum to 1; a pooled token hands 1/16 to each child)
  * scale invariance      -> sum(q * dq) = sum(k * dk): scores see q and k only through q.k
"""
import math

import pytest
import torch

import parity_cases as P

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available()
    from llsa_amd._lib import get_lib
    get_lib()
    return torch.device("cuda:0")


def test_c1_inputs_in_bf16(dev):
    """Benchmark configuration 1 (llsa_l1, B=1, H=6, N=1024, topk 8, N(0,1) inputs) is an fp32 CPU case
    of the reference; the kernels are bf16, so the same inputs are rounded to bf16 and checked against
    the oracle in bf16 (forward and backward), and the output against the fp32 oracle on the
    operator's own selection within the bf16 tolerance."""
    import llsa_amd
    from oracle import llsa_oracle as O
    from llsa_amd.kernel.torch_op._fused import selection
    P.check_op_l1(dev, B=1, H=6, N=1024, T=8, fused=True, rope=False)
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(1, 6, 1024, 64, generator=g) for _ in range(3))
    out = llsa_amd.llsa_l1(*(t.bfloat16().to(dev).requires_grad_(True) for t in (q, k, v)), 8, 16)
    idx = selection(out)[0].cpu().long()
    ref, _ = O.llsa_l1_fwd(q, k, v, 8, 16, indices=idx)
    err = (out.detach().float().cpu() - ref)
    assert err.norm() / ref.norm() <= 1e-2 and err.abs().max() <= 2e-2


def test_c2_full_size_against_oracle(dev):
    P.check_op_l1(dev, B=4, H=6, N=4096, T=16, fused=True, rope=False, smooth=True)


def test_c3_full_size_against_oracle(dev):
    P.check_op_l2(dev, B=2, H=6, N=16384, T=16, T2=16, fused=True, rope=True, smooth=True)


def test_c5_full_size_two_heads_against_oracle(dev):
    """Benchmark configuration 5 at its shape, B=1, H=6, N=262144, topk 16/16, RoPE in the kernel (six (b,h) in the
    split-form index transpose and the workspace strides); the oracle runs on the first and the last head."""
    P.check_op_l2(dev, B=1, H=6, N=262144, T=16, T2=16, fused=True, rope=True, smooth=True, slices=[(0, 0), (0, 5)])


@pytest.mark.parametrize("H,T,T2,T3,rope,qk_norm", [(1, 16, 16, 16, True, False), (2, 8, 4, 8, False, True)])
def test_three_levels_against_oracle(dev, H, T, T2, T3, rope, qk_norm):
    """llsa_l3 (no counterpart in the reference) at its smallest size, N = 262144, against the oracle's
    three-level composition."""
    P.check_op_l3(dev, B=1, H=H, N=262144, T=T, T2=T2, T3=T3, rope=rope, qk_norm=qk_norm)


def _rel(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-30)).item()


def test_four_levels_single_queries_against_enumeration(dev):
    """llsa_lk with four pooled levels at the smallest size it admits, N = 4194304 = 64 * 16^4."""
    P.check_op_lk_samples(dev, N=4194304, topks=(16, 16, 16, 16))


@pytest.mark.parametrize("N,topks,H", [(4194304, (16, 16, 16, 16), 1), (262144, (8, 4, 8), 2), (16384, (16, 16), 2)])
def test_dk_dv_elementwise_with_sparse_dout(dev, N, topks, H):
    """Every element of dK and dV at two, three and four levels: dO is zero outside three query blocks, so the whole
    gradient follows from 48 queries, enumerated on the CPU in fp64 from the device's selection."""
    P.check_op_lk_sparse_dout(dev, N=N, topks=topks, H=H)


def test_three_levels_single_queries_against_enumeration(dev):
    P.check_op_lk_samples(dev, N=262144, topks=(8, 4, 8), H=2)


@pytest.mark.parametrize("N,H,levels", [(65536, 2, 2), (262144, 1, 2), (1048576, 1, 3), (4194304, 1, 4)])
def test_large_n_properties(dev, N, H, levels):
    import llsa_amd
    from llsa_amd.utils.rope_table import rope_table
    q, k, v, do = P.smooth_inputs(1, H, N, 64, dev)
    freq = rope_table(math.isqrt(N), dtype=torch.bfloat16).to(dev)
    if levels >= 3:
        op = lambda q_, k_, v_: llsa_amd.llsa_lk(q_, k_, v_, (16,) * levels, 16, rope=freq)
    else:
        op = lambda q_, k_, v_: llsa_amd.llsa_l2(q_, k_, v_, 16, 16, 16, rope=freq)

    with torch.no_grad():
        const = torch.full_like(v, 0.625)
        assert (op(q, k, const).float() - 0.625).abs().max().item() < 4e-3, "constant V must come out unchanged"
        v2 = P.smooth_inputs(1, H, N, 64, dev, seeds=(5, 6, 7, 8))[2]
        o1, o2 = op(q, k, v).float(), op(q, k, v2).float()
        mix = (0.5 * v.float() - 0.25 * v2.float()).bfloat16()
        want = 0.5 * o1 - 0.25 * o2
        assert _rel(op(q, k, mix).float(), want) < 1e-2, "O must be linear in V"

    q, k, v = (t.detach().requires_grad_(True) for t in (q, k, v))
    op(q, k, v).backward(do)
    torch.cuda.synchronize()
    assert all(torch.isfinite(t.grad).all() for t in (q, k, v))
    col_dv, col_do = v.grad.double().sum(dim=2), do.double().sum(dim=2)
    assert _rel(col_dv, col_do) < 1e-2, f"column sums of dV and dO differ: {_rel(col_dv, col_do):.3e}"
    # the gradients are bf16 and both sums cancel heavily, so compare them on the scale of their terms
    qdq, kdk = (q.detach().double() * q.grad.double()).sum(), (k.detach().double() * k.grad.double()).sum()
    scale = (q.detach().double() * q.grad.double()).abs().sum()
    assert abs(qdq - kdk) / scale < 2e-3, f"sum(q dq) = {qdq:.6e} but sum(k dk) = {kdk:.6e} (terms sum to {scale:.3e})"
