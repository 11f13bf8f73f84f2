"""The parity cases of tests/parity_cases.py at tiny sizes on the CPU, through the x86
emulation build of the HIP sources (tests/cpu_emu).  This checks index arithmetic, operand
layouts and the Python/autograd glue without a GPU; the GPU run of the same cases is
tests/test_gpu_parity.py."""
import pytest
import torch

import parity_cases as P
from emu_util import emu_lib
from llsa_amd._lib import override_library_for_tests

DEV = torch.device("cpu")


@pytest.fixture(autouse=True)
def _emu():
    with override_library_for_tests(emu_lib()):
        yield


def test_pool_pyramid():
    P.check_pool_pyramid(DEV, N=512, strided=True, rope=True)
    P.check_pool_pyramid(DEV, N=256, strided=False, rope=False)
    P.check_pool_pyramid(DEV, B=1, H=1, N=4096, strided=True, rope=False)       # with the tiles of the level-2 rows


def test_mean_pool1d():
    P.check_mean_pool1d(DEV, torch.bfloat16, 16, 64, 64, 'bhsc')
    P.check_mean_pool1d(DEV, torch.float32, 4, 24, 32, 'bhsc')
    P.check_mean_pool1d(DEV, torch.bfloat16, 8, 100, 32, 'bsc')


def test_rope():
    P.check_rope(DEV, side=8, strided=True)


def test_topk_dense():
    P.check_topk_dense(DEV, n=64, T=8, round_scores=True)
    P.check_topk_dense(DEV, n=64, T=8, round_scores=False, min_safe=0.9)
    P.check_topk_dense_ties(DEV)


def test_topk_dense_multi_chunk():
    P.check_topk_dense(DEV, B=1, H=1, n=1088, T=16, round_scores=False, min_safe=0.9)


def test_topk_sparse():
    P.check_topk_sparse(DEV, N1=256, T=8, T2=4)
    P.check_topk_cascade(DEV, B=1, H=1, N1=512, T=8, T2=4)


def test_permute():
    P.check_permute(DEV, B=2, side=8, C=24, dtype=torch.bfloat16)
    P.check_permute(DEV, B=1, side=4, C=4, dtype=torch.float32)


def test_rms_norm():
    P.check_rms_norm(DEV, B=1, H=2, N=64, strided=True)
    P.check_rms_norm(DEV, B=1, H=33, N=2048, strided=False)       # 264 partial rows: the weights' gradient is folded in two launches


def test_op_l1_qk_norm():
    P.check_op_l1(DEV, B=1, H=1, N=1024, T=8, fused=True, rope=True, qk_norm=True)


def test_transpose():
    P.check_transpose(DEV, Mb=64, T=8)
    P.check_transpose(DEV, B=1, H=1, Mb=64, T=4, Kb=16)
    P.check_transpose(DEV, B=1, H=2, Mb=4096, T=16, chunk=64)        # 65536 entries: the split form
    P.check_transpose_hot_block(DEV)
    P.check_transpose_levels(DEV, B=1, H=2, sizes=((256, 8), (16, 4)))
    P.check_transpose(DEV, B=1, H=1, Mb=40, T=4, Kb=2048, chunk=2)   # more key blocks than threads
    P.check_transpose(DEV, B=1, H=1, Mb=200, T=12, Kb=200)           # a last word that is not full


def test_attn_l1():
    P.check_attn_l1(DEV, B=1, H=2, N=1024, T=8, strided=True)


def test_attn_l1_hot_block():
    P.check_attn_l1(DEV, B=1, H=1, N=2048, T=4, hot=5)        # 128 query blocks on one key block: 4 chunks


def test_attn_special_cases():
    P.check_attn_reduces_to_sdpa(DEV, B=1, H=1, N=1024)
    P.check_constant_v(DEV)
    P.check_attn_fwd_repeated_block(DEV, B=1, H=1, N=1024, T=8)


@pytest.mark.parametrize("fused,rope", [(True, False), (True, True), (False, False)])
def test_op_l1(fused, rope):
    P.check_op_l1(DEV, B=1, H=1, N=1024, T=8, fused=fused, rope=rope, strided=True)


def test_attn_l2_hot_coarse_block():
    # (the smallest two-level case takes two minutes in the emulation, so the two-level kernels get one
    # run here, the one that also cuts a list into chunks; the plain case runs on the GPU)
    P.check_attn_l2(DEV, B=1, H=1, N=16384, T=4, T2=4, hot=3)  # 64 parents on one coarse block: 8 chunks


def test_op_l2_fused_rope():
    P.check_op_l2(DEV, B=1, H=1, N=16384, T=4, T2=4, fused=True, rope=True)


def test_sparse_dout_enumeration_two_levels():
    """The element-wise dK / dV check that the GPU suite runs at three and four levels, at two levels and N = 16384 here
    (where the whole-tensor oracle agrees too: test_op_l2_fused_rope): the enumeration itself is what this pins."""
    P.check_op_lk_sparse_dout(DEV, N=16384, topks=(8, 4), H=1, query_blocks=(0, 517, -1), rope=True)


def test_unfused_backward_rejects_a_repeated_parent():
    """A caller's own p_indices that name a block twice in a row are an error, not a wrong gradient."""
    from llsa_amd.kernel.hip import _attention as A
    B, H, N = 1, 1, 16384
    g = torch.Generator().manual_seed(3)
    q, k, v, do, o = (torch.randn(B, H, N, 64, generator=g).bfloat16() for _ in range(5))
    pk, pv = (torch.randn(B, H, N // 16, 64, generator=g).bfloat16() for _ in range(2))
    pk2, pv2 = (torch.randn(B, H, N // 256, 64, generator=g).bfloat16() for _ in range(2))
    lse = torch.zeros(B, H, N)
    idx = torch.arange(8).expand(B, H, N // 16, 8).contiguous()
    pidx = torch.tensor([0, 1, 2, 2]).expand(B, H, N // 256, 4).contiguous()
    with pytest.raises(ValueError, match="names a block twice"):
        A.attn_bwd(do, q, k, v, pk, pv, o, lse, idx, 16.0, 16.0, pk2=pk2, pv2=pv2, p_indices=pidx, token_weight_2=256.0)
