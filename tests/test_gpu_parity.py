"""GPU parity: the HIP kernels (through libllsa_hip.so and the Python operator API) against
the CPU oracle on the same seeded inputs.  Run with `pytest -m gpu` on an MI355X."""
import pytest
import torch

import parity_cases as P

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available()
    from llsa_amd._lib import get_lib
    get_lib()                       # fails loudly if the HIP library is not built
    return torch.device("cuda:0")


def test_library_loaded(dev):
    from llsa_amd._lib import EXPORTS, get_lib
    lib = get_lib()
    assert lib.device_library and lib.version() >= 100
    for name in EXPORTS:
        assert hasattr(lib.cdll, name)


def test_cpu_tensors_are_rejected(dev):
    import llsa_amd
    x = torch.randn(1, 1, 1024, 64).bfloat16()
    with pytest.raises(RuntimeError, match="GPU only"):
        llsa_amd.llsa_l1(x, x, x, 8, 16)


@pytest.mark.parametrize("N,strided,rope", [(512, True, True), (4096, False, False), (16384, True, True)])
def test_pool_pyramid(dev, N, strided, rope):
    P.check_pool_pyramid(dev, B=2, H=3, N=N, strided=strided, rope=rope)


def test_mean_pool1d(dev):
    P.check_mean_pool1d(dev, torch.bfloat16, 16, 64, 1024, 'bhsc')
    P.check_mean_pool1d(dev, torch.float32, 4, 24, 32, 'bhsc')
    P.check_mean_pool1d(dev, torch.bfloat16, 8, 100, 64, 'bsc')


def test_rope(dev):
    P.check_rope(dev, B=2, H=3, side=32, strided=True)
    P.check_rope(dev, B=1, H=2, side=8, strided=False)


def test_permute(dev):
    P.check_permute(dev, B=2, side=128, C=384, dtype=torch.bfloat16)
    P.check_permute(dev, B=3, side=16, C=12, dtype=torch.float32)


def test_rms_norm(dev):
    P.check_rms_norm(dev, B=2, H=3, N=4096, strided=True)
    P.check_rms_norm(dev, B=1, H=1, N=16, strided=False)
    P.check_rms_norm(dev, B=4, H=6, N=16384, strided=True)        # 1536 partial rows: folded in two launches


def test_op_with_qk_norm(dev):
    P.check_op_l1(dev, B=2, H=2, N=4096, T=16, fused=True, rope=True, strided=True, qk_norm=True)
    P.check_op_l2(dev, B=1, H=2, N=16384, T=16, T2=16, fused=True, rope=True, smooth=True, qk_norm=True)


def test_topk_dense(dev):
    P.check_topk_dense(dev, B=2, H=3, n=256, T=16, round_scores=True)
    P.check_topk_dense(dev, B=1, H=2, n=64, T=16, round_scores=False, min_safe=0.9)
    P.check_topk_dense(dev, B=1, H=2, n=1024, T=16, round_scores=False, min_safe=0.9)
    P.check_topk_dense(dev, B=1, H=2, n=2048, T=16, round_scores=False, min_safe=0.9)     # rows longer than the radix kernel keeps: chunked arg-max
    P.check_topk_dense(dev, B=1, H=1, n=4096, T=8, round_scores=True)
    P.check_topk_dense_ties(dev)


def test_topk_sparse(dev):
    P.check_topk_sparse(dev, B=2, H=3, N1=1024, T=16, T2=16)
    P.check_topk_sparse(dev, B=1, H=1, N1=256, T=8, T2=4)
    P.check_topk_cascade(dev, B=2, H=3, N1=1024, T=16, T2=16)
    P.check_topk_cascade(dev, B=1, H=1, N1=4096, T=16, T2=32)        # 256 parent tokens: the most the cascade takes
    P.check_topk_cascade(dev, B=1, H=2, N1=256, T=4, T2=4)


def test_transpose(dev):
    P.check_transpose(dev, B=2, H=3, Mb=1024, T=16)
    P.check_transpose(dev, B=1, H=2, Mb=64, T=16)
    P.check_transpose(dev, B=1, H=1, Mb=64, T=4, Kb=16)
    P.check_transpose_hot_block(dev)
    P.check_transpose_levels(dev)                                    # two levels, one launch
    P.check_transpose(dev, B=1, H=2, Mb=64, T=8, Kb=8192, chunk=4)   # more key blocks than threads, two words a row
    P.check_transpose(dev, B=1, H=1, Mb=1000, T=12, Kb=1000)         # a last word that is not full, topk not a power of two
    P.check_transpose_levels(dev, B=1, H=2, sizes=((256, 16),))


def test_transpose_largest(dev):
    P.check_transpose(dev, B=1, H=1, Mb=16384, T=16)
    P.check_transpose(dev, B=1, H=2, Mb=16384, T=16, chunk=64)       # with the work list: the split form
    P.check_transpose(dev, B=1, H=1, Mb=262144, T=16, chunk=64)      # the fine level of four pooled levels: 128 KB of sort bitmaps
    P.check_transpose(dev, B=1, H=1, Mb=524288, T=2, Kb=8192, chunk=64)   # two sort waves a workgroup


@pytest.mark.parametrize("strided,smooth", [(False, False), (True, False), (False, True)])
def test_attn_l1(dev, strided, smooth):
    P.check_attn_l1(dev, B=2, H=3, N=4096, T=16, strided=strided, smooth=smooth)


def test_attn_l1_small(dev):
    P.check_attn_l1(dev, B=1, H=2, N=1024, T=8)


def test_attn_more_than_64_selected(dev):
    """top-k above 64: the kernels fetch the indices of a query block 64 at a time, and every key
    block's list (128 entries here: every query block selects every key block) has two chunks."""
    P.check_attn_l1(dev, B=1, H=2, N=2048, T=128)
    P.check_attn_reduces_to_sdpa(dev, B=1, H=1, N=2048)


def test_attn_hot_blocks(dev):
    P.check_attn_l1(dev, B=1, H=2, N=4096, T=8, hot=5)
    P.check_attn_l2(dev, B=1, H=1, N=16384, T=8, T2=8, hot=3)
    P.check_attn_l1(dev, B=1, H=1, N=32768, T=4, hot=5)          # beyond 16384 tokens a work item holds up to 256 entries: 8 full ones here


def test_attn_special_cases(dev):
    P.check_attn_reduces_to_sdpa(dev, B=1, H=2, N=1024)
    P.check_constant_v(dev)
    P.check_attn_fwd_repeated_block(dev)


@pytest.mark.parametrize("smooth", [False, True])
def test_attn_l2(dev, smooth):
    P.check_attn_l2(dev, B=1, H=2, N=16384, T=16, T2=16, smooth=smooth)


@pytest.mark.parametrize("fused,rope,strided", [(True, False, False), (True, True, True), (False, False, True), (False, True, False)])
def test_op_l1(dev, fused, rope, strided):
    P.check_op_l1(dev, B=2, H=2, N=4096, T=16, fused=fused, rope=rope, strided=strided, smooth=not strided)


@pytest.mark.parametrize("fused,rope", [(True, False), (True, True), (False, True)])
def test_op_l2(dev, fused, rope):
    P.check_op_l2(dev, B=1, H=2, N=16384, T=16, T2=16, fused=fused, rope=rope, smooth=True)


@pytest.mark.parametrize("B,H,N,T", [(1, 1, 1024, 4), (3, 1, 3072, 12), (1, 5, 5120, 16), (2, 3, 2048, 32), (1, 2, 7168, 64),
                                     (1, 7, 1024, 64), (1, 1, 32768, 16)])
def test_op_l1_shapes(dev, B, H, N, T):
    """Token counts that are not powers of two (any multiple of 1024), odd batch and head counts, every
    topk the kernels take (multiples of 4 up to N/16)."""
    P.check_op_l1(dev, B=B, H=H, N=N, T=T, fused=True, rope=False, strided=(B + H) % 2 == 1)


@pytest.mark.parametrize("B,H,N,T,T2", [(1, 1, 16384, 4, 4), (1, 3, 32768, 12, 8), (2, 1, 49152, 16, 12), (1, 2, 16384, 32, 16),
                                        (1, 1, 16384, 64, 32), (3, 2, 16384, 8, 8)])
def test_op_l2_shapes(dev, B, H, N, T, T2):
    """Multiples of 16384 tokens that are not squares, topk1 up to 64 and topk2 up to 32, the largest the
    selection kernels take."""
    P.check_op_l2(dev, B=B, H=H, N=N, T=T, T2=T2, fused=True, rope=False)


@pytest.mark.parametrize("levels", [1, 2])
def test_step_is_deterministic(dev, levels):
    """Every reduction has a fixed order (sorted CSR segments, partial sums added in chunk order, no
    atomics in the floating-point path), so two runs give the same bits -- with hot key blocks, whose
    lists are cut into chunks, and with other work in between."""
    import math
    import llsa_amd
    from llsa_amd.utils.rope_table import rope_table
    B, H, N = 2, 3, 16384
    q, k, v, do = P.smooth_inputs(B, H, N, 64, dev)
    k[:, :, 160:176] *= 3.0                            # a key block that very many query blocks select
    freq = rope_table(math.isqrt(N), dtype=torch.bfloat16).to(dev)
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)

    def step():
        q.grad = k.grad = v.grad = None
        o = llsa_amd.llsa_l2(q, k, v, 16, 16, 16, rope=freq) if levels == 2 else llsa_amd.llsa_l1(q, k, v, 16, 16, rope=freq)
        o.backward(do)
        torch.cuda.synchronize()
        return [t.clone() for t in (o, q.grad, k.grad, v.grad)]

    first = step()
    torch.randn(1 << 22, device=dev).sum().item()      # other kernels and allocations in between
    for name, a, b in zip(("o", "dq", "dk", "dv"), first, step()):
        assert torch.equal(a, b), f"{name} differs between two runs of the same step"


def test_mixed_layouts_and_partial_grads(dev):
    """q in (B,N,H,D) memory, k contiguous, v a slice of a packed projection; the output of a no-grad call
    equals the output of a call that records the backward; gradients arrive in the layout of their
    inputs, and asking for only some of them changes none of the values."""
    import llsa_amd
    B, H, N = 2, 3, 4096
    g = torch.Generator().manual_seed(3)
    q = torch.randn(B, N, H, 64, generator=g).bfloat16().to(dev).transpose(1, 2)
    k = torch.randn(B, H, N, 64, generator=g).bfloat16().to(dev)
    packed = torch.randn(B, N, 2 * H * 64, generator=g).bfloat16().to(dev)
    v = packed[..., H * 64:].reshape(B, N, H, 64).transpose(1, 2)
    do = torch.randn(B, N, H, 64, generator=g).bfloat16().to(dev).transpose(1, 2)
    with torch.no_grad():
        o0 = llsa_amd.llsa_l1(q, k, v, 8, 16)
    qa, ka, va = (t.detach().requires_grad_(True) for t in (q, k, v))
    o1 = llsa_amd.llsa_l1(qa, ka, va, 8, 16)
    assert torch.equal(o0, o1) and o1.stride() == q.stride()
    from llsa_amd.kernel.torch_op._fused import selection
    idx = selection(o1)[0].cpu().long()              # (the node's saved tensors are gone after the backward)
    o1.backward(do)
    assert qa.grad.stride() == q.stride() and ka.grad.is_contiguous()
    qb, kb, vb = q.detach(), k.detach(), v.detach().requires_grad_(True)       # only dV asked for
    llsa_amd.llsa_l1(qb, kb, vb, 8, 16).backward(do)
    assert torch.equal(vb.grad, va.grad)
    # and against the oracle on the same inputs
    from oracle import llsa_oracle as O
    ro, ctx = O.llsa_l1_fwd(q.cpu().contiguous(), k.cpu(), v.cpu().contiguous(), 8, 16, indices=idx)
    rq, rk, rv, _ = O.llsa_l1_bwd(do.cpu().contiguous(), ctx)
    for name, a, b in (("o", o1, ro), ("dq", qa.grad, rq), ("dk", ka.grad, rk), ("dv", va.grad, rv)):
        P.close(name, a, b)


def test_selection_limits_are_errors(dev):
    import llsa_amd
    from llsa_amd._lib import LlsaError
    x = torch.randn(1, 1, 16384, 64).bfloat16().to(dev)
    with pytest.raises(LlsaError, match="T2 <= min"):
        llsa_amd.llsa_l2(x, x, x, 16, 64, 16)
    with pytest.raises(LlsaError, match="T <= min"):
        llsa_amd.llsa_l2(x, x, x, 128, 16, 16)
    with pytest.raises(ValueError, match="multiple of 16384"):
        llsa_amd.llsa_l2(x[:, :, :4096], x[:, :, :4096], x[:, :, :4096], 8, 8, 16)


@pytest.mark.skip(reason="capturing this case (B=1, H=2, N=16384, topk 8/4) ended in a segmentation fault of the host "
                         "process inside torch.cuda.graph's capture_end (hipStreamEndCapture), twice; the cause is not "
                         "known, so the case stays off the GPU and GraphedStep's constructor raises.  The same capture and replay at the bench shapes "
                         "(B=2,H=6,N=16384,16/16 and B=4,H=6,N=4096,16) completed and matched the eager step bit for bit.")
def test_graphed_step_matches_eager(dev):
    """A forward + backward captured in one HIP graph gives, on every replay, bit for bit what the
    same step gives launched kernel by kernel -- with eager work and synchronisations between the
    replays, and after the inputs were changed in place."""
    import math
    import llsa_amd
    from llsa_amd.utils.rope_table import rope_table
    B, H, N = 1, 2, 16384
    q, k, v, do = P.smooth_inputs(B, H, N, 64, dev)
    freq = rope_table(math.isqrt(N), dtype=torch.bfloat16).to(dev)
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    fn = lambda q_, k_, v_: llsa_amd.llsa_l2(q_, k_, v_, 8, 4, 16, rope=freq)

    def eager():
        q.grad = k.grad = v.grad = None
        o = fn(q, k, v)
        o.backward(do)
        torch.cuda.synchronize()
        return [t.clone() for t in (o, q.grad, k.grad, v.grad)]

    ref = eager()
    from llsa_amd.utils.graphed import GraphedStep
    g = GraphedStep(fn, [q, k, v], do)
    for rep in range(3):
        if rep == 2:                                  # new inputs, written into the graph's static buffers
            with torch.no_grad():
                q.copy_(q.flip(2))
                do.mul_(0.5)
            ref = eager()
        out, grads = g.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("o", "dq", "dk", "dv"), [out] + grads, ref):
            assert torch.equal(a, b), f"replay {rep}: {name} differs from the eager step"
        eager()                                       # the program's own eager work between replays


def test_op_l2_largest_topk_and_odd_shapes(dev):
    """The largest top-k the selection kernels take (64 fine blocks: 65536 list entries per (b,h) through the one-launch
    transposes, key blocks with several work items) and a batch x heads that is no power of two with top-k values that
    are none either."""
    P.check_op_l2(dev, B=1, H=1, N=16384, T=64, T2=32, fused=True, rope=True)
    P.check_op_l2(dev, B=3, H=5, N=16384, T=12, T2=20, fused=True, rope=True, smooth=True, slices=[(0, 0), (2, 4)])
    P.check_op_l1(dev, B=2, H=2, N=4096, T=64, fused=True, rope=True)
