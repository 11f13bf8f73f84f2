"""llsa_rmsnorm_bwd_static, the entry point that allocates nothing (its partial sums live in a static device
array inside the library), against llsa_rmsnorm_bwd with a caller-owned buffer: same kernels, same order of
additions, so the results must be bit-identical.  Two calls in a row share the static array, the second with a
smaller input that leaves stale rows of the first behind it."""
import ctypes as C

import pytest
import torch


def _call(lib, static, dy, x, gamma, eps, stream):
    B, H, N, _ = x.shape
    s3 = lambda t: (C.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2))
    dx = torch.empty_like(dy)
    dg = torch.empty(64, device=x.device, dtype=torch.float32)
    if static:
        rc = lib.rmsnorm_bwd_static(dy.data_ptr(), s3(dy), x.data_ptr(), s3(x), gamma.data_ptr(), eps, dx.data_ptr(), s3(dx),
                                    dg.data_ptr(), B, H, N, stream)
    else:
        part = torch.empty(lib.rmsnorm_bwd_partials(B, H, N), device=x.device, dtype=torch.float32)
        rc = lib.rmsnorm_bwd(dy.data_ptr(), s3(dy), x.data_ptr(), s3(x), gamma.data_ptr(), eps, dx.data_ptr(), s3(dx),
                             dg.data_ptr(), part.data_ptr(), B, H, N, stream)
    lib.check(rc, "rmsnorm_bwd")
    return dx, dg


def _two_calls_in_a_row(lib, dev, shapes, stream_of):
    gen = torch.Generator().manual_seed(77)
    gamma = (1.0 + 0.1 * torch.randn(64, generator=gen)).to(dev)
    for B, H, N in shapes:
        x = torch.randn(B, H, N, 64, generator=gen).to(torch.bfloat16).to(dev)
        dy = torch.randn(B, H, N, 64, generator=gen).to(torch.bfloat16).to(dev)
        stream = stream_of(x)
        dx_s, dg_s = _call(lib, True, dy, x, gamma, 1e-5, stream)
        dx_r, dg_r = _call(lib, False, dy, x, gamma, 1e-5, stream)
        assert torch.equal(dx_s.cpu(), dx_r.cpu()), f"dx differs at {(B, H, N)}"
        assert torch.equal(dg_s.cpu(), dg_r.cpu()), f"dgamma differs at {(B, H, N)}"
        assert torch.isfinite(dg_s).all()


@pytest.mark.gpu
def test_static_scratch_matches_caller_buffer_on_two_calls():
    from llsa_amd._lib import get_lib
    from llsa_amd.kernel.hip._common import stream_of
    lib = get_lib()
    dev = torch.device("cuda:0")
    # 4 * 6 * 64 = 1536 rows of partial sums (two folding launches), then 2 * 3 * 2 = 12 rows (one)
    _two_calls_in_a_row(lib, dev, [(4, 6, 16384), (2, 3, 512)], lambda t: stream_of(lib, t))
    torch.cuda.synchronize()


@pytest.mark.gpu
def test_static_scratch_rejects_sizes_beyond_its_limit():
    from llsa_amd._lib import STATIC_PARTIALS_MAX, get_lib
    lib = get_lib()
    n = 256 * (STATIC_PARTIALS_MAX // 64 + 1)          # one row of partial sums too many
    s = (C.c_int64 * 3)(8, 8, 8)
    assert lib.rmsnorm_bwd_static(16, s, 16, s, 16, 1e-5, 16, s, 16, 1, 1, n, None) != 0
    assert b"exceed the static scratch" in lib.last_error_string()


def test_static_scratch_in_the_cpu_build_of_the_kernels():
    """The same two calls through the x86 build of the sources (host logic: limit, per-device pointer, launches)."""
    from emu_util import emu_lib
    lib = emu_lib()
    _two_calls_in_a_row(lib, torch.device("cpu"), [(1, 33, 2048), (1, 2, 64)], lambda t: None)
    from llsa_amd._lib import STATIC_PARTIALS_MAX
    s = (C.c_int64 * 3)(8, 8, 8)
    assert lib.rmsnorm_bwd_static(16, s, 16, s, 16, 1e-5, 16, s, 16, 1, 1, 256 * (STATIC_PARTIALS_MAX // 64 + 1), None) != 0
    assert b"exceed the static scratch" in lib.last_error_string()
