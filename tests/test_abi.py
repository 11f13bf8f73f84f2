"""The C-ABI library builds, loads, and exports every function include/llsa_hip.h declares; argument checks of the
entry points reject bad input before any kernel is launched (no GPU needed: a rejected call launches nothing)."""
import ctypes as C
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "llsa_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(llsa_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from llsa_amd._lib import LIB_PATH, Lib
    if not os.path.exists(LIB_PATH):
        from llsa_amd import build
        build.build(verbose=False)
    return Lib(LIB_PATH)


def test_header_and_binding_agree(lib):
    from llsa_amd._lib import EXPORTS
    names = declared_functions()
    assert len(names) >= 14
    assert sorted(EXPORTS) == names, "llsa_amd/_lib.py and include/llsa_hip.h must list the same functions"
    for n in names:
        assert hasattr(lib.cdll, n), f"library does not export {n}"
    assert lib.version() >= 100


def test_struct_sizes_match_header():
    """ctypes mirrors of the argument structs must have the size the compiler gives them."""
    import subprocess, tempfile
    from llsa_amd._lib import AttnBwdArgs, AttnFwdArgs, PoolItem
    src = '#include "llsa_hip.h"\n#include <stdio.h>\nint main(){printf("%zu %zu %zu\\n", sizeof(llsa_pool_item), sizeof(llsa_attn_fwd_args), sizeof(llsa_attn_bwd_args));return 0;}\n'
    with tempfile.TemporaryDirectory() as d:
        open(os.path.join(d, "s.c"), "w").write(src)
        subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), os.path.join(d, "s.c"), "-o", os.path.join(d, "s")])
        out = subprocess.check_output([os.path.join(d, "s")]).decode().split()
    assert [int(x) for x in out] == [C.sizeof(PoolItem), C.sizeof(AttnFwdArgs), C.sizeof(AttnBwdArgs)]


def test_entry_points_reject_bad_arguments(lib):
    from llsa_amd._lib import AttnFwdArgs, PoolItem
    assert lib.pool_pyramid_fwd(None, 0, None, 1, 1, None) != 0
    assert b"items" in lib.last_error_string()
    it = PoolItem()
    it.x, it.n = 16, 24                      # n not a multiple of 16
    assert lib.pool_pyramid_fwd(C.byref(it), 1, None, 1, 1, None) != 0
    assert b"multiple of 16" in lib.last_error_string()
    assert lib.topk_dense(16, 16, 16, 1, 1, 64, 128, 1, None) != 0          # T > n
    a = AttnFwdArgs()
    a.levels, a.B, a.H, a.N, a.T = 1, 1, 1, 1000, 8
    a.qr = a.kr = a.vt = a.idx = a.o = a.lse = 16
    a.lvl[0].kr = a.lvl[0].vt = 16
    a.lvl[0].w = 16.0
    assert lib.attn_fwd(C.byref(a), None) != 0
    assert b"1024" in lib.last_error_string()
    a.N, a.T = 1024, 6
    assert lib.attn_fwd(C.byref(a), None) != 0
    assert b"multiple of 4" in lib.last_error_string()
    a.levels, a.N, a.T = 4, 262144, 8                   # four levels need N % 4194304 == 0
    assert lib.attn_fwd(C.byref(a), None) != 0
    assert b"4194304" in lib.last_error_string()
    a.levels = 5
    assert lib.attn_fwd(C.byref(a), None) != 0
    topk = lambda *t: (C.c_int32 * len(t))(*t)
    assert lib.attn_bwd_workspace_bytes(2, 6, 16384, topk(16, 16), 2) > 0
    assert lib.attn_bwd_workspace_bytes(1, 1, 262144, topk(16, 16, 16), 3) > lib.attn_bwd_workspace_bytes(1, 1, 262144, topk(16, 16), 2) > 0
    assert lib.attn_bwd_workspace_bytes(2, 6, 16384, topk(16, 16, 16, 16, 16), 5) < 0
    # a token count the coarsest level cannot tile is an error, not a division by zero in the work split
    assert lib.attn_bwd_workspace_bytes(1, 1, 512, topk(8), 1) < 0
    assert lib.attn_bwd_workspace_bytes(1, 1, 4096, topk(8, 8), 2) < 0
    assert lib.attn_bwd_workspace_bytes(1, 1, 1024, topk(8), 1) > 0
    a.levels, a.N, a.T = 3, 262144, 8                   # forward and backward share the limit on the pooled levels' topk
    for l in range(3):
        a.lvl[l].kr = a.lvl[l].vt = a.lvl[l].sel = 16
        a.lvl[l].w = 16.0
    a.lvl[0].T = a.lvl[1].T = 32
    assert lib.attn_fwd(C.byref(a), None) != 0
    assert b"must not exceed 56" in lib.last_error_string()
    assert lib.work_list_len(1024, 1024, 16, 32) == 4 + 4 * (512 + 1024) + 4 * 513 + 1024
    assert lib.fine_chunk(16384) == 64 and lib.fine_chunk(65536) == 256 and lib.fine_chunk(262144) <= 256      # <= LLSA_CHUNK_FINE_MAX


def test_python_layer_rejects_unsupported_inputs():
    from llsa_amd._lib import override_library_for_tests
    from llsa_amd.kernel.hip._attention import attn_fwd
    from emu_util import emu_lib
    with override_library_for_tests(emu_lib()):
        q = torch.zeros(1, 1, 1024, 64, dtype=torch.bfloat16)
        pk = torch.zeros(1, 1, 64, 64, dtype=torch.bfloat16)
        idx = torch.zeros(1, 1, 64, 4, dtype=torch.int32)
        with pytest.raises(NotImplementedError, match="bf16"):
            attn_fwd(q.float(), q.float(), q.float(), pk.float(), pk.float(), idx, 16.0)
        with pytest.raises(NotImplementedError, match="head dim"):
            attn_fwd(q[..., :32], q[..., :32], q[..., :32], pk[..., :32], pk[..., :32], idx, 16.0)
        with pytest.raises(ValueError, match="multiple of 1024"):
            attn_fwd(q[:, :, :512], q[:, :, :512], q[:, :, :512], pk[:, :, :32], pk[:, :, :32], idx[:, :, :32], 16.0)
        with pytest.raises(ValueError, match="same shape"):
            attn_fwd(q, q[:, :, :512], q, pk, pk, idx, 16.0)


def test_utils_match_oracle():
    from llsa_amd.utils import rope_table as R, zorder as Z
    from oracle import llsa_oracle as O
    for side in (2, 8, 64):
        p, ip = Z.zorder_perm(side)
        op, oip = O.zorder_perm(side)
        assert torch.equal(p, op) and torch.equal(ip, oip)
    assert torch.equal(Z.gen_permutations(2)[0], O.zorder_perm(8)[0])
    x = torch.arange(64)[None, :, None].float()
    assert torch.equal(Z.from_zorder(Z.to_zorder(x, 8), 8), x)
    for dt in (torch.float64, torch.bfloat16):
        assert torch.equal(R.rope_table(16, dtype=dt), O.rope_table(16, dtype=dt))
