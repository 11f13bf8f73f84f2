"""llsa_amd -- log-linear sparse attention (llsa_l1 / llsa_l2) on AMD MI355X.

Hand-written HIP kernels for gfx950 behind the operator API of SingleZombie/LLSA.  Importing
this package loads llsa_amd/lib/libllsa_hip.so lazily on first use and fails loudly if it has
not been built (python -m llsa_amd.build)."""
from .kernel.hip.mean_pool import mean_pool1d
from .kernel.hip.permute import gather_tokens, permute_tokens
from .kernel.hip.rms_norm import my_rms_norm_fn
from .kernel.hip.rope import my_rope_fn
from .kernel.torch_op.flash_sparse_attention_res_1 import (flash_sparse_residual_attention_l1_op, llsa_l1,
                                                           llsa_l1_unfused)
from .kernel.torch_op.flash_sparse_attention_res_2 import (flash_sparse_residual_attention_l2_op, llsa_l2,
                                                           llsa_l2_unfused, llsa_l3, llsa_lk)

__all__ = ["llsa_l1", "llsa_l2", "llsa_l3", "llsa_lk", "llsa_l1_unfused", "llsa_l2_unfused", "flash_sparse_residual_attention_l1_op",
           "flash_sparse_residual_attention_l2_op", "mean_pool1d", "my_rope_fn", "my_rms_norm_fn", "permute_tokens",
           "gather_tokens"]
