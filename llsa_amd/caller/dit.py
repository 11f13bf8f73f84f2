"""The caller of llsa_l2 in the reference, restated small: a pixel-space DiT with adaLN-zero blocks
(models/rope_dit_transformer_2d.py: block :295-337 and :581-711, model :827-828, :891-897,
:940-1049, attention call site :180-260) and one flow-matching training step
(trainers/dit_trainer.py:243-315, schedulers/flow_training_scheduler.py:540-565,
trainers/ddpm_trainer.py:97-103).  Plain torch modules around this package's operators: the
attention, the qk RMS norms, the RoPE rotation and the Z-order permutation run in the HIP kernels,
everything else (linear layers, layer norms, GELU, AdamW) is torch's.

The reference builds its model from diffusers classes, which are neither part of its checkout nor
installed here; the layer shapes below follow the arguments it passes to them (biases on q/k/v and
on the output projection, `gelu-approximate` MLP of 4x width, layer norms without weights, eps 1e-5
in the block and 1e-6 in the adaLN norms, 256 sinusoidal timestep channels with cos first).  It is
a workload for timing the operator inside a training step, not a weight-compatible model.
"""
from __future__ import annotations

import math
from typing import Sequence, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..kernel.hip.permute import permute_tokens
from ..kernel.hip.rms_norm import my_rms_norm_fn
from ..kernel.hip.rope import my_rope_fn
from ..kernel.torch_op.flash_sparse_attention_res_1 import llsa_l1
from ..kernel.torch_op.flash_sparse_attention_res_2 import llsa_l2, llsa_l3
from ..utils.rope_table import rope_table
from ..utils.zorder import zorder_perm


def timestep_channels(t: torch.Tensor, channels: int = 256, max_period: float = 10000.0) -> torch.Tensor:
    """Sinusoidal embedding of the timesteps as the model's `Timesteps(256, flip_sin_to_cos=True,
    downscale_freq_shift=1)` makes it (:267-268): frequencies max_period^(-i/(half-1)), cosines
    first."""
    half = channels // 2
    freqs = torch.exp(-math.log(max_period) * torch.arange(half, dtype=torch.float32, device=t.device) / (half - 1))
    ang = t.float()[:, None] * freqs[None]
    return torch.cat([ang.cos(), ang.sin()], dim=-1)


class TimestepEmbedding(nn.Module):
    def __init__(self, dim: int):
        super().__init__()
        self.linear_1 = nn.Linear(256, dim)
        self.linear_2 = nn.Linear(dim, dim)

    def forward(self, t: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
        return self.linear_2(F.silu(self.linear_1(timestep_channels(t).to(dtype))))


class AdaLayerNormZero(nn.Module):
    """:295-337: six modulation vectors from the timestep embedding; returns the modulated
    normalised tokens and the other four vectors."""

    def __init__(self, dim: int):
        super().__init__()
        self.emb = TimestepEmbedding(dim)
        self.linear = nn.Linear(dim, 6 * dim)
        self.norm = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)

    def forward(self, x, t):
        shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = self.linear(F.silu(self.emb(t, x.dtype))).chunk(6, dim=1)
        return self.norm(x) * (1 + scale_msa[:, None]) + shift_msa[:, None], gate_msa, shift_mlp, scale_mlp, gate_mlp


class LlsaSelfAttention(nn.Module):
    """The attention module with RopeAttnProcessor (:180-260).  q, k, v stay in the (B, N, H, D)
    memory of their linear layers (the kernels read the transposed views in place), and the output
    comes back in that layout, so the output projection reads it without a copy.

    fused_prologue=True hands the RMS-norm weights and the RoPE table to the operator, which
    normalises and rotates inside its pooling pass; False composes my_rms_norm_fn, my_rope_fn and
    the operator as the reference does."""

    def __init__(self, dim: int, heads: int, head_dim: int, levels: int = 2, sparse_topk: Tuple[int, int] = (16, 16),
                 block_size: int = 16, qk_norm: bool = True, eps: float = 1e-5, fused_prologue: bool = True):
        super().__init__()
        inner = heads * head_dim
        self.heads, self.head_dim, self.levels = heads, head_dim, levels
        self.sparse_topk, self.block_size, self.eps, self.fused_prologue = tuple(sparse_topk), block_size, eps, fused_prologue
        self.to_q, self.to_k, self.to_v = nn.Linear(dim, inner), nn.Linear(dim, inner), nn.Linear(dim, inner)
        self.to_out = nn.Linear(inner, dim)
        if qk_norm:
            self.norm_q_weight = nn.Parameter(torch.ones(head_dim))
            self.norm_k_weight = nn.Parameter(torch.ones(head_dim))
        else:
            self.norm_q_weight = self.norm_k_weight = None

    def forward(self, x: torch.Tensor, freq: torch.Tensor) -> torch.Tensor:
        B, N, _ = x.shape
        split = lambda y: y.view(B, N, self.heads, self.head_dim).transpose(1, 2)
        q, k, v = split(self.to_q(x)), split(self.to_k(x)), split(self.to_v(x))
        norm = None
        if self.norm_q_weight is not None:
            norm = (self.norm_q_weight.float(), self.norm_k_weight.float(), self.eps)
        rope = freq
        if not self.fused_prologue:
            if norm is not None:
                q, k = my_rms_norm_fn(q, norm[0], self.eps), my_rms_norm_fn(k, norm[1], self.eps)
            q, k = my_rope_fn(q, freq), my_rope_fn(k, freq)
            norm = rope = None
        tk = self.sparse_topk                                   # coarsest level first, fine blocks last
        if self.levels == 1:
            o = llsa_l1(q, k, v, tk[-1], self.block_size, rope=rope, qk_norm=norm)
        elif self.levels == 2:      # the reference passes (sparse_topk[1], sparse_topk[0]) as (topk1, topk2), :249-250
            o = llsa_l2(q, k, v, tk[-1], tk[-2], self.block_size, rope=rope, qk_norm=norm)
        else:                       # three levels: no counterpart in the reference
            o = llsa_l3(q, k, v, tk[-1], tk[-2], tk[-3], self.block_size, rope=rope, qk_norm=norm)
        return self.to_out(o.transpose(1, 2).reshape(B, N, self.heads * self.head_dim))


class RopeTransformerBlock(nn.Module):
    """:581-711 with norm_type 'ada_norm_zero' and no cross attention."""

    def __init__(self, dim: int, heads: int, head_dim: int, **attn):
        super().__init__()
        self.norm1 = AdaLayerNormZero(dim)
        self.attn1 = LlsaSelfAttention(dim, heads, head_dim, **attn)
        self.norm3 = nn.LayerNorm(dim, eps=1e-5, elementwise_affine=False)
        self.ff_in, self.ff_out = nn.Linear(dim, 4 * dim), nn.Linear(4 * dim, dim)

    def forward(self, x, t, freq):
        h, gate_msa, shift_mlp, scale_mlp, gate_mlp = self.norm1(x, t)
        x = gate_msa.unsqueeze(1) * self.attn1(h, freq) + x
        h = self.norm3(x) * (1 + scale_mlp[:, None]) + shift_mlp[:, None]
        return gate_mlp.unsqueeze(1) * self.ff_out(F.gelu(self.ff_in(h), approximate="tanh")) + x


class PixelDiT(nn.Module):
    """RopeDiTTransformer2DModel (:735-1058) at patch size 1 with token_permutation.  The defaults
    are configs/models/model_rope_dit_S_128_rms_llsa_l2.json (that file's sparse_topk is 8; the
    benchmark configuration uses 16)."""

    def __init__(self, num_attention_heads: int = 6, attention_head_dim: int = 64, num_layers: int = 12, in_channels: int = 3,
                 out_channels: int = 3, sample_size: int = 128, axes_dims_rope: Sequence[int] = (32, 32), levels: int = 2,
                 sparse_topk=16, qk_norm: bool = True, fused_prologue: bool = True):
        super().__init__()
        dim = num_attention_heads * attention_head_dim
        if isinstance(sparse_topk, int):
            sparse_topk = (sparse_topk,) * max(levels, 2)
        self.sample_size, self.out_channels = sample_size, out_channels
        self.proj_in = nn.Conv2d(in_channels, dim, kernel_size=1)
        self.transformer_blocks = nn.ModuleList(
            RopeTransformerBlock(dim, num_attention_heads, attention_head_dim, levels=levels, sparse_topk=sparse_topk,
                                 qk_norm=qk_norm, fused_prologue=fused_prologue) for _ in range(num_layers))
        self.norm_out = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
        self.proj_out_1 = nn.Linear(dim, 2 * dim)
        self.proj_out_2 = nn.Linear(dim, out_channels)
        perm, inv = zorder_perm(sample_size)
        self.register_buffer("bwd_perm", perm.to(torch.int32), persistent=False)     # Z-order -> raster
        self.register_buffer("fwd_perm", inv.to(torch.int32), persistent=False)      # raster -> Z-order
        # the table is kept in Z-order and in bf16, as register_rope_emb builds it (:153-173)
        self.register_buffer("freq", rope_table(sample_size, tuple(axes_dims_rope), dtype=torch.bfloat16), persistent=False)

    def forward(self, images: torch.Tensor, timestep: torch.Tensor) -> torch.Tensor:
        B, _, Hh, Ww = images.shape
        if Hh != self.sample_size or Ww != self.sample_size:
            raise ValueError(f"this model is built for {self.sample_size} x {self.sample_size} images")
        x = self.proj_in(images).reshape(B, -1, Hh * Ww).transpose(1, 2)                 # :942-945
        x = permute_tokens(x, self.fwd_perm, self.bwd_perm)                              # :963-965
        for block in self.transformer_blocks:
            x = block(x, timestep, self.freq)
        x = permute_tokens(x, self.bwd_perm, self.fwd_perm)                              # :1028-1030
        cond = self.transformer_blocks[0].norm1.emb(timestep, x.dtype)                   # :1033-1034
        shift, scale = self.proj_out_1(F.silu(cond)).chunk(2, dim=1)
        x = self.proj_out_2(self.norm_out(x) * (1 + scale[:, None]) + shift[:, None])
        return x.reshape(B, Hh, Ww, self.out_channels).permute(0, 3, 1, 2)               # :1039-1049 at patch size 1


class FlowMatchingStep:
    """One optimisation step of the trainer with is_flow_matching and v-prediction
    (dit_trainer.py:243-315, 346-349): noisy = (1 - sigma) x + sigma noise with sigma = t / 1000,
    target = noise - x, mean squared error in fp32, gradient norm clipped to 1, AdamW with the
    trainer's defaults (ddpm_trainer.py:39-43, 97-103), the model under bf16 autocast."""

    def __init__(self, model: nn.Module, lr: float = 1e-4, betas=(0.9, 0.999), weight_decay: float = 1e-2, eps: float = 1e-8,
                 num_train_timesteps: int = 1000, clip: float = 1.0):
        self.model, self.T, self.clip = model, num_train_timesteps, clip
        self.optimizer = torch.optim.AdamW(model.parameters(), lr=lr, betas=betas, weight_decay=weight_decay, eps=eps)

    def loss(self, images, noise, timesteps):
        sigma = (timesteps.float() / self.T)[:, None, None, None]
        noisy = (1.0 - sigma) * images + sigma * noise
        with torch.autocast(device_type=images.device.type, dtype=torch.bfloat16):
            out = self.model(noisy, timesteps)
        return F.mse_loss(out.float(), (noise - images).float())

    def __call__(self, images, noise, timesteps) -> torch.Tensor:
        loss = self.loss(images, noise, timesteps)
        loss.backward()
        if self.clip:
            torch.nn.utils.clip_grad_norm_(self.model.parameters(), self.clip)
        self.optimizer.step()
        self.optimizer.zero_grad(set_to_none=True)
        return loss.detach()
