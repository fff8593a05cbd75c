"""Rotate-half rotary position encoding."""
from __future__ import annotations

import torch

from ..ops import kernels
from .base import DeferredNorm, PositionEncoding
from .registry import register_part


@register_part("position", "rotary_half")
class RotaryHalf(PositionEncoding):
    """Pairs (j, j + rotary_dim/2) are rotated by position * theta^(-2j/rotary_dim)
    (pico_vllm/model.py:80-86,116-123).  Angles, cosines and sines are float32
    and are computed inside the kernel from the position, so there is no table
    whose length bounds the sequence (the reference keeps a [131072, d] table)."""

    graph_safe_prompts = True

    def __init__(self, rotary_dim: int, theta: float, act_dtype: torch.dtype = torch.bfloat16):
        if rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even, got {rotary_dim}")
        self.rotary_dim, self.theta = rotary_dim, theta
        self.inv_freq = None

    def load(self, tensors, device, dtype) -> None:
        d = self.rotary_dim
        # same float32 arithmetic as pico_vllm/model.py:80-82
        inv = 1.0 / (self.theta ** (torch.arange(0, d, 2).float() / d))
        self.inv_freq = inv.to(device).contiguous()

    def table(self, ctx) -> torch.Tensor:
        """cos and sin of every token's angles, [T, rotary_dim / 2, 2]; the first layer of a step
        that asks computes them, the others find them in ``ctx.shared``."""
        key = ("rotary_half", self.rotary_dim, self.theta)
        if key not in ctx.shared:
            ctx.shared[key] = kernels.rope_table(ctx.positions[:ctx.num_tokens], self.inv_freq)
        return ctx.shared[key]

    def rotate_and_store(self, qkv, ctx, kv, block_table, nq, nkv, d) -> None:
        kernels.rope_kv_store(qkv, self.table(ctx), ctx.slot_mapping[kv.group], kv.k, kv.v, nq, nkv, d, self.rotary_dim)

    takes_deferred_norm = True

    def project_rotate_store(self, x, linear, ctx, kv, block_table, nq, nkv, d) -> torch.Tensor:
        fusable = (self.rotary_dim == d and d % 32 == 0 and kv.k.dtype == torch.bfloat16
                   and kv.k.shape[2] & (kv.k.shape[2] - 1) == 0)
        if isinstance(x, DeferredNorm):
            # one token: the norm in front rides on the same kernel
            if fusable and x.kind == "rms" and kernels.skinny_norm_ok(x.resid_in, x.delta, linear.weight):
                q, x.resid = kernels.gemm_skinny_rope_norm(x.resid_in, x.delta, x.weight, x.eps, linear.weight, linear.bias_f32,
                                                           self.table(ctx), ctx.slot_mapping[kv.group], kv.k, kv.v, nq, nkv, d)
                return q
            x = x.run()
        # few tokens in bfloat16: projection, bias, rotation and cache store are one weight-streaming kernel
        if fusable and kernels.skinny_ok(x, linear.weight):
            return kernels.gemm_skinny_rope(x, linear.weight, linear.bias_f32, self.table(ctx), ctx.slot_mapping[kv.group],
                                            kv.k, kv.v, nq, nkv, d)
        return super().project_rotate_store(x, linear, ctx, kv, block_table, nq, nkv, d)


@register_part("position", "none")
class NoPosition(PositionEncoding):
    """No position encoding: keys and values are stored as they are."""
    graph_safe_prompts = True

    def __init__(self, act_dtype: torch.dtype = torch.bfloat16):
        pass

    def rotate_and_store(self, qkv, ctx, kv, block_table, nq, nkv, d) -> None:
        kernels.rope_kv_store(qkv, None, ctx.slot_mapping[kv.group], kv.k, kv.v, nq, nkv, d, 0)
