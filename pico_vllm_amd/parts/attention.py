"""Grouped-query attention over the paged cache."""
from __future__ import annotations

import dataclasses
import math
from typing import Dict, List, Optional

import torch

from ..ops import kernels
from ..ops.linear import Linear
from .base import DeferredNorm, Mixer, StepContext
from .registry import build_part, register_part
from .spec import CacheSpec, PageTensor, ParamSpec, PartSpec


def kv_page_tensors(num_kv_heads: int, head_dim: int):
    """The layout of a page that this package's attention and store kernels read and write: in ``k`` a token's key
    is contiguous ([kv heads, page, head size]); in ``v`` a head dimension's values of the page's tokens are
    ([kv heads, head size, page]: the matrix-core kernels contract over keys).  The reference keeps V like K
    (pico_vllm/blockmanager.py:39-42)."""
    return (PageTensor("k", (num_kv_heads, "page", head_dim)), PageTensor("v", (num_kv_heads, head_dim, "page")))


@register_part("mixer", "gqa_attention")
class GQAAttention(Mixer):
    """qkv = x Wqkv^T (+ b); position encoding on q, k; k, v into the cache;
    attention of every new token over its request's cache; o = a Wo^T.

    Order and shapes follow pico_vllm/model.py:187-228 (fused qkv with bias
    :148-152, rows [q; k; v] :42-43 of weights.py, o_proj without bias :147).
    Keys and values of the new tokens are written first and attention then
    reads old and new alike from the cache (model.py:216-221), which is what
    makes a prompt cut into portions equal the whole prompt.  A run that was
    given another run's cache (``cache.read_only``) stores nothing and attends
    over what the owner stored in the same step.  The checkpoint
    holds q_proj, k_proj and v_proj separately; they are concatenated at load.
    ``window`` > 0 restricts every query to the last ``window`` keys."""

    takes_deferred_norm = True
    graph_safe_prompts = True       # what the host chooses (the shape of the prefill workgroups) is the graph's variant

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 qkv_bias: bool, position: PartSpec, window: int = 0,
                 act_dtype: torch.dtype = torch.bfloat16):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} kv heads")
        if not 1 <= head_dim <= kernels.MAX_HEAD_DIM:
            raise ValueError(f"head size {head_dim} is outside what the attention kernels take (1 to {kernels.MAX_HEAD_DIM})")
        if window < 0:
            raise ValueError(f"window must not be negative, got {window}")
        self.hidden_size, self.nq, self.nkv, self.d = hidden_size, num_heads, num_kv_heads, head_dim
        self.qkv_bias, self.window, self.act_dtype = qkv_bias, window, act_dtype
        self.scale = 1.0 / math.sqrt(head_dim)          # pico_vllm/kernels/attention.py:92,231
        self.position = build_part("position", position, act_dtype=act_dtype)
        self.qkv: Optional[Linear] = None
        self.o: Optional[Linear] = None
        self.fast = None                                # matrix-core kernels, chosen at load

    def cache_spec(self) -> CacheSpec:
        return CacheSpec("paged_kv", window=self.window, page_tensors=kv_page_tensors(self.nkv, self.d))

    def flops(self, tokens: int, pairs: int) -> float:
        # the projections, and q.k and p.v for every (query, key) pair of every head
        return super().flops(tokens, pairs) + 4.0 * self.nq * self.d * pairs

    def param_specs(self) -> List[ParamSpec]:
        H, nq, nkv, d = self.hidden_size, self.nq, self.nkv, self.d
        out = [ParamSpec("q_proj.weight", (nq * d, H)), ParamSpec("k_proj.weight", (nkv * d, H)),
               ParamSpec("v_proj.weight", (nkv * d, H)), ParamSpec("o_proj.weight", (H, nq * d))]
        if self.qkv_bias:
            out += [ParamSpec("q_proj.bias", (nq * d,), role="bias"), ParamSpec("k_proj.bias", (nkv * d,), role="bias"),
                    ParamSpec("v_proj.bias", (nkv * d,), role="bias")]
        return out + [ParamSpec("position." + p.name, p.shape, p.role, p.std) for p in self.position.param_specs()]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        ws = [tensors[f"{n}_proj.weight"] for n in "qkv"]
        wdt = torch.float32 if any(w.dtype == torch.float32 for w in ws) else ws[0].dtype
        w = torch.cat([t.to(wdt) for t in ws], dim=0).to(device)
        b = None
        if self.qkv_bias:
            b = torch.cat([tensors[f"{n}_proj.bias"].float() for n in "qkv"], dim=0).to(device)
        self.qkv = Linear(w, b)
        self.o = Linear(tensors["o_proj.weight"].to(device))
        self.position.load({k[len("position."):]: v for k, v in tensors.items() if k.startswith("position.")},
                           device, dtype)
        if self.act_dtype == torch.bfloat16:
            from ..ops import attention_fast
            self.fast = attention_fast.choose(self.nq, self.nkv, self.d, self.window)

    def graph_variant(self, ctx: StepContext) -> tuple:
        own = (("gqa_attention",) + self.fast.plan(ctx),) if self.fast is not None and not ctx.all_decode else ()
        return own + super().graph_variant(ctx)

    def forward(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        nq, nkv, d = self.nq, self.nkv, self.d
        bt = ctx.block_tables[cache.group]
        if isinstance(x, DeferredNorm) and not getattr(self.position, "takes_deferred_norm", False):
            x = x.run()
        if getattr(cache, "read_only", False):
            # another run's keys and values: this run encodes its queries and attends over them; every token's slot
            # reads as "none", which the stores of all position encodings honour
            if "no_slots" not in ctx.shared:
                ctx.shared["no_slots"] = torch.full_like(ctx.slot_mapping[cache.group], -1)
            ctx = dataclasses.replace(ctx, slot_mapping=[ctx.shared["no_slots"]] * len(ctx.slot_mapping))
        # [T, >= nq d]: the encoded queries first; keys and values are in the cache after this
        qkv = self.position.project_rotate_store(x, self.qkv, ctx, cache, bt, nq, nkv, d)
        if self.fast is not None and cache.k.dtype == torch.bfloat16:
            a = self.fast(qkv, cache, bt, ctx, self.scale)
        else:
            a = kernels.paged_attention_ref(qkv, cache.k, cache.v, bt, ctx.positions, ctx.token_seq,
                                            nq, nkv, d, self.scale, self.window)
        return self.o.partial(a)
