"""Arrangements of parts into a layer."""
from __future__ import annotations

from .base import Block
from .registry import register_part


@register_part("block", "prenorm")
class PreNormBlock(Block):
    """x += mixer(norm1(x)); x += ff(norm2(x))   (pico_vllm/model.py:361-374).

    Each residual sum is fused into the norm that follows it: the block hands
    its last delta on as ``pending`` and the next block's (or the model's
    final) norm adds it.  The sums are float32."""
    slot_categories = {"norm1": "norm", "mixer": "mixer", "norm2": "norm", "ff": "feed_forward"}

    def forward(self, resid, pending, ctx, cache):
        p = self.parts
        h = p["norm1"].add_norm(resid, pending)
        a = p["mixer"].forward(h, ctx, cache)
        h = p["norm2"].add_norm(resid, a)
        return resid, p["ff"].forward(h, ctx)
