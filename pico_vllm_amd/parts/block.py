"""Arrangements of parts into a layer."""
from __future__ import annotations

from .base import Block, DeferredNorm
from .registry import register_part


@register_part("block", "prenorm")
class PreNormBlock(Block):
    """x += mixer(norm1(x)); x += ff(norm2(x))   (pico_vllm/model.py:361-374).

    Each residual sum is fused into the norm that follows it: the block hands
    its last delta on as ``pending`` and the next block's (or the model's
    final) norm adds it.  The sums are float32."""
    slot_categories = {"norm1": "norm", "mixer": "mixer", "norm2": "norm", "ff": "feed_forward"}
    graph_safe_prompts = True

    @staticmethod
    def _normed(norm, consumer, resid, delta):
        """The normed activations for ``consumer``, or the norm left to it where both sides can."""
        if getattr(consumer, "takes_deferred_norm", False):
            later = norm.deferred(resid, delta)
            if later is not None:
                return later
        return norm.add_norm(resid, delta)

    @staticmethod
    def _after(h, resid):
        if isinstance(h, DeferredNorm):
            if h.resid is None:
                raise RuntimeError("a part took a deferred norm and neither ran nor fused it")
            return h.resid
        return resid

    def forward(self, resid, pending, ctx, cache):
        p = self.parts
        h = self._normed(p["norm1"], p["mixer"], resid, pending)
        a = p["mixer"].forward(h, ctx, cache)
        resid = self._after(h, resid)
        h = self._normed(p["norm2"], p["ff"], resid, a)
        f = p["ff"].forward(h, ctx)
        return self._after(h, resid), f
