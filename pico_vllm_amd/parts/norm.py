"""RMSNorm with the residual sum fused in front of it."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels
from .base import DeferredNorm, Norm
from .registry import register_part
from .spec import ParamSpec


@register_part("norm", "rms_norm")
class RMSNorm(Norm):
    """y = x / sqrt(mean(x^2) + eps) * weight, in float32 (pico_vllm/RMSNorm.py:22-31)."""
    graph_safe_prompts = True

    def __init__(self, size: int, eps: float, act_dtype: torch.dtype = torch.bfloat16):
        self.size, self.eps, self.act_dtype = size, eps, act_dtype
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> List[ParamSpec]:
        return [ParamSpec("weight", (self.size,), role="norm")]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        self.weight = tensors["weight"].to(device=device, dtype=torch.float32).contiguous()

    def add_norm(self, resid, delta, rows=None):
        return kernels.add_rmsnorm(resid, delta, self.weight, self.eps, self.act_dtype, rows)

    def deferred(self, resid, delta):
        # the one row of a bfloat16 step: the projection behind the norm can norm it itself
        if (self.act_dtype == torch.bfloat16 and resid.shape[0] <= kernels.SKINNY_NORM_ROWS
                and (delta is None or delta.dtype == torch.float32)):
            return DeferredNorm(self, resid, delta, "rms", self.weight, self.eps)
        return None
