"""The dense SwiGLU feed-forward."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops.linear import Linear
from .base import FeedForward, StepContext
from .registry import register_part
from .spec import ParamSpec


@register_part("feed_forward", "swiglu_mlp")
class SwiGLUMLP(FeedForward):
    """down( silu(gate) * up ), [gate; up] = x Wgu^T, no biases
    (pico_vllm/model.py:309-318; gate rows first, weights.py:58).  The
    checkpoint holds gate_proj and up_proj separately; they are concatenated
    at load so one GEMM makes both."""

    takes_deferred_norm = True      # Linear.swiglu runs or fuses it
    graph_safe_prompts = True

    def __init__(self, hidden_size: int, intermediate_size: int, act_dtype: torch.dtype = torch.bfloat16):
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.gate_up: Optional[Linear] = None
        self.down: Optional[Linear] = None

    def param_specs(self) -> List[ParamSpec]:
        H, I = self.hidden_size, self.intermediate_size
        return [ParamSpec("gate_proj.weight", (I, H)), ParamSpec("up_proj.weight", (I, H)),
                ParamSpec("down_proj.weight", (H, I))]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        g, u = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        wdt = torch.float32 if torch.float32 in (g.dtype, u.dtype) else g.dtype
        self.gate_up = Linear(torch.cat([g.to(wdt), u.to(wdt)], dim=0).to(device))
        self.down = Linear(tensors["down_proj.weight"].to(device))

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        return self.down.partial(self.gate_up.swiglu(x))
