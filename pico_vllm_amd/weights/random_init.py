"""Random-weights mode: write a model folder (config.json, model.safetensors)
from a configuration and a seed.

Distributions: matrices and biases N(0, 0.02), norm weights 1 + U(-0.1, 0.1),
integer tables zero.  Each tensor has its own generator seeded from (seed,
tensor name), so the file does not depend on the order of tensors.  Floating
tensors are stored in bfloat16, norm weights in float32.  The reference has no
such mode; it always loads the released weights (pico_vllm/run_single.py:12).
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Dict, Optional

import torch

from ..config.registry import resolve_architecture
from ..parts.spec import ParamSpec
from .safetensors_io import write_safetensors


def _generator(seed: int, name: str) -> torch.Generator:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    g = torch.Generator(device="cpu")
    g.manual_seed(int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF)
    return g


def stored_dtype(spec: ParamSpec) -> torch.dtype:
    return {"norm": torch.float32, "table": torch.int32}.get(spec.role, torch.bfloat16)


def random_tensor(spec: ParamSpec, seed: int, std: Optional[float] = None) -> torch.Tensor:
    g = _generator(seed, spec.name)
    std = spec.std if std is None else std
    if spec.role == "table":
        return torch.zeros(spec.shape, dtype=torch.int32)
    if spec.role == "norm":
        return 1.0 + (torch.rand(spec.shape, generator=g, dtype=torch.float32) * 0.2 - 0.1)
    return (torch.randn(spec.shape, generator=g, dtype=torch.float32) * std).to(torch.bfloat16)


def write_random_model(model_dir: str, config: Dict[str, Any], seed: int = 0,
                       std_overrides: Optional[Dict[str, float]] = None) -> str:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` (a dict
    with the architecture's config.json keys, ``architectures`` included).
    ``std_overrides`` maps a substring of tensor names to another standard
    deviation (tests use it to make attention scores spread out)."""
    from ..parts.model import model_param_specs
    arch = resolve_architecture(config)
    cfg = arch.config_from_dict(config)
    spec = arch.build_spec(cfg)
    params = model_param_specs(spec)
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w") as f:
        json.dump(config, f, indent=1, sort_keys=True)
    by_name = {p.name: p for p in params}

    def _std_for(name: str) -> Optional[float]:
        for sub, std in (std_overrides or {}).items():
            if sub in name:
                return std
        return None
    write_safetensors(
        os.path.join(model_dir, "model.safetensors"),
        [(p.name, tuple(p.shape), stored_dtype(p)) for p in params],
        lambda name: random_tensor(by_name[name], seed, _std_for(name)),
        metadata={"format": "pt", "seed": str(seed)})
    return model_dir
