"""Typed configuration of the Qwen2 dense decoder, read from config.json.

The field names are the keys of the architecture's own config.json; they are
also the field names of the reference's dataclass (pico_vllm/model.py:16-26),
which hard-codes the 1.5B values and never reads a file.  Here no size has a
default: a missing size is an error.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, asdict
from typing import Any, Dict, Optional, Tuple


class ConfigError(ValueError):
    """A config.json that this engine cannot run, with the reason."""


_REQUIRED = ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
             "num_key_value_heads", "intermediate_size", "rms_norm_eps", "rope_theta",
             "tie_word_embeddings")


def _integer(d: Dict[str, Any], key: str, value: Any = None) -> int:
    v = d[key] if value is None else value
    if isinstance(v, bool) or not isinstance(v, int):
        raise ConfigError(f"{key} must be an integer, got {v!r}")
    return v


def _number(d: Dict[str, Any], key: str) -> float:
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"{key} must be a number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class Qwen2Config:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    intermediate_size: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    head_dim: int
    max_position_embeddings: int = 131072
    hidden_act: str = "silu"
    eos_token_id: Optional[int] = None
    architectures: Tuple[str, ...] = ("Qwen2ForCausalLM",)
    torch_dtype: str = "bfloat16"
    ignored_keys: Tuple[str, ...] = field(default=(), compare=False)

    # derived (pico_vllm/model.py:41-43)
    @property
    def num_kv_groups(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "Qwen2Config":
        missing = [k for k in _REQUIRED if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks required keys: {', '.join(missing)}")
        head_dim = d.get("head_dim")
        if head_dim is None:
            # pico_vllm/model.py:37-38
            width, heads = _integer(d, "hidden_size"), _integer(d, "num_attention_heads")
            if heads < 1 or width % heads:
                raise ConfigError("hidden_size is not a multiple of num_attention_heads and head_dim is not given")
            head_dim = width // heads
        eos = d.get("eos_token_id")
        if isinstance(eos, (list, tuple)):
            eos = eos[0] if eos else None
        if eos is not None:
            eos = _integer(d, "eos_token_id", eos)
        if not isinstance(d["tie_word_embeddings"], bool):
            raise ConfigError(f"tie_word_embeddings must be true or false, got {d['tie_word_embeddings']!r}")
        architectures = d.get("architectures") or ("Qwen2ForCausalLM",)
        if isinstance(architectures, str) or not all(isinstance(a, str) for a in architectures):
            raise ConfigError(f"architectures must be a list of names, got {architectures!r}")
        known = set(cls.__dataclass_fields__) | {"use_sliding_window", "sliding_window", "max_window_layers",
                                                 "rope_scaling", "attention_bias", "model_type"}
        cfg = cls(
            vocab_size=_integer(d, "vocab_size"), hidden_size=_integer(d, "hidden_size"),
            num_hidden_layers=_integer(d, "num_hidden_layers"),
            num_attention_heads=_integer(d, "num_attention_heads"),
            num_key_value_heads=_integer(d, "num_key_value_heads"),
            intermediate_size=_integer(d, "intermediate_size"),
            rms_norm_eps=_number(d, "rms_norm_eps"), rope_theta=_number(d, "rope_theta"),
            tie_word_embeddings=d["tie_word_embeddings"], head_dim=_integer(d, "head_dim", head_dim),
            max_position_embeddings=_integer(d, "max_position_embeddings", d.get("max_position_embeddings", 131072)),
            hidden_act=str(d.get("hidden_act", "silu")), eos_token_id=eos,
            architectures=tuple(architectures),
            torch_dtype=str(d.get("torch_dtype", "bfloat16")),
            ignored_keys=tuple(sorted(k for k in d if k not in known)),
        )
        cfg._validate(d)
        return cfg

    def _validate(self, raw: Dict[str, Any]) -> None:
        pos = ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
               "num_key_value_heads", "intermediate_size", "head_dim", "max_position_embeddings")
        for k in pos:
            least = 0 if k == "num_hidden_layers" else 1
            if getattr(self, k) < least:
                raise ConfigError(f"{k} must be at least {least}, got {getattr(self, k)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(f"num_attention_heads ({self.num_attention_heads}) is not a multiple of "
                              f"num_key_value_heads ({self.num_key_value_heads})")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim ({self.head_dim}) must be even for rotate-half position encoding")
        if self.hidden_act != "silu":
            raise ConfigError(f"hidden_act {self.hidden_act!r} is not supported (only 'silu')")
        if not (self.rms_norm_eps > 0):
            raise ConfigError("rms_norm_eps must be positive")
        if not (self.rope_theta > 0):
            raise ConfigError("rope_theta must be positive")
        if raw.get("use_sliding_window"):
            raise ConfigError("use_sliding_window=true is not supported for this architecture")
        if raw.get("rope_scaling"):
            raise ConfigError("rope_scaling is not supported for this architecture")
        if raw.get("attention_bias") is False:
            raise ConfigError("attention_bias=false: this architecture has biases on q, k and v")

    def to_dict(self) -> Dict[str, Any]:
        d = asdict(self)
        d.pop("ignored_keys")
        d["architectures"] = list(self.architectures)
        d["model_type"] = "qwen2"
        return d


def read_config_json(model_dir: str) -> Dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{path} does not exist")
    with open(path) as f:
        try:
            return json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path} is not valid JSON: {e}") from None
