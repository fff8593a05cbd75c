"""The Qwen2 dense decoder as a model description.

Layer make-up and order follow pico_vllm/model.py:340-374 (pre-norm block:
norm1 -> attention -> add -> norm2 -> SwiGLU -> add) and :427-445 (embedding,
blocks, final norm, output matrix).  Tensor names are those the reference's
loader reads (pico_vllm/weights.py:18-68).
"""
from __future__ import annotations

from ..parts.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from .model_config import Qwen2Config
from .registry import register_architecture


def qwen2_spec(cfg: Qwen2Config) -> ModelSpec:
    norm = PartSpec("rms_norm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    attn = PartSpec("gqa_attention", {
        "hidden_size": cfg.hidden_size,
        "num_heads": cfg.num_attention_heads,
        "num_kv_heads": cfg.num_key_value_heads,
        "head_dim": cfg.head_dim,
        "qkv_bias": True,                       # pico_vllm/model.py:148-152
        "window": 0,
        "position": PartSpec("rotary_half", {"rotary_dim": cfg.head_dim, "theta": cfg.rope_theta}),
    })
    ff = PartSpec("swiglu_mlp", {"hidden_size": cfg.hidden_size,
                                 "intermediate_size": cfg.intermediate_size})
    layers = [
        LayerSpec(prefix=f"model.layers.{i}", block="prenorm", slots={
            "norm1": ("input_layernorm", norm),
            "mixer": ("self_attn", attn),
            "norm2": ("post_attention_layernorm", norm),
            "ff": ("mlp", ff),
        })
        for i in range(cfg.num_hidden_layers)
    ]
    return ModelSpec(
        hidden_size=cfg.hidden_size, vocab_size=cfg.vocab_size,
        embed_name="model.embed_tokens.weight",
        layers=layers,
        run_order=[RunEntry(i) for i in range(cfg.num_hidden_layers)],
        final_norm=norm, final_norm_name="model.norm",
        head_name=None if cfg.tie_word_embeddings else "lm_head.weight",
        eos_token_id=cfg.eos_token_id,
        max_position=cfg.max_position_embeddings,
        # a tied model's file may still hold the output matrix; the reference never reads it (weights.py:67-68)
        ignored_tensors=("lm_head.weight",) if cfg.tie_word_embeddings else (),
    )


def qwen2_sizes(cfg: Qwen2Config) -> dict:
    """The sizes of a configuration as a flat record (for a benchmark's report)."""
    return {"layers": cfg.num_hidden_layers, "hidden": cfg.hidden_size, "q_heads": cfg.num_attention_heads,
            "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size,
            "vocab": cfg.vocab_size, "tied": cfg.tie_word_embeddings}


def qwen2_with_layers(raw: dict, layers: int) -> dict:
    """The same layer sizes with ``layers`` layers (a measurement that memory or time limits to fewer)."""
    return dict(raw, num_hidden_layers=layers)


register_architecture("Qwen2ForCausalLM", Qwen2Config.from_dict, qwen2_spec, qwen2_sizes, qwen2_with_layers)
