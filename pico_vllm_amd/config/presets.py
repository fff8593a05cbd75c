"""Named configurations for random-weight runs: the sizes of the published Qwen2.5 models and two
tiny ones for quick checks.  Each is what the model's config.json would hold (the keys that
``Qwen2Config.from_dict`` reads); nothing else in the package refers to these sizes."""
from __future__ import annotations

from typing import Dict


def _qwen2(vocab, hidden, layers, heads, kv_heads, inter, tied, eps=1e-6, theta=1e6, max_pos=131072, **more) -> Dict:
    cfg = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "vocab_size": vocab, "hidden_size": hidden,
           "num_hidden_layers": layers, "num_attention_heads": heads, "num_key_value_heads": kv_heads,
           "intermediate_size": inter, "rms_norm_eps": eps, "rope_theta": theta, "tie_word_embeddings": tied,
           "max_position_embeddings": max_pos, "hidden_act": "silu"}
    cfg.update(more)
    return cfg


PRESETS: Dict[str, Dict] = {
    "tiny-a": _qwen2(256, 64, 2, 4, 1, 172, True, theta=1e4, max_pos=2048, eos_token_id=255),
    "tiny-b": _qwen2(384, 192, 3, 6, 3, 320, False, eps=1e-5, max_pos=4096, eos_token_id=383),
    "1.5b": _qwen2(151936, 1536, 28, 12, 2, 8960, True),
    "7b": _qwen2(152064, 3584, 28, 28, 4, 18944, False),
    "32b": _qwen2(152064, 5120, 64, 40, 8, 27648, False),
}


def preset(name: str) -> Dict:
    try:
        return dict(PRESETS[name.lower()])
    except KeyError:
        raise ValueError(f"unknown configuration {name!r}; known: {', '.join(sorted(PRESETS))}") from None
