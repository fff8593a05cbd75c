"""The small configurations the tests run: they differ in every size and option."""
import tempfile

TINY_A = {   # MQA, tied, head 16
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "vocab_size": 256, "hidden_size": 64, "num_hidden_layers": 2, "num_attention_heads": 4,
    "num_key_value_heads": 1, "intermediate_size": 172, "rms_norm_eps": 1e-6, "rope_theta": 10000.0,
    "tie_word_embeddings": True, "max_position_embeddings": 2048, "hidden_act": "silu", "eos_token_id": 255,
}
TINY_B = {   # groups of 2, untied, head 32
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "vocab_size": 384, "hidden_size": 192, "num_hidden_layers": 3, "num_attention_heads": 6,
    "num_key_value_heads": 3, "intermediate_size": 320, "rms_norm_eps": 1e-5, "rope_theta": 1000000.0,
    "tie_word_embeddings": False, "max_position_embeddings": 4096, "hidden_act": "silu", "eos_token_id": 383,
}
TINY_C = {   # head size 48 given explicitly (hidden != heads * head), 5 heads without grouping, odd vocabulary
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "vocab_size": 301, "hidden_size": 136, "num_hidden_layers": 1, "num_attention_heads": 5,
    "num_key_value_heads": 5, "head_dim": 48, "intermediate_size": 200, "rms_norm_eps": 1e-6,
    "rope_theta": 50000.0, "tie_word_embeddings": True, "max_position_embeddings": 1024, "hidden_act": "silu",
}
TINY_D = {   # sizes that no vector access divides: a width of 100, an odd intermediate size and vocabulary
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "vocab_size": 257, "hidden_size": 100, "num_hidden_layers": 2, "num_attention_heads": 4,
    "num_key_value_heads": 2, "head_dim": 16, "intermediate_size": 123, "rms_norm_eps": 1e-6,
    "rope_theta": 10000.0, "tie_word_embeddings": False, "max_position_embeddings": 1024, "hidden_act": "silu",
}
TINY_E = {   # head size 96 (three chunks of 32; its 12 chunks of 16 bytes a key divide no workgroup), groups of 3
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "vocab_size": 333, "hidden_size": 168, "num_hidden_layers": 2, "num_attention_heads": 6,
    "num_key_value_heads": 2, "head_dim": 96, "intermediate_size": 232, "rms_norm_eps": 3e-6,
    "rope_theta": 100000.0, "tie_word_embeddings": True, "max_position_embeddings": 2048, "hidden_act": "silu",
}
TINY_F = {   # for contexts of thousands of tokens: two heads of 64 on one kv head, positions up to 16,384
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "vocab_size": 299, "hidden_size": 128, "num_hidden_layers": 2, "num_attention_heads": 2,
    "num_key_value_heads": 1, "intermediate_size": 264, "rms_norm_eps": 1e-6, "rope_theta": 1000000.0,
    "tie_word_embeddings": False, "max_position_embeddings": 16384, "hidden_act": "silu",
}
TINY_G = {   # head size 24, between the steps of 16 that the matrix-core attention takes: groups of 3, pages of 8
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "vocab_size": 271, "hidden_size": 144, "num_hidden_layers": 2, "num_attention_heads": 6,
    "num_key_value_heads": 2, "intermediate_size": 208, "rms_norm_eps": 1e-5,
    "rope_theta": 10000.0, "tie_word_embeddings": False, "max_position_embeddings": 1024, "hidden_act": "silu",
}
TINY_H = {   # head size 40 given explicitly, five heads on one kv head, a width that is not heads * head
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "vocab_size": 263, "hidden_size": 120, "num_hidden_layers": 3, "num_attention_heads": 5,
    "num_key_value_heads": 1, "head_dim": 40, "intermediate_size": 176, "rms_norm_eps": 1e-6,
    "rope_theta": 1000000.0, "tie_word_embeddings": True, "max_position_embeddings": 1024, "hidden_act": "silu",
}
TINY_Z = dict(TINY_B, num_hidden_layers=0)       # no layer at all: embedding, final norm, untied output matrix
PAGE_SIZE = {"A": 16, "B": 8, "C": 16, "D": 16, "E": 16, "F": 16, "G": 8, "H": 16, "Z": 8}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E, "F": TINY_F, "G": TINY_G, "H": TINY_H,
           "Z": TINY_Z}


def drawn(seed: int):
    """A configuration drawn at random (the same for a seed on every machine): head sizes in steps of 16,
    any number of heads and groups, a width, an intermediate size and a vocabulary that are no powers of
    two, with or without a head size of its own, tied or not; and a page size."""
    import random
    rng = random.Random(1000 + seed)
    d = rng.choice([16, 32, 48, 64, 80, 96, 128])
    nkv = rng.choice([1, 2, 3, 4])
    nq = nkv * rng.choice([1, 2, 3, 5, 7])
    while nq * d > 1024:
        nq -= nkv
    cfg = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
           "num_attention_heads": nq, "num_key_value_heads": nkv,
           "num_hidden_layers": rng.choice([1, 2, 3]), "vocab_size": rng.randrange(200, 700) | 1,
           "intermediate_size": 8 * rng.randrange(9, 50), "rms_norm_eps": rng.choice([1e-6, 3e-6, 1e-5]),
           "rope_theta": rng.choice([1e4, 5e4, 1e6]), "tie_word_embeddings": rng.random() < 0.5,
           "max_position_embeddings": 2048}
    if rng.random() < 0.5:
        cfg["hidden_size"] = nq * d
    else:
        cfg["hidden_size"] = 8 * rng.randrange(9, 40)
        cfg["head_dim"] = d
    return cfg, rng.choice([8, 16, 32])


for _seed in range(10):
    CONFIGS[f"R{_seed}"], PAGE_SIZE[f"R{_seed}"] = drawn(_seed)



def _real(hidden, heads, kv_heads, inter, layers, vocab, tied):
    return {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "vocab_size": vocab, "hidden_size": hidden,
            "num_hidden_layers": layers, "num_attention_heads": heads, "num_key_value_heads": kv_heads,
            "intermediate_size": inter, "rms_norm_eps": 1e-6, "rope_theta": 1000000.0, "tie_word_embeddings": tied,
            "max_position_embeddings": 32768, "hidden_act": "silu"}


# Layers of the sizes of real models (the vocabulary cut down so that the plain implementation stays quick): two
# layers of Qwen2.5-1.5B, one each of 7B (groups of 7 heads) and 32B (groups of 5, a width beyond 4,096)
REAL = {"L1.5B": _real(1536, 12, 2, 8960, 2, 20011, True), "L7B": _real(3584, 28, 4, 18944, 1, 4099, False),
        "L32B": _real(5120, 40, 8, 27648, 1, 3001, False),
        # the whole Qwen2.5-1.5B shape: all 28 layers and the whole vocabulary
        "F1.5B": _real(1536, 12, 2, 8960, 28, 151936, True)}
for _name, _cfg in REAL.items():
    CONFIGS[_name], PAGE_SIZE[_name] = _cfg, 16


def balanced(config) -> dict:
    """Standard deviations for the real sizes: every part changes the residual stream by about as much as it
    holds (rows of unit length into unit-variance activations), and attention scores have a spread of about 3."""
    H, I = config["hidden_size"], config["intermediate_size"]
    return {"q_proj.weight": (3.0 / H) ** 0.5, "k_proj.weight": (3.0 / H) ** 0.5, "v_proj.weight": H ** -0.5,
            "o_proj.weight": H ** -0.5, "gate_proj": 1.5 * H ** -0.5, "up_proj": H ** -0.5, "down_proj": 2.0 * I ** -0.5,
            "_proj.bias": 0.2, "embed_tokens": 1.0, "lm_head": H ** -0.5}


_made = {}


def strong(config) -> dict:
    """Standard deviations larger than N(0, 0.02), so that a fault shows in the logits: with q and k
    weights of sqrt(3 / hidden) the attention scores have a spread of about 3, which makes attention
    pick out keys (a wrong rotation, mask or page changes the result) without making the softmax so
    sharp that rounding is amplified; the other matrices change the residual stream visibly."""
    qk = (3.0 / config["hidden_size"]) ** 0.5
    return {"q_proj.weight": qk, "k_proj.weight": qk, "v_proj.weight": 0.1, "o_proj.weight": 0.1,
            "gate_proj": 0.1, "up_proj": 0.1, "down_proj": 0.1, "_proj.bias": 0.2, "embed_tokens": 0.1,
            "lm_head": 0.1}


STRONG = strong(TINY_B)


def model_dir(name: str, seed: int = 0, strong: bool = True) -> str:
    """A random-weights model folder in a temporary place, made once per process."""
    from pico_vllm_amd.weights.random_init import write_random_model
    key = (name, seed, strong)
    if key not in _made:
        d = tempfile.mkdtemp(prefix=f"pico_tiny_{name}_")
        stds = (balanced if name in REAL else globals()['strong'])(CONFIGS[name]) if strong else None
        write_random_model(d, CONFIGS[name], seed, stds)
        _made[key] = d
    return _made[key]
