"""Plain, slow, whole-sequence implementation of the Qwen2 dense decoder.

Written from the formulas of the reference (paths below are relative to the
reference checkout, ``pico_vllm/...``).  One function per part, float32
everywhere, no cache, no batching, no code shared with the engine.  It is the
oracle every engine test compares against.

Two places differ from the reference on purpose, both documented where they
occur: rotation tables stay in float32 (the reference's tables become bfloat16
only because the whole module is cast, run_single.py:13), and an untied model
multiplies by ``lm_head.weight`` (the reference always multiplies by the
embedding matrix, model.py:445, even when ``tie_word_embeddings`` is false).
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import torch
from safetensors import safe_open


# --------------------------------------------------------------------------
# configuration and weights (read with the safetensors package, not with the
# engine's own reader)
# --------------------------------------------------------------------------
def f32(x: torch.Tensor) -> torch.Tensor:
    """At least float32: what is float64 stays so.  With float64 weights the whole computation runs in
    float64, which tells the engine's rounding from this implementation's own."""
    return x if x.dtype == torch.float64 else x.float()


@dataclass
class PlainConfig:
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


def read_config(model_dir: str) -> PlainConfig:
    """Field names are the reference dataclass's (model.py:16-26); head_dim
    defaults to hidden/heads (model.py:37-38)."""
    with open(os.path.join(model_dir, "config.json")) as f:
        c = json.load(f)
    hd = c.get("head_dim") or c["hidden_size"] // c["num_attention_heads"]
    return PlainConfig(
        vocab_size=c["vocab_size"], hidden_size=c["hidden_size"],
        num_hidden_layers=c["num_hidden_layers"],
        num_attention_heads=c["num_attention_heads"],
        num_key_value_heads=c["num_key_value_heads"],
        intermediate_size=c["intermediate_size"],
        rms_norm_eps=c["rms_norm_eps"], rope_theta=c["rope_theta"],
        tie_word_embeddings=c["tie_word_embeddings"], head_dim=hd)


def read_weights(model_dir: str) -> Dict[str, torch.Tensor]:
    """Every tensor as float32, by its name in the file (weights.py:10-15)."""
    out: Dict[str, torch.Tensor] = {}
    for name in sorted(os.listdir(model_dir)):
        if name.endswith(".safetensors"):
            with safe_open(os.path.join(model_dir, name), framework="pt", device="cpu") as st:
                for key in st.keys():
                    out[key] = st.get_tensor(key).float()
    return out


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x * 1/sqrt(mean(x^2) + eps) * w   (RMSNorm.py:22-31; eager twin
    model.py:63-66).  eps sits inside the square root; the weight multiplies
    (it is not 1+w)."""
    x = f32(x)
    var = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x * (1.0 / torch.sqrt(var + eps)) * f32(weight).to(x.dtype)


def rope_tables(positions: torch.Tensor, head_dim: int, theta: float, dtype: torch.dtype = torch.float32):
    """cos/sin rows for the given absolute positions (model.py:80-90).

    f_j = 1 / theta^(2j/d), j < d/2; angle = p * f_j in float32; each table
    row is the half-row repeated twice.  The angle is the float32 product by
    definition; ``dtype`` is that of its cosine and sine."""
    freqs = 1.0 / (theta ** (torch.arange(0, head_dim, 2).float() / head_dim))
    angles = torch.outer(positions.float(), freqs).to(dtype)
    cos = torch.cat([angles.cos(), angles.cos()], dim=-1)
    sin = torch.cat([angles.sin(), angles.sin()], dim=-1)
    return cos, sin


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x: [S, heads, d]; cos/sin: [S, d].  x*cos + rotate_half(x)*sin with
    rotate_half(x) = [-x2, x1], the halves being the first and last d/2
    entries (model.py:116-123).  So pairs are (j, j + d/2)."""
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    rot = torch.cat([-x2, x1], dim=-1)
    return x * cos[:, None, :] + rot * sin[:, None, :]


def split_qkv(qkv: torch.Tensor, n_q: int, n_kv: int, d: int):
    """Rows of the fused projection are [q; k; v] (weights.py:42-43), split
    into sizes [nq*d, nkv*d, nkv*d] and viewed per head (model.py:205-208)."""
    q, k, v = qkv.split([n_q * d, n_kv * d, n_kv * d], dim=-1)
    S = qkv.shape[0]
    return q.reshape(S, n_q, d), k.reshape(S, n_kv, d), v.reshape(S, n_kv, d)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                     q_positions: Optional[torch.Tensor] = None,
                     window: int = 0, rnd_p=None) -> torch.Tensor:
    """q: [M, nq, d]; k, v: [N, nkv, d]; returns [M, nq, d].

    Query head h reads KV head h // (nq/nkv) (kernels/attention.py:31,139).
    Scores (q.k) * d^-0.5 (attention.py:92,231); key n is visible to the
    query at absolute position p iff n <= p (attention.py:193-197); softmax
    over visible keys; weighted sum of V.  Without q_positions the M queries
    are the last M of the N positions (tests/test_prefill_paged_attn.py:38-44).
    ``window`` > 0 additionally hides keys with n <= p - window (not in the
    reference; used only for the windowed-attention part test).  ``rnd_p``
    rounds the probabilities before they multiply V, as the reference's
    prefill kernel does in bfloat16 (attention.py:206)."""
    M, nq, d = q.shape
    N, nkv, _ = k.shape
    G = nq // nkv
    if q_positions is None:
        q_positions = torch.arange(N - M, N)
    scale = 1.0 / math.sqrt(d)
    out = torch.empty(M, nq, d, dtype=f32(q).dtype)
    k_pos = torch.arange(N)
    visible = k_pos[None, :] <= q_positions[:, None]
    if window > 0:
        visible &= k_pos[None, :] > (q_positions[:, None] - window)
    for h in range(nq):
        g = h // G
        s = (f32(q[:, h, :]) @ f32(k[:, g, :]).T) * scale
        s = s.masked_fill(~visible, float("-inf"))
        p = torch.softmax(s, dim=-1)
        if rnd_p is not None:
            p = rnd_p(p)
        out[:, h, :] = p @ f32(v[:, g, :])
    return out


def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    """gate = first half, up = second half of the last dim (weights.py:58);
    out = gate * sigmoid(gate) * up  (kernels/swiglu.py:36-41, model.py:318)."""
    I = gate_up.shape[-1] // 2
    gate, up = f32(gate_up[..., :I]), f32(gate_up[..., I:])
    return gate * torch.sigmoid(gate) * up


def _same(x: torch.Tensor) -> torch.Tensor:
    return x


def to_bf16(x: torch.Tensor) -> torch.Tensor:
    """Round to bfloat16 and back: what storing an activation in bfloat16 does to it."""
    return x.to(torch.bfloat16).float()


def dithered_bf16(generator: torch.Generator):
    """A rounding to bfloat16 whose error is drawn anew at every call (subtractive dither): x + d is rounded, d uniform
    within one unit in the last place of x, and d is taken off again.  The error is that of a bfloat16 rounding, uniform
    within half a unit in the last place, but independent of x and of every other call: runs of the plain
    implementation with it are independent draws of what bfloat16 storage of activations does to the logits."""
    def rnd(x: torch.Tensor) -> torch.Tensor:
        _, e = torch.frexp(x)                                        # |x| in [2^(e-1), 2^e)
        ulp = torch.ldexp(torch.ones_like(x), e - 8)                 # bfloat16 keeps 8 significant bits
        d = (torch.rand(x.shape, generator=generator, dtype=x.dtype) - 0.5) * ulp
        return (x + d).to(torch.bfloat16).to(x.dtype) - d
    return rnd


def attention_layer(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str,
                    cfg: PlainConfig, positions: torch.Tensor, rnd=_same) -> torch.Tensor:
    """qkv = h W^T + b with bias on q, k, v only (model.py:148-152); RoPE on
    q and k (model.py:211); attention; o_proj without bias (model.py:147,225)."""
    nq, nkv, d = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    W = torch.cat([w[f"{prefix}.self_attn.q_proj.weight"],
                   w[f"{prefix}.self_attn.k_proj.weight"],
                   w[f"{prefix}.self_attn.v_proj.weight"]], dim=0)
    b = torch.cat([w[f"{prefix}.self_attn.q_proj.bias"],
                   w[f"{prefix}.self_attn.k_proj.bias"],
                   w[f"{prefix}.self_attn.v_proj.bias"]], dim=0)
    qkv = rnd(h @ W.T + b)
    q, k, v = split_qkv(qkv, nq, nkv, d)
    cos, sin = rope_tables(positions, d, cfg.rope_theta, qkv.dtype)
    q, k = rnd(apply_rope(q, cos, sin)), rnd(apply_rope(k, cos, sin))
    o = rnd(causal_attention(q, k, v, q_positions=positions - positions[0], rnd_p=None if rnd is _same else rnd))
    return rnd(o.reshape(h.shape[0], nq * d) @ w[f"{prefix}.self_attn.o_proj.weight"].T)


def mlp_layer(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, rnd=_same) -> torch.Tensor:
    """down( swiglu( h [gate; up]^T ) ), no biases (model.py:309-318)."""
    Wgu = torch.cat([w[f"{prefix}.mlp.gate_proj.weight"], w[f"{prefix}.mlp.up_proj.weight"]], dim=0)
    return rnd(rnd(swiglu(rnd(h @ Wgu.T))) @ w[f"{prefix}.mlp.down_proj.weight"].T)


def block(x: torch.Tensor, w: Dict[str, torch.Tensor], i: int, cfg: PlainConfig,
          positions: torch.Tensor, rnd=_same) -> torch.Tensor:
    """x += attn(norm1(x)); x += ffn(norm2(x))   (model.py:361-374)."""
    p = f"model.layers.{i}"
    x = x + attention_layer(rnd(rms_norm(x, w[f"{p}.input_layernorm.weight"], cfg.rms_norm_eps)),
                            w, p, cfg, positions, rnd)
    x = x + mlp_layer(rnd(rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], cfg.rms_norm_eps)), w, p, rnd)
    return x


def forward(tokens: Sequence[int], w: Dict[str, torch.Tensor], cfg: PlainConfig,
            first_position: int = 0, rnd=_same) -> torch.Tensor:
    """Logits [S, V] for one whole sequence (model.py:427-445): embedding,
    L blocks, final norm, output matrix.  Tied models multiply by the
    embedding matrix; untied ones by lm_head.weight (our deliberate
    difference, see the module docstring).

    ``rnd`` is applied to every activation between the parts (not to the
    residual stream, not to the logits); with ``to_bf16`` it shows how far
    bfloat16 storage of activations moves the logits of this model, which is
    the yardstick for the bfloat16 engine's tolerance."""
    ids = torch.as_tensor(list(tokens), dtype=torch.long)
    x = f32(w["model.embed_tokens.weight"][ids])
    positions = torch.arange(first_position, first_position + len(ids))
    for i in range(cfg.num_hidden_layers):
        x = block(x, w, i, cfg, positions, rnd)
    x = rnd(rms_norm(x, w["model.norm.weight"], cfg.rms_norm_eps))
    out_w = w["model.embed_tokens.weight"] if cfg.tie_word_embeddings else w["lm_head.weight"]
    return x @ f32(out_w).T


def permute_inner_dimensions(w: Dict[str, torch.Tensor], cfg: PlainConfig, generator: torch.Generator) -> Dict[str, torch.Tensor]:
    """The same model with its hidden and intermediate dimensions in another (random) order: every matrix and norm
    weight is permuted consistently, so the function from tokens to logits is unchanged (model.py:361-374 adds and
    norms along the hidden dimension, model.py:309-318 contracts over the intermediate one; neither cares about the
    order), but every sum over those dimensions runs in another order.  In float32 each such model is an independent
    draw of what float32 rounding does to the logits.  Head dimensions keep their order (rotation pairs j with
    j + d/2, model.py:116-123)."""
    ph = torch.randperm(cfg.hidden_size, generator=generator)
    pi = torch.randperm(cfg.intermediate_size, generator=generator)
    out = {}
    for name, t in w.items():
        if name.endswith("embed_tokens.weight") or name.endswith("lm_head.weight"):
            t = t[:, ph]
        elif name.endswith("layernorm.weight") or name == "model.norm.weight":
            t = t[ph]
        elif name.endswith(("q_proj.weight", "k_proj.weight", "v_proj.weight")):
            t = t[:, ph]
        elif name.endswith("o_proj.weight"):
            t = t[ph, :]
        elif name.endswith(("gate_proj.weight", "up_proj.weight")):
            t = t[pi][:, ph]
        elif name.endswith("down_proj.weight"):
            t = t[ph][:, pi]
        out[name] = t.contiguous()
    return out


class PlainModel:
    """A model folder read once; ``logits(tokens)`` runs the whole sequence."""

    def __init__(self, model_dir: str, dtype: torch.dtype = torch.float32):
        """``dtype`` float64: the same weights (they are exact in float64) and every sum in float64."""
        self.cfg = read_config(model_dir)
        self.w = {k: v.to(dtype) for k, v in read_weights(model_dir).items()}

    def logits(self, tokens: Sequence[int], rnd=_same) -> torch.Tensor:
        with torch.no_grad():
            return forward(tokens, self.w, self.cfg, rnd=rnd)

    def greedy(self, prompt: Sequence[int], n: int) -> List[int]:
        toks = list(prompt)
        out: List[int] = []
        for _ in range(n):
            t = int(torch.argmax(self.logits(toks)[-1]))
            out.append(t)
            toks.append(t)
        return out


# --------------------------------------------------------------------------
# sampling
# --------------------------------------------------------------------------
def sample_greedy(logits: torch.Tensor) -> int:
    """argmax (sampler.py:8); the first index wins a tie."""
    return int(torch.argmax(logits.float()))


def temperature_probs(logits: torch.Tensor, temperature: float) -> torch.Tensor:
    """softmax(logits / T)  (sampler.py:16)."""
    return torch.softmax(logits.double() / temperature, dim=-1)


def top_p_probs(logits: torch.Tensor, temperature: float, top_p: float) -> torch.Tensor:
    """Sort descending, drop entries whose preceding cumulative mass is
    >= top_p (so the first token that crosses is kept), renormalise
    (sampler.py:25-32).  Returned in vocabulary order.  Of tokens with equal
    probability a prefix in sorted order survives; which of them come first is
    the sort's choice in the reference (torch.sort is not stable there), the
    lowest indices here (a stable sort)."""
    probs = temperature_probs(logits, temperature)
    sp, si = torch.sort(probs, descending=True, stable=True)
    cum = torch.cumsum(sp, dim=-1)
    sp = sp.masked_fill(cum - sp >= top_p, 0.0)
    sp = sp / sp.sum()
    out = torch.zeros_like(probs)
    out[si] = sp
    return out


def inverse_cdf(probs: torch.Tensor, u: float) -> int:
    """Smallest index whose cumulative probability exceeds u * total: how the
    engine turns one uniform number into a draw from ``probs`` (the reference
    draws with torch.multinomial, sampler.py:17, which fixes only the
    distribution)."""
    cum = torch.cumsum(probs.double(), dim=-1)
    idx = int(torch.searchsorted(cum, torch.tensor(u * float(cum[-1]), dtype=torch.float64), right=True))
    nz = torch.nonzero(probs > 0).flatten()
    return min(max(idx, int(nz[0])), int(nz[-1]))
