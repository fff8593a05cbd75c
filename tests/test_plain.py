"""Pins of the plain implementation: each formula is fixed by something besides the
reference's text: a library routine it must reduce to, an invariant, or a vector the
reference's own tests hold."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_qwen2 as P
from tiny_configs import model_dir

torch.manual_seed(0)


# ---- RMSNorm -------------------------------------------------------------
def test_rmsnorm_unit_weight_is_x_over_rms():
    x = torch.randn(5, 37)
    y = P.rms_norm(x, torch.ones(37), 1e-6)
    want = x.numpy() / np.sqrt(np.mean(x.numpy().astype(np.float64) ** 2, axis=-1, keepdims=True) + 1e-6)
    assert np.allclose(y.numpy(), want, rtol=1e-5, atol=1e-6)
    # rows have RMS 1 when eps vanishes against the data
    assert torch.allclose((y * y).mean(-1).sqrt(), torch.ones(5), atol=1e-4)


def test_rmsnorm_eps_inside_the_root_and_weight_multiplies():
    x = torch.full((1, 8), 1e-4)
    # mean(x^2) = 1e-8 << eps = 1e-2: y = x / sqrt(eps); eps outside the root would give ~1
    y = P.rms_norm(x, torch.ones(8), 1e-2)
    assert torch.allclose(y, x / math.sqrt(1e-8 + 1e-2), rtol=1e-5)
    w = torch.linspace(0.5, 2.0, 8)
    big = torch.randn(3, 8) * 10
    assert torch.allclose(P.rms_norm(big, w, 1e-6), P.rms_norm(big, torch.ones(8), 1e-6) * w)  # not (1 + w)
    # scale equivariance
    assert torch.allclose(P.rms_norm(3 * big, w, 1e-12), P.rms_norm(big, w, 1e-12), rtol=1e-4, atol=1e-5)


# ---- rotation ------------------------------------------------------------
def test_rope_tables_shapes_and_unit_circle():
    # shapes as in the reference's test (tests/test_model.py:51-63)
    cos, sin = P.rope_tables(torch.arange(10), 128, 1e6)
    assert cos.shape == (10, 128) and sin.shape == (10, 128)
    assert torch.allclose(cos * cos + sin * sin, torch.ones_like(cos), atol=1e-3)
    assert torch.equal(cos[:, :64], cos[:, 64:])          # halves duplicated (model.py:88-89)
    # frequency j is theta^(-2j/d)
    assert math.isclose(float(sin[1, 1]), math.sin(1e6 ** (-2 / 128)), rel_tol=1e-5)


def test_rope_position_zero_is_identity_and_pairs_are_j_and_j_plus_half():
    d = 16
    x = torch.randn(1, 2, d)
    cos, sin = P.rope_tables(torch.tensor([0]), d, 1e4)
    assert torch.allclose(P.apply_rope(x, cos, sin), x)
    e = torch.zeros(1, 1, d)
    e[0, 0, 3] = 1.0
    cos, sin = P.rope_tables(torch.tensor([5]), d, 1e4)
    y = P.apply_rope(e, cos, sin)[0, 0]
    ang = 5 * 1e4 ** (-2 * 3 / d)
    assert set(torch.nonzero(y.abs() > 1e-7).flatten().tolist()) == {3, 3 + d // 2}    # not (2j, 2j+1)
    assert math.isclose(float(y[3]), math.cos(ang), abs_tol=1e-6)
    assert math.isclose(float(y[3 + d // 2]), math.sin(ang), abs_tol=1e-6)            # +sin: counter-clockwise


def test_rope_keeps_pair_norms_and_scores_depend_on_distance_only():
    d = 32
    q, k = torch.randn(1, 1, d), torch.randn(1, 1, d)

    def rot(x, p):
        c, s = P.rope_tables(torch.tensor([p]), d, 1e4)
        return P.apply_rope(x, c, s)[0, 0]
    qr = rot(q, 7)
    pair = lambda v: v[:d // 2] ** 2 + v[d // 2:] ** 2
    assert torch.allclose(pair(qr), pair(q[0, 0]), atol=1e-5)
    a = torch.dot(rot(q, 7), rot(k, 3))
    b = torch.dot(rot(q, 107), rot(k, 103))
    c = torch.dot(rot(q, 7), rot(k, 4))
    assert math.isclose(float(a), float(b), rel_tol=1e-3, abs_tol=1e-4)
    assert not math.isclose(float(a), float(c), rel_tol=1e-3, abs_tol=1e-4)


# ---- attention -----------------------------------------------------------
def _sdpa(q, k, v):
    G = q.shape[1] // k.shape[1]
    kk, vv = k.repeat_interleave(G, dim=1), v.repeat_interleave(G, dim=1)
    o = F.scaled_dot_product_attention(q.transpose(0, 1)[None], kk.transpose(0, 1)[None], vv.transpose(0, 1)[None],
                                       is_causal=True)
    return o[0].transpose(0, 1)


@pytest.mark.parametrize("nq,nkv", [(4, 4), (4, 1), (6, 3), (12, 2)])
def test_attention_reduces_to_library_routine(nq, nkv):
    S, d = 19, 16
    q, k, v = torch.randn(S, nq, d), torch.randn(S, nkv, d), torch.randn(S, nkv, d)
    assert torch.allclose(P.causal_attention(q, k, v), _sdpa(q, k, v), atol=1e-5)


def test_attention_head_map_is_h_div_group_not_h_mod_kv():
    S, nq, nkv, d = 5, 6, 3, 8
    q, k = torch.randn(S, nq, d), torch.randn(S, nkv, d)
    v = torch.zeros(S, nkv, d)
    v[:, 1, :] = 1.0                      # only kv head 1 carries anything
    o = P.causal_attention(q, k, v)
    live = [h for h in range(nq) if o[:, h].abs().sum() > 0]
    assert live == [2, 3]                 # h // 2 == 1; h % 3 == 1 would give [1, 4]


def test_first_token_sees_only_itself_and_scale_is_inverse_root_d():
    S, d = 6, 16
    q, k, v = torch.randn(S, 2, d), torch.randn(S, 2, d), torch.randn(S, 2, d)
    o = P.causal_attention(q, k, v)
    assert torch.allclose(o[0], v[0], atol=1e-6)
    # two keys, explicit weights
    s = (q[1, 0] @ k[:2, 0].T) / math.sqrt(d)
    w = torch.softmax(s, -1)
    assert torch.allclose(o[1, 0], w @ v[:2, 0], atol=1e-6)


# the (new_lens, prefix_lens) cases of the reference's kernel test (tests/test_prefill_paged_attn.py:183-260)
REFERENCE_CASES = [([32], [0]), ([64], [0]), ([37], [0]), ([16], [32]), ([16], [20]), ([15], [20]), ([20], [200]),
                   ([1], [32]), ([16, 32, 8], [0, 48, 20]), ([16, 24, 32, 8], [0, 0, 0, 0]),
                   ([8, 16, 4, 12], [32, 48, 16, 64]), ([64, 128, 48, 96], [100, 50, 200, 30])]


@pytest.mark.parametrize("new_lens,prefix_lens", REFERENCE_CASES[:9])
def test_attention_with_prefix_equals_tail_of_whole(new_lens, prefix_lens):
    # queries that are the last M of N positions equal the last M rows of attention over all N
    for M, pre in zip(new_lens, prefix_lens):
        N = M + pre
        q, k, v = torch.randn(N, 12, 16) * 0.5, torch.randn(N, 2, 16) * 0.5, torch.randn(N, 2, 16)
        whole = _sdpa(q, k, v)
        tail = P.causal_attention(q[pre:], k, v)
        assert torch.allclose(tail, whole[pre:], atol=1e-5)


def test_attention_window():
    S, d, W = 12, 8, 4
    q, k, v = torch.randn(S, 1, d), torch.randn(S, 1, d), torch.randn(S, 1, d)
    o = P.causal_attention(q, k, v, window=W)
    for p in (0, 3, 4, 11):
        lo = max(0, p - W + 1)
        w = torch.softmax((q[p, 0] @ k[lo:p + 1, 0].T) / math.sqrt(d), -1)
        assert torch.allclose(o[p, 0], w @ v[lo:p + 1, 0], atol=1e-6)


# ---- feed-forward ----------------------------------------------------------
def test_swiglu_reduces_to_silu_and_halves_are_gate_then_up():
    g = torch.randn(4, 10)
    assert torch.allclose(P.swiglu(torch.cat([g, torch.ones(4, 10)], -1)), F.silu(g), atol=1e-6)
    assert torch.count_nonzero(P.swiglu(torch.cat([torch.zeros(4, 10), g], -1))) == 0    # gate = 0 gives 0
    u = torch.randn(4, 10)
    # exchanging the halves changes the result: the gate is the FIRST half
    assert not torch.allclose(P.swiglu(torch.cat([g, u], -1)), P.swiglu(torch.cat([u, g], -1)))
    assert torch.allclose(P.swiglu(torch.cat([g, u], -1)), F.silu(g) * u, atol=1e-6)


# ---- block and model -------------------------------------------------------
def _plain(name):
    return P.PlainModel(model_dir(name))


def test_block_with_zero_projections_is_identity():
    m = _plain("A")
    w = dict(m.w)
    for k in list(w):
        if "o_proj" in k or "down_proj" in k:
            w[k] = torch.zeros_like(w[k])
    x = torch.randn(7, m.cfg.hidden_size)
    assert torch.equal(P.block(x, w, 0, m.cfg, torch.arange(7)), x)


def test_prenorm_feeds_the_normed_stream_but_adds_to_the_raw_one():
    m = _plain("A")
    x = torch.randn(5, m.cfg.hidden_size) * 3
    pos = torch.arange(5)
    p = "model.layers.0"
    a = P.attention_layer(P.rms_norm(x, m.w[f"{p}.input_layernorm.weight"], m.cfg.rms_norm_eps), m.w, p, m.cfg, pos)
    x1 = x + a
    f = P.mlp_layer(P.rms_norm(x1, m.w[f"{p}.post_attention_layernorm.weight"], m.cfg.rms_norm_eps), m.w, p)
    assert torch.allclose(P.block(x, m.w, 0, m.cfg, pos), x1 + f, atol=1e-6)


@pytest.mark.parametrize("name", ["A", "B"])
def test_model_without_layers_is_norm_times_output_matrix(name):
    m = _plain(name)
    cfg0 = P.PlainConfig(**{**m.cfg.__dict__, "num_hidden_layers": 0})
    ids = [3, 9, 200]
    E = m.w["model.embed_tokens.weight"]
    out = E if cfg0.tie_word_embeddings else m.w["lm_head.weight"]
    want = P.rms_norm(E[ids], m.w["model.norm.weight"], cfg0.rms_norm_eps) @ out.T
    assert torch.allclose(P.forward(ids, m.w, cfg0), want, atol=1e-6)
    if not cfg0.tie_word_embeddings:      # an untied model must not use the embedding matrix
        assert not torch.allclose(want, P.rms_norm(E[ids], m.w["model.norm.weight"], cfg0.rms_norm_eps) @ E.T)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_model_is_causal_and_shift_invariant(name):
    m = _plain(name)
    V = m.cfg.vocab_size
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(0, V, (24,), generator=g).tolist()
    full = m.logits(ids)
    assert torch.allclose(m.logits(ids[:10]), full[:10], atol=1e-5)              # later tokens do not matter
    shifted = P.forward(ids, m.w, m.cfg, first_position=64)                       # only distances count
    assert torch.allclose(shifted, full, atol=2e-3)
    ids2 = list(ids)
    ids2[0] = (ids2[0] + 1) % V
    assert not torch.allclose(m.logits(ids2)[-1], full[-1], atol=1e-4)            # the far token does matter


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_a_model_with_its_inner_dimensions_permuted_is_the_same_function(name):
    # the yardstick of the float32 replay tests: in float64 the permuted model gives the same logits to the last
    # places, in float32 it rounds differently (an independent draw of float32 rounding)
    d = model_dir(name)
    m64, m32 = P.PlainModel(d, torch.float64), _plain(name)
    g = torch.Generator().manual_seed(2)
    ids = torch.randint(0, m64.cfg.vocab_size, (20,), generator=g).tolist()
    ref = m64.logits(ids)
    w64 = P.permute_inner_dimensions(m64.w, m64.cfg, g)
    assert any(not torch.equal(w64[k], m64.w[k]) for k in w64)
    with torch.no_grad():
        assert float((P.forward(ids, w64, m64.cfg) - ref).abs().max()) < 1e-11 * float(ref.std())
        a = m32.logits(ids).double()
        b = P.forward(ids, P.permute_inner_dimensions(m32.w, m32.cfg, g), m32.cfg).double()
    assert not torch.equal(a, b)                                         # other roundings
    assert float((b - ref).abs().max()) < 1e-4 * float(ref.std())        # of the same, small, size


def test_dithered_rounding_errs_like_a_bfloat16_rounding_but_anew_every_time():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(200000, generator=g) * 3
    rnd = P.dithered_bf16(g)
    e0, e1, e2 = P.to_bf16(x) - x, rnd(x) - x, rnd(x) - x
    ulp = torch.ldexp(torch.ones_like(x), torch.frexp(x)[1] - 8)
    assert float((e1.abs() / ulp).max()) <= 0.5 + 1e-3                   # within half a unit in the last place (of x + d)
    size = lambda e: float((e / x).pow(2).mean().sqrt())
    assert abs(size(e1) / size(e0) - 1) < 0.02                           # the size of a rounding
    corr = lambda a, b: float((a * b).mean() / (a.pow(2).mean() * b.pow(2).mean()).sqrt())
    assert abs(corr(e1, e0)) < 0.02 and abs(corr(e1, e2)) < 0.02         # drawn anew


def test_qkv_bias_is_used():
    m = _plain("A")
    w = {k: (torch.zeros_like(v) if k.endswith("_proj.bias") else v) for k, v in m.w.items()}
    assert not torch.allclose(P.forward([1, 2, 3], w, m.cfg), m.logits([1, 2, 3]), atol=1e-4)


# ---- sampling --------------------------------------------------------------
def test_top_p_keeps_the_token_that_crosses_and_drops_at_equality():
    logits = torch.log(torch.tensor([0.5, 0.3, 0.15, 0.05]))
    p = P.top_p_probs(logits, 1.0, 0.81)
    assert torch.allclose(p, torch.tensor([0.5, 0.3, 0.15, 0.0]).double() / 0.95, atol=1e-9)
    p = P.top_p_probs(logits, 1.0, 0.79)
    assert torch.allclose(p, torch.tensor([0.5, 0.3, 0.0, 0.0]).double() / 0.8, atol=1e-9)
    p = P.top_p_probs(logits, 1.0, 0.2)           # the first token always stays
    assert torch.allclose(p, torch.tensor([1.0, 0, 0, 0]).double())


def test_temperature_limits_and_inverse_cdf():
    logits = torch.tensor([1.0, 3.0, 2.0, 3.0])
    assert P.sample_greedy(logits) == 1                                            # first maximum
    p = P.temperature_probs(logits, 0.01)
    assert float(p[1] + p[3]) > 0.999999
    p = P.temperature_probs(logits, 1.0)
    assert P.inverse_cdf(p, 0.0) == 0 and P.inverse_cdf(p, 0.999999) == 3
    cum = torch.cumsum(p, 0)
    assert P.inverse_cdf(p, float(cum[0]) + 1e-9) == 1
    onehot = torch.tensor([0.0, 0.0, 1.0, 0.0])
    assert all(P.inverse_cdf(onehot, u) == 2 for u in (0.0, 0.3, 0.99))
