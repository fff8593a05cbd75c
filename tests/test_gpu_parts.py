"""Each part alone against the plain function of the same part, a model whose run order names a
layer twice, and toy parts of every kind (a mixer with state of its own, a feed-forward with routing, a position
encoding, a norm, an arrangement) that the tests register without touching the framework."""

import pytest
import torch

import plain_qwen2 as P
from gpu_util import DEV, DTYPES, tol
from tiny_configs import PAGE_SIZE, model_dir

pytestmark = pytest.mark.gpu


def close(a, b, dtype, scale=1.0):
    rtol, atol = tol(dtype)
    if dtype == torch.float32:
        rtol, atol = 1e-4, 1e-4         # several chained kernels
    a, b = a.float().cpu(), b.float().cpu()
    err = (a - b).abs()
    assert bool((err <= atol * scale + rtol * b.abs()).all()), f"max err {float(err.max()):.3e}"


def close_to_plain(got, exact, rounded, dtype):
    """float32: summation order only.  bfloat16: within twice the error that rounding every
    activation to bfloat16 causes in the plain computation of the same thing (``rounded``)."""
    got, exact = got.float().cpu(), exact.float()
    err = (got - exact).abs()
    if dtype == torch.float32:
        assert float(err.max()) <= 1e-4 * max(1.0, float(exact.abs().max())), f"max err {float(err.max()):.3e}"
    else:
        noise = (rounded.float() - exact).abs()
        assert float(err.max()) <= 2.0 * float(noise.max()), f"max {float(err.max()):.3e} vs noise {float(noise.max()):.3e}"
        assert float((err ** 2).mean().sqrt()) <= 1.5 * float((noise ** 2).mean().sqrt())


def one_seq_context(n_new, n_cached, runner, req="r"):
    """A StepContext for one request bringing n_new tokens after n_cached cached ones."""
    from pico_vllm_amd.engine.batch import SeqStep, build_context
    m = runner.manager
    if req not in m.requests:
        m.add_request(req)
    m.advance(req, n_cached)
    assert m.grow(req, n_cached + n_new)
    seq = SeqStep(req, [0] * n_new, [])
    return build_context([seq], m, runner.buffers, runner.model.dtype, runner.model.spec.vocab_size)


def runner_for(name, dtype):
    from pico_vllm_amd.engine.step import ModelRunner
    from pico_vllm_amd.parts.model import load_model
    model = load_model(model_dir(name), "float32" if dtype == torch.float32 else "bfloat16", DEV)
    return ModelRunner(model, PAGE_SIZE[name], 64, 4, 256, 256)


def whole(delta):
    """What a part hands to the next norm may be a float32 stack of partial sums over ranges of k."""
    return delta.float().sum(0) if delta.dim() == 3 else delta.float()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_attention_and_mlp_and_block_parts(name, dtype):
    r = runner_for(name, dtype)
    plain = P.PlainModel(model_dir(name))
    cfg = plain.cfg
    H, S = cfg.hidden_size, 37
    blk = r.model.layers[0]
    g = torch.Generator().manual_seed(0)
    x = torch.randn(S, H, generator=g)
    h = x.to(dtype)
    pos = torch.arange(S)
    # mixer alone: whole sequence in one step, then the same in two portions through the cache
    ctx = one_seq_context(S, 0, r)
    out = blk.mixer.forward(h.to(DEV), ctx, r.storage.layer(0))
    want = P.attention_layer(h.float(), plain.w, "model.layers.0", cfg, pos)
    rounded = P.attention_layer(h.float(), plain.w, "model.layers.0", cfg, pos, rnd=P.to_bf16)
    close_to_plain(out, want, rounded, dtype)
    r.manager.free_request("r")
    ctx = one_seq_context(20, 0, r)
    first = blk.mixer.forward(h[:20].to(DEV), ctx, r.storage.layer(0))
    ctx = one_seq_context(S - 20, 20, r)
    second = blk.mixer.forward(h[20:].to(DEV), ctx, r.storage.layer(0))
    close_to_plain(torch.cat([first, second]), want, rounded, dtype)
    # feed-forward alone
    f = whole(blk.parts["ff"].forward(h.to(DEV), ctx))
    wantf = P.mlp_layer(h.float(), plain.w, "model.layers.0")
    close_to_plain(f, wantf, P.mlp_layer(h.float(), plain.w, "model.layers.0", rnd=P.to_bf16), dtype)
    # norm alone (the part, with the fused add)
    delta = torch.randn(S, H, generator=g).to(dtype)
    resid = x.clone().to(DEV)
    n = blk.parts["norm1"].add_norm(resid, delta.to(DEV))
    close(n, P.rms_norm(x + delta.float(), plain.w["model.layers.0.input_layernorm.weight"], cfg.rms_norm_eps), dtype, 3)
    # the whole block: pending delta in, pending delta out
    r.manager.free_request("r")
    ctx = one_seq_context(S, 0, r)
    resid = x.clone().to(DEV)
    resid2, pending = blk.forward(resid, None, ctx, r.storage.layer(0))
    wantb = P.block(x, plain.w, 0, cfg, pos)
    close_to_plain(resid2 + whole(pending), wantb, P.block(x, plain.w, 0, cfg, pos, rnd=P.to_bf16), dtype)


@pytest.mark.parametrize("d", [16, 64, 24, 40])
@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_part_with_a_window(dtype, d):
    """The same mixer class with window = 24: its cache group gives pages back, and the result is
    the plain windowed attention (head size 16: the 32-query matrix-core kernels in bfloat16, 64: the 16-query ones,
    24 and 40: no multiple of 16, the plain kernel in both precisions)."""
    from pico_vllm_amd.cache.manager import CacheManager
    from pico_vllm_amd.cache.storage import CacheStorage
    from pico_vllm_amd.engine.batch import BatchBuffers, SeqStep, build_context
    from pico_vllm_amd.parts.registry import build_part
    from pico_vllm_amd.parts.spec import PartSpec
    H, nq, nkv, W, Pg = 96, 6, 2, 24, 8
    spec = PartSpec("gqa_attention", dict(hidden_size=H, num_heads=nq, num_kv_heads=nkv, head_dim=d, qkv_bias=True,
                                          window=W, position=PartSpec("rotary_half", {"rotary_dim": d, "theta": 1e4})))
    mixer = build_part("mixer", spec, act_dtype=dtype)
    g = torch.Generator().manual_seed(1)
    w = {p.name: (torch.randn(p.shape, generator=g) * (0.3 if p.role == "matrix" else 0.1)).to(torch.bfloat16)
         for p in mixer.param_specs()}
    mixer.load({k: v.to(dtype) for k, v in w.items()}, torch.device(DEV), dtype)
    mgr = CacheManager({0: mixer.cache_spec()}, Pg, 8, 1)          # 8 pages of 8: a 100-token request only fits
    store = CacheStorage(mgr, {0: mixer.cache_spec()}, dtype, torch.device(DEV))   # because the window frees pages
    buf = BatchBuffers(torch.device(DEV), 64, 1, 16, 1)
    S = 100
    x = torch.randn(S, H, generator=g).to(dtype)
    mgr.add_request("r")
    outs, i = [], 0
    for n in [13, 2, 30, 1, 1, 17, 36]:
        assert mgr.grow("r", i + n)
        ctx = build_context([SeqStep("r", [0] * n, [])], mgr, buf, dtype, 10)
        out = mixer.forward(x[i:i + n].to(DEV), ctx, store.layer(0))
        outs.append(out.float().sum(0) if out.dim() == 3 else out.float())      # partial sums over ranges of k, or the product
        i += n
        mgr.advance("r", i)
        mgr.check()
    assert i == S and mgr.groups[0].pool.reuse_count > 0
    # plain: same projections, windowed attention
    wf = {k: v.float() for k, v in w.items()}
    qkv = x.float() @ torch.cat([wf["q_proj.weight"], wf["k_proj.weight"], wf["v_proj.weight"]]).T \
        + torch.cat([wf["q_proj.bias"], wf["k_proj.bias"], wf["v_proj.bias"]])
    q, k, v = P.split_qkv(qkv, nq, nkv, d)
    cos, sin = P.rope_tables(torch.arange(S), d, 1e4)
    o = P.causal_attention(P.apply_rope(q, cos, sin), P.apply_rope(k, cos, sin), v, window=W)
    want = o.reshape(S, nq * d) @ wf["o_proj.weight"].T
    close(torch.cat(outs), want, dtype, scale=float(want.abs().max()))


@pytest.mark.parametrize("dtype", DTYPES)
def test_run_order_may_name_a_layer_twice(dtype):
    """Layers run in the order [0, 1, 0]: layer 0's weights twice, each run with a cache of its own."""
    import dataclasses
    from pico_vllm_amd.config.registry import load_model_description
    from pico_vllm_amd.engine.batch import SeqStep
    from pico_vllm_amd.engine.step import ModelRunner
    from pico_vllm_amd.parts.model import DecoderModel
    from pico_vllm_amd.parts.spec import RunEntry
    from pico_vllm_amd.weights.loader import load_checkpoint
    d = model_dir("A")
    _, cfg, spec = load_model_description(d)
    spec = dataclasses.replace(spec, run_order=[RunEntry(0), RunEntry(1), RunEntry(0)])
    model = DecoderModel(spec, dtype, torch.device(DEV))
    model.load(load_checkpoint(d, model.param_specs(), dtype))
    assert sorted(model.cache_specs()) == [0, 1, 2]
    r = ModelRunner(model, 16, 32, 2, 128, 128)
    plain = P.PlainModel(d)
    toks = torch.randint(0, 255, (45,), generator=torch.Generator().manual_seed(2)).tolist()
    x = plain.w["model.embed_tokens.weight"][toks].float()
    pos = torch.arange(len(toks))
    for i in (0, 1, 0):
        x = P.block(x, plain.w, i, plain.cfg, pos)
    want = P.rms_norm(x, plain.w["model.norm.weight"], plain.cfg.rms_norm_eps) @ plain.w["model.embed_tokens.weight"].T
    xr = plain.w["model.embed_tokens.weight"][toks].float()
    for i in (0, 1, 0):
        xr = P.block(xr, plain.w, i, plain.cfg, pos, rnd=P.to_bf16)
    rounded = P.to_bf16(P.rms_norm(xr, plain.w["model.norm.weight"], plain.cfg.rms_norm_eps)) \
        @ plain.w["model.embed_tokens.weight"].T
    r.manager.add_request("r")
    got, i = [], 0
    for n in (20, 3, 1, 21):
        assert r.manager.grow("r", i + n)
        seq = [SeqStep("r", toks[i:i + n], list(range(n)))]
        got.append(r.step(seq))
        r.advance(seq)
        i += n
    close_to_plain(torch.cat(got), want, rounded, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_toy_mixer_with_state_of_its_own_registers_builds_and_steps(dtype):
    """A mixer that keeps a running mean of its inputs per request (a fixed-size state, no pages)
    is defined here, registered, put into a new architecture together with the framework's norm
    and feed-forward, loaded from a random-weights folder and stepped in portions; the framework's
    files are not changed for it."""
    import tempfile
    from pico_vllm_amd.config.registry import register_architecture
    from pico_vllm_amd.engine.batch import SeqStep
    from pico_vllm_amd.engine.step import ModelRunner
    from pico_vllm_amd.parts.base import Mixer
    from pico_vllm_amd.parts.model import load_model
    from pico_vllm_amd.parts.registry import register_part
    from pico_vllm_amd.parts.spec import CacheSpec, LayerSpec, ModelSpec, ParamSpec, PartSpec, RunEntry
    from pico_vllm_amd.weights.random_init import write_random_model

    @register_part("mixer", "toy_running_mean")
    class RunningMean(Mixer):
        """y_t = W * mean(x_0 .. x_t); state per request: [sum (H values), count]."""

        def __init__(self, hidden_size, act_dtype=torch.bfloat16):
            self.H, self.act_dtype = hidden_size, act_dtype

        def cache_spec(self):
            return CacheSpec("state", state_shape=(self.H + 1,), state_dtype="float32")

        def param_specs(self):
            return [ParamSpec("mix.weight", (self.H, self.H), std=0.2)]

        def load(self, tensors, device, dtype):
            self.w = tensors["mix.weight"].to(device).float()

        def forward(self, x, ctx, cache):
            H = self.H
            if ctx.all_decode:
                # one token a sequence: device work only, so the step may be recorded into a graph and replayed
                # (padding rows of a recorded batch all point at the spare slot)
                slots = ctx.state_slots[:ctx.num_seqs].long()
                st = cache.state.index_select(0, slots)
                sums = st[:, :H] + x.float()
                counts = st[:, H] + 1
                cache.state.index_copy_(0, slots, torch.cat([sums, counts[:, None]], 1))
                return ((sums / counts[:, None]) @ self.w.T).to(x.dtype)
            out = torch.empty_like(x)
            cu = ctx.host["cu_seqlens"]
            slots = ctx.state_slots.tolist()
            for b in range(ctx.num_seqs):
                lo, hi = int(cu[b]), int(cu[b + 1])
                st = cache.state[slots[b]]                      # zero when the request is new: the framework sees to it
                xs = x[lo:hi].float()
                sums = st[:self.H] + torch.cumsum(xs, 0)
                counts = st[self.H] + torch.arange(1, hi - lo + 1, device=x.device)
                out[lo:hi] = ((sums / counts[:, None]) @ self.w.T).to(x.dtype)
                st[:self.H] = sums[-1]
                st[self.H] = counts[-1]
            return out

    def toy_spec(cfg):
        H = cfg["hidden_size"]
        norm = PartSpec("rms_norm", {"size": H, "eps": 1e-5})
        layers = [LayerSpec(f"toy.layers.{i}", "prenorm", {
            "norm1": ("ln1", norm), "mixer": ("mixer", PartSpec("toy_running_mean", {"hidden_size": H})),
            "norm2": ("ln2", norm), "ff": ("mlp", PartSpec("swiglu_mlp", {"hidden_size": H, "intermediate_size": 2 * H}))})
            for i in range(cfg["num_hidden_layers"])]
        return ModelSpec(H, cfg["vocab_size"], "toy.embed.weight", layers, [RunEntry(i) for i in range(len(layers))],
                         norm, "toy.norm", None)

    register_architecture("ToyRunningMeanLM", lambda raw: raw, toy_spec)
    cfg = {"architectures": ["ToyRunningMeanLM"], "hidden_size": 48, "vocab_size": 100, "num_hidden_layers": 2}
    with tempfile.TemporaryDirectory() as d:
        write_random_model(d, cfg, seed=0, std_overrides={"mlp": 0.2, "embed": 0.5})
        model = load_model(d, "float32" if dtype == torch.float32 else "bfloat16", DEV)
        r = ModelRunner(model, 16, 4, 3, 64, 64)
        assert r.manager.state_layers == [0, 1] and not r.manager.groups
        toks = {"a": list(range(1, 30)), "b": list(range(50, 61))}
        # whole
        whole = {}
        for rid, t in toks.items():
            r.manager.add_request(rid)
            s = [SeqStep(rid, t, list(range(len(t))))]
            whole[rid] = r.step(s)
            r.manager.free_request(rid)
        # in portions, both requests in the same steps, state carried between steps in their slots
        for rid in toks:
            r.manager.add_request(rid)
        got = {rid: [] for rid in toks}
        cuts = {"a": [5, 1, 10, 13], "b": [2, 7, 1, 1]}
        fed = {rid: 0 for rid in toks}
        for k in range(4):
            seqs = []
            for rid in toks:
                n = cuts[rid][k]
                seqs.append(SeqStep(rid, toks[rid][fed[rid]:fed[rid] + n], list(range(n))))
            out = r.step(seqs)
            r.advance(seqs)
            o = 0
            for s in seqs:
                got[s.req].append(out[o:o + len(s.tokens)])
                o += len(s.tokens)
                fed[s.req] += len(s.tokens)
        for rid in toks:
            close(torch.cat(got[rid]), whole[rid], dtype, scale=float(whole[rid].std()) * 3)
        assert whole["a"].shape == (29, 100) and float(whole["a"].std()) > 0.01
        del r, model

        # through the entry point, with graphs: five requests through two state slots (every slot is taken again by a
        # later request and must start from zero), decode steps replayed from graphs; the same tokens as without graphs
        # and as each request alone in an engine of its own
        from pico_vllm_amd import LLM, SamplingParams
        prompts = [list(range(1, 12)), [7, 3], list(range(40, 70)), [9], list(range(80, 97))]
        sp = SamplingParams(max_new_tokens=12, temperature=0.0, ignore_eos=True)
        kind = "float32" if dtype == torch.float32 else "bfloat16"

        def run(ps, **kw):
            llm = LLM(model=d, dtype=kind, block_size=16, num_gpu_blocks=8, max_seq_len=64, max_num_batched_tokens=64, **kw)
            outs = [o.token_ids for o in llm.generate(ps, sp)]
            return outs, llm.engine.runner
        graphed, runner = run(prompts, max_num_seqs=2, use_cuda_graph=True, max_batch_size=2)
        assert runner.use_graph and runner._graphs, "the toy mixer is graph-safe: decode steps were to be replayed"
        eager, _ = run(prompts, max_num_seqs=2, use_cuda_graph=False)
        assert graphed == eager
        if dtype == torch.float32:          # alone the batch has another shape: in bfloat16 the library's product may round otherwise
            alone = [run([p], max_num_seqs=1, use_cuda_graph=False)[0][0] for p in prompts]
            assert eager == alone
        one_slot, _ = run(prompts, max_num_seqs=1, use_cuda_graph=False)      # every request takes slot 0 after another
        assert one_slot == eager or dtype != torch.float32


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_toy_mixer_that_keeps_nothing_beside_a_layer_with_attention(dtype):
    """A mixer that works on every token by itself (y = (x Wv) * sigmoid(x Wg)) says nothing about a cache: the
    default is none, its run gets no pages and no state, and the attention layer behind it has the model's only
    group of pages.  Whole against a plain computation, portions against whole, and generation with recorded decode
    steps against generation without."""
    import tempfile
    from pico_vllm_amd.config.registry import register_architecture
    from pico_vllm_amd.engine.batch import SeqStep
    from pico_vllm_amd.engine.step import ModelRunner
    from pico_vllm_amd.parts.base import Mixer
    from pico_vllm_amd.parts.model import load_model
    from pico_vllm_amd.parts.registry import register_part
    from pico_vllm_amd.parts.spec import LayerSpec, ModelSpec, ParamSpec, PartSpec, RunEntry
    from pico_vllm_amd.weights.random_init import write_random_model
    H, V, NQ, NKV, D, I = 48, 120, 3, 1, 16, 80

    @register_part("mixer", "toy_gated_linear")
    class GatedLinear(Mixer):
        def __init__(self, hidden_size, act_dtype=torch.bfloat16):
            self.H = hidden_size

        def param_specs(self):
            return [ParamSpec("value.weight", (self.H, self.H), std=0.3), ParamSpec("gate.weight", (self.H, self.H), std=0.3)]

        def load(self, tensors, device, dtype):
            self.wv, self.wg = tensors["value.weight"].to(device), tensors["gate.weight"].to(device)

        def forward(self, x, ctx, cache):
            assert cache is None
            return ((x @ self.wv.T).float() * torch.sigmoid((x @ self.wg.T).float())).to(x.dtype)

    def toy_spec(cfg):
        norm = PartSpec("rms_norm", {"size": H, "eps": 1e-5})
        attn = PartSpec("gqa_attention", {"hidden_size": H, "num_heads": NQ, "num_kv_heads": NKV, "head_dim": D, "qkv_bias": True,
                                          "window": 0, "position": PartSpec("rotary_half", {"rotary_dim": D, "theta": 100.0})})
        ff = PartSpec("swiglu_mlp", {"hidden_size": H, "intermediate_size": I})
        mixers = [PartSpec("toy_gated_linear", {"hidden_size": H}), attn]
        layers = [LayerSpec(f"toy.layers.{i}", "prenorm", {"norm1": ("ln1", norm), "mixer": ("mix", mixers[i]), "norm2": ("ln2", norm),
                                                          "ff": ("ff", ff)}) for i in range(2)]
        return ModelSpec(H, V, "toy.embed.weight", layers, [RunEntry(0), RunEntry(1)], norm, "toy.norm", None)

    register_architecture("ToyGatedLinearLM", lambda raw: raw, toy_spec)
    rnd = P._same if dtype == torch.float32 else P.to_bf16
    kind = "float32" if dtype == torch.float32 else "bfloat16"
    with tempfile.TemporaryDirectory() as d:
        write_random_model(d, {"architectures": ["ToyGatedLinearLM"]}, seed=6, std_overrides={"mix": 0.3, "embed": 0.5, "ff": 0.3})
        w = {k: v.float() for k, v in P.read_weights(d).items()}
        model = load_model(d, kind, DEV)
        r = ModelRunner(model, 8, 16, 3, 64, 64)
        assert [g.layers for g in r.manager.groups] == [[1]] and not r.manager.state_layers
        assert r.storage.layer(0) is None and r.storage.layer(1) is not None
        toks = torch.randint(0, V, (37,), generator=torch.Generator().manual_seed(2)).tolist()

        def plain(rnd):
            pos = torch.arange(len(toks))
            x = w["toy.embed.weight"][toks]
            h = rnd(P.rms_norm(x, w["toy.layers.0.ln1.weight"], 1e-5))
            x = x + rnd(rnd(h @ w["toy.layers.0.mix.value.weight"].T) * torch.sigmoid(rnd(h @ w["toy.layers.0.mix.gate.weight"].T)))
            for i in range(2):
                p = f"toy.layers.{i}"
                if i == 1:
                    h = rnd(P.rms_norm(x, w[f"{p}.ln1.weight"], 1e-5))
                    W = torch.cat([w[f"{p}.mix.{n}_proj.weight"] for n in "qkv"], 0)
                    b = torch.cat([w[f"{p}.mix.{n}_proj.bias"] for n in "qkv"], 0)
                    q, k, v = P.split_qkv(rnd(h @ W.T + b), NQ, NKV, D)
                    cos, sin = P.rope_tables(pos, D, 100.0)
                    o = rnd(P.causal_attention(rnd(P.apply_rope(q, cos, sin)), rnd(P.apply_rope(k, cos, sin)), v,
                                               rnd_p=None if rnd is P._same else rnd))
                    x = x + rnd(o.reshape(len(toks), NQ * D) @ w[f"{p}.mix.o_proj.weight"].T)
                h = rnd(P.rms_norm(x, w[f"{p}.ln2.weight"], 1e-5))
                gu = torch.cat([w[f"{p}.ff.gate_proj.weight"], w[f"{p}.ff.up_proj.weight"]], 0)
                x = x + rnd(rnd(P.swiglu(rnd(h @ gu.T))) @ w[f"{p}.ff.down_proj.weight"].T)
            return rnd(P.rms_norm(x, w["toy.norm.weight"], 1e-5)) @ w["toy.embed.weight"].T

        r.manager.add_request("w")
        assert r.manager.grow("w", len(toks))
        whole = r.step([SeqStep("w", toks, list(range(len(toks))))])
        r.manager.free_request("w")
        close_to_plain(whole, plain(P._same), plain(rnd), dtype)
        r.manager.add_request("a")
        got, fed = [], 0
        for n in (11, 1, 2, 20, 1, 1, 1):
            assert r.manager.grow("a", fed + n)
            seqs = [SeqStep("a", toks[fed:fed + n], list(range(n)))]
            got.append(r.step(seqs))
            r.advance(seqs)
            fed += n
        close(torch.cat(got), whole, dtype, scale=float(whole.std()) * 3)
        r.manager.check()
        del r, model
        from pico_vllm_amd import LLM, SamplingParams
        prompts = [toks[:9], toks[9:12], toks[12:]]
        sp = SamplingParams(max_new_tokens=10, temperature=0.0, ignore_eos=True)

        def run(**kw):
            llm = LLM(model=d, dtype=kind, block_size=8, num_gpu_blocks=24, max_seq_len=64, max_num_seqs=2, max_num_batched_tokens=64, **kw)
            return [o.token_ids for o in llm.generate(prompts, sp)], llm.engine.runner
        graphed, runner = run(use_cuda_graph=True, max_batch_size=2)
        assert runner.use_graph and runner._graphs
        assert graphed == run(use_cuda_graph=False)[0]


def test_a_part_that_decides_on_the_host_keeps_the_model_out_of_graphs():
    """``graph_safe = False`` on any part: the runner never records a graph, whatever the options say."""
    import dataclasses
    from pico_vllm_amd.config.registry import load_model_description
    from pico_vllm_amd.engine.step import ModelRunner
    from pico_vllm_amd.parts.base import FeedForward
    from pico_vllm_amd.parts.model import DecoderModel
    from pico_vllm_amd.parts.registry import register_part
    from pico_vllm_amd.parts.spec import LayerSpec, PartSpec

    @register_part("feed_forward", "toy_host_decides")
    class HostDecides(FeedForward):
        graph_safe = False

        def __init__(self, act_dtype=torch.bfloat16):
            pass

        def forward(self, x, ctx):
            return x * float(len(ctx.host["cu_seqlens"]))

    _, cfg, spec = load_model_description(model_dir("A"))
    safe = DecoderModel(spec, torch.bfloat16, torch.device(DEV))
    assert safe.is_graph_safe()
    l0 = spec.layers[0]
    layers = [LayerSpec(l0.prefix, l0.block, {**l0.slots, "ff": ("mlp", PartSpec("toy_host_decides", {}))})] + list(spec.layers[1:])
    model = DecoderModel(dataclasses.replace(spec, layers=layers), torch.bfloat16, torch.device(DEV))
    assert not model.is_graph_safe()
    assert ModelRunner(safe, 16, 8, 2, 64, 64, use_graph=True).use_graph
    assert not ModelRunner(model, 16, 8, 2, 64, 64, use_graph=True).use_graph


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_toy_feed_forward_with_routing_and_a_toy_position_encoding(dtype):
    """Two more toy parts, defined and registered here: a feed-forward that sends every token to the
    one of three small experts whose router logit is largest (router in float32), and a position
    encoding that multiplies the entries of q and k by cosines of the position.  Layer 0 has the
    routed feed-forward, layer 1 the framework's dense one; both use the framework's attention with the toy
    encoding.  The engine's whole prompt equals a plain computation written out below, and portions
    equal the whole."""
    import tempfile
    from pico_vllm_amd.config.registry import register_architecture
    from pico_vllm_amd.engine.batch import SeqStep
    from pico_vllm_amd.engine.step import ModelRunner
    from pico_vllm_amd.ops import kernels
    from pico_vllm_amd.ops.linear import Linear
    from pico_vllm_amd.parts.base import FeedForward, PositionEncoding
    from pico_vllm_amd.parts.model import load_model
    from pico_vllm_amd.parts.registry import register_part
    from pico_vllm_amd.parts.spec import LayerSpec, ModelSpec, ParamSpec, PartSpec, RunEntry
    from pico_vllm_amd.weights.random_init import write_random_model

    H, V, NQ, NKV, D, E, I = 40, 90, 3, 1, 16, 3, 24

    def gate_of(positions, d, base):
        return torch.cos(positions.float()[:, None] / (base ** (torch.arange(d, device=positions.device).float() / d)))

    @register_part("position", "toy_cosine_gate")
    class CosineGate(PositionEncoding):
        def __init__(self, base, act_dtype=torch.bfloat16):
            self.base = base

        def rotate_and_store(self, qkv, ctx, kv, block_table, nq, nkv, d):
            T = qkv.shape[0]
            qk = qkv[:, :(nq + nkv) * d].view(T, nq + nkv, d)
            qk.copy_((qk.float() * gate_of(ctx.positions[:T], d, self.base)[:, None, :]).to(qkv.dtype))
            kernels.rope_kv_store(qkv, None, ctx.slot_mapping[kv.group], kv.k, kv.v, nq, nkv, d, 0)

    @register_part("feed_forward", "toy_top1_experts")
    class Top1Experts(FeedForward):
        def __init__(self, hidden_size, num_experts, expert_size, act_dtype=torch.bfloat16):
            self.H, self.E, self.I = hidden_size, num_experts, expert_size

        def param_specs(self):
            out = [ParamSpec("router.weight", (self.E, self.H), std=1.0)]
            for e in range(self.E):
                out += [ParamSpec(f"experts.{e}.in.weight", (self.I, self.H), std=0.3),
                        ParamSpec(f"experts.{e}.out.weight", (self.H, self.I), std=0.3)]
            return out

        def load(self, tensors, device, dtype):
            self.router = tensors["router.weight"].to(device).float()
            # the experts' matrices in lists: what the part reports as streamed bytes finds them there
            self.w_in = [Linear(tensors[f"experts.{e}.in.weight"].to(device)) for e in range(self.E)]
            self.w_out = [Linear(tensors[f"experts.{e}.out.weight"].to(device)) for e in range(self.E)]

        def weight_bytes(self):
            return super().weight_bytes() + self.router.numel() * self.router.element_size()

        def flops(self, tokens, pairs):
            # the router for every token, and the one expert it chose: not what the default counts (every matrix)
            return 2.0 * tokens * (self.E * self.H + 2 * self.I * self.H)

        def forward(self, x, ctx):
            choice = (x.float() @ self.router.T).argmax(-1)            # router logits in float32
            out = torch.zeros_like(x)
            for e in range(self.E):
                rows = (choice == e).nonzero().flatten()
                if rows.numel():
                    h = torch.relu(x[rows] @ self.w_in[e].weight.T)
                    out[rows] = h @ self.w_out[e].weight.T
            return out

    def toy_spec(cfg):
        norm = PartSpec("rms_norm", {"size": H, "eps": 1e-5})
        attn = PartSpec("gqa_attention", {"hidden_size": H, "num_heads": NQ, "num_kv_heads": NKV, "head_dim": D, "qkv_bias": False,
                                          "window": 0, "position": PartSpec("toy_cosine_gate", {"base": 50.0})})
        ffs = [PartSpec("toy_top1_experts", {"hidden_size": H, "num_experts": E, "expert_size": I}),
               PartSpec("swiglu_mlp", {"hidden_size": H, "intermediate_size": I})]
        layers = [LayerSpec(f"toy.layers.{i}", "prenorm", {"norm1": ("ln1", norm), "mixer": ("attn", attn), "norm2": ("ln2", norm),
                                                          "ff": ("ff", ffs[i])}) for i in range(2)]
        return ModelSpec(H, V, "toy.embed.weight", layers, [RunEntry(0), RunEntry(1)], norm, "toy.norm", None)

    register_architecture("ToyRoutedLM", lambda raw: raw, toy_spec)
    cfg = {"architectures": ["ToyRoutedLM"]}
    rnd = P._same if dtype == torch.float32 else P.to_bf16
    with tempfile.TemporaryDirectory() as d:
        write_random_model(d, cfg, seed=4, std_overrides={"attn": 0.4, "embed": 0.5, "ff.gate": 0.3, "ff.up": 0.3, "ff.down": 0.3})
        w = {k: v.float() for k, v in P.read_weights(d).items()}
        model = load_model(d, "float32" if dtype == torch.float32 else "bfloat16", DEV)
        r = ModelRunner(model, 8, 16, 3, 64, 64)
        toks = torch.randint(0, V, (43,), generator=torch.Generator().manual_seed(1)).tolist()
        # what a step streams and computes is asked of the parts: all three experts' matrices and the router, the dense
        # feed-forward of the other layer, both attentions, the tied output matrix
        size = 4 if dtype == torch.float32 else 2
        attn_w = (NQ + 2 * NKV) * D * H + H * NQ * D
        assert model.num_weight_bytes() == size * (2 * attn_w + E * 2 * I * H + 3 * I * H + V * H) + 4 * E * H
        assert r.decode_bytes([10, 5]) == model.num_weight_bytes() + 15 * 2 * (2 * NKV * D * size)
        T, pairs = 7, 7 * 8 // 2
        assert model.flops(T, pairs, 2) == 2.0 * T * (2 * attn_w + (E * H + 2 * I * H) + 3 * I * H) \
            + 2 * 4.0 * NQ * D * pairs + 2.0 * 2 * V * H

        # the plain computation, whole sequence, no cache
        def plain(rnd):
            pos = torch.arange(len(toks))
            x = w["toy.embed.weight"][toks]
            margins = []
            for i in range(2):
                p = f"toy.layers.{i}"
                h = rnd(P.rms_norm(x, w[f"{p}.ln1.weight"], 1e-5))
                W = torch.cat([w[f"{p}.attn.{n}_proj.weight"] for n in "qkv"], 0)
                q, k, v = P.split_qkv(rnd(h @ W.T), NQ, NKV, D)
                g = gate_of(pos, D, 50.0)[:, None, :]
                o = rnd(P.causal_attention(rnd(q * g), rnd(k * g), v))
                x = x + rnd(o.reshape(len(toks), NQ * D) @ w[f"{p}.attn.o_proj.weight"].T)
                h = rnd(P.rms_norm(x, w[f"{p}.ln2.weight"], 1e-5))
                if i == 0:
                    logits = h @ w[f"{p}.ff.router.weight"].T
                    top = logits.topk(2, -1).values
                    margins.append(float((top[:, 0] - top[:, 1]).min()))
                    f = torch.zeros_like(h)
                    for t, e in enumerate(logits.argmax(-1).tolist()):
                        f[t] = rnd(rnd(torch.relu(h[t] @ w[f"{p}.ff.experts.{e}.in.weight"].T)) @ w[f"{p}.ff.experts.{e}.out.weight"].T)
                    assert len(set(logits.argmax(-1).tolist())) == E          # every expert has tokens
                else:
                    gu = torch.cat([w[f"{p}.ff.gate_proj.weight"], w[f"{p}.ff.up_proj.weight"]], 0)
                    f = rnd(rnd(P.swiglu(rnd(h @ gu.T))) @ w[f"{p}.ff.down_proj.weight"].T)
                x = x + f
            return rnd(P.rms_norm(x, w["toy.norm.weight"], 1e-5)) @ w["toy.embed.weight"].T, min(margins)

        want, margin = plain(P._same)
        assert margin > 0.05, "a token sits between two experts: take another seed"
        r.manager.add_request("w")
        assert r.manager.grow("w", len(toks))
        whole_logits = r.step([SeqStep("w", toks, list(range(len(toks))))])
        r.manager.free_request("w")
        close_to_plain(whole_logits, want, plain(rnd)[0], dtype)
        # in portions, a second request beside it
        r.manager.add_request("a")
        r.manager.add_request("b")
        got, fed = [], 0
        for n, nb in ((9, 2), (1, 1), (2, 5), (24, 1), (7, 1)):
            assert r.manager.grow("a", fed + n) and r.manager.grow("b", r.manager.num_computed("b") + nb)
            seqs = [SeqStep("b", toks[:nb], []), SeqStep("a", toks[fed:fed + n], list(range(n)))]
            got.append(r.step(seqs))
            r.advance(seqs)
            fed += n
        close(torch.cat(got), whole_logits, dtype, scale=float(whole_logits.std()) * 3)


def test_a_block_leaves_the_norm_of_a_single_row_to_a_part_that_takes_it():
    """With one row in bfloat16 the block hands a part that says so the norm's operands instead of
    normed activations.  A part that runs the norm itself sees what the norm's kernel gives, the
    residual stream is summed either way, parts that do not say so get tensors, and a part that
    takes the operands and drops them is caught."""
    from pico_vllm_amd.parts.base import DeferredNorm, FeedForward, Mixer
    from pico_vllm_amd.parts.block import PreNormBlock
    from pico_vllm_amd.parts.norm import RMSNorm
    H = 128
    g = torch.Generator().manual_seed(0)
    seen = []

    class Plain(Mixer):                       # does not take deferred norms
        def forward(self, x, ctx, cache):
            seen.append(("mixer", type(x)))
            return 0.5 * x.float()

    class Runs(FeedForward):
        takes_deferred_norm = True

        def forward(self, x, ctx):
            seen.append(("ff", type(x)))
            h = x.run() if isinstance(x, DeferredNorm) else x
            return 2.0 * h.float()

    class Drops(FeedForward):
        takes_deferred_norm = True

        def forward(self, x, ctx):
            return torch.zeros(x.resid_in.shape, device=DEV)

    def block(ff):
        norms = [RMSNorm(H, 1e-5, torch.bfloat16) for _ in range(2)]
        for n in norms:
            n.load({"weight": 1 + 0.1 * torch.randn(H, generator=g)}, DEV, torch.bfloat16)
        return PreNormBlock({"norm1": norms[0], "mixer": Plain(), "norm2": norms[1], "ff": ff}), norms

    for T in (1, 3):
        seen.clear()
        blk, norms = block(Runs())
        x0 = torch.randn(T, H, generator=g)
        pend = torch.randn(T, H, generator=g)
        resid, out = blk.forward(x0.clone().to(DEV), pend.to(DEV), None, None)
        assert seen[0] == ("mixer", torch.Tensor)
        assert seen[1] == ("ff", DeferredNorm if T == 1 else torch.Tensor)
        r1 = x0 + pend
        h1 = P.rms_norm(r1, norms[0].weight.cpu(), 1e-5).bfloat16().float()
        r2 = r1 + 0.5 * h1
        close(resid, r2, torch.float32, scale=4)
        close(out, 2.0 * P.rms_norm(r2, norms[1].weight.cpu(), 1e-5), torch.bfloat16, scale=8)
    blk, _ = block(Drops())
    with pytest.raises(RuntimeError, match="deferred norm"):
        blk.forward(torch.randn(1, H).to(DEV), None, None, None)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_description_with_an_embedding_multiplier_a_head_bias_and_a_soft_cap(dtype):
    """What surrounds the layers is data of the model description too: the framework's layers between an embedding
    times 3, an output matrix with a bias and logits capped at 2 tanh(x / 2), registered here as an architecture of
    its own, written with random weights, stepped in portions and compared with the plain parts."""
    import dataclasses
    import tempfile
    from pico_vllm_amd.config.model_config import Qwen2Config
    from pico_vllm_amd.config.qwen2 import qwen2_spec
    from pico_vllm_amd.config.registry import register_architecture
    from pico_vllm_amd.engine.batch import SeqStep
    from pico_vllm_amd.engine.step import ModelRunner
    from pico_vllm_amd.parts.model import load_model
    from pico_vllm_amd.weights.random_init import write_random_model
    from tiny_configs import TINY_B, strong
    SCALE, CAP = 3.0, 2.0
    register_architecture("ToyCappedLM", Qwen2Config.from_dict,
                          lambda cfg: dataclasses.replace(qwen2_spec(cfg), embed_scale=SCALE, logit_softcap=CAP,
                                                          head_bias_name="toy_head.bias"))
    cfg = dict(TINY_B, architectures=["ToyCappedLM"])
    with tempfile.TemporaryDirectory() as d:
        write_random_model(d, cfg, seed=4, std_overrides=dict(strong(cfg), **{"toy_head.bias": 0.5}))
        model = load_model(d, "float32" if dtype == torch.float32 else "bfloat16", DEV)
        r = ModelRunner(model, 8, 16, 2, 64, 64)
        plain = P.PlainModel(d)
        toks = torch.randint(0, 383, (37,), generator=torch.Generator().manual_seed(6)).tolist()

        def want(rnd):
            x = plain.w["model.embed_tokens.weight"][toks].float() * SCALE
            for i in range(plain.cfg.num_hidden_layers):
                x = P.block(x, plain.w, i, plain.cfg, torch.arange(len(toks)), rnd)
            h = rnd(P.rms_norm(x, plain.w["model.norm.weight"], plain.cfg.rms_norm_eps))
            return CAP * torch.tanh((h @ plain.w["lm_head.weight"].T + plain.w["toy_head.bias"]) / CAP)
        exact, rounded = want(lambda x: x), want(P.to_bf16)
        assert float(plain.w["toy_head.bias"].abs().max()) > 0.5 and float(exact.abs().max()) > 1.5      # bias and cap both bite
        r.manager.add_request("r")
        got, i = [], 0
        for n in (20, 1, 2, 14):
            assert r.manager.grow("r", i + n)
            seq = [SeqStep("r", toks[i:i + n], list(range(n)))]
            got.append(r.step(seq))
            r.advance(seq)
            i += n
        close_to_plain(torch.cat(got), exact, rounded, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_run_may_read_another_runs_cache(dtype):
    """Run order [layer 0, layer 1 with the cache of run 0]: layer 1 projects and encodes its own queries, attends over
    the keys and values that layer 0 stored, and stores nothing (the cache of run 0 is the model's only one).  In
    portions and token by token the result is the plain computation of that model."""
    import dataclasses
    from pico_vllm_amd.config.registry import load_model_description
    from pico_vllm_amd.engine.batch import SeqStep
    from pico_vllm_amd.engine.step import ModelRunner
    from pico_vllm_amd.parts.model import DecoderModel
    from pico_vllm_amd.parts.spec import RunEntry
    from pico_vllm_amd.weights.loader import load_checkpoint
    d = model_dir("A")
    _, cfg, spec = load_model_description(d)
    spec = dataclasses.replace(spec, run_order=[RunEntry(0), RunEntry(1, cache_of=0)])
    model = DecoderModel(spec, dtype, torch.device(DEV))
    model.load(load_checkpoint(d, model.param_specs(), dtype))
    assert sorted(model.cache_specs()) == [0]
    r = ModelRunner(model, 16, 8, 2, 128, 128)
    plain = P.PlainModel(d)
    w, c = plain.w, plain.cfg
    toks = torch.randint(0, 255, (45,), generator=torch.Generator().manual_seed(4)).tolist()
    pos = torch.arange(len(toks))

    def want(rnd):
        nq, nkv, hd = c.num_attention_heads, c.num_key_value_heads, c.head_dim
        x = w["model.embed_tokens.weight"][toks].float()
        kv = None
        for i in (0, 1):
            p = f"model.layers.{i}"
            h = rnd(P.rms_norm(x, w[f"{p}.input_layernorm.weight"], c.rms_norm_eps))
            W = torch.cat([w[f"{p}.self_attn.{n}_proj.weight"] for n in "qkv"])
            b = torch.cat([w[f"{p}.self_attn.{n}_proj.bias"] for n in "qkv"])
            q, k, v = P.split_qkv(rnd(h @ W.T + b), nq, nkv, hd)
            cos, sin = P.rope_tables(pos, hd, c.rope_theta)
            q, k = rnd(P.apply_rope(q, cos, sin)), rnd(P.apply_rope(k, cos, sin))
            if i == 0:
                kv = (k, v)                      # what run 0 stores is what run 1 reads
            o = rnd(P.causal_attention(q, kv[0], kv[1], rnd_p=None if rnd is P._same else rnd))
            x = x + rnd(o.reshape(len(toks), nq * hd) @ w[f"{p}.self_attn.o_proj.weight"].T)
            x = x + P.mlp_layer(rnd(P.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], c.rms_norm_eps)), w, p, rnd)
        return rnd(P.rms_norm(x, w["model.norm.weight"], c.rms_norm_eps)) @ w["model.embed_tokens.weight"].T
    exact, rounded = want(P._same), want(P.to_bf16)
    ordinary = plain.logits(toks)
    assert float((exact - ordinary).abs().max()) > 0.05 * float(ordinary.std())       # it is another model than the ordinary one
    r.manager.add_request("r")
    got, i = [], 0
    for n in (20, 3, 1, 1, 20):
        assert r.manager.grow("r", i + n)
        seq = [SeqStep("r", toks[i:i + n], list(range(n)))]
        got.append(r.step(seq))
        r.advance(seq)
        i += n
    close_to_plain(torch.cat(got), exact, rounded, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_layers_with_and_without_a_window_in_one_model(dtype):
    """Layer 0 reads the last 24 keys only, layers 1 and 2 all of them: two groups of layers with pages of their own, the
    windowed group giving pages back while the request runs.  A request of 120 tokens in portions and token by token,
    and a second one beside it, in pools so small that the windowed group's pages are used again; against the plain
    computation of that model."""
    import dataclasses
    import tempfile
    from pico_vllm_amd.config.model_config import Qwen2Config
    from pico_vllm_amd.config.qwen2 import qwen2_spec
    from pico_vllm_amd.config.registry import register_architecture
    from pico_vllm_amd.engine.batch import SeqStep
    from pico_vllm_amd.engine.step import ModelRunner
    from pico_vllm_amd.parts.model import load_model
    from pico_vllm_amd.parts.spec import LayerSpec, PartSpec
    from pico_vllm_amd.weights.random_init import write_random_model
    from tiny_configs import TINY_B, strong
    W = 24

    def spec_with_window(cfg):
        spec = qwen2_spec(cfg)
        l0 = spec.layers[0]
        name, attn = l0.slots["mixer"]
        windowed = PartSpec(attn.kind, dict(attn.params, window=W))
        return dataclasses.replace(spec, layers=[LayerSpec(l0.prefix, l0.block, {**l0.slots, "mixer": (name, windowed)})] + list(spec.layers[1:]))
    register_architecture("ToyWindowFirstLM", Qwen2Config.from_dict, spec_with_window)
    cfg = dict(TINY_B, architectures=["ToyWindowFirstLM"])
    with tempfile.TemporaryDirectory() as d:
        write_random_model(d, cfg, seed=8, std_overrides=strong(cfg))
        model = load_model(d, "float32" if dtype == torch.float32 else "bfloat16", DEV)
        r = ModelRunner(model, 8, 20, 2, 64, 160)          # 20 pages of 8 a group: 160 tokens, two requests of 120 + 30 need the give-back
        m = r.manager
        assert len(m.groups) == 2 and sorted(g.window for g in m.groups) == [0, W]
        plain = P.PlainModel(d)
        w, c = plain.w, plain.cfg

        def want(toks, rnd):
            nq, nkv, hd = c.num_attention_heads, c.num_key_value_heads, c.head_dim
            pos = torch.arange(len(toks))
            x = w["model.embed_tokens.weight"][toks].float()
            for i in range(c.num_hidden_layers):
                p = f"model.layers.{i}"
                h = rnd(P.rms_norm(x, w[f"{p}.input_layernorm.weight"], c.rms_norm_eps))
                Wm = torch.cat([w[f"{p}.self_attn.{n}_proj.weight"] for n in "qkv"])
                b = torch.cat([w[f"{p}.self_attn.{n}_proj.bias"] for n in "qkv"])
                q, k, v = P.split_qkv(rnd(h @ Wm.T + b), nq, nkv, hd)
                cos, sin = P.rope_tables(pos, hd, c.rope_theta)
                q, k = rnd(P.apply_rope(q, cos, sin)), rnd(P.apply_rope(k, cos, sin))
                o = rnd(P.causal_attention(q, k, v, window=W if i == 0 else 0, rnd_p=None if rnd is P._same else rnd))
                x = x + rnd(o.reshape(len(toks), nq * hd) @ w[f"{p}.self_attn.o_proj.weight"].T)
                x = x + P.mlp_layer(rnd(P.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], c.rms_norm_eps)), w, p, rnd)
            return rnd(P.rms_norm(x, w["model.norm.weight"], c.rms_norm_eps)) @ w["lm_head.weight"].T
        g = torch.Generator().manual_seed(9)
        a, b = torch.randint(0, 383, (120,), generator=g).tolist(), torch.randint(0, 383, (30,), generator=g).tolist()
        assert float((want(a, P._same) - plain.logits(a)).abs().max()) > 0.05 * float(plain.logits(a).std())   # the window matters
        m.add_request("a")
        m.add_request("b")
        got = {"a": [], "b": []}
        fed = {"a": 0, "b": 0}
        plan = [(40, 0), (13, 7), (1, 1), (1, 1), (30, 2), (1, 19), (34, 0)]
        for na, nb in plan:
            seqs = []
            for rid, n, toks in (("a", na, a), ("b", nb, b)):
                if n:
                    assert m.grow(rid, fed[rid] + n)
                    seqs.append(SeqStep(rid, toks[fed[rid]:fed[rid] + n], list(range(n))))
            out = r.step(seqs)
            r.advance(seqs)
            o = 0
            for s in seqs:
                got[s.req].append(out[o:o + len(s.tokens)])
                o += len(s.tokens)
                fed[s.req] += len(s.tokens)
            m.check()
        assert fed == {"a": 120, "b": 30}
        windowed = [gr for gr in m.groups if gr.window][0]
        assert windowed.pool.peak_used < 20 and windowed.pool.num_used < [gr for gr in m.groups if not gr.window][0].pool.num_used
        for rid, toks in (("a", a), ("b", b)):
            close_to_plain(torch.cat(got[rid]), want(toks, P._same), want(toks, P.to_bf16), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_layer_without_position_encoding_between_layers_with_rotation(dtype):
    """The framework's own "none" position encoding in layer 1, rotation in the others: keys and values of that layer are
    stored as they are.  A prompt in portions, then token by token (in bfloat16 a single row reaches the attention as a
    norm still to be run, which this encoding does not take over), with and without recorded steps; against the plain
    computation of that model, which differs from the one with rotation everywhere."""
    import dataclasses
    import tempfile
    from pico_vllm_amd.config.model_config import Qwen2Config
    from pico_vllm_amd.config.qwen2 import qwen2_spec
    from pico_vllm_amd.config.registry import register_architecture
    from pico_vllm_amd.engine.batch import SeqStep
    from pico_vllm_amd.engine.step import ModelRunner
    from pico_vllm_amd.parts.model import load_model
    from pico_vllm_amd.parts.spec import LayerSpec, PartSpec
    from pico_vllm_amd.weights.random_init import write_random_model
    from tiny_configs import TINY_B, strong

    def spec_with_a_bare_layer(cfg):
        spec = qwen2_spec(cfg)
        l1 = spec.layers[1]
        name, attn = l1.slots["mixer"]
        bare = PartSpec(attn.kind, dict(attn.params, position=PartSpec("none", {})))
        layers = list(spec.layers)
        layers[1] = LayerSpec(l1.prefix, l1.block, {**l1.slots, "mixer": (name, bare)})
        return dataclasses.replace(spec, layers=layers)
    register_architecture("ToyBareLayerLM", Qwen2Config.from_dict, spec_with_a_bare_layer)
    cfg = dict(TINY_B, architectures=["ToyBareLayerLM"])
    with tempfile.TemporaryDirectory() as d:
        write_random_model(d, cfg, seed=12, std_overrides=strong(cfg))
        model = load_model(d, "float32" if dtype == torch.float32 else "bfloat16", DEV)
        plain = P.PlainModel(d)
        w, c = plain.w, plain.cfg

        def want(toks, rnd):
            nq, nkv, hd = c.num_attention_heads, c.num_key_value_heads, c.head_dim
            pos = torch.arange(len(toks))
            x = w["model.embed_tokens.weight"][toks].float()
            for i in range(c.num_hidden_layers):
                p = f"model.layers.{i}"
                h = rnd(P.rms_norm(x, w[f"{p}.input_layernorm.weight"], c.rms_norm_eps))
                Wm = torch.cat([w[f"{p}.self_attn.{n}_proj.weight"] for n in "qkv"])
                b = torch.cat([w[f"{p}.self_attn.{n}_proj.bias"] for n in "qkv"])
                q, k, v = P.split_qkv(rnd(h @ Wm.T + b), nq, nkv, hd)
                if i != 1:
                    cos, sin = P.rope_tables(pos, hd, c.rope_theta)
                    q, k = rnd(P.apply_rope(q, cos, sin)), rnd(P.apply_rope(k, cos, sin))
                o = rnd(P.causal_attention(q, k, v, rnd_p=None if rnd is P._same else rnd))
                x = x + rnd(o.reshape(len(toks), nq * hd) @ w[f"{p}.self_attn.o_proj.weight"].T)
                x = x + P.mlp_layer(rnd(P.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], c.rms_norm_eps)), w, p, rnd)
            return rnd(P.rms_norm(x, w["model.norm.weight"], c.rms_norm_eps)) @ w["lm_head.weight"].T
        toks = torch.randint(0, 383, (70,), generator=torch.Generator().manual_seed(5)).tolist()
        assert float((want(toks, P._same) - plain.logits(toks)).abs().max()) > 0.05 * float(plain.logits(toks).std())
        for graphs in (False, True):
            r = ModelRunner(model, 8, 24, 2, 64, 96, use_graph=graphs, max_graph_batch=2)
            assert r.use_graph == graphs
            r.manager.add_request("a")
            got, fed = [], 0
            for n in [23, 2, 17] + [1] * 28:
                assert r.manager.grow("a", fed + n)
                seqs = [SeqStep("a", toks[fed:fed + n], [n - 1] if graphs else list(range(n)))]
                got.append(r.step(seqs).clone())
                r.advance(seqs)
                fed += n
            assert fed == 70
            rows = [22, 24, 41] + list(range(42, 70)) if graphs else list(range(70))
            close_to_plain(torch.cat(got), want(toks, P._same)[rows], want(toks, P.to_bf16)[rows], dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_toy_norm_and_a_toy_arrangement_of_the_parts(dtype):
    """The two remaining kinds of part, defined and registered here: a norm that centres on the mean and has a
    bias (the framework's subtracts nothing and has none), and an arrangement in which the mixer and the
    feed-forward read the same normed activations and their outputs are added together,
    x += mixer(norm(x)) + ff(norm(x)), one norm a layer.  Mixer, feed-forward and position encoding are the
    framework's.  The whole prompt equals a plain computation written out below, portions beside another request
    equal the whole, and the entry point generates with the model from graphs as without."""
    import tempfile
    from pico_vllm_amd import LLM, SamplingParams
    from pico_vllm_amd.config.registry import register_architecture
    from pico_vllm_amd.engine.batch import SeqStep
    from pico_vllm_amd.engine.step import ModelRunner
    from pico_vllm_amd.parts.base import Block, Norm
    from pico_vllm_amd.parts.model import load_model
    from pico_vllm_amd.parts.registry import register_part
    from pico_vllm_amd.parts.spec import LayerSpec, ModelSpec, ParamSpec, PartSpec, RunEntry
    from pico_vllm_amd.weights.random_init import write_random_model

    H, V, NQ, NKV, D, I, EPS, THETA = 48, 77, 3, 3, 16, 40, 1e-4, 300.0

    def flat(delta):                 # a part's output: [T, H], or a float32 stack of partial sums
        delta = delta.float()
        return delta.sum(0) if delta.dim() == 3 else delta

    @register_part("norm", "toy_centred_norm")
    class CentredNorm(Norm):
        def __init__(self, size, eps, act_dtype=torch.bfloat16):
            self.size, self.eps, self.act_dtype = size, eps, act_dtype

        def param_specs(self):
            return [ParamSpec("weight", (self.size,), role="norm"), ParamSpec("bias", (self.size,), role="bias")]

        def load(self, tensors, device, dtype):
            self.weight, self.bias = tensors["weight"].to(device).float(), tensors["bias"].to(device).float()

        def add_norm(self, resid, delta, rows=None):
            if rows is None:
                if delta is not None:
                    resid += flat(delta)
                x = resid
            else:
                x = resid[rows.long()] + (flat(delta)[rows.long()] if delta is not None else 0.0)
            x = x - x.mean(-1, keepdim=True)
            return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.eps) * self.weight + self.bias).to(self.act_dtype)

    @register_part("block", "toy_side_by_side")
    class SideBySide(Block):
        slot_categories = {"norm": "norm", "mixer": "mixer", "ff": "feed_forward"}

        def forward(self, resid, pending, ctx, cache):
            h = self.parts["norm"].add_norm(resid, pending)
            return resid, flat(self.parts["mixer"].forward(h, ctx, cache)) + flat(self.parts["ff"].forward(h, ctx))

    def toy_spec(cfg):
        norm = PartSpec("toy_centred_norm", {"size": H, "eps": EPS})
        attn = PartSpec("gqa_attention", {"hidden_size": H, "num_heads": NQ, "num_kv_heads": NKV, "head_dim": D, "qkv_bias": True,
                                          "window": 0, "position": PartSpec("rotary_half", {"rotary_dim": D, "theta": THETA})})
        ff = PartSpec("swiglu_mlp", {"hidden_size": H, "intermediate_size": I})
        layers = [LayerSpec(f"toy.layers.{i}", "toy_side_by_side", {"norm": ("ln", norm), "mixer": ("attn", attn), "ff": ("ff", ff)})
                  for i in range(3)]
        return ModelSpec(H, V, "toy.embed.weight", layers, [RunEntry(i) for i in range(3)], norm, "toy.norm", None)

    register_architecture("ToySideBySideLM", lambda raw: raw, toy_spec)
    rnd = P._same if dtype == torch.float32 else P.to_bf16
    with tempfile.TemporaryDirectory() as d:
        write_random_model(d, {"architectures": ["ToySideBySideLM"]}, seed=6,
                           std_overrides={"attn": 0.4, "embed": 0.5, "ff.gate": 0.3, "ff.up": 0.3, "ff.down": 0.3, ".bias": 0.3})
        w = {k: v.float() for k, v in P.read_weights(d).items()}
        assert float(w["toy.layers.0.ln.bias"].abs().max()) > 0.1
        model = load_model(d, "float32" if dtype == torch.float32 else "bfloat16", DEV)
        assert not model.is_graph_safe(prompts=True) and model.is_graph_safe()      # the toy parts did not opt in for prompts
        r = ModelRunner(model, 8, 16, 3, 64, 64)
        toks = torch.randint(0, V, (41,), generator=torch.Generator().manual_seed(2)).tolist()

        def centred(x, p):
            x = x - x.mean(-1, keepdim=True)
            return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + EPS) * w[f"{p}.weight"] + w[f"{p}.bias"]

        def plain(rnd):              # the whole sequence, no cache
            pos = torch.arange(len(toks))
            x = w["toy.embed.weight"][toks]
            cos, sin = P.rope_tables(pos, D, THETA)
            for i in range(3):
                p = f"toy.layers.{i}"
                h = rnd(centred(x, f"{p}.ln"))
                W = torch.cat([w[f"{p}.attn.{n}_proj.weight"] for n in "qkv"], 0)
                b = torch.cat([w[f"{p}.attn.{n}_proj.bias"] for n in "qkv"], 0)
                q, k, v = P.split_qkv(rnd(h @ W.T + b), NQ, NKV, D)
                o = rnd(P.causal_attention(rnd(P.apply_rope(q, cos, sin)), rnd(P.apply_rope(k, cos, sin)), v,
                                           rnd_p=None if rnd is P._same else rnd))
                a = rnd(o.reshape(len(toks), NQ * D) @ w[f"{p}.attn.o_proj.weight"].T)
                gu = torch.cat([w[f"{p}.ff.gate_proj.weight"], w[f"{p}.ff.up_proj.weight"]], 0)
                f = rnd(rnd(P.swiglu(rnd(h @ gu.T))) @ w[f"{p}.ff.down_proj.weight"].T)
                x = x + a + f                                            # both read h, neither the other's output
            return rnd(centred(x, "toy.norm")) @ w["toy.embed.weight"].T

        want = plain(P._same)
        r.manager.add_request("w")
        assert r.manager.grow("w", len(toks))
        whole_logits = r.step([SeqStep("w", toks, list(range(len(toks))))])
        r.manager.free_request("w")
        close_to_plain(whole_logits, want, plain(rnd), dtype)
        r.manager.add_request("a")
        r.manager.add_request("b")
        got, fed = [], 0
        for n, nb in ((9, 2), (1, 1), (2, 5), (22, 1), (7, 1)):
            assert r.manager.grow("a", fed + n) and r.manager.grow("b", r.manager.num_computed("b") + nb)
            seqs = [SeqStep("b", toks[:nb], []), SeqStep("a", toks[fed:fed + n], list(range(n)))]
            got.append(r.step(seqs))
            r.advance(seqs)
            fed += n
        close(torch.cat(got), whole_logits, dtype, scale=float(whole_logits.std()) * 3)
        del r, model
        # through the entry point, decode steps from graphs and without: the same tokens, and the plain argmax
        outs = []
        for graphs in (True, False):
            llm = LLM(model=d, dtype="float32" if dtype == torch.float32 else "bfloat16", max_seq_len=64, max_num_seqs=2,
                      num_gpu_blocks=16, block_size=8, use_cuda_graph=graphs)
            assert llm.engine.runner.use_graph == graphs and not llm.engine.runner.graph_prompts
            outs.append([o.token_ids for o in llm.generate([toks[:9], toks[5:20]], SamplingParams(max_new_tokens=6, temperature=0.0))])
            del llm
        assert outs[0] == outs[1]


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_parts_around_the_layers_learned_positions_in_front_and_a_gain_behind(dtype):
    """``ModelSpec.before_layers`` / ``after_layers``: parts of the category "stream" that work on the residual stream
    outside the layers, defined and registered here: learned absolute positions added to the embeddings (a table of the
    checkpoint, looked up by ``ctx.positions``) and a gain per channel behind the last layer.  The attention layers carry
    no position encoding, so positions reach the logits through the table alone.  Portions, single tokens (recorded
    steps too) and the whole prompt against the plain computation."""
    import dataclasses
    import tempfile
    from pico_vllm_amd.config.model_config import Qwen2Config
    from pico_vllm_amd.config.qwen2 import qwen2_spec
    from pico_vllm_amd.config.registry import register_architecture
    from pico_vllm_amd.engine.batch import SeqStep
    from pico_vllm_amd.engine.step import ModelRunner
    from pico_vllm_amd.parts.base import StreamPart
    from pico_vllm_amd.parts.model import load_model
    from pico_vllm_amd.parts.registry import register_part
    from pico_vllm_amd.parts.spec import LayerSpec, ParamSpec, PartSpec
    from pico_vllm_amd.weights.random_init import write_random_model
    from tiny_configs import TINY_A, strong

    @register_part("stream", "toy_learned_positions")
    class LearnedPositions(StreamPart):
        graph_safe_prompts = True

        def __init__(self, size, most, act_dtype=torch.bfloat16):
            self.size, self.most = size, most

        def param_specs(self):
            return [ParamSpec("weight", (self.most, self.size), std=0.5)]

        def load(self, tensors, device, dtype):
            self.table = tensors["weight"].to(device).float()

        def forward(self, resid, ctx):
            T = resid.shape[0]
            resid += self.table.index_select(0, ctx.positions[:T].long())       # device work only: may be recorded
            return resid

    @register_part("stream", "toy_gain")
    class Gain(StreamPart):
        graph_safe_prompts = True

        def __init__(self, size, act_dtype=torch.bfloat16):
            self.size = size

        def param_specs(self):
            return [ParamSpec("weight", (self.size,), role="norm")]

        def load(self, tensors, device, dtype):
            self.gain = tensors["weight"].to(device).float()

        def forward(self, resid, ctx):
            return resid * self.gain

    MOST = 96

    def spec_with_parts_around(cfg):
        spec = qwen2_spec(cfg)
        layers = []
        for l in spec.layers:
            name, attn = l.slots["mixer"]
            layers.append(LayerSpec(l.prefix, l.block, {**l.slots, "mixer": (name, PartSpec(attn.kind, dict(attn.params, position=PartSpec("none", {}))))}))
        return dataclasses.replace(spec, layers=layers,
                                   before_layers=(("model.wpe", PartSpec("toy_learned_positions", {"size": cfg.hidden_size, "most": MOST})),),
                                   after_layers=(("model.out_gain", PartSpec("toy_gain", {"size": cfg.hidden_size})),))
    register_architecture("ToyLearnedPositionsLM", Qwen2Config.from_dict, spec_with_parts_around)
    cfg = dict(TINY_A, architectures=["ToyLearnedPositionsLM"])
    with tempfile.TemporaryDirectory() as d:
        write_random_model(d, cfg, seed=21, std_overrides=strong(cfg))
        model = load_model(d, "float32" if dtype == torch.float32 else "bfloat16", DEV)
        plain = P.PlainModel(d)
        w, c = plain.w, plain.cfg
        assert w["model.wpe.weight"].shape == (MOST, c.hidden_size) and w["model.out_gain.weight"].shape == (c.hidden_size,)

        def want(toks, rnd, first=0):
            nq, nkv, hd = c.num_attention_heads, c.num_key_value_heads, c.head_dim
            x = w["model.embed_tokens.weight"][toks].float() + w["model.wpe.weight"][first:first + len(toks)]
            for i in range(c.num_hidden_layers):
                p = f"model.layers.{i}"
                h = rnd(P.rms_norm(x, w[f"{p}.input_layernorm.weight"], c.rms_norm_eps))
                Wm = torch.cat([w[f"{p}.self_attn.{n}_proj.weight"] for n in "qkv"])
                b = torch.cat([w[f"{p}.self_attn.{n}_proj.bias"] for n in "qkv"])
                q, k, v = P.split_qkv(rnd(h @ Wm.T + b), nq, nkv, hd)
                o = rnd(P.causal_attention(q, k, v, rnd_p=None if rnd is P._same else rnd))
                x = x + rnd(o.reshape(len(toks), nq * hd) @ w[f"{p}.self_attn.o_proj.weight"].T)
                x = x + P.mlp_layer(rnd(P.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], c.rms_norm_eps)), w, p, rnd)
            x = x * w["model.out_gain.weight"]
            return rnd(P.rms_norm(x, w["model.norm.weight"], c.rms_norm_eps)) @ w["model.embed_tokens.weight"].T
        toks = torch.randint(0, 255, (70,), generator=torch.Generator().manual_seed(6)).tolist()
        exact = want(toks, P._same)
        # positions do reach the logits, and through the table: the same tokens from another first position differ
        assert float((want(toks, P._same, first=9) - exact).abs().max()) > 0.05 * float(exact.std())
        for graphs in (False, True):
            r = ModelRunner(model, 16, 12, 2, 64, 96, use_graph=graphs, max_graph_batch=2)
            assert r.use_graph == graphs and r.graph_prompts == graphs
            r.manager.add_request("a")
            got, fed = [], 0
            for n in [23, 2, 17] + [1] * 28:
                assert r.manager.grow("a", fed + n)
                seqs = [SeqStep("a", toks[fed:fed + n], [n - 1] if graphs else list(range(n)))]
                got.append(r.step(seqs).clone())
                r.advance(seqs)
                fed += n
            rows = [22, 24, 41] + list(range(42, 70)) if graphs else list(range(70))
            close_to_plain(torch.cat(got), exact[rows], want(toks, P.to_bf16)[rows], dtype)
            if graphs:
                assert r._graphs and r._prompt_graphs


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_toy_mixer_whose_pages_hold_what_it_says(dtype):
    """The tensors of a cache page are the mixer's to name (``CacheSpec.page_tensors``): this toy mixer keeps ONE latent
    vector of 12 numbers per token, in float32 whatever the engine's dtype, in pages [page, 12], beside a second
    tensor [3, page] of the positions' powers that it never needs again but stores to show two tensors of different
    shapes; it mixes by the causal mean of the cached latents (y_t = Wu mean_{s <= t} Wd x_s).  Layer 0 has it, layer 1
    the framework's attention: two groups of pages with one block table each.  Whole against a plain computation,
    portions and mixed steps against whole, pages given back and used again, and generation through the scheduler."""
    import tempfile
    from pico_vllm_amd.config.registry import register_architecture
    from pico_vllm_amd.engine.batch import SeqStep
    from pico_vllm_amd.engine.step import ModelRunner
    from pico_vllm_amd.parts.base import Mixer
    from pico_vllm_amd.parts.model import load_model
    from pico_vllm_amd.parts.registry import register_part
    from pico_vllm_amd.parts.spec import CacheSpec, LayerSpec, ModelSpec, PageTensor, ParamSpec, PartSpec, RunEntry
    from pico_vllm_amd.weights.random_init import write_random_model

    H, V, R, NQ, NKV, D = 40, 90, 12, 2, 1, 16

    @register_part("mixer", "toy_latent_mean")
    class LatentMean(Mixer):
        graph_safe = False                   # it sizes a gather by the longest context of the step, on the host

        def __init__(self, hidden_size, latent, act_dtype=torch.bfloat16):
            self.H, self.R = hidden_size, latent

        def cache_spec(self):
            return CacheSpec("paged_kv", page_tensors=(PageTensor("latent", ("page", self.R), "float32"),
                                                       PageTensor("powers", (3, "page"), "float32")))

        def param_specs(self):
            return [ParamSpec("down.weight", (self.R, self.H), std=0.4), ParamSpec("up.weight", (self.H, self.R), std=0.4)]

        def load(self, tensors, device, dtype):
            self.wd, self.wu = tensors["down.weight"].to(device).float(), tensors["up.weight"].to(device).float()

        def forward(self, x, ctx, cache):
            T, P = x.shape[0], cache.page_size
            assert cache.latent.shape[1:] == (P, self.R) and cache.powers.shape[1:] == (3, P) and cache.latent.dtype == torch.float32
            seq, pos = ctx.token_seq[:T].long(), ctx.positions[:T].long()
            slots = ctx.slot_mapping[cache.group][:T].long()                 # page * P + place in the page
            flat = cache.latent.view(-1, self.R)
            flat.index_copy_(0, slots, x.float() @ self.wd.T)
            pw = cache.powers.permute(0, 2, 1).reshape(-1, 3)                # a copy: written back below
            pw[slots] = torch.stack([pos.float(), pos.float() ** 2, pos.float() ** 3], 1)
            cache.powers.copy_(pw.view(-1, P, 3).permute(0, 2, 1))
            # every token's mean over the latents of its request up to its own position, from the pages
            longest = int(ctx.host["context_lens"][:ctx.num_seqs].max())
            keys = torch.arange(longest, device=x.device)
            pages = ctx.block_tables[cache.group][seq][:, keys // P].long()     # [T, longest]; -1 beyond a request's pages
            seen = keys[None, :] <= pos[:, None]
            lat = flat[(pages * P + keys % P).clamp(min=0)] * seen[..., None]
            mean = lat.sum(1) / (pos + 1).float()[:, None]
            return (mean @ self.wu.T).to(x.dtype)

    def toy_spec(cfg):
        norm = PartSpec("rms_norm", {"size": H, "eps": 1e-5})
        attn = PartSpec("gqa_attention", {"hidden_size": H, "num_heads": NQ, "num_kv_heads": NKV, "head_dim": D, "qkv_bias": True,
                                          "window": 0, "position": PartSpec("rotary_half", {"rotary_dim": D, "theta": 1e4})})
        mixers = [("lat", PartSpec("toy_latent_mean", {"hidden_size": H, "latent": R})), ("attn", attn)]
        ff = PartSpec("swiglu_mlp", {"hidden_size": H, "intermediate_size": 56})
        layers = [LayerSpec(f"toy.layers.{i}", "prenorm", {"norm1": ("ln1", norm), "mixer": mixers[i], "norm2": ("ln2", norm),
                                                          "ff": ("ff", ff)}) for i in range(2)]
        return ModelSpec(H, V, "toy.embed.weight", layers, [RunEntry(0), RunEntry(1)], norm, "toy.norm", None)

    register_architecture("ToyLatentPagesLM", lambda raw: raw, toy_spec)
    cfg = {"architectures": ["ToyLatentPagesLM"]}
    rnd = P._same if dtype == torch.float32 else P.to_bf16
    with tempfile.TemporaryDirectory() as d:
        write_random_model(d, cfg, seed=8, std_overrides={"attn": 0.3, "embed": 0.5, "ff": 0.2})
        w = {k: v.float() for k, v in P.read_weights(d).items()}
        model = load_model(d, "float32" if dtype == torch.float32 else "bfloat16", DEV)
        r = ModelRunner(model, 8, 14, 3, 64, 64)
        assert len(r.manager.groups) == 2 and not r.use_graph
        lat_layer = r.storage.layer(0)
        assert set(lat_layer.tensors) == {"latent", "powers"} and lat_layer.latent.shape == (14, 8, R)
        assert r.storage.bytes_per_token() == 4 * (R + 3) + 2 * NKV * D * (4 if dtype == torch.float32 else 2)

        def plain(toks, rnd):
            n = len(toks)
            pos = torch.arange(n)
            x = w["toy.embed.weight"][toks]
            p = "toy.layers.0"
            h = rnd(P.rms_norm(x, w[f"{p}.ln1.weight"], 1e-5))
            lat = h @ w[f"{p}.lat.down.weight"].T
            mean = torch.cumsum(lat, 0) / (pos + 1).float()[:, None]
            x = x + rnd(mean @ w[f"{p}.lat.up.weight"].T)
            x = x + P.mlp_layer(rnd(P.rms_norm(x, w[f"{p}.ln2.weight"], 1e-5)), {k.replace(".ff.", ".mlp."): v for k, v in w.items()}, p, rnd)
            p = "toy.layers.1"
            h = rnd(P.rms_norm(x, w[f"{p}.ln1.weight"], 1e-5))
            Wm = torch.cat([w[f"{p}.attn.{n}_proj.weight"] for n in "qkv"])
            b = torch.cat([w[f"{p}.attn.{n}_proj.bias"] for n in "qkv"])
            q, k, v = P.split_qkv(rnd(h @ Wm.T + b), NQ, NKV, D)
            cos, sin = P.rope_tables(pos, D, 1e4)
            o = rnd(P.causal_attention(rnd(P.apply_rope(q, cos, sin)), rnd(P.apply_rope(k, cos, sin)), v, rnd_p=None if rnd is P._same else rnd))
            x = x + rnd(o.reshape(n, NQ * D) @ w[f"{p}.attn.o_proj.weight"].T)
            x = x + P.mlp_layer(rnd(P.rms_norm(x, w[f"{p}.ln2.weight"], 1e-5)), {k.replace(".ff.", ".mlp."): v for k, v in w.items()}, p, rnd)
            return rnd(P.rms_norm(x, w["toy.norm.weight"], 1e-5)) @ w["toy.embed.weight"].T

        g = torch.Generator().manual_seed(2)
        reqs = {rid: torch.randint(0, V, (n,), generator=g).tolist() for rid, n in (("a", 43), ("b", 21), ("c", 30))}
        whole = {}
        for rid, toks in reqs.items():
            r.manager.add_request(rid)
            assert r.manager.grow(rid, len(toks))
            whole[rid] = r.step([SeqStep(rid, toks, list(range(len(toks))))])
            r.manager.free_request(rid)
            close_to_plain(whole[rid], plain(toks, P._same), plain(toks, rnd), dtype)
        # a and b in portions beside each other; b ends, c takes its pages (14 pages of 8 do not hold all three)
        got = {rid: [] for rid in reqs}
        fed = {rid: 0 for rid in reqs}
        plan = [(("a", 9), ("b", 2)), (("b", 1), ("a", 1)), (("a", 2), ("b", 18)), (("a", 24),), (("c", 13), ("a", 1)), (("a", 6), ("c", 17))]
        r.manager.add_request("a"); r.manager.add_request("b")
        for step in plan:
            if step[0][0] == "c" and "c" not in r.manager.requests:
                r.manager.free_request("b")
                r.manager.add_request("c")
            seqs = []
            for rid, n in step:
                assert r.manager.grow(rid, fed[rid] + n), (rid, fed[rid], n)
                seqs.append(SeqStep(rid, reqs[rid][fed[rid]:fed[rid] + n], list(range(n))))
            out = r.step(seqs)
            r.advance(seqs)
            at = 0
            for rid, n in step:
                got[rid].append(out[at:at + n])
                at += n
                fed[rid] += n
            r.manager.check()
        for rid in reqs:
            assert fed[rid] == len(reqs[rid])
            close(torch.cat(got[rid]), whole[rid], dtype, scale=float(whole[rid].std()) * 3)
        assert all(g.pool.reuse_count > 0 for g in r.manager.groups)
        del r, model
        # through the scheduler: generation with a pool so small that requests wait for pages
        from pico_vllm_amd import LLM, SamplingParams
        kind = "float32" if dtype == torch.float32 else "bfloat16"
        prompts = [reqs["a"][:20], reqs["b"][:9], reqs["c"][:15]]
        sp = SamplingParams(max_new_tokens=10, temperature=0.0, ignore_eos=True)
        llm = LLM(model=d, dtype=kind, block_size=8, num_gpu_blocks=9, max_seq_len=64, max_num_seqs=3, max_num_batched_tokens=16)
        assert not llm.engine.runner.use_graph
        outs = llm.generate(prompts, sp)
        for prompt, o in zip(prompts, outs):
            toks = list(prompt)
            for t in o.token_ids:
                logits = plain(toks, P._same)[-1]
                assert float(logits[t]) >= float(logits.max()) - (1e-4 if dtype == torch.float32 else 0.05 * float(logits.std()))
                toks.append(t)
        llm.engine.runner.manager.check()
        assert all(g.pool.num_free == 9 for g in llm.engine.runner.manager.groups)
