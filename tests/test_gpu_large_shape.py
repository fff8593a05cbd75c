"""The engine at the layer sizes of real models, with random weights.

The tiny configurations of the other tests never reach the paths that only large sizes take (two key
teams over a 2,048-token triangle, the 8960-wide contraction cut into seven ranges, a vocabulary of
151,936, the library's matrix products for many rows, groups of 5 and 7 query heads of size 128, a width
beyond what the fused norm takes).

Against the plain implementation in float64: two layers of the Qwen2.5-1.5B sizes and one layer each of
the 7B and 32B sizes with a vocabulary cut to a few thousand, a prompt of 200 tokens whole, in portions
of changing size and with its tail token by token, in 32-bit and in bfloat16, with the bounds of the
replay tests (the reference's own bar is equality of generations with an outside model at the real
size, pico_vllm/tests/test_engine.py:59-93).
With the whole vocabulary of 151,936 and a prompt beyond one 2,048-token portion the plain implementation
is too slow; there the yardstick is the engine's own 32-bit path, which the tests above pin.
"""
import random
import tempfile

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SHAPE = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "vocab_size": 151936, "hidden_size": 1536,
    "num_hidden_layers": 2, "num_attention_heads": 12, "num_key_value_heads": 2, "intermediate_size": 8960,
    "rms_norm_eps": 1e-6, "rope_theta": 1000000.0, "tie_word_embeddings": True, "max_position_embeddings": 32768,
    "hidden_act": "silu",
}
N = 2300          # prompt: more than one 2,048-token portion


@pytest.fixture(scope="module")
def folder():
    from pico_vllm_amd.weights.random_init import write_random_model
    with tempfile.TemporaryDirectory(prefix="pico_large_") as d:
        # queries and keys strong enough that attention is not uniform: a wrong key shows
        write_random_model(d, SHAPE, 3, {"q_proj.weight": (3.0 / 1536) ** 0.5, "k_proj.weight": (3.0 / 1536) ** 0.5})
        yield d


def replay(folder, dtype, steps):
    from pico_vllm_amd.engine.replay import TraceReplayer
    rep = TraceReplayer(folder, dtype, max_tokens=2 * 64 * (-(-N // 64)))
    out = {}
    for s in steps:
        got = rep.run_step(s)
        if got is not None:
            out[s["step"]] = got
    del rep
    torch.cuda.empty_cache()
    return out


def test_bfloat16_follows_the_32_bit_path_at_the_1_5b_shape(folder):
    rng = random.Random(1)
    toks = [rng.randrange(SHAPE["vocab_size"]) for _ in range(N)]
    # after the two large portions come portions of 40, 17 and 9 tokens (the weight-streaming kernels for 33 to 64,
    # 17 to 32 and 9 to 16 rows at these matrix sizes), then single tokens
    small = [40, 17, 9]
    cut = N - 32 - sum(small)                      # where the second large portion ends
    ends = [cut + sum(small[:i + 1]) - 1 for i in range(len(small))]
    want = [0, 1, 63, 64, 1000, 2047, 2048] + ends + [N - 1]
    whole = [{"step": 0, "entries": [{"id": "a", "tokens": toks, "want": want}], "end": ["a"]}]
    ref = replay(folder, "float32", whole)[0]
    spread = float(ref.std())
    assert np.isfinite(ref).all() and spread > 0.1

    def check(got, rows, label):
        err = got - ref[rows]
        rms = float(np.sqrt((err ** 2).mean())) / spread
        print(f"[large] {label}: rms error {rms:.2e} of the spread, argmax equal in {int((got.argmax(1) == ref[rows].argmax(1)).sum())}/{len(rows)} rows")
        # bfloat16 rounding through two layers and the output matrix measures 1.7e-2 .. 2.7e-2 here; a wrong key,
        # slice or page gives an error of the order of the spread itself
        assert np.isfinite(got).all() and rms < 5e-2, (label, rms)

    # whole: one step of 2,300 tokens (library GEMMs, key teams)
    check(replay(folder, "bfloat16", whole)[0], list(range(len(want))), "whole")
    # portions of 2,048 + the rest of the large part (prefix attention), the small portions, then the last 32 one by
    # one (skinny GEMMs, decode attention)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:2048], "want": [0, 1, 63, 64, 1000, 2047]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[2048:cut], "want": [0]}], "end": []}]
    at = cut
    for n in small:
        steps.append({"step": len(steps), "entries": [{"id": "a", "tokens": toks[at:at + n], "want": [n - 1]}], "end": []})
        at += n
    first_single = len(steps)
    for i in range(N - 32, N):
        steps.append({"step": len(steps), "entries": [{"id": "a", "tokens": [toks[i]], "want": [0] if i == N - 1 else []}], "end": []})
    last = len(steps) - 1
    assert at == N - 32 and last == first_single + 31
    got = replay(folder, "bfloat16", steps)
    check(got[0], [0, 1, 2, 3, 4, 5], "first portion")
    check(got[1], [6], "second portion")
    for j, n in enumerate(small):
        check(got[2 + j], [7 + j], f"portion of {n}")
    check(got[last], [len(want) - 1], "last token after 32 single steps")
    # the 32-bit path itself: portions and single tokens give what the whole prompt gives
    got32 = replay(folder, "float32", steps)
    for key, rows in ((0, [0, 1, 2, 3, 4, 5]), (1, [6]), (2, [7]), (3, [8]), (4, [9]), (last, [len(want) - 1])):
        assert float(np.abs(got32[key] - ref[rows]).max()) <= 2e-4 * spread, key


def test_decoding_40_requests_together_gives_what_each_gives_alone(folder):
    """At these sizes a batch of 40 decoding requests takes the kernels for 33 to 64 rows and another
    split of the context than a request alone; the logits of a request must not depend on it beyond
    the rounding of bfloat16 (the sums of the weight-streaming kernels are the same bit for bit, the
    attention merges its splits in another order)."""
    from pico_vllm_amd.engine.replay import TraceReplayer
    rng = random.Random(2)
    R = 40
    prompts = [[rng.randrange(SHAPE["vocab_size"]) for _ in range((5 if i % 2 else 500) + i)] for i in range(R)]    # short and long contexts
    nexts = [[rng.randrange(SHAPE["vocab_size"]) for _ in range(2)] for _ in range(R)]
    rep = TraceReplayer(folder, "bfloat16", max_tokens=R * 576, max_live=R)

    def prefill(i):
        return rep.run_step({"step": 0, "entries": [{"id": str(i), "tokens": prompts[i], "want": [len(prompts[i]) - 1]}], "end": []})

    # alone: prompt, then two single tokens
    alone = []
    for i in range(R):
        rows = [prefill(i)[0]]
        for t in nexts[i]:
            rows.append(rep.run_step({"step": 1, "entries": [{"id": str(i), "tokens": [t], "want": [0]}], "end": []})[0])
        rep.run_step({"step": 2, "entries": [], "end": [str(i)]})
        alone.append(rows)
    # together: the prompts one after the other (as above), then all 40 decode in one step, twice
    for i in range(R):
        got = prefill(i)[0]
        assert np.array_equal(got, alone[i][0]), i          # the same kernels on the same inputs
    for k in range(2):
        got = rep.run_step({"step": 3 + k, "entries": [{"id": str(i), "tokens": [nexts[i][k]], "want": [0]} for i in range(R)],
                            "end": []})
        ref = np.stack([alone[i][1 + k] for i in range(R)])
        spread = float(ref.std())
        rms = float(np.sqrt(((got - ref) ** 2).mean())) / spread
        same = int((got.argmax(1) == ref.argmax(1)).sum())
        print(f"[large] 40 together, decode step {k}: rms difference {rms:.2e} of the spread, argmax equal in {same}/{R} rows")
        assert rms < 5e-3 and same >= R - 2, (k, rms, same)
    del rep
    torch.cuda.empty_cache()


# ---- against the plain implementation ----------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["L1.5B", "L7B", "L32B"])
def test_real_layer_sizes_against_the_plain_implementation(name, dtype):
    import test_gpu_replay as R
    reqs = R.make_requests(name, [200], seed=21)
    print(f"[real sizes] {name} {dtype}", flush=True)
    for label, trace in (("whole", R.whole(reqs)), ("portions", R.portions(reqs)), ("tail", R.tail_one_by_one(reqs))):
        got, _ = R.replay(name, dtype, trace)
        R.compare(name, dtype, reqs, got, f"real {label}")
    torch.cuda.empty_cache()


def test_real_layer_sizes_mixed_in_a_small_pool():
    # seven requests of the 7B sizes, three live at a time, portions of some beside single tokens of others, pages used again
    import test_gpu_replay as R
    reqs = R.make_requests("L7B", [90, 70, 120, 64, 100, 80, 75], seed=22)
    trace = R.mixed(reqs, seed=5, max_live=3)
    for dtype in ("float32", "bfloat16"):
        got, pool = R.replay("L7B", dtype, trace)
        assert pool.reuse_count > 0
        R.compare("L7B", dtype, reqs, got, "real mixed")
    torch.cuda.empty_cache()


def test_graph_replay_and_the_step_in_flight_at_head_size_128():
    """Decode steps replayed from a HIP graph (recorded with the longest context's kernel choices and padded rows) and the
    decode step in flight, at the 1.5B layer sizes (heads of 128, groups of 6): batches of 1, 3 (a graph of 4) and 8;
    the same tokens in all four modes, each the plain implementation's argmax within bfloat16 rounding
    (the reference's graph path: pico_vllm/engine.py:139-191, its test tests/test_cuda_graph_model.py:64-197)."""
    import plain_qwen2 as P
    from tiny_configs import CONFIGS, model_dir
    from pico_vllm_amd import LLM, SamplingParams
    name = "L1.5B"
    V = CONFIGS[name]["vocab_size"]
    plain = P.PlainModel(model_dir(name))
    rng = random.Random(5)
    sp = SamplingParams(max_new_tokens=40, temperature=0.0, ignore_eos=True)
    for batch in (1, 3, 8):
        prompts = [[rng.randrange(V) for _ in range(rng.choice([3, 17, 40, 70]))] for _ in range(batch)]
        seen = {}
        for graph in (False, True):
            for pipeline in (False, True):
                llm = LLM(model=model_dir(name), dtype="bfloat16", block_size=16, num_gpu_blocks=8 * 8, max_seq_len=128,
                          max_num_seqs=8, max_num_batched_tokens=256, use_cuda_graph=graph, max_batch_size=8,
                          pipeline_decode=pipeline)
                outs = llm.generate(prompts, sp)
                if graph:
                    assert (1 if batch == 1 else 4 if batch == 3 else 8) in llm.engine.runner._graphs
                seen[graph, pipeline] = [o.token_ids for o in outs]
                del llm
                torch.cuda.empty_cache()
        first = seen[False, False]
        assert all(len(t) == 40 for t in first)
        for mode, toks in seen.items():
            assert toks == first, (batch, mode)
        for p, gen in zip(prompts, first):
            logits = plain.logits(p + gen)
            for k, t in enumerate(gen):
                row = logits[len(p) + k - 1]
                assert float(row[t]) >= float(row.max()) - 0.05 * float(row.std()), (batch, len(p), k, t, int(row.argmax()))


def test_prompt_steps_replayed_from_graphs_at_sizes_that_take_the_library_products():
    """A prompt portion that is a step of its own replays a graph recorded at the next of a few sizes, padded with
    filler tokens in a sequence of their own.  At the 1.5B layer sizes such a step holds library matrix products;
    whatever those record into a graph must give the same on every replay: every replay (prompts of other lengths
    and contents at the same recorded size, portions after a prefix, decode steps and synchronisations between them)
    is compared bit for bit with the same padded step run unrecorded, and with the plain implementation."""
    import plain_qwen2 as P
    from tiny_configs import CONFIGS, model_dir
    from pico_vllm_amd.engine.batch import SeqStep, build_context
    from pico_vllm_amd.engine.step import ModelRunner
    from pico_vllm_amd.parts.model import load_model
    name = "L1.5B"
    V = CONFIGS[name]["vocab_size"]
    model = load_model(model_dir(name), "bfloat16", "cuda:0")
    rec = ModelRunner(model, 16, 448, 4, 2048, 6144, use_graph=True, max_graph_batch=4)
    raw = ModelRunner(model, 16, 448, 4, 2048, 6144, use_graph=False)
    assert rec.graph_prompts and 320 in rec.prompt_sizes and 1024 in rec.prompt_sizes
    plain = P.PlainModel(model_dir(name))
    rng = random.Random(9)

    def both(rid, toks, want):
        """The step on both runners; the unrecorded one is padded by hand to the size the recorded one takes."""
        outs = []
        for r in (rec, raw):
            m = r.manager
            if rid not in m.requests:
                assert m.add_request(rid)
            assert m.grow(rid, m.num_computed(rid) + len(toks))
            seq = SeqStep(rid, toks, want)
            if r is rec:
                size = r._prompt_size([seq])
                outs.append(r.step([seq]).clone())
            elif size:
                ctx = build_context([seq], m, r.buffers, model.dtype, V, pad_tokens_to=size)
                outs.append(model.forward(ctx, r.storage).clone())
            else:
                outs.append(r.step([seq]).clone())
            r.advance([seq])
        torch.cuda.synchronize()
        return outs[0], outs[1], size

    sizes_seen = []
    for i, (n_first, n_second) in enumerate([(300, 290), (310, 17), (257, 200), (300, 0), (1000, 24), (318, 5)]):
        rid = f"p{i}"
        toks = [rng.randrange(V) for _ in range(n_first + n_second + 3)]
        a, b, size = both(rid, toks[:n_first], [n_first - 1])
        sizes_seen.append(size)
        assert size >= n_first and torch.equal(a, b), (i, "first portion", size)
        ref = plain.logits(toks[:n_first])[-1]
        assert float((a[0].cpu() - ref).abs().max()) < 0.1 * float(ref.std())
        if n_second:
            a, b, size2 = both(rid, toks[n_first:n_first + n_second], [n_second - 1])     # a portion after a prefix
            assert torch.equal(a, b), (i, "second portion", size2)
            ref = plain.logits(toks[:n_first + n_second])[-1]
            assert float((a[0].cpu() - ref).abs().max()) < 0.1 * float(ref.std())
        for t in toks[n_first + n_second:]:                                              # decode steps in between
            a, b, _ = both(rid, [t], [0])
            assert torch.equal(a, b)
        for r in (rec, raw):
            r.manager.free_request(rid)
    assert sizes_seen.count(320) >= 3 and 1024 in sizes_seen          # a recorded size was replayed after other work
    assert len(rec._prompt_graphs) >= 4 and not raw._prompt_graphs
    # Steps of decoding requests and one prompt portion are recorded too: the single tokens padded to a power of two
    # with empty rows, the portion to a recorded size with filler.  Each replay against the same padded step unrecorded,
    # bit for bit, and against the plain implementation.
    def both_mixed(seqs):
        outs = []
        singles = len(seqs) - 1
        for r in (rec, raw):
            m = r.manager
            for q in seqs:
                if q.req not in m.requests:
                    assert m.add_request(q.req)
                assert m.grow(q.req, m.num_computed(q.req) + len(q.tokens))
            if r is rec:
                size = r._prompt_size(seqs)
                before = len(r._prompt_graphs)
                outs.append(r.step(seqs).clone())
            else:
                rows = 1
                while rows < singles:
                    rows *= 2
                ctx = build_context(seqs, m, wide, model.dtype, V, pad_to=rows, pad_tokens_to=size)
                ctx.max_context = r.max_seq_len
                out = model.forward(ctx, r.storage)
                outs.append(torch.cat([out[:singles], out[rows:]]).clone())
            r.advance(seqs)
        torch.cuda.synchronize()
        return outs[0], outs[1], size, len(rec._prompt_graphs) - before

    from pico_vllm_amd.engine.batch import BatchBuffers
    wide = BatchBuffers(model.device, 2048 + 4, 6, raw.max_pages, 1)      # room for the padding, which the unrecording runner never needs
    lens = {"d0": 40, "d1": 333, "d2": 7}
    text = {rid: [rng.randrange(V) for _ in range(n + 8)] for rid, n in lens.items()}
    text["new"] = [rng.randrange(V) for _ in range(700)]
    at = dict(lens, new=0)
    for rid, n in lens.items():
        both(rid, text[rid][:n], [n - 1])
    recorded = 0
    for live, n in ((["d0", "d1", "d2"], 100), (["d1"], 37), (["d0", "d2"], 250), (["d2", "d0", "d1"], 2), (["d1", "d0", "d2"], 120),
                    (["d0"], 40), (["d1", "d2"], 110)):
        seqs = [SeqStep(rid, text[rid][at[rid]:at[rid] + 1], [0]) for rid in live] + [SeqStep("new", text["new"][at["new"]:at["new"] + n], [n - 1])]
        a, b, size, fresh = both_mixed(seqs)
        recorded += fresh
        assert size >= n and a.shape == (len(live) + 1, V) and torch.equal(a, b), (live, n, size)
        for q, row in zip(seqs, a):
            at[q.req] += len(q.tokens)
            ref = plain.logits(text[q.req][:at[q.req]])[-1]
            assert float((row.cpu() - ref).abs().max()) < 0.1 * float(ref.std()), (live, n, q.req)
    # seven steps, five shapes: (4 rows, 128), (1, 64), (2, 256), (4, 16) and (2, 128) were recorded, two were replays of them
    assert recorded == 5 and sorted(k[:2] for k in rec._prompt_graphs if k[0]) == [(1, 64), (2, 128), (2, 256), (4, 16), (4, 128)]
    big = [SeqStep("d0", [1], [0]), SeqStep("new", [1] * 140, [139])]
    assert rec._prompt_size(big[1:]) == 192 and rec._prompt_size(big) == 192
    big[1] = SeqStep("new", [1] * 1100, [0])
    assert rec._prompt_size(big[1:]) == 1280 and not rec._prompt_size(big)              # beyond 1,024 tokens only alone
    for r in (rec, raw):
        for rid in at:
            r.manager.free_request(rid)
    # What the attention chooses on the host (the shape of its prefill workgroups) differs between a first portion and
    # one behind thousands of tokens: the two are recorded apart, and each replay is the unrecorded step bit for bit.
    toks = [rng.randrange(V) for _ in range(6000)]
    for at, n in ((0, 2048), (2048, 2048), (4096, 1900)):
        a, b, size = both("long", toks[at:at + n], [n - 1])
        assert size == 2048 and torch.equal(a, b), (at, n)
    variants = {key[3] for key in rec._prompt_graphs if key[1] == 2048}
    assert len(variants) >= 2, variants
    del rec, raw, model
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_all_28_layers_of_the_1_5b_shape_against_the_plain_implementation(dtype):
    """The benchmark's own configuration, every layer and the whole vocabulary of 151,936, with random weights: a prompt
    of 48 tokens whole and with its last 8 tokens one by one against the plain implementation in float64, with the
    yardsticks of the replay tests (in float32: eight permuted float32 runs of the plain implementation)."""
    import test_gpu_replay as R
    reqs = R.make_requests("F1.5B", [48], seed=23)
    print(f"[real sizes] F1.5B {dtype}", flush=True)
    for label, trace in (("whole", R.whole(reqs)), ("tail", R.tail_one_by_one(reqs, tail=8))):
        got, _ = R.replay("F1.5B", dtype, trace)
        R.compare("F1.5B", dtype, reqs, got, f"28 layers {label}")
    torch.cuda.empty_cache()
    if dtype == "bfloat16":
        for key in [k for k in R._plain_cache if k == "F1.5B" or (isinstance(k, tuple) and k[0] == "F1.5B")]:
            del R._plain_cache[key]          # 18 GB of float32 and float64 weights
