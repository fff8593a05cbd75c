"""Generation through the entry point against the plain implementation: the workloads of the two
tiny configurations, greedy and with temperature, chunked prompts mixed with decoding, HIP graph
replay of decode steps, and what happens when pages run out."""
import os

import pytest
import torch

import plain_qwen2 as P
from tiny_configs import CONFIGS, PAGE_SIZE, TINY_A, model_dir

pytestmark = pytest.mark.gpu


def llm(name, dtype, **kw):
    from pico_vllm_amd import LLM
    args = dict(block_size=PAGE_SIZE[name], num_gpu_blocks=64, max_seq_len=256, max_num_seqs=4,
                max_num_batched_tokens=64, use_cuda_graph=False)
    args.update(kw)
    return LLM(model=model_dir(name), dtype=dtype, **args)


def prompts_for(name, lengths, seed=0):
    g = torch.Generator().manual_seed(seed)
    V = CONFIGS[name]["vocab_size"]
    return [torch.randint(0, V - 1, (n,), generator=g).tolist() for n in lengths]     # never the eos id


def check_greedy(name, dtype, prompts, outs):
    """Every generated token is the plain argmax given the same prefix (bfloat16: or within the
    rounding error of the logits of it)."""
    plain = P.PlainModel(model_dir(name))
    for p, o in zip(prompts, outs):
        toks = list(p)
        for t in o.token_ids:
            logits = plain.logits(toks)[-1]
            slack = 1e-4 if dtype == "float32" else 0.05 * float(logits.std())
            assert float(logits[t]) >= float(logits.max()) - slack, (name, dtype, len(p), o.token_ids)
            toks.append(t)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_tiny_a_workload_greedy(dtype):
    from pico_vllm_amd import SamplingParams
    prompts = prompts_for("A", [5, 11, 23])
    outs = llm("A", dtype).generate(prompts, SamplingParams(max_new_tokens=8, temperature=0.0, ignore_eos=True))
    assert [len(o.token_ids) for o in outs] == [8, 8, 8] and all(o.finish_reason == "length" for o in outs)
    check_greedy("A", dtype, prompts, outs)
    if dtype == "float32":
        plain = P.PlainModel(model_dir("A"))
        assert [o.token_ids for o in outs] == [plain.greedy(p, 8) for p in prompts]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_tiny_b_workload_chunks_of_13_temperature(dtype):
    """4 requests, prompts 1/7/19/40, prefilled in portions of at most 13 tokens mixed with decoding,
    10 tokens each at temperature 0.8 with a fixed seed."""
    from pico_vllm_amd import SamplingParams
    from pico_vllm_amd.sampling.sampler import uniform
    prompts = prompts_for("B", [1, 7, 19, 40], seed=1)
    sp = [SamplingParams(max_new_tokens=10, temperature=0.8, seed=100 + i, ignore_eos=True) for i in range(4)]
    eng = llm("B", dtype, max_num_batched_tokens=13)
    outs = eng.generate(prompts, sp)
    assert eng.engine.stats["steps"] > 10 + 3            # prompts were cut: 67 prompt tokens at <= 13 a step
    again = llm("B", dtype, max_num_batched_tokens=64).generate(prompts, sp)
    plain = P.PlainModel(model_dir("B"))
    for i, (p, o) in enumerate(zip(prompts, outs)):
        assert len(o.token_ids) == 10
        toks = list(p)
        for k, t in enumerate(o.token_ids):
            probs = P.temperature_probs(plain.logits(toks)[-1], 0.8)
            u = uniform(100 + i, k)
            want = P.inverse_cdf(probs, u)
            if t != want:        # only where u falls within the engine's rounding of a CDF boundary
                cum = torch.cumsum(probs, 0)
                edge = float(cum[min(t, want)])
                assert abs(edge - u) < (1e-4 if dtype == "float32" else 2e-2), (dtype, i, k, t, want, u, edge)
            toks.append(t)
        if dtype == "float32":
            assert o.token_ids == again[i].token_ids     # same seed, other batching: same tokens


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_top_p_and_eos(dtype):
    from pico_vllm_amd import SamplingParams
    prompts = prompts_for("B", [9, 9], seed=2)
    outs = llm("B", dtype).generate(prompts, [SamplingParams(max_new_tokens=12, temperature=1.0, top_p=0.5, seed=7),
                                               SamplingParams(max_new_tokens=12, temperature=0.0)])
    plain = P.PlainModel(model_dir("B"))
    toks = list(prompts[0])
    for t in outs[0].token_ids:                         # every draw lies in the nucleus of the plain rule
        p = P.top_p_probs(plain.logits(toks)[-1], 1.0, 0.5 if dtype == "float32" else 0.55)
        assert float(p[t]) > 0
        toks.append(t)
    eos = CONFIGS["B"]["eos_token_id"]
    for o in outs:
        assert (o.finish_reason == "eos") == (o.token_ids[-1] == eos and len(o.token_ids) <= 12)
        assert eos not in o.token_ids[:-1]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_replayed_from_a_graph_give_the_same_tokens(dtype):
    from pico_vllm_amd import SamplingParams
    prompts = prompts_for("A", [5, 11, 23, 40, 3], seed=3)
    sp = SamplingParams(max_new_tokens=40, temperature=0.0, ignore_eos=True)
    eager = llm("A", dtype, num_gpu_blocks=128).generate(prompts, sp)
    graph_llm = llm("A", dtype, num_gpu_blocks=128, use_cuda_graph=True, max_batch_size=4)
    graphed = graph_llm.generate(prompts, sp)
    assert graph_llm.engine.runner._graphs, "no decode step went through a graph"
    # the same kernels with the same choices on the same inputs: the same tokens, in bfloat16 too
    assert [o.token_ids for o in graphed] == [o.token_ids for o in eager]
    check_greedy("A", dtype, prompts, graphed)
    # a second batch on the same engine replays the graphs captured by the first
    more = graph_llm.generate(prompts[:2], sp)
    check_greedy("A", dtype, prompts[:2], more)


def test_decode_steps_of_many_unequal_requests_cut_their_contexts_alike_recorded_or_not(monkeypatch):
    # 21 requests (a recorded step of them is padded to 32) with prompts of 3 to 120 tokens: their decode steps cut the
    # contexts of all sequences into pieces of one length; recorded and padded or not, the same tokens in bfloat16
    # (that the logits of such steps are the plain implementation's within rounding: test_gpu_replay.py)
    from pico_vllm_amd import SamplingParams
    from pico_vllm_amd.ops.attention_fast import FastAttention
    cuts = []
    real = FastAttention.decode_cut
    monkeypatch.setattr(FastAttention, "decode_cut", lambda self, n, ns, dev: cuts.append((n, ns, real(self, n, ns, dev))) or cuts[-1][2])
    lengths = [3, 120, 17, 64, 5, 99, 33, 2, 80, 47, 111, 9, 65, 28, 1, 73, 16, 104, 55, 12, 90]
    prompts = prompts_for("B", lengths, seed=21)
    sp = SamplingParams(max_new_tokens=25, temperature=0.0, ignore_eos=True)
    kw = dict(num_gpu_blocks=21 * 20 + 8, max_num_seqs=21, max_num_batched_tokens=512, max_seq_len=192)
    eager = llm("B", "bfloat16", **kw).generate(prompts, sp)
    assert any(c is not None and n == 21 for n, _, c in cuts), "no decode step cut its contexts over all sequences"
    cuts.clear()
    graph_llm = llm("B", "bfloat16", use_cuda_graph=True, max_batch_size=32, **kw)
    graphed = graph_llm.generate(prompts, sp)
    assert 32 in graph_llm.engine.runner._graphs and any(c is not None and n == 32 for n, _, c in cuts)
    assert [o.token_ids for o in graphed] == [o.token_ids for o in eager]


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("B", "bfloat16")])
def test_steps_of_decoding_requests_and_a_prompt_portion_replayed_from_graphs_give_the_same_tokens(name, dtype):
    # a small token budget: while prompts are still coming in, most steps are a few decoding requests and one portion of a
    # prompt; those are recorded with the single tokens padded to a power of two and the portion to a recorded size
    from pico_vllm_amd import SamplingParams
    prompts = prompts_for(name, [40, 9, 77, 23, 51, 30, 64], seed=5)
    sps = [SamplingParams(max_new_tokens=n, temperature=t, top_p=0.9, seed=i, ignore_eos=True)
           for i, (n, t) in enumerate([(30, 0.0), (45, 0.0), (12, 0.7), (40, 0.0), (25, 0.0), (33, 0.9), (8, 0.0)])]
    kw = dict(num_gpu_blocks=160, max_num_seqs=4, max_num_batched_tokens=32, max_seq_len=128)
    eager = llm(name, dtype, **kw).generate(prompts, sps)
    graph_llm = llm(name, dtype, use_cuda_graph=True, max_batch_size=4, **kw)
    graphed = graph_llm.generate(prompts, sps)
    keys = list(graph_llm.engine.runner._prompt_graphs)
    assert any(k[0] > 0 for k in keys), "no step of single tokens and a portion went through a graph"
    assert any(k[0] == 0 for k in keys) and graph_llm.engine.runner._graphs
    assert {k[0] for k in keys} <= {0, 1, 2, 4}
    assert [o.token_ids for o in graphed] == [o.token_ids for o in eager]
    check_greedy(name, dtype, [prompts[i] for i in (0, 1, 3, 4, 6)], [graphed[i] for i in (0, 1, 3, 4, 6)])
    # nothing is recorded when the option says so
    off = llm(name, dtype, use_cuda_graph=True, max_batch_size=4, graph_prompts=False, **kw)
    assert [o.token_ids for o in off.generate(prompts, sps)] == [o.token_ids for o in eager]
    assert not off.engine.runner._prompt_graphs and off.engine.runner._graphs


def test_running_out_of_pages_preempts_and_recomputes_to_the_same_tokens():
    from pico_vllm_amd import SamplingParams
    prompts = prompts_for("A", [30, 30, 30], seed=4)
    sp = SamplingParams(max_new_tokens=40, temperature=0.0, ignore_eos=True)
    roomy = llm("A", "float32", num_gpu_blocks=64).generate(prompts, sp)
    tight_llm = llm("A", "float32", num_gpu_blocks=8)               # 8 pages of 16: three requests of 70 do not fit
    tight = tight_llm.generate(prompts, sp)
    assert tight_llm.engine.stats["preemptions"] > 0 and sum(o.num_preemptions for o in tight) > 0
    assert tight[0].num_preemptions == 0                             # the oldest request is never the victim
    assert [o.token_ids for o in tight] == [o.token_ids for o in roomy]
    m = tight_llm.engine.runner.manager
    m.check()
    assert m.groups[0].pool.num_free == 8 and m.groups[0].pool.reuse_count > 0


@pytest.mark.parametrize("name", ["A", "B"])
def test_tokens_recomputed_after_a_preemption_in_bfloat16_are_still_the_plain_argmax(name):
    # In bfloat16 a preempted request's earlier tokens come back through the prompt kernels, so its later tokens need
    # not be the bits of an undisturbed run; they must still be right: every token the plain argmax given the
    # engine's own prefix, within the rounding of the logits.
    from pico_vllm_amd import SamplingParams
    prompts = prompts_for(name, [30, 30, 30, 17], seed=14)
    sp = SamplingParams(max_new_tokens=40, temperature=0.0, ignore_eos=True)
    pages = 8 * 16 // PAGE_SIZE[name]                               # room for 128 tokens: four requests of up to 70 do not fit
    for graphs in (False, True):
        tight_llm = llm(name, "bfloat16", num_gpu_blocks=pages, use_cuda_graph=graphs, max_batch_size=4)
        tight = tight_llm.generate(prompts, sp)
        assert tight_llm.engine.stats["preemptions"] > 0 and sum(o.num_preemptions for o in tight) > 0
        assert tight[0].num_preemptions == 0
        assert [len(o.token_ids) for o in tight] == [40] * 4 and all(o.finish_reason == "length" for o in tight)
        check_greedy(name, "bfloat16", prompts, tight)
        m = tight_llm.engine.runner.manager
        m.check()
        assert m.groups[0].pool.num_free == pages and m.groups[0].pool.reuse_count > 0 and not m.requests


def test_submit_step_is_done_in_the_reference_manner():
    from pico_vllm_amd import EngineArgs
    from pico_vllm_amd.engine.llm import LLMEngine
    eng = LLMEngine(EngineArgs(model=model_dir("A"), dtype="float32", num_gpu_blocks=32, max_seq_len=128,
                               use_cuda_graph=False, pipeline_decode=False))
    a = eng.submit([1, 2, 3], max_new_tokens=1, temperature=0, top_p=1.0)
    b = eng.submit([4, 5, 6, 7], max_new_tokens=3, temperature=0, top_p=1.0, ignore_eos=True)
    done = []
    steps = 0
    while not eng.is_done():
        done += eng.step()
        steps += 1
    # a request that finishes in its prefill step is reported once and not decoded again
    assert [o.request_id for o in done] == [a, b] and steps == 3
    assert len(done[0].token_ids) == 1 and len(done[1].token_ids) == 3
    with pytest.raises(ValueError):
        eng.submit([1] * 200, max_new_tokens=10)
    with pytest.raises(ValueError):
        eng.submit([999], max_new_tokens=1)
    # after mark_finished nothing more is taken (the reference returns -1 then, engine.py:250-251)
    c = eng.submit([7, 8], max_new_tokens=2, ignore_eos=True)
    eng.mark_finished()
    assert eng.submit([1, 2, 3], max_new_tokens=1) == -1 and not eng.is_done()
    while not eng.is_done():
        done += eng.step()
    assert done[-1].request_id == c and len(done[-1].token_ids) == 2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("graph", [False, True])
def test_a_decode_step_in_flight_changes_nothing(dtype, graph):
    # with pipeline_decode the next decode step starts from the tokens on the device before the host has
    # read them; requests end by length and by the end-of-sequence token at different steps, one is
    # sampled with a temperature, and pages are so few that requests are preempted
    from pico_vllm_amd import SamplingParams
    name = "B"
    eos = CONFIGS[name]["eos_token_id"]
    g = torch.Generator().manual_seed(8)
    V = CONFIGS[name]["vocab_size"]
    prompts = [torch.randint(0, V, (n,), generator=g).tolist() for n in (9, 30, 17, 5, 41)]
    sps = [SamplingParams(max_new_tokens=n, temperature=t, top_p=p, seed=3, ignore_eos=ig)
           for n, t, p, ig in ((25, 0.0, 1.0, False), (7, 0.0, 1.0, True), (40, 0.9, 0.8, False), (1, 0.0, 1.0, True),
                               (33, 0.0, 1.0, False))]
    outs = {}
    for pipe in (False, True):
        for blocks in (64, 14):
            eng = llm(name, dtype, num_gpu_blocks=blocks, max_num_seqs=3, use_cuda_graph=graph, max_batch_size=4,
                      pipeline_decode=pipe)
            outs[pipe, blocks] = eng.generate(prompts, sps)
            eng.engine.runner.manager.check()
            assert eng.engine._inflight is None
            assert eng.engine.runner.manager.groups[0].pool.num_free == blocks
    base = outs[False, 64]
    for o, sp in zip(base, sps):
        assert 1 <= len(o.token_ids) <= sp.max_new_tokens
        assert (o.finish_reason == "eos") == (not sp.ignore_eos and o.token_ids[-1] == eos)
    if dtype == "float32":       # float32 logits do not depend on the batch, so neither do the tokens
        for key, got in outs.items():
            assert [(o.token_ids, o.finish_reason) for o in got] == [(o.token_ids, o.finish_reason) for o in base], key
    else:                        # bfloat16: rounding depends on the batch; every greedy token is the plain argmax within rounding
        greedy = [i for i, sp in enumerate(sps) if sp.temperature == 0.0]
        for got in outs.values():
            check_greedy(name, dtype, [prompts[i] for i in greedy], [got[i] for i in greedy])
            for o, sp in zip(got, sps):
                assert 1 <= len(o.token_ids) <= sp.max_new_tokens
                assert (o.finish_reason == "eos") == (not sp.ignore_eos and o.token_ids[-1] == eos)
    assert any(o.num_preemptions for o in outs[True, 14])


def test_stop_tokens_end_a_request_like_the_end_of_sequence_token():
    from pico_vllm_amd import SamplingParams
    prompts = prompts_for("A", [12], seed=6)
    base = llm("A", "float32").generate(prompts, SamplingParams(max_new_tokens=12, temperature=0.0, ignore_eos=True))[0]
    stop = base.token_ids[4]
    first = base.token_ids.index(stop)
    out = llm("A", "float32").generate(prompts, SamplingParams(max_new_tokens=12, temperature=0.0, ignore_eos=True,
                                                               stop_token_ids=[stop]))[0]
    assert out.finish_reason == "stop" and out.token_ids == base.token_ids[:first + 1]     # the stop token is kept


def test_command_line_on_random_weights_of_a_named_size(capsys):
    from pico_vllm_amd import run
    assert run.main(["--random-config", "tiny-a", "--prompt-ids", "5,17,3", "--prompt-ids", "9", "--max-new-tokens", "6",
                     "--ignore-eos", "--dtype", "float32", "--num-gpu-blocks", "16", "--max-seq-len", "64"]) == 0
    lines = [l for l in capsys.readouterr().out.splitlines() if l.startswith("[")]
    assert len(lines) == 2 and all("(length)" in l and len(l.split(")")[1].split()) == 6 for l in lines)



def test_command_line_with_a_text_prompt_and_a_tokenizer_in_the_model_folder(capsys, tmp_path):
    """--prompt TEXT goes through the tokenizer files of the model folder, as the reference's entry script
    does (pico_vllm/run_single.py:15,31); the answer is the decoded prompt + generated tokens
    (pico_vllm/engine.py:385); the end-of-sequence token comes from the tokenizer when config.json names none
    (engine.py:48)."""
    import json
    from tokenizers import Tokenizer
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import WhitespaceSplit
    from pico_vllm_amd import run
    from pico_vllm_amd.weights.random_init import write_random_model
    folder = str(tmp_path / "model")
    config = {k: v for k, v in TINY_A.items() if k not in ("model_type", "eos_token_id")}
    write_random_model(folder, config, 0)
    tok = Tokenizer(WordLevel({f"w{i}": i for i in range(config["vocab_size"])}, unk_token="w0"))
    tok.pre_tokenizer = WhitespaceSplit()
    tok.save(os.path.join(folder, "tokenizer.json"))
    common = ["--model", folder, "--max-new-tokens", "8", "--dtype", "float32", "--num-gpu-blocks", "16", "--max-seq-len", "64"]
    with open(os.path.join(folder, "tokenizer_config.json"), "w") as f:
        json.dump({"tokenizer_class": "PreTrainedTokenizerFast"}, f)
    assert run.main(common + ["--prompt-ids", "5,17,3"]) == 0
    ids = [l for l in capsys.readouterr().out.splitlines() if l.startswith("[")][0].split(")")[1].split()
    assert len(ids) == 8
    assert run.main(common + ["--prompt", "w5 w17 w3"]) == 0
    text = [l for l in capsys.readouterr().out.splitlines() if l.startswith("[")][0].split(")", 1)[1].strip()
    assert text == " ".join(["w5", "w17", "w3"] + [f"w{i}" for i in ids])
    # the tokenizer names the third generated token as the end of a sequence: generation stops there and keeps it
    with open(os.path.join(folder, "tokenizer_config.json"), "w") as f:
        json.dump({"tokenizer_class": "PreTrainedTokenizerFast", "eos_token": f"w{ids[2]}"}, f)
    assert run.main(common + ["--prompt", "w5 w17 w3"]) == 0
    line = [l for l in capsys.readouterr().out.splitlines() if l.startswith("[")][0]
    first = ids.index(ids[2])
    assert "(eos)" in line and line.split(")", 1)[1].split() == ["w5", "w17", "w3"] + [f"w{i}" for i in ids[:first + 1]]


def test_what_the_model_cannot_run_is_refused_before_serving_starts():
    from pico_vllm_amd import EngineArgs
    from pico_vllm_amd.engine.llm import LLMEngine
    from pico_vllm_amd.parts.attention import GQAAttention
    from pico_vllm_amd.parts.spec import PartSpec
    # a request could reach positions beyond what the model was made for
    with pytest.raises(ValueError, match="max_position_embeddings"):
        LLMEngine(EngineArgs(model=model_dir("A"), dtype="float32", max_seq_len=TINY_A["max_position_embeddings"] + 1))
    # a head size no attention kernel takes: refused when the part is built, not at the first step
    with pytest.raises(ValueError, match="head size"):
        GQAAttention(1024, 2, 1, 512, True, PartSpec("none", {}))


def test_a_finished_request_leaves_the_engine():
    from pico_vllm_amd import SamplingParams
    eng = llm("A", "float32")
    eng.generate(prompts_for("A", [5, 9, 3]), SamplingParams(max_new_tokens=4, ignore_eos=True))
    assert eng.engine.requests == {} and not eng.engine.runner.manager.requests


def test_phase_timers_behind_their_flag_change_nothing(monkeypatch):
    from pico_vllm_amd import SamplingParams
    from pico_vllm_amd.engine.phases import PhaseTimers
    monkeypatch.setattr(PhaseTimers, "COLLECT_EVERY", 6)        # events are read while the run goes on, not only by a report
    prompts = prompts_for("A", [5, 30, 11], seed=6)
    sp = SamplingParams(max_new_tokens=12, temperature=0.0, ignore_eos=True)
    plain_run = llm("A", "bfloat16", use_cuda_graph=True, max_batch_size=4)
    timed = llm("A", "bfloat16", use_cuda_graph=True, max_batch_size=4, profile_phases=True)
    a, b = plain_run.generate(prompts, sp), timed.generate(prompts, sp)
    assert [o.token_ids for o in a] == [o.token_ids for o in b]
    assert "phases" not in plain_run.engine.report()
    assert len(timed.engine.timers._pending) < 4 * 6 and timed.engine.timers.device_s["model"] > 0
    rep = timed.engine.report()
    steps = rep["steps"]
    assert steps >= 12 and rep["decode_tokens"] > 0 and rep["prefill_tokens"] == 46
    assert rep["phases"]["model"]["calls"] == steps == rep["phases"]["sample"]["calls"]
    assert rep["phases"]["model"]["device_ms"] > 0 and rep["phases"]["model"]["host_ms_per_call"] > 0
    assert rep["phases"]["schedule"]["calls"] >= steps and rep["phases"]["read"]["calls"] == steps
    assert rep["pages"][0]["in_use"] == 0 and rep["pages"][0]["peak"] > 0 and rep["graphs"]


def test_what_generate_and_the_step_refuse_and_the_defaults_they_fall_back_to():
    from pico_vllm_amd import LLM, SamplingParams
    from pico_vllm_amd.engine.batch import BatchError, SeqStep
    # no number of pages given: room for max_num_seqs requests of max_seq_len tokens
    eng = LLM(model=model_dir("A"), dtype="float32", block_size=16, max_seq_len=100, max_num_seqs=3, max_num_batched_tokens=64,
              use_cuda_graph=False)
    assert eng.engine.runner.manager.groups[0].pool.num_pages == 3 * 7
    sizing = eng.engine.report()["pool_sizing"]
    assert sizing["pages"] == 21 == sizing["wanted"] and sizing["from"] == "max_num_seqs * max_seq_len" and sizing["fit"] > 21
    # 2 layers x (k and v) x 1 kv head x 16 x 16 tokens x 4 bytes
    assert sizing["bytes_per_page"] == 2 * 2 * 16 * 16 * 4
    # ... or as many as a share of the free memory holds, when that is fewer; none for a whole request is refused
    free = torch.cuda.mem_get_info()[0]
    share = 40.5 * sizing["bytes_per_page"] / free
    small = LLM(model=model_dir("A"), dtype="float32", block_size=16, max_seq_len=100, max_num_seqs=30, max_num_batched_tokens=64,
                use_cuda_graph=False, kv_memory_fraction=share)
    sizing = small.engine.report()["pool_sizing"]
    assert sizing["from"] == "memory" and sizing["wanted"] == 210 and 30 <= sizing["pages"] <= 41
    assert small.engine.runner.manager.groups[0].pool.num_pages == sizing["pages"]
    with pytest.raises(ValueError, match="not one request of max_seq_len"):
        LLM(model=model_dir("A"), dtype="float32", block_size=16, max_seq_len=100, max_num_seqs=30, max_num_batched_tokens=64,
            use_cuda_graph=False, kv_memory_fraction=3.5 * sizing["bytes_per_page"] / free)
    # portions of a prompt capped beside the budget
    capped = LLM(model=model_dir("A"), dtype="float32", block_size=16, max_seq_len=100, max_num_seqs=3, max_num_batched_tokens=64,
                 use_cuda_graph=False, prefill_chunk=7)
    prompts = prompts_for("A", [30, 9], seed=2)
    outs = capped.generate(prompts, SamplingParams(max_new_tokens=5, ignore_eos=True))
    assert capped.engine.stats["steps"] >= 5 + 4                       # 30 tokens in portions of at most 7
    check_greedy("A", "float32", prompts, outs)
    prompts = prompts_for("A", [5, 9], seed=2)
    outs = eng.generate(prompts)                                       # no options given: greedy, 16 tokens at most
    assert all(1 <= len(o.token_ids) <= 16 for o in outs)
    check_greedy("A", "float32", prompts, outs)
    with pytest.raises(ValueError, match="one SamplingParams per prompt"):
        eng.generate(prompts, [SamplingParams()] * 3)
    with pytest.raises(ValueError, match="needs a tokenizer"):
        eng.generate(["some text"])
    with pytest.raises(ValueError, match="temperature"):
        eng.generate(prompts, SamplingParams(temperature=float("nan")))
    assert eng.engine.is_done()
    # the step function itself
    r = eng.engine.runner
    m = r.manager
    m.add_request("a"); m.add_request("b")
    assert m.grow("a", 4) and m.grow("b", 1)
    with pytest.raises(BatchError, match="single-token sequences only"):
        r.step([SeqStep("a", [1, 2, 3, 4], [3]), SeqStep("b", [1], [0])], device_tokens=torch.zeros(2, dtype=torch.int32, device="cuda"))
    m.advance("a", 4)
    assert m.grow("a", 100)
    with pytest.raises(BatchError, match="beyond max_seq_len=100"):
        r.step([SeqStep("a", [1] * 97, [])])
    logits = r.step([SeqStep("a", [1] * 60, [59]), SeqStep("b", [1], [0])])
    assert logits.shape == (2, CONFIGS["A"]["vocab_size"]) and bool(torch.isfinite(logits).all())
    m.free_request("a"); m.free_request("b")
    m.check()


def test_the_sizes_that_reports_are_made_of_and_the_measured_peaks():
    from pico_vllm_amd.ops import peaks
    from pico_vllm_amd.sampling.sampler import Sampler
    eng = llm("B", "bfloat16").engine
    c = CONFIGS["B"]
    H, I, V, L = c["hidden_size"], c["intermediate_size"], c["vocab_size"], c["num_hidden_layers"]
    nq, nkv = c["num_attention_heads"], c["num_key_value_heads"]
    d = c.get("head_dim", H // nq)
    per_layer = (nq + 2 * nkv) * d * H + H * nq * d + 2 * I * H + H * I          # q/k/v, o, gate/up, down
    assert not c["tie_word_embeddings"]
    assert eng.model.num_weight_bytes() == 2 * (L * per_layer + V * H)           # and the output matrix once
    per_token = L * 2 * nkv * d * 2
    assert eng.runner.storage.bytes_per_token() == per_token
    assert eng.runner.storage.num_bytes() == per_token * 64 * PAGE_SIZE["B"]     # 64 pages
    assert eng.runner.decode_bytes([10, 300]) == eng.model.num_weight_bytes() + 310 * per_token
    tied = llm("A", "bfloat16").engine
    a = CONFIGS["A"]
    assert a["tie_word_embeddings"]
    da = a.get("head_dim", a["hidden_size"] // a["num_attention_heads"])
    per_layer = ((a["num_attention_heads"] + 2 * a["num_key_value_heads"]) * da * a["hidden_size"]
                 + a["hidden_size"] * a["num_attention_heads"] * da + 3 * a["intermediate_size"] * a["hidden_size"])
    assert tied.model.num_weight_bytes() == 2 * (a["num_hidden_layers"] * per_layer + a["vocab_size"] * a["hidden_size"])
    # the two yardsticks of the benchmark: what a read stream and a loop of matrix-core products reach on this GPU
    stream = peaks.read_bandwidth(num_bytes=1 << 30, reps=5)
    flops, seconds = peaks.mfma_peak(reps=3, iters=4000)
    assert 2e12 < stream < 8e12 and 0.8e15 < flops < 2.6e15 and seconds > 0, (stream, flops)
    # the sampler's own refusals, and one call that launches and reads
    sm = Sampler(torch.device("cuda:0"), 2)
    logits = torch.zeros(3, 50, device="cuda")
    logits[0, 7] = logits[1, 9] = 1.0
    assert sm.sample(logits[:2], [0.0, 0.0], [1.0, 1.0], [1, 2], [0, 0]) == [7, 9]
    with pytest.raises(ValueError, match="one set of sampling parameters per row"):
        sm.launch(logits[:2], [0.0], [1.0, 1.0], [1, 2], [0, 0])
    with pytest.raises(ValueError, match="3 rows to sample, the sampler was made for 2"):
        sm.launch(logits, [0.0] * 3, [1.0] * 3, [1, 2, 3], [0] * 3)


def test_a_stop_token_that_arrives_while_the_other_request_is_being_preempted():
    # With a step in flight the next step is planned before the tokens of the one in flight are read.  Two requests, so
    # few pages that the younger one is preempted when both want their third page; the older one's stop token is placed
    # at every position in turn, so that at one of them it arrives in the very step whose plan preempted the younger:
    # all that the plan held has then ended, and the engine has to plan anew instead of finding nothing to run.
    from pico_vllm_amd import SamplingParams
    prompts = prompts_for("A", [20, 20], seed=11)
    free = SamplingParams(max_new_tokens=40, temperature=0.0, ignore_eos=True)
    roomy = dict(num_gpu_blocks=16, max_num_seqs=2, max_num_batched_tokens=64, max_seq_len=64, use_cuda_graph=False)
    ref = [o.token_ids for o in llm("A", "float32", **roomy).generate(prompts, free)]
    assert len(ref[0]) == 40 and len(ref[1]) == 40
    tight = dict(roomy, num_gpu_blocks=5)
    preempted = 0
    for k in range(40):
        stop = ref[0][k]
        first = ref[0].index(stop)                              # the request ends where the token first appears
        sps = [SamplingParams(max_new_tokens=40, temperature=0.0, ignore_eos=True, stop_token_ids=[stop]), free]
        for pipe in (True, False):
            eng = llm("A", "float32", pipeline_decode=pipe, **tight)
            outs = eng.generate(prompts, sps)
            assert [o.token_ids for o in outs] == [ref[0][:first + 1], ref[1]], (k, pipe)
            assert outs[0].finish_reason == ("stop" if first < 39 or stop == ref[0][39] else "length") and outs[1].finish_reason == "length"
            preempted += eng.engine.stats["preemptions"]
            m = eng.engine.runner.manager
            m.check()
            assert all(g.pool.num_free == g.pool.num_pages for g in m.groups)
    assert preempted > 0


@pytest.mark.parametrize("seed", range(3))
def test_drawn_serving_scenarios_give_the_same_tokens_in_every_mode(seed):
    # requests of drawn lengths and options (greedy and sampled, stop tokens, the end-of-sequence token honoured or not)
    # served with and without recorded steps, with and without the step in flight, in a roomy and in a tight pool that
    # forces preemption: in float32 the same tokens and finish reasons in all eight, no page lost, nothing left behind
    import random
    from pico_vllm_amd import LLM, SamplingParams
    rng = random.Random(1000 + seed)
    for _ in range(8):
        name = rng.choice(["A", "B", "C", "D", "E"])
        V, page = CONFIGS[name]["vocab_size"], PAGE_SIZE[name]
        n = rng.randint(2, 7)
        prompts = [[rng.randrange(V - 1) for _ in range(rng.choice([1, 2, 3, 7, 15, 16, 17, 33, 64, 65, 100]))] for _ in range(n)]
        sps = [SamplingParams(max_new_tokens=rng.choice([1, 2, 5, 17, 40]), temperature=rng.choice([0.0, 0.0, 0.8]), top_p=rng.choice([1.0, 0.9]),
                              seed=rng.randrange(1000), ignore_eos=rng.random() < 0.7,
                              stop_token_ids=[rng.randrange(V)] if rng.random() < 0.3 else []) for _ in range(n)]
        longest = max(len(p) + sp.max_new_tokens for p, sp in zip(prompts, sps))
        need = -(-longest // page)
        max_seqs, budget = rng.randint(2, 5), rng.choice([16, 33, 64, 128])
        tight = need + rng.randint(0, need)
        ref = None
        for graphs in (False, True):
            for pipe in (False, True):
                for pages in (need * max_seqs + 4, tight):
                    eng = LLM(model=model_dir(name), dtype="float32", block_size=page, num_gpu_blocks=pages, max_seq_len=max(longest, 16),
                              max_num_seqs=max_seqs, max_num_batched_tokens=budget, use_cuda_graph=graphs, pipeline_decode=pipe,
                              max_batch_size=4)
                    got = [(o.token_ids, o.finish_reason) for o in eng.generate(prompts, sps)]
                    m = eng.engine.runner.manager
                    m.check()
                    assert all(g.pool.num_free == g.pool.num_pages for g in m.groups) and not eng.engine.requests
                    ref = ref or got
                    assert got == ref, (name, graphs, pipe, pages, [len(p) for p in prompts])


@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_a_recorded_prompt_step_gives_the_bits_of_the_step_unrecorded_and_unpadded(name):
    # in bfloat16 too: the filler and the empty rows of a recorded step take no part in what the kernels choose (the
    # attention's workgroup shapes, the splits of the single tokens' contexts), and with few rows every product is a
    # kernel of this package in which a row does not depend on the others (A and D have inner sizes that are no
    # multiple of 8: the plain matrix-core product instead of the weight-streaming one)
    from pico_vllm_amd.engine.batch import SeqStep
    from pico_vllm_amd.engine.step import ModelRunner
    from pico_vllm_amd.parts.model import load_model
    model = load_model(model_dir(name), "bfloat16", "cuda:0")
    V, page = CONFIGS[name]["vocab_size"], PAGE_SIZE[name]
    rec = ModelRunner(model, page, 64, 4, 64, 256, use_graph=True, max_graph_batch=4)
    raw = ModelRunner(model, page, 64, 4, 64, 256, use_graph=False)
    g = torch.Generator().manual_seed(4)
    text = {r: torch.randint(0, V, (200,), generator=g).tolist() for r in "abcd"}
    at = dict.fromkeys(text, 0)

    def both(parts):
        outs = []
        for r in (rec, raw):
            seqs = []
            for rid, n in parts:
                if rid not in r.manager.requests:
                    assert r.manager.add_request(rid)
                assert r.manager.grow(rid, at[rid] + n)
                seqs.append(SeqStep(rid, text[rid][at[rid]:at[rid] + n], [n - 1]))
            outs.append(r.step(seqs).clone())
            r.advance(seqs)
        for rid, n in parts:
            at[rid] += n
        assert torch.equal(outs[0], outs[1]), parts

    for parts in ([("a", 15)], [("b", 40)], [("a", 1), ("b", 1), ("c", 23)], [("a", 1), ("c", 2)], [("a", 1), ("b", 1), ("c", 1), ("d", 50)],
                  [("b", 1), ("d", 7)], [("a", 1), ("b", 1), ("c", 1), ("d", 1)], [("c", 33)], [("a", 1), ("b", 1), ("d", 1), ("c", 60)]):
        both(parts)
    assert {k[:2] for k in rec._prompt_graphs} >= {(0, 16), (2, 32), (1, 16), (4, 64)} and rec._graphs and not raw._prompt_graphs
