#!/usr/bin/env python3
"""Decode and prefill throughput at the Qwen2.5-1.5B shape with random weights on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W]
  python bench.py --shape 7b --layers 8 --context 8192      (other sizes and context lengths)
  python bench.py --workload serve --shape 7b --layers 8 --context 8192
                                                            (64 requests, prompts of 128..4096 tokens, 256 new tokens each,
                                                             continuous batching with prompts cut into portions)

  python bench.py --workload long --shape 32b --device-weights --context 32768
                                                            (one 16k-token prompt in portions of 2,048, then decode at
                                                             batch 1 and 8 with contexts ending at the context length;
                                                             --device-weights draws the weights on the GPU, no file)

A step is one decode step of the engine (scheduler, model step from a HIP graph, sampling) at
batch 8 with every request's context ending at 4096 tokens.  One JSON line goes to stdout:
decoded tokens a second as ``value`` (K steps between two synchronisations, the contract's clock);
``ms_per_step_median`` from device events around every step; ``prefill`` (one 2,048-token prompt in one
step, median of device-event times) with its TFLOP/s and its fraction of the bf16 matrix-core peak;
``roofline`` (bytes the decode step has to read: every weight once plus the cache of the live requests,
over its time, against 8 TB/s); ``points`` with decode at batch 1 and 64; ``points_other`` with the Qwen2.5-7B shape
(all 28 layers, weights drawn on the GPU): decode at batch 8 with contexts ending at 8,192 tokens and the 2,048-token
prefill.  What a step reads and computes is asked of the model's parts (``DecoderModel.num_weight_bytes`` /
``flops``), its sizes for the record of the architecture's registry entry: this program reads no key of any
architecture's configuration.  Beside the published peaks
stand measured ones (``measured_peak``): a read stream over 2 GiB and a loop of matrix-core products, by
this package's own kernels on the same GPU in the same run.
"""
from __future__ import annotations

import argparse
import json
import os
import shutil
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12            # bytes/s, MI355X HBM3E
MFMA_PEAK = {"bfloat16": 2.5e15, "float32": 157.3e12}

from pico_vllm_amd.config.presets import preset   # noqa: E402  (needs ROOT on the path)

# name -> (what the record calls it, the configuration as its config.json would hold it); the default run is the
# Qwen2.5-1.5B shape, the others are measured with fewer layers when asked (--layers)
SHAPES = {"1.5b": ("Qwen2.5-1.5B shape", preset("1.5b")), "7b": ("Qwen2.5-7B shape", preset("7b")),
          "32b": ("Qwen2.5-32B shape", preset("32b"))}
CONFIG = SHAPES["1.5b"][1]   # the shape being measured (set in main)
CONTEXT = 4096
PREFILL_TOKENS = 2048
OTHER_SHAPE, OTHER_CONTEXT = "7b", 8192      # ``points_other``


def describe(raw):
    """(registry entry, typed configuration, model description) of a configuration."""
    from pico_vllm_amd.config.registry import resolve_architecture
    arch = resolve_architecture(raw)
    typed = arch.config_from_dict(raw)
    return arch, typed, arch.build_spec(typed)


def log(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def prefill_flops(model, T: int) -> float:
    """What a prompt of T tokens alone costs: the matrices for every token, attention over the T (T + 1) / 2 (query,
    key) pairs of a causal mask, and the output matrix on one row; each part of the model reports its own."""
    return model.flops(T, T * (T + 1) // 2, 1)


def measured_peaks():
    """(read stream in bytes/s, bf16 matrix-core loop in flop/s) on this GPU, once per run."""
    global _PEAKS
    if _PEAKS is None:
        from pico_vllm_amd.ops import peaks
        _PEAKS = (peaks.read_bandwidth(), peaks.mfma_peak()[0])
        log(f"measured peaks: read stream {_PEAKS[0] / 1e12:.2f} TB/s, bf16 matrix cores {_PEAKS[1] / 1e15:.2f} PFLOP/s")
    return _PEAKS


_PEAKS = None


def device_model(cfg, dtype, seed=0):
    """The model of ``cfg`` with random weights drawn on the GPU (same distributions as the random-weights
    folders: matrices and biases N(0, 0.02), norm weights 1 + U(-0.1, 0.1)): for sizes whose file would take
    longer to write and read than the measurement."""
    import torch
    from pico_vllm_amd.parts.model import DecoderModel
    _, typed, spec = describe(cfg)
    model = DecoderModel(spec, {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype], torch.device("cuda:0"))
    g = torch.Generator(device="cuda:0").manual_seed(seed)
    tensors = {}
    for p in model.param_specs():
        if p.role == "norm":
            tensors[p.name] = 1.0 + (torch.rand(p.shape, generator=g, device="cuda:0") * 0.2 - 0.1)
        elif p.role == "table":
            tensors[p.name] = torch.zeros(p.shape, dtype=torch.int32, device="cuda:0")
        else:
            t = torch.empty(p.shape, dtype=model.dtype, device="cuda:0")
            t.normal_(0.0, p.std, generator=g)
            tensors[p.name] = t
    model.load(tensors)
    model.config = typed
    return model


def make_engine(model_dir, dtype, batch, layers_model=None, context=None):
    from pico_vllm_amd import EngineArgs
    from pico_vllm_amd.engine.llm import LLMEngine
    block = 16
    context = context or CONTEXT
    args = EngineArgs(model=model_dir, dtype=dtype, block_size=block,
                      num_gpu_blocks=batch * (context // block + 1) + 8, max_seq_len=context + 16,
                      max_num_seqs=batch, max_num_batched_tokens=max(PREFILL_TOKENS, batch),
                      use_cuda_graph=True, max_batch_size=64, tune_library_gemm=True)
    return LLMEngine(args, model=layers_model)


def decode_point(model_dir, model, dtype, batch, steps, warmup, context=None):
    """Fill `batch` requests so that the timed steps end at the context length, then time `steps` decode steps."""
    import torch
    context = context or CONTEXT
    eng = make_engine(model_dir, dtype, batch, model, context)
    V = eng.model.spec.vocab_size
    g = torch.Generator().manual_seed(batch)
    # while later prompts are still being prefilled the earlier requests already decode: leave room for that
    slack = batch * (-(-context // PREFILL_TOKENS)) + 2
    prompt_len = context - (warmup + steps) - 1 - slack
    for i in range(batch):
        ids = torch.randint(0, V, (prompt_len,), generator=g).tolist()
        eng.submit(ids, max_new_tokens=warmup + steps + 1 + slack, temperature=0.0, ignore_eos=True)
    t0 = time.time()
    said = time.time()
    while any(r.num_uncomputed > 1 or not r.generated_ids for r in eng.requests.values()):
        eng.step()                                   # prompt portions (and the first decodes of early requests)
        if time.time() - said > 20:
            said = time.time()
            log(f"batch {batch}: {sum(r.num_computed for r in eng.requests.values())} of {batch * prompt_len} prompt tokens in the cache")
    torch.cuda.synchronize()
    log(f"batch {batch}: prompts of {prompt_len} tokens in the cache after {time.time() - t0:.1f}s")
    # bring every request to the same number of generated tokens is not needed: all decode from here on
    for _ in range(warmup):
        eng.step()
    torch.cuda.synchronize()
    ctx_start = [r.total_len - 1 for r in eng.requests.values()]
    pool = eng.runner.manager.groups[0].pool
    pages_in_use = pool.num_used
    # the contract's clock: K steps between two synchronisations; and an event behind every step's launches, whose
    # distances are the steps' times on the device
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(steps):
        done = eng.step()
        marks[i + 1].record()
        if done:
            raise RuntimeError("a request finished inside the timed region")
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(steps))
    ctx_mean = [c + (steps - 1) / 2 + 1 for c in ctx_start]          # keys read per step, averaged over the region
    nbytes = eng.runner.decode_bytes([int(c) for c in ctx_mean])
    ms = dt / steps * 1e3
    res = {"prompt_len": prompt_len, "tok_s": batch * steps / dt, "ms_per_step": ms, "bytes": nbytes, "gbps": nbytes / (dt / steps) / 1e9,
           "context": sum(ctx_mean) / batch, "ms_median": per_step[len(per_step) // 2], "ms_min": per_step[0],
           "pages_in_use": pages_in_use, "pages": pool.num_pages}
    model = eng.model
    del eng
    torch.cuda.empty_cache()
    return res, model


def prefill_point(model_dir, model, dtype, reps=7, tokens=PREFILL_TOKENS, context=None):
    import torch
    from pico_vllm_amd.engine.batch import SeqStep
    peak = measured_peaks()[1] if dtype == "bfloat16" else None       # before the timed steps: a profile ends with them
    eng = make_engine(model_dir, dtype, 1, model, context)
    V = eng.model.spec.vocab_size
    ids = torch.randint(0, V, (tokens,), generator=torch.Generator().manual_seed(7)).tolist()
    m = eng.runner.manager
    times = []
    for i in range(reps + 1):
        rid = f"p{i}"
        m.add_request(rid)
        assert m.grow(rid, tokens)
        seq = [SeqStep(rid, ids, [tokens - 1])]
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        eng.runner.step(seq)
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1) * 1e-3)
        m.free_request(rid)
    times = sorted(times[1:])                         # the first run builds, tunes and warms
    dt = times[len(times) // 2]
    flops = prefill_flops(eng.model, tokens)
    out = {"value": tokens / dt, "tokens": tokens, "ms": dt * 1e3, "ms_min": times[0] * 1e3,
           "tflops": flops / dt / 1e12, "frac": flops / dt / MFMA_PEAK[dtype]}
    if peak is not None:
        out["measured_peak_tflops"] = peak / 1e12
        out["frac_of_measured"] = flops / dt / peak
    return out


def sweep_point(model_dir, model, dtype, batch, bin_width=256):
    """Decode from a prompt of 16 tokens up to the context length, an event behind every step: the median time of a
    step for every `bin_width` positions of context (the reference sweeps sequence lengths 16 to 4096 this way,
    pico_vllm/profiling/profile_pagedkvcacheTritoncompile.py:43-113, for its successive engines)."""
    import torch
    eng = make_engine(model_dir, dtype, batch, model)
    V = eng.model.spec.vocab_size
    g = torch.Generator().manual_seed(11)
    new = CONTEXT - 16
    for _ in range(batch):
        eng.submit(torch.randint(0, V, (16,), generator=g).tolist(), max_new_tokens=new, temperature=0.0, ignore_eos=True)
    eng.step()                                        # the prompts
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True)]
    marks[0].record()
    while not eng.is_done():
        eng.step()
        e = torch.cuda.Event(enable_timing=True)
        e.record()
        marks.append(e)
    torch.cuda.synchronize()
    ms = [marks[i].elapsed_time(marks[i + 1]) for i in range(len(marks) - 1)]
    rows = []
    for lo in range(0, len(ms), bin_width):
        part = sorted(ms[lo:lo + bin_width])
        if len(part) >= bin_width // 2:
            med = part[len(part) // 2]
            rows.append({"context": 16 + lo + len(part) // 2, "ms_per_step": round(med, 4), "tok_s": round(batch / med * 1e3, 1)})
    return rows


def long_prompt_point(model_dir, model, dtype, prompt_len):
    """One prompt of ``prompt_len`` tokens through the scheduler, cut into portions of PREFILL_TOKENS; the time
    until its first token is sampled."""
    import torch
    eng = make_engine(model_dir, dtype, 1, model)
    V = eng.model.spec.vocab_size
    g = torch.Generator().manual_seed(3)
    warm = eng.submit(torch.randint(0, V, (prompt_len,), generator=g).tolist(), max_new_tokens=2, ignore_eos=True)
    while not eng.is_done():
        eng.step()                                   # kernels built, library products chosen, steps recorded
    torch.cuda.synchronize()
    rid = eng.submit(torch.randint(0, V, (prompt_len,), generator=g).tolist(), max_new_tokens=2, temperature=0.0, ignore_eos=True)
    req = eng.requests[rid]
    steps = 0
    t0 = time.perf_counter()
    while not req.generated_ids:
        eng.step()
        steps += 1
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    while not eng.is_done():
        eng.step()
    model = eng.model
    del eng
    torch.cuda.empty_cache()
    return {"tokens": prompt_len, "portions": steps, "ms": dt * 1e3, "tok_s": prompt_len / dt,
            "tflops": prefill_flops(model, prompt_len) / dt / 1e12}, model


def serve_point(model_dir, dtype, requests, max_new, model=None):
    """The mixed workload: `requests` requests with prompt lengths uniform in 128..4096 (seeded) and
    `max_new` new tokens each, all submitted at once; the scheduler admits, cuts prompts into portions of at most
    2,048 tokens beside the decoding requests, decodes, finishes and frees."""
    import torch
    from pico_vllm_amd import EngineArgs
    from pico_vllm_amd.engine.llm import LLMEngine
    g = torch.Generator().manual_seed(requests)
    lens = torch.randint(128, 4097, (requests,), generator=g).tolist()
    block = 16
    longest = max(lens) + max_new
    if longest > CONTEXT:
        raise SystemExit(f"bench.py: --context must be at least {longest} for this workload")
    pages = sum(-(-(n + max_new) // block) for n in lens) + 8
    eng = LLMEngine(EngineArgs(model=model_dir, dtype=dtype, block_size=block, num_gpu_blocks=pages, max_seq_len=CONTEXT,
                               max_num_seqs=requests, max_num_batched_tokens=PREFILL_TOKENS, use_cuda_graph=True,
                               max_batch_size=64, tune_library_gemm=True), model=model)
    V = eng.model.spec.vocab_size
    # a short run first: kernels built and tuned, graphs captured for the batch sizes of the run's tail
    for n in (PREFILL_TOKENS, 300):
        eng.submit(torch.randint(0, V, (n,), generator=g).tolist(), max_new_tokens=4, ignore_eos=True)
    while not eng.is_done():
        eng.step()
    torch.cuda.synchronize()
    for n in lens:
        eng.submit(torch.randint(0, V, (n,), generator=g).tolist(), max_new_tokens=max_new, temperature=0.0, ignore_eos=True)
    steps0 = eng.stats["steps"]
    t0 = time.perf_counter()
    finished = 0
    while not eng.is_done():
        finished += len(eng.step())
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert finished == requests
    return {"seconds": dt, "steps": eng.stats["steps"] - steps0, "prompt_tokens": sum(lens), "new_tokens": requests * max_new,
            "preemptions": eng.stats["preemptions"]}


def attention_point(cfg, nseq, new_len, prefix, shape=0, reps=20, chunk_len=0):
    """The prefill attention kernel alone on ``nseq`` portions of ``new_len`` tokens after ``prefix`` cached ones,
    with the shape's heads; ``shape``: what FastAttention.prefill_teams would return, 0 = ask it."""
    import torch
    from pico_vllm_amd.ops.attention_fast import FastAttention
    mixer = describe(cfg)[2].layers[0].slots["mixer"][1].params          # the constants of the first layer's attention part
    nq, nkv, d = mixer["num_heads"], mixer["num_kv_heads"], mixer["head_dim"]
    P, dev = 16, "cuda"
    g = torch.Generator(device=dev).manual_seed(0)
    ctx = new_len + prefix
    per = -(-ctx // P)
    pages = nseq * per + 8
    kc = torch.randn(pages, nkv, P, d, device=dev, generator=g).bfloat16()
    vc = torch.randn(pages, nkv, d, P, device=dev, generator=g).bfloat16()
    bt = torch.randperm(pages, device=dev, generator=g)[: nseq * per].int().reshape(nseq, per).contiguous()
    q = torch.randn(nseq * new_len, (nq + 2 * nkv) * d, device=dev, generator=g).bfloat16()
    cu = torch.arange(0, (nseq + 1) * new_len, new_len, dtype=torch.int32, device=dev)
    cl = torch.full((nseq,), ctx, dtype=torch.int32, device=dev)
    fa = FastAttention(nq, nkv, d)
    shape = shape or fa.prefill_teams([new_len] * nseq, [ctx] * nseq)
    out = torch.empty(nseq * new_len, nq * d, dtype=torch.bfloat16, device=dev)
    order = fa.order_list(nseq * new_len, nseq, dev) if nseq > 1 else None      # the tiles of all sequences, longest first
    run = lambda build=False: fa.prefill(q, kc, vc, bt, cu, cl, nseq, d ** -0.5, out=out, teams=shape, chunk_len=chunk_len,
                                         max_chunks=-(-ctx // chunk_len) if chunk_len else 0, order=order, order_build=build)
    run(True)          # the list is written once a step, by the first layer
    for _ in range(5):
        run()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        run()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) / reps * 1e3
    flops = 4.0 * nq * d * nseq * (new_len * prefix + new_len * (new_len + 1) / 2)
    return {"us": round(us, 1), "shape": shape, "tflops": round(flops / us / 1e6, 1), "frac": round(flops / (us * 1e-6) / MFMA_PEAK["bfloat16"], 4),
            "heads": nq, "kv_heads": nkv}


def sampling_point(cfg, rows, top_p, reps=50):
    """The sampling call alone on ``rows`` rows of float32 logits of the shape's vocabulary: greedy, temperature 0.8,
    and temperature 0.8 with ``top_p``; microseconds a call."""
    import torch
    from pico_vllm_amd.ops import kernels
    dev, V = "cuda", describe(cfg)[2].vocab_size
    g = torch.Generator(device=dev).manual_seed(0)
    logits = torch.randn(rows, V, device=dev, generator=g) * 3.0
    u = torch.rand(rows, device=dev, generator=g)
    out = torch.empty(rows, dtype=torch.int32, device=dev)
    work = kernels.sample_workspace(rows, dev)
    res = {}
    for name, temp, p in (("greedy", 0.0, 1.0), ("temperature", 0.8, 1.0), ("top_p", 0.8, top_p)):
        t = torch.full((rows,), temp, device=dev)
        pp = torch.full((rows,), p, device=dev)
        run = lambda: kernels.sample(logits, t, pp, u, out=out, work=work, top_p_rows=temp > 0 and p < 1)
        for _ in range(5):
            run()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            run()
        e1.record()
        torch.cuda.synchronize()
        res[name] = round(e0.elapsed_time(e1) / reps * 1e3, 1)
    res["vocab"] = V
    return res


def other_shape_points(dtype, steps, warmup):
    """``points_other``: the OTHER_SHAPE shape with all its layers (weights drawn on the GPU), decode at batch 8 with
    contexts ending at OTHER_CONTEXT tokens and the 2,048-token prefill."""
    import torch
    name, raw = SHAPES[OTHER_SHAPE]
    arch, typed, _ = describe(raw)
    t0 = time.time()
    model = device_model(raw, dtype)
    torch.cuda.synchronize()
    log(f"{name}: {model.num_weight_bytes() / 1e9:.1f} GB of matrices drawn on the GPU in {time.time() - t0:.0f}s")
    r, model = decode_point("", model, dtype, 8, steps, warmup, OTHER_CONTEXT)
    log(f"{name} decode batch 8 at context {OTHER_CONTEXT}: {r['tok_s']:.0f} tok/s, {r['ms_per_step']:.3f} ms/step")
    pf = prefill_point("", model, dtype, reps=5, context=OTHER_CONTEXT)
    log(f"{name} prefill: {pf}")
    del model
    torch.cuda.empty_cache()
    return {"model": name, "layers": arch.sizes(typed)["layers"], "context": OTHER_CONTEXT,
            "decode_b8": round(r["tok_s"], 1), "decode_b8_ms_per_step": round(r["ms_per_step"], 4),
            "decode_b8_gbytes_per_step": round(r["bytes"] / 1e9, 3), "decode_b8_hbm_frac": round(r["gbps"] * 1e9 / HBM_PEAK, 4),
            "prefill_tokens": pf["tokens"], "prefill_tok_s": round(pf["value"], 1), "prefill_ms": round(pf["ms"], 4),
            "prefill_tflops": round(pf["tflops"], 1), "prefill_frac": round(pf["frac"], 4)}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points, the prefill and the other shape (long workload: the decode points)")
    ap.add_argument("--no-other", action="store_true", help="skip ``points_other`` (the 7B shape)")
    ap.add_argument("--prefill-only", action="store_true", help="measure only the 2,048-token prefill (for profiling)")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS,
                    help="with --prefill-only: the prompt's length (2 to 2048; the contract's prefill is of 2,048 tokens)")
    ap.add_argument("--write-model", metavar="DIR", default=None,
                    help="only write the random-weights model folder to DIR (to reuse with --model) and exit")
    ap.add_argument("--model", default=None, help="measure this model folder (config.json + model.safetensors, any registered "
                    "architecture) instead of writing random weights of --shape")
    ap.add_argument("--shape", default="1.5b", choices=sorted(SHAPES), help="layer sizes (default: the 1.5B shape)")
    ap.add_argument("--layers", type=int, default=0, help="run only this many layers of the shape (0: all)")
    ap.add_argument("--context", type=int, default=4096, help="context length at which the decode steps end")
    ap.add_argument("--workload", default="decode", choices=["decode", "serve", "long", "sweep"],
                    help="decode: the contract's steady decode steps; serve: many requests of mixed lengths at once; "
                         "long: one prompt of --prompt tokens in portions, then decode at batch 1 and 8 at the context length; "
                         "sweep: decode from context 16 to the context length, the time of a step by context")
    ap.add_argument("--prompt", type=int, default=16384, help="prompt tokens of the long workload")
    ap.add_argument("--device-weights", action="store_true",
                    help="draw the random weights on the GPU instead of writing and reading a model folder")
    ap.add_argument("--requests", type=int, default=64, help="requests of the serve workload")
    ap.add_argument("--max-new", type=int, default=256, help="new tokens per request of the serve workload")
    ap.add_argument("--attention", metavar="SEQS,NEW,PREFIX[,SHAPE[,CHUNK]]", default=None,
                    help="time only the prefill attention kernel on SEQS portions of NEW tokens after PREFIX cached ones")
    ap.add_argument("--sampling", metavar="ROWS[,TOP_P]", default=None,
                    help="time only the sampling call on ROWS rows of the shape's vocabulary (greedy, temperature, top-p)")
    a = ap.parse_args()
    global CONFIG, CONTEXT
    shape_name, full = SHAPES[a.shape]
    if a.model:
        # a model folder says itself what it is (any registered architecture); it keeps the shape's name if it has the shape's sizes
        from pico_vllm_amd.config.model_config import read_config_json
        own = read_config_json(a.model)
        if a.layers:
            print("bench.py: --layers cuts a named shape; a model folder has the layers it has")
            return 2
        arch_own = describe(own)[0]
        if arch_own.sizes is None:
            print(f"bench.py: the architecture of {a.model} registers no sizes for the record")
            return 2
        if arch_own.sizes(arch_own.config_from_dict(own)) != describe(full)[0].sizes(describe(full)[1]):
            shape_name = f"{arch_own.name} in {os.path.basename(os.path.normpath(a.model))}"
        full = own
    arch, typed_full, _ = describe(full)
    layers_full = arch.sizes(typed_full)["layers"]
    CONFIG = dict(full)
    if a.layers:
        if not 0 < a.layers <= layers_full:
            print(f"bench.py: --layers must be 1..{layers_full}")
            return 2
        CONFIG = arch.with_layers(full, a.layers)
    sizes = arch.sizes(arch.config_from_dict(CONFIG))       # flat: layers, hidden, q_heads, kv_heads, head_dim, intermediate, vocab, tied
    CONTEXT = a.context
    if a.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {a.gpus} is not supported")
        return 2
    if not 2 <= a.prefill_tokens <= PREFILL_TOKENS:
        print(f"bench.py: --prefill-tokens must be 2..{PREFILL_TOKENS}")
        return 2
    if CONTEXT < 2 * PREFILL_TOKENS or a.steps + a.warmup >= CONTEXT // 2 - 200:
        print(f"bench.py: the context must be at least {2 * PREFILL_TOKENS} and steps + warmup below {CONTEXT // 2 - 200}")
        return 2
    import torch
    from pico_vllm_amd.weights.random_init import write_random_model
    if a.attention:
        nums = [int(x) for x in a.attention.split(",")]
        r = attention_point(CONFIG, nums[0], nums[1], nums[2], nums[3] if len(nums) > 3 else 0,
                            chunk_len=nums[4] if len(nums) > 4 else 0)
        print(json.dumps({"metric": "prefill attention kernel", "unit": "us", "value": r["us"], "workgroup_shape": r["shape"],
                          "tflops": r["tflops"], "frac_of_bf16_peak": r["frac"], "sequences": nums[0], "new_tokens": nums[1],
                          "prefix": nums[2], "heads": r["heads"], "kv_heads": r["kv_heads"]}))
        return 0
    if a.sampling:
        parts = a.sampling.split(",")
        rows, top_p = int(parts[0]), float(parts[1]) if len(parts) > 1 else 0.9
        if not (1 <= rows <= 1024 and 0 < top_p <= 1):
            print("bench.py: --sampling takes 1..1024 rows and a top-p in (0, 1]")
            return 2
        r = sampling_point(CONFIG, rows, top_p)
        print(json.dumps({"metric": "sampling call", "unit": "us", "value": r["top_p"], "greedy": r["greedy"],
                          "temperature": r["temperature"], "top_p": r["top_p"], "rows": rows, "vocab": r["vocab"],
                          "p": top_p}))
        return 0
    if a.write_model:
        write_random_model(a.write_model, CONFIG, seed=0)
        print(f"wrote {a.write_model}")
        return 0
    tmp = None
    model_dir = a.model
    preloaded = None
    if a.device_weights:
        t0 = time.time()
        log(f"drawing random weights of the {shape_name}, {sizes['layers']} layers, on the GPU ...")
        preloaded = device_model(CONFIG, a.dtype)
        torch.cuda.synchronize()
        log(f"... {time.time() - t0:.0f}s, {preloaded.num_weight_bytes() / 1e9:.1f} GB of matrices")
        model_dir = ""
    elif model_dir is None:
        tmp = tempfile.mkdtemp(prefix="pico_bench_")
        model_dir = tmp
        t0 = time.time()
        log(f"writing random weights of the {shape_name}, {sizes['layers']} layers ...")
        write_random_model(model_dir, CONFIG, seed=0)
        log(f"... {time.time() - t0:.0f}s")
    try:
        if a.workload == "serve":
            r = serve_point(model_dir, a.dtype, a.requests, a.max_new, preloaded)
            total = r["prompt_tokens"] + r["new_tokens"]
            print(json.dumps({
                "metric": f"tokens/s (prompt + new) serving {a.requests} requests at once, {shape_name.split()[0]} bf16",
                "value": round(total / r["seconds"], 1), "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True,
                "new_tokens_per_s": round(r["new_tokens"] / r["seconds"], 1), "seconds": round(r["seconds"], 3),
                "steps": r["steps"], "ms_per_step": round(r["seconds"] / r["steps"] * 1e3, 4),
                "dtype": "bf16" if a.dtype == "bfloat16" else "fp32",
                "data": "synthetic: random weights N(0, 0.02), uniform random token ids, prompt lengths uniform in 128..4096",
                "config": {"model": shape_name, "requests": a.requests, "new_tokens_each": a.max_new,
                           "prompt_tokens": r["prompt_tokens"], "layers": layers_full,
                           "layers_run": sizes["layers"], "hidden": sizes["hidden"],
                           "max_num_batched_tokens": PREFILL_TOKENS, "max_seq_len": CONTEXT, "page_size": 16,
                           "preemptions": r["preemptions"]}}), flush=True)
            return 0
        if a.prefill_only:
            print(json.dumps({"prefill": prefill_point(model_dir, preloaded, a.dtype, tokens=a.prefill_tokens)}), flush=True)
            return 0
        if a.workload == "sweep":
            rows = sweep_point(model_dir, preloaded, a.dtype, a.batch)
            print(json.dumps({"metric": f"decode ms/step by context, batch {a.batch}, {shape_name.split()[0]} {a.dtype}",
                              "unit": "ms", "n_gpus": 1, "batch": a.batch, "layers_run": sizes["layers"],
                              "layers": layers_full, "rows": rows}), flush=True)
            return 0
        if a.workload == "long":
            if a.prompt + 8 > CONTEXT:
                print(f"bench.py: --prompt {a.prompt} does not fit --context {CONTEXT}")
                return 2
            lp, model = long_prompt_point(model_dir, preloaded, a.dtype, a.prompt)
            log(f"prompt of {a.prompt} tokens in {lp['portions']} portions: {lp['ms']:.1f} ms, {lp['tok_s']:.0f} tok/s")
            pts = {}
            for b in (() if a.no_points else (1, 8)):
                r, model = decode_point(model_dir, model, a.dtype, b, a.steps, a.warmup)
                log(f"decode batch {b} at context {CONTEXT}: {r['tok_s']:.0f} tok/s, {r['ms_per_step']:.3f} ms/step, {r['gbps'] / 1e3:.2f} TB/s")
                pts[f"decode_b{b}"] = {"tok_s": round(r["tok_s"], 1), "ms_per_step": round(r["ms_per_step"], 4),
                                       "ms_per_step_median": round(r["ms_median"], 4), "gbytes_per_step": round(r["bytes"] / 1e9, 2),
                                       "hbm_frac": round(r["gbps"] * 1e9 / HBM_PEAK, 4), "pages_in_use": r["pages_in_use"]}
            print(json.dumps({
                "metric": f"decode tok/s @ batch 8 at context {CONTEXT} after a {a.prompt}-token prompt in portions of {PREFILL_TOKENS}, {shape_name.split()[0]} bf16",
                "value": pts["decode_b8"]["tok_s"] if pts else None, "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
                "ms_per_step": pts["decode_b8"]["ms_per_step"] if pts else None, "higher_is_better": True,
                "dtype": "bf16" if a.dtype == "bfloat16" else "fp32",
                "data": "synthetic: random weights N(0, 0.02)" + (" drawn on the GPU" if a.device_weights else "") + ", uniform random token ids",
                "config": {"model": shape_name, "layers": layers_full, "layers_run": sizes["layers"],
                           "hidden": sizes["hidden"], "q_heads": sizes["q_heads"],
                           "kv_heads": sizes["kv_heads"], "intermediate": sizes["intermediate"],
                           "vocab": sizes["vocab"], "seq_len": CONTEXT, "prompt": a.prompt, "portion": PREFILL_TOKENS,
                           "page_size": 16, "weight_gbytes": round(model.num_weight_bytes() / 1e9, 1)},
                "long_prompt": {k: (round(v, 2) if isinstance(v, float) else v) for k, v in lp.items()},
                "points": pts}), flush=True)
            return 0
        main_res, model = decode_point(model_dir, preloaded, a.dtype, a.batch, a.steps, a.warmup)
        log(f"decode batch {a.batch}: {main_res['tok_s']:.0f} tok/s, {main_res['ms_per_step']:.3f} ms/step")
        out = {
            "metric": f"decode tok/s @ batch {a.batch}, {shape_name.split()[0]} bf16 (plus batch 1/64 and prefill @ 2048 tok)",
            "value": round(main_res["tok_s"], 1), "unit": "tokens/s", "n_gpus": 1, "steps": a.steps,
            "warmup": a.warmup, "ms_per_step": round(main_res["ms_per_step"], 4),
            "ms_per_step_median": round(main_res["ms_median"], 4), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if a.dtype == "bfloat16" else "fp32",
            "data": "synthetic: random weights N(0, 0.02), uniform random token ids",
            "config": {"model": shape_name, "global_batch": a.batch, "seq_len": CONTEXT,
                       "parallelism": "single GPU", "layers": layers_full,
                       "layers_run": sizes["layers"], "hidden": sizes["hidden"],
                       "q_heads": sizes["q_heads"], "kv_heads": sizes["kv_heads"],
                       "head_dim": sizes["head_dim"],
                       "intermediate": sizes["intermediate"], "vocab": sizes["vocab"],
                       "tied": sizes["tied"],
                       "page_size": 16, "prompt_len": int(main_res["prompt_len"]),
                       "context_in_timed_steps": round(main_res["context"], 1)},
            "roofline": {"bound": "hbm", "achieved": round(main_res["gbps"], 1), "peak": HBM_PEAK / 1e9,
                         "unit": "GB/s", "frac": round(main_res["gbps"] * 1e9 / HBM_PEAK, 4),
                         "gbytes_per_step": round(main_res["bytes"] / 1e9, 3)},
            "pages_in_use": main_res["pages_in_use"], "pages": main_res["pages"],
        }
        if a.dtype == "bfloat16":
            stream = measured_peaks()[0]
            out["roofline"]["measured_peak"] = round(stream / 1e9, 1)
            out["roofline"]["frac_of_measured"] = round(main_res["gbps"] * 1e9 / stream, 4)
        if not a.no_points:
            out["prefill"] = {k: (round(v, 4) if isinstance(v, float) else v)
                              for k, v in prefill_point(model_dir, model, a.dtype).items()}
            log(f"prefill: {out['prefill']}")
            pts = {}
            for b, steps in ((1, min(a.steps, 200)), (64, min(a.steps, 100))):
                r, model = decode_point(model_dir, model, a.dtype, b, steps, min(a.warmup, 10))
                pts[f"decode_b{b}"] = round(r["tok_s"], 1)
                pts[f"decode_b{b}_hbm_frac"] = round(r["gbps"] * 1e9 / HBM_PEAK, 4)
                log(f"decode batch {b}: {r['tok_s']:.0f} tok/s, {r['ms_per_step']:.3f} ms/step")
            if a.shape == "1.5b" and not a.layers and a.dtype == "bfloat16" and shape_name == SHAPES["1.5b"][0]:
                # the one figure the reference publishes for this model: 97 tok/s at batch 1 on its authors' card
                # (README.md:9,43-45 of the reference); other hardware, so a context, not a baseline
                pts["decode_b1_vs_reference_published"] = round(pts["decode_b1"] / 97.0, 2)
            out["points"] = pts
            if a.shape == "1.5b" and not a.layers and a.dtype == "bfloat16" and not a.no_other and not a.model:
                # a second shape, driver-visible: the larger the matrices, the nearer a step comes to what the memory allows
                del model
                torch.cuda.empty_cache()
                out["points_other"] = other_shape_points(a.dtype, min(a.steps, 50), min(a.warmup, 5))
        print(json.dumps(out), flush=True)
    finally:
        if tmp:
            shutil.rmtree(tmp, ignore_errors=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
