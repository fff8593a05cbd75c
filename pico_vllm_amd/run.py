"""Command line in the manner of the reference's entry script
(pico_vllm/run_single.py:10-37), whose constants become options with the same
names: --num-gpu-blocks 500 --block-size 16 (run_single.py:17-22),
--use-cuda-graph (:26), --max-new-tokens 20 --temperature 0 --top-p 1.0 (:31).

  python -m pico_vllm_amd.run --model DIR --prompt-ids 1,2,3 --max-new-tokens 20
  python -m pico_vllm_amd.run --model DIR --prompt "The capital of France is"
  python -m pico_vllm_amd.run --write-random DIR --config config.json --seed 0
  python -m pico_vllm_amd.run --random-config tiny-b --prompt-ids 5,17,3     (random weights of a named size)
"""
from __future__ import annotations

import argparse
import json
import shutil
import sys
import tempfile


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="pico_vllm_amd.run", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", help="folder with config.json and model.safetensors")
    ap.add_argument("--prompt", action="append", default=[], help="text prompt (needs tokenizer files in --model)")
    ap.add_argument("--prompt-ids", action="append", default=[], help="prompt as comma-separated token ids")
    ap.add_argument("--max-new-tokens", type=int, default=20)
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=None)
    ap.add_argument("--ignore-eos", action="store_true")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--num-gpu-blocks", type=lambda v: None if v == "auto" else int(v), default=500,
                    help="cache pages per group of layers (the reference's 500), or 'auto': what --max-num-seqs requests of "
                         "--max-seq-len can use, within --kv-memory-fraction of the free GPU memory")
    ap.add_argument("--kv-memory-fraction", type=float, default=0.9)
    ap.add_argument("--prefill-chunk", type=int, default=None, help="longest portion of one prompt in a step (default: the step's budget)")
    ap.add_argument("--max-seq-len", type=int, default=4096)
    ap.add_argument("--max-num-seqs", type=int, default=4)
    ap.add_argument("--max-num-batched-tokens", type=int, default=2048)
    ap.add_argument("--max-batch-size", type=int, default=8)
    ap.add_argument("--use-cuda-graph", dest="use_cuda_graph", action="store_true", default=True)
    ap.add_argument("--no-cuda-graph", dest="use_cuda_graph", action="store_false")
    ap.add_argument("--manual-seed", type=int, default=42)
    ap.add_argument("--write-random", metavar="DIR", help="write a random-weights model folder and exit")
    ap.add_argument("--config", help="config.json to use with --write-random")
    ap.add_argument("--random-config", metavar="NAME", help="run on random weights of a named size "
                    "(tiny-a, tiny-b, 1.5b, 7b, 32b) instead of --model; with --write-random: that size")
    ap.add_argument("--no-pipeline-decode", dest="pipeline_decode", action="store_false", default=True,
                    help="read every step's tokens before the next step starts")
    ap.add_argument("--profile-phases", action="store_true",
                    help="time the phases of every step, mark them for rocprofv3 --marker-trace, and print the report to stderr")
    args = ap.parse_args(argv)

    if args.write_random:
        if not (args.config or args.random_config):
            ap.error("--write-random needs --config or --random-config")
        from .config.presets import preset
        from .weights.random_init import write_random_model
        if args.config:
            with open(args.config) as f:
                cfg = json.load(f)
        else:
            cfg = preset(args.random_config)
        write_random_model(args.write_random, cfg, args.seed or 0)
        print(f"wrote {args.write_random}")
        return 0
    tmp = None
    if args.random_config and not args.model:
        from .config.presets import preset
        from .weights.random_init import write_random_model
        tmp = tempfile.mkdtemp(prefix="pico_random_")
        write_random_model(tmp, preset(args.random_config), args.seed or 0)
        args.model = tmp
    if not args.model:
        ap.error("--model or --random-config is required")
    try:
        return _generate(ap, args)
    finally:
        if tmp:
            shutil.rmtree(tmp, ignore_errors=True)


def _generate(ap, args) -> int:
    prompts = list(args.prompt) + [[int(t) for t in p.split(",") if t.strip()] for p in args.prompt_ids]
    if not prompts:
        ap.error("give at least one --prompt or --prompt-ids")

    from .config.engine_args import EngineArgs
    from .engine.llm import LLM
    from .sampling.params import SamplingParams
    tokenizer = None
    if args.prompt:
        try:
            from transformers import AutoTokenizer      # the reference's tokenizer, run_single.py:15
            tokenizer = AutoTokenizer.from_pretrained(args.model)
        except Exception as e:
            print(f"cannot load a tokenizer from {args.model}: {e}", file=sys.stderr)
            return 2
    ea = EngineArgs(model=args.model, dtype=args.dtype, block_size=args.block_size,
                    num_gpu_blocks=args.num_gpu_blocks, max_seq_len=args.max_seq_len,
                    max_num_seqs=args.max_num_seqs, max_num_batched_tokens=args.max_num_batched_tokens,
                    prefill_chunk=args.prefill_chunk, kv_memory_fraction=args.kv_memory_fraction,
                    use_cuda_graph=args.use_cuda_graph, max_batch_size=args.max_batch_size,
                    manual_seed=args.manual_seed, pipeline_decode=args.pipeline_decode, profile_phases=args.profile_phases)
    llm = LLM(tokenizer=tokenizer, engine_args=ea)
    sp = SamplingParams(args.max_new_tokens, args.temperature, args.top_p, args.seed, args.ignore_eos)
    for o in llm.generate(prompts, sp):
        shown = o.text if o.text is not None else " ".join(map(str, o.token_ids))
        print(f"[{o.request_id}] ({o.finish_reason}) {shown}")
    if args.profile_phases:
        print(json.dumps(llm.engine.report(), indent=1), file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
