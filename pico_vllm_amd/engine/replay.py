"""Trace replay: feed given token ids through the model step by step and write
the logits at the wanted places.  Nothing is sampled.  It drives the same
model, step function, cache manager and kernels as generation does.

Input, one JSON object a line:
  {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
Output for a step that wants something: <out>/<step>.f32, little-endian float32
[wanted, vocab] in the order of the entries and of ``want``; after every step
the line ``done <step>``.  Beside them <out>/pages.jsonl gets one JSON object a
step: for every entry the cache pages its tokens of that step landed on, per
group of layers, so that a reader of the output alone can tell that a page was
used again by another request:
  {"step": 0, "entries": [{"id": "a", "first_position": 0, "pages": [[7, 2]]}], "end": []}
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import Dict, IO, List

import numpy as np


class TraceReplayer:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, page_size: int = 16, max_live: int = 8,
                 device: str = "cuda:0"):
        import torch
        from ..parts.model import load_model
        from .step import ModelRunner
        if not torch.cuda.is_available():
            raise RuntimeError("trace replay runs on the GPU; no GPU is visible")
        if dtype == "float32":
            # nothing in the 32-bit path calls a library matrix product, but make sure none could use a
            # reduced-precision mode
            torch.backends.cuda.matmul.allow_tf32 = False
        self.model = load_model(model_dir, dtype, device)
        num_pages = max(1, -(-max_tokens // page_size))
        self.runner = ModelRunner(self.model, page_size, num_pages, max_live,
                                  max_tokens_per_step=max(max_tokens, 1), max_seq_len=max(max_tokens, 1),
                                  use_graph=False)
        self.live: Dict[str, bool] = {}
        self.last_pages: List[dict] = []       # of the last step: per entry its id, first position and pages per group

    def run_step(self, step: dict):
        """Returns the logits [wanted, vocab] as a numpy array, or None if nothing is wanted."""
        import torch
        from .batch import SeqStep
        m = self.runner.manager
        seqs: List[SeqStep] = []
        for e in step.get("entries", []):
            rid = str(e["id"])
            if rid not in self.live:
                if not m.add_request(rid):
                    raise RuntimeError(f"step {step.get('step')}: no room for another live request ({rid})")
                self.live[rid] = True
            toks = [int(t) for t in e["tokens"]]
            if not m.grow(rid, m.num_computed(rid) + len(toks)):
                raise RuntimeError(f"step {step.get('step')}: out of cache pages for request {rid} "
                                   f"({m.num_free_pages()} pages free)")
            seqs.append(SeqStep(rid, toks, [int(w) for w in e.get("want", [])]))
        P = m.page_size
        self.last_pages = []
        for s in seqs:
            lo = m.num_computed(s.req)
            span = range(lo // P, -(-(lo + len(s.tokens)) // P)) if s.tokens else range(0)
            self.last_pages.append({"id": s.req, "first_position": lo,
                                    "pages": [[int(m.block_table(s.req, gi)[j]) for j in span] for gi in range(len(m.groups))]})
        out = None
        if seqs:
            logits = self.runner.step(seqs)
            self.runner.advance(seqs)
            if logits.shape[0]:
                out = logits.detach().to("cpu", torch.float32).numpy()
        for rid in step.get("end", []):
            rid = str(rid)
            if rid in self.live:
                m.free_request(rid)
                del self.live[rid]
        return out


def main(argv=None, stdin: IO[str] = None, stdout: IO[str] = None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time, each request's count rounded up to whole cache "
                         "pages (--block-size tokens; a multiple of 64 is a multiple of every page size up to 64)")
    ap.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    args = ap.parse_args(argv)
    stdin = stdin or sys.stdin
    stdout = stdout or sys.stdout
    os.makedirs(args.out, exist_ok=True)
    rp = TraceReplayer(args.model, args.dtype, args.max_tokens, args.block_size)
    pages_log = open(os.path.join(args.out, "pages.jsonl"), "w")
    for line in stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        logits = rp.run_step(step)
        if logits is not None:
            np.ascontiguousarray(logits, dtype="<f4").tofile(os.path.join(args.out, f"{step['step']}.f32"))
        pages_log.write(json.dumps({"step": step["step"], "entries": rp.last_pages,
                                    "end": [str(r) for r in step.get("end", [])]}) + "\n")
        pages_log.flush()
        stdout.write(f"done {step['step']}\n")
        stdout.flush()
    pages_log.close()
    return 0
