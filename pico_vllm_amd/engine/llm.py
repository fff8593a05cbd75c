"""The engine and its Python entry point.

In the manner of the reference's entry script (pico_vllm/run_single.py:10-37:
build the model, load weights, make the block manager and the engine, then
``submit`` and loop ``step()`` until done): ``LLMEngine.submit`` /
``step`` / ``is_done`` have the reference's names and meanings
(engine.py:243,282,465); ``LLM.generate`` wraps the loop.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Union

import torch

from ..cache.storage import bytes_per_page
from ..config.engine_args import EngineArgs
from ..ops import linear
from ..parts.model import DecoderModel, load_model
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .batch import SeqStep
from .phases import PhaseTimers
from .request import Request, RequestStatus
from .scheduler import Scheduler
from .step import ModelRunner


@dataclass
class RequestOutput:
    request_id: int
    prompt_token_ids: List[int]
    token_ids: List[int]
    finish_reason: str
    text: Optional[str] = None
    num_preemptions: int = 0


@dataclass
class _Inflight:
    sampling: list          # the ScheduledSeq that get a token from this step, in the order of the sampled rows
    ticket: tuple           # what Sampler.read wants


class LLMEngine:
    def __init__(self, args: EngineArgs, model: Optional[DecoderModel] = None, tokenizer=None):
        args.validate()
        if not torch.cuda.is_available():
            raise RuntimeError("pico_vllm_amd runs on an AMD GPU only; no GPU is visible to torch")
        self.args = args
        self.model = model if model is not None else load_model(args.model, args.dtype, args.device)
        if args.max_seq_len > self.model.spec.max_position:
            raise ValueError(f"max_seq_len = {args.max_seq_len} exceeds the model's max_position_embeddings = "
                             f"{self.model.spec.max_position}")
        if args.tune_library_gemm:
            # a mode of the whole process (torch's tuner): an engine only ever switches it on, so that building a
            # second engine does not change what the first one runs
            linear.set_library_tuning(True)
        num_pages = args.num_gpu_blocks
        self.pool_sizing = {"pages": num_pages, "from": "num_gpu_blocks"}
        if num_pages is None:
            num_pages, self.pool_sizing = self._pages_from_memory(args)
        self.runner = ModelRunner(self.model, args.block_size, num_pages, args.max_num_seqs,
                                  args.max_num_batched_tokens, args.max_seq_len,
                                  use_graph=args.use_cuda_graph, max_graph_batch=args.max_batch_size,
                                  graph_prompts=args.graph_prompts)
        self.scheduler = Scheduler(self.runner.manager, args.max_num_seqs, args.max_num_batched_tokens,
                                   args.max_seq_len, args.prefill_chunk)
        self.sampler = Sampler(self.model.device, args.max_num_seqs)
        self.eos_token_id = self.model.spec.eos_token_id
        if self.eos_token_id is None and tokenizer is not None:     # the reference's source for it, pico_vllm/engine.py:48
            self.eos_token_id = getattr(tokenizer, "eos_token_id", None)
        self.tokenizer = tokenizer
        self._next_id = 0
        self.no_more_requests = False
        self.requests: Dict[int, Request] = {}
        self.stats = {"steps": 0, "prefill_tokens": 0, "decode_tokens": 0, "preemptions": 0}
        self.timers = PhaseTimers(args.profile_phases)
        self._inflight: Optional[_Inflight] = None      # a launched step whose tokens have not been read

    def _pages_from_memory(self, args: EngineArgs):
        """Pages per group when ``num_gpu_blocks`` is not given: as many as ``max_num_seqs`` requests of ``max_seq_len``
        can use at once (more would never be touched), or fewer if ``kv_memory_fraction`` of the GPU memory that is free
        now, with the weights loaded, does not hold that many.  (The reference fixes 500 blocks in its script,
        pico_vllm/run_single.py:17-22.)  Returns (pages, how they were found, for ``report()``)."""
        want = args.max_num_seqs * (-(-args.max_seq_len // args.block_size))
        per_page = bytes_per_page(self.model.cache_specs(), args.block_size, self.model.dtype)
        free, total = torch.cuda.mem_get_info(self.model.device)
        fit = int(free * args.kv_memory_fraction) // per_page if per_page else want
        pages = max(1, min(want, fit))
        sizing = {"pages": pages, "from": "memory" if fit < want else "max_num_seqs * max_seq_len", "wanted": want,
                  "fit": fit, "bytes_per_page": per_page, "free_bytes": int(free), "kv_memory_fraction": args.kv_memory_fraction}
        if pages * args.block_size < args.max_seq_len:
            raise ValueError(f"the GPU has {free / 2**30:.1f} GiB free, of which {args.kv_memory_fraction:.0%} hold {fit} cache pages "
                             f"of {args.block_size} tokens ({per_page} bytes each over all layers): not one request of "
                             f"max_seq_len = {args.max_seq_len}; lower max_seq_len or give num_gpu_blocks")
        return pages, sizing

    # ---- the reference's trio -------------------------------------------
    def submit(self, prompt: Union[str, Sequence[int]], max_new_tokens: int = 16, temperature: float = 0.0,
               top_p: float = 1.0, seed: Optional[int] = None, ignore_eos: bool = False,
               stop_token_ids: Sequence[int] = ()) -> int:
        """Queue a request; returns its id, or -1 once ``mark_finished`` has been called (pico_vllm/engine.py:243-276)."""
        if self.no_more_requests:
            return -1
        params = SamplingParams(max_new_tokens, temperature, top_p, seed, ignore_eos, [int(t) for t in stop_token_ids])
        params.validate()
        ids = self._encode(prompt)
        V = self.model.spec.vocab_size
        if any(not 0 <= t < V for t in ids):
            raise ValueError(f"prompt holds a token id outside [0, {V})")
        rid = self._next_id
        self._next_id += 1
        req = Request(rid, list(ids), params, seed=seed if seed is not None else self.args.manual_seed * 1000003 + rid)
        self.scheduler.add_request(req)
        self.requests[rid] = req
        return rid

    def step(self) -> List[RequestOutput]:
        """One scheduling decision and one model step; returns the requests found finished.

        With ``pipeline_decode`` a step whose successor can be foreseen (every running request
        decodes on, nobody waits, nobody reaches its length) stays in flight: the next call starts
        that successor from the tokens on the device and only then reads this step's tokens, so
        the GPU does not wait for the host between decode steps.  The tokens of a step in flight
        are reported by the call that reads them; what is generated does not change."""
        prev, self._inflight = self._inflight, None
        done: List[RequestOutput] = []
        plan = None
        if prev is not None:
            if self._foreseeable(prev):
                with self.timers.phase("schedule"):
                    plan = self.scheduler.schedule()
                if not plan.preempted and [s.request for s in plan.seqs] == [s.request for s in prev.sampling] \
                        and all(s.num_tokens == 1 for s in plan.seqs):
                    nxt = self._launch(plan, from_device=True)
                    done = self._resolve(prev)
                    self._inflight = nxt
                    return done
            # not foreseeable after all (pages ran out): the tokens first, then what is left of the plan
            done = self._resolve(prev)
            if plan is not None:
                plan.seqs = [s for s in plan.seqs if s.request.status is RequestStatus.RUNNING]
                if not plan.seqs:
                    # everything it planned has ended with the tokens just read (a stop token cannot be foreseen), and
                    # what it preempted waits: plan anew
                    self.stats["preemptions"] += len(plan.preempted)
                    plan = None
        if plan is None:
            with self.timers.phase("schedule"):
                plan = self.scheduler.schedule()
        self.stats["preemptions"] += len(plan.preempted)
        if not plan.seqs:
            if self.scheduler.has_unfinished():
                raise RuntimeError("the scheduler found nothing to run although requests are unfinished")
            return done
        launched = self._launch(plan)
        if self.args.pipeline_decode and self._foreseeable(launched):
            self._inflight = launched
        else:
            done += self._resolve(launched)
        return done

    def mark_finished(self) -> None:
        """No further request will be submitted (pico_vllm/engine.py:278-280): ``submit`` returns -1 from now on."""
        self.no_more_requests = True

    def is_done(self) -> bool:
        """Nothing is queued, running or in flight.  (The reference's also waits for ``mark_finished``,
        engine.py:472-475; here a loop over ``step`` may end whenever the engine has run dry, and more may be
        submitted afterwards.)"""
        return self._inflight is None and not self.scheduler.has_unfinished()

    # ---- a step in two halves -------------------------------------------
    def _foreseeable(self, step: "_Inflight") -> bool:
        """Whether the step after ``step`` is known before its tokens are: every running request
        got a token in it and goes on decoding, nobody waits for admission, and nobody reaches
        its length with that token (an end-of-sequence token cannot be foreseen: the request
        then simply drops the one token computed too many)."""
        if not self.args.pipeline_decode or self.scheduler.waiting:
            return False
        if [s.request for s in step.sampling] != self.scheduler.running:
            return False
        return all(not r.is_max_len_finished() and r.total_len < self.args.max_seq_len for r in self.scheduler.running)

    def _launch(self, plan, from_device: bool = False) -> "_Inflight":
        """Start the model step and the sampling of ``plan`` and advance what does not depend on the
        values of the new tokens."""
        seqs = []
        for s in plan.seqs:
            r = s.request
            toks = [0] if from_device else r.all_ids[r.num_computed:r.num_computed + s.num_tokens]
            seqs.append(SeqStep(r.request_id, toks, [s.num_tokens - 1] if s.samples else []))
        with self.timers.phase("model", device=True):
            logits = self.runner.step(seqs, self.sampler.device_tokens if from_device else None)
        sampling = [s for s in plan.seqs if s.samples]
        with self.timers.phase("sample", device=True):
            ticket = self.sampler.launch(
                logits,
                [s.request.params.temperature for s in sampling], [s.request.params.top_p for s in sampling],
                [s.request.seed for s in sampling], [s.request.num_generated for s in sampling])
        for s in plan.seqs:
            self.stats["decode_tokens" if s.num_tokens == 1 and s.request.num_generated else "prefill_tokens"] += s.num_tokens
            self.scheduler.on_step_done(s)
        for s in sampling:
            s.request.num_pending += 1
        self.stats["steps"] += 1
        return _Inflight(sampling, ticket)

    def _resolve(self, step: "_Inflight") -> List[RequestOutput]:
        """Read the tokens of a launched step and finish what they finish."""
        done: List[RequestOutput] = []
        with self.timers.phase("read"):
            tokens = self.sampler.read(step.ticket)
        for s, tok in zip(step.sampling, tokens):
            r = s.request
            if r.status is RequestStatus.FINISHED:      # ended by the token before this one: computed too many
                continue
            r.num_pending -= 1
            r.generated_ids.append(int(tok))
            reason = None
            # the end-of-sequence token is kept in the output (pico_vllm/engine.py:380-385)
            if not r.params.ignore_eos and self.eos_token_id is not None and tok == self.eos_token_id:
                reason = "eos"
            elif tok in r.params.stop_token_ids:
                reason = "stop"
            elif len(r.generated_ids) >= r.params.max_new_tokens:    # the first sampled token counts (pico_vllm/scheduler.py:55-56)
                reason = "length"
            if reason:
                r.num_pending = 0
                self.scheduler.finish(r, reason)
                done.append(self._output(r))
        return done

    # ---- counters -------------------------------------------------------
    def report(self) -> Dict[str, object]:
        """Counters of the engine: steps, prompt and decoded tokens, preemptions, pages in use and at the peak per
        group of layers, and, with ``profile_phases``, the time of every phase."""
        m = self.runner.manager
        out: Dict[str, object] = dict(self.stats)
        out["pages"] = [{"window": g.window, "layers": len(g.layers), "total": g.pool.num_pages, "in_use": g.pool.num_used,
                         "peak": g.pool.peak_used, "reused": g.pool.reuse_count} for g in m.groups]
        out["pool_sizing"] = dict(self.pool_sizing)      # how the number of pages was found (given, or from the free memory)
        out["graphs"] = sorted(self.runner._graphs)
        out["prompt_graphs"] = sorted((key[0], key[1]) for key in self.runner._prompt_graphs)   # (single tokens, portion)
        if self.timers.enabled:
            out["phases"] = self.timers.report()
        return out

    # ---- helpers --------------------------------------------------------
    def _encode(self, prompt) -> List[int]:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("a text prompt needs a tokenizer; pass token ids or give the engine a tokenizer")
            return list(self.tokenizer.encode(prompt))
        return [int(t) for t in prompt]

    def _output(self, r: Request) -> RequestOutput:
        # a finished request leaves the engine's books with its report (the reference keeps every request
        # for the life of the engine, pico_vllm/engine.py:262)
        self.requests.pop(r.request_id, None)
        text = None
        if self.tokenizer is not None:
            text = self.tokenizer.decode(r.input_ids + r.generated_ids)     # prompt + generated, engine.py:385
        return RequestOutput(r.request_id, list(r.input_ids), list(r.generated_ids), r.finish_reason or "",
                             text, r.num_preemptions)


class LLM:
    """``LLM(model=DIR, dtype=...).generate(prompts, sampling_params)``."""

    def __init__(self, model: str = "", tokenizer=None, engine_args: Optional[EngineArgs] = None, **kw):
        args = engine_args or EngineArgs(model=model, **kw)
        if model:
            args.model = model
        self.engine = LLMEngine(args, tokenizer=tokenizer)

    def generate(self, prompts: Sequence[Union[str, Sequence[int]]],
                 sampling_params: Union[SamplingParams, Sequence[SamplingParams], None] = None) -> List[RequestOutput]:
        if sampling_params is None:
            sampling_params = SamplingParams()
        if isinstance(sampling_params, SamplingParams):
            sampling_params = [sampling_params] * len(prompts)
        if len(sampling_params) != len(prompts):
            raise ValueError("one SamplingParams per prompt, or one for all")
        ids = [self.engine.submit(p, sp.max_new_tokens, sp.temperature, sp.top_p, sp.seed, sp.ignore_eos, sp.stop_token_ids)
               for p, sp in zip(prompts, sampling_params)]
        outs: Dict[int, RequestOutput] = {}
        while not self.engine.is_done():
            for o in self.engine.step():
                outs[o.request_id] = o
        return [outs[i] for i in ids]
