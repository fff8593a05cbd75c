"""Engine options in one place.

Names and meanings follow the reference where it has them: ``block_size``
and ``num_gpu_blocks`` (pico_vllm/blockmanager.py:21-28; run_single.py:17-22
uses 500 blocks of 16), ``max_seq_len`` (engine.py:41), ``max_num_seqs``
(scheduler.py:84), ``use_cuda_graph`` and ``max_batch_size`` (engine.py:21-22;
the graph here is a HIP graph), ``manual_seed`` (engine.py:30).
``max_num_batched_tokens`` and ``prefill_chunk`` (the token budget of a step and the longest
portion of one prompt in it; the reference prefills whole prompts, engine.py:305-306, and lists
portions as future work, TODO.md:3), ``kv_memory_fraction`` (the reference fixes 500 blocks,
run_single.py:17-22), ``dtype`` and ``pipeline_decode`` (start the next decode
step from the tokens on the device before the host has read them) have no counterpart there.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass
class EngineArgs:
    model: str = ""                      # folder with config.json and model.safetensors
    dtype: str = "bfloat16"              # "bfloat16" or "float32" (true 32-bit everywhere)
    block_size: int = 16                 # tokens per cache page
    num_gpu_blocks: Optional[int] = None  # pages per layer group; None: what max_num_seqs requests of max_seq_len can use, or
                                          # fewer if kv_memory_fraction of the memory free after loading does not hold that
    kv_memory_fraction: float = 0.9      # with num_gpu_blocks=None: the share of the free GPU memory the cache may take
    max_seq_len: int = 4096              # longest request (prompt + generated)
    max_num_seqs: int = 4                # requests running at once
    max_num_batched_tokens: int = 2048   # token budget of one step
    prefill_chunk: Optional[int] = None  # longest portion of one prompt in a step; None: whatever the budget leaves
    use_cuda_graph: bool = True          # replay pure-decode steps from a captured HIP graph
    max_batch_size: int = 8              # largest decode batch that has a graph
    graph_prompts: bool = True           # with use_cuda_graph: a step that is one prompt portion, alone or behind decoding requests, replays a graph too
    manual_seed: int = 42
    pipeline_decode: bool = True         # keep one decode step in flight while the host prepares the next
    tune_library_gemm: bool = False      # let the library time its solutions for whole prompt portions (stalls the first such step)
    profile_phases: bool = False         # time the phases of every step (host clock and device events) and mark them for a profiler
    device: str = "cuda:0"

    def validate(self) -> None:
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {self.dtype!r}")
        if self.block_size < 8 or self.block_size & (self.block_size - 1):
            raise ValueError(f"block_size must be a power of two of at least 8, got {self.block_size}")
        if self.max_num_seqs < 1 or self.max_num_batched_tokens < 1 or self.max_seq_len < 1:
            raise ValueError("max_num_seqs, max_num_batched_tokens and max_seq_len must be positive")
        if self.prefill_chunk is not None and self.prefill_chunk < 1:
            raise ValueError(f"prefill_chunk must be positive (or None for the step's budget), got {self.prefill_chunk}")
        if self.num_gpu_blocks is not None and self.num_gpu_blocks < 1:
            raise ValueError(f"num_gpu_blocks must be positive (or None to size the pool from memory), got {self.num_gpu_blocks}")
        if not 0.0 < self.kv_memory_fraction <= 1.0:
            raise ValueError(f"kv_memory_fraction must be in (0, 1], got {self.kv_memory_fraction}")
