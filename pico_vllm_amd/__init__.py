"""pico_vllm_amd: a small, whole LLM inference engine for one AMD MI355X.

Public entry points: ``LLM``, ``SamplingParams``, ``EngineArgs`` (generation),
``load_model`` / ``write_random_model`` (weights), and ``bin/trace_run``.
"""
from .config import EngineArgs

__all__ = ["EngineArgs", "LLM", "SamplingParams", "load_model", "write_random_model"]


def __getattr__(name):
    # the heavy modules (torch, the HIP library) load on first use
    if name in ("LLM", "LLMEngine"):
        from .engine import llm
        return getattr(llm, name)
    if name == "SamplingParams":
        from .sampling.params import SamplingParams
        return SamplingParams
    if name == "load_model":
        from .parts.model import load_model
        return load_model
    if name == "write_random_model":
        from .weights.random_init import write_random_model
        return write_random_model
    raise AttributeError(name)
