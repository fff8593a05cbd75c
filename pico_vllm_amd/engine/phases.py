"""Timers for the phases of an engine step, behind ``EngineArgs.profile_phases``.

The reference carries such timers as commented-out ``perf_counter`` prints around the parts of its step
(pico_vllm/engine.py:283-391) and brackets decode steps for an external profiler
(profiling/profile_nsys.py:94-113).  Here a phase is a ``with`` block: its host time is added up under its
name, a pair of device events measures what the GPU did between its start and its end (read back lazily, so
that timing does not stall the step), and the block is a marker range that ``rocprofv3 --marker-trace`` shows.
Switched off, a phase is a no-op.
"""
from __future__ import annotations

import time
from typing import Dict, List, Tuple

import torch


class _Off:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_OFF = _Off()


class _Phase:
    def __init__(self, owner: "PhaseTimers", name: str, device: bool):
        self.owner, self.name, self.device = owner, name, device

    def __enter__(self):
        torch.cuda.nvtx.range_push(self.name)
        if self.device:
            self.e0 = torch.cuda.Event(enable_timing=True)
            self.e0.record()
        self.t0 = time.perf_counter()
        return self

    def __exit__(self, *exc):
        dt = time.perf_counter() - self.t0
        o = self.owner
        o.host_s[self.name] = o.host_s.get(self.name, 0.0) + dt
        o.calls[self.name] = o.calls.get(self.name, 0) + 1
        if self.device:
            e1 = torch.cuda.Event(enable_timing=True)
            e1.record()
            o._pending.append((self.name, self.e0, e1))
            if len(o._pending) >= PhaseTimers.COLLECT_EVERY:      # a long run that never asks for a report keeps few events
                o._collect(wait=False)
                if len(o._pending) >= 4 * PhaseTimers.COLLECT_EVERY:
                    o._collect(wait=True)
        torch.cuda.nvtx.range_pop()
        return False


class PhaseTimers:
    COLLECT_EVERY = 64      # pending pairs of events beyond which finished ones are read (and all of them at four times that)

    def __init__(self, enabled: bool):
        self.enabled = enabled
        self.host_s: Dict[str, float] = {}
        self.device_s: Dict[str, float] = {}
        self.calls: Dict[str, int] = {}
        self._pending: List[Tuple[str, torch.cuda.Event, torch.cuda.Event]] = []

    def phase(self, name: str, device: bool = False):
        """``with timers.phase("launch", device=True): ...``"""
        return _Phase(self, name, device) if self.enabled else _OFF

    def _collect(self, wait: bool) -> None:
        left = []
        for name, e0, e1 in self._pending:
            if wait or e1.query():
                if wait:
                    e1.synchronize()
                self.device_s[name] = self.device_s.get(name, 0.0) + e0.elapsed_time(e1) * 1e-3
            else:
                left.append((name, e0, e1))
        self._pending = left

    def report(self) -> Dict[str, Dict[str, float]]:
        """Per phase: calls, host milliseconds in all and per call, and device milliseconds where measured."""
        self._collect(wait=True)
        out = {}
        for name, n in self.calls.items():
            row = {"calls": n, "host_ms": self.host_s[name] * 1e3, "host_ms_per_call": self.host_s[name] * 1e3 / n}
            if name in self.device_s:
                row["device_ms"] = self.device_s[name] * 1e3
                row["device_ms_per_call"] = self.device_s[name] * 1e3 / n
            out[name] = row
        return out
