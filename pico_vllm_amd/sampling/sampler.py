"""Sampling one token per row of logits on the GPU.

Strategy per row as in pico_vllm/sampler.py:40-88 (greedy / temperature /
temperature with top-p), but in one call with per-row parameters for the whole
batch (a short chain of launches, several workgroups a row) instead of torch
calls per group of equal parameters.  Randomness comes from
a counter-based generator on the host: the uniform number of a draw depends
only on (seed, index of the token in its request), so a request samples the
same tokens whatever else is in the batch.
"""
from __future__ import annotations

from typing import List, Sequence

import torch

from ..ops import kernels

_MASK = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform(seed: int, index: int) -> float:
    """A number in [0, 1) with 24 random bits, a pure function of (seed, index)."""
    z = _splitmix64(_splitmix64(seed & _MASK) ^ ((index * 0xD6E8FEB86659FD93) & _MASK))
    return (z >> 40) / float(1 << 24)


class Sampler:
    def __init__(self, device: torch.device, max_rows: int):
        self.device = device
        self.max_rows = max_rows
        # two sets of host buffers, used in turn: a step's tokens may be read, and its parameters
        # may still wait for their copy, after the next step was launched
        self._host = [torch.zeros(3, max_rows, dtype=torch.float32, pin_memory=torch.cuda.is_available()) for _ in range(2)]
        self._dev = torch.zeros(3, max_rows, dtype=torch.float32, device=device)
        self._out = torch.zeros(max_rows, dtype=torch.int32, device=device)
        self._argmax_work = kernels.argmax_workspace(max_rows, device) if torch.cuda.is_available() else None
        self._sample_work = kernels.sample_workspace(max_rows, device) if torch.cuda.is_available() else None
        self._host_np = [h.numpy() for h in self._host]
        self._landing = [torch.zeros(max_rows, dtype=torch.int32, pin_memory=torch.cuda.is_available()) for _ in range(2)]
        self._landed = [torch.cuda.Event() if torch.cuda.is_available() else None for _ in range(2)]
        self._turn = 0

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], top_ps: Sequence[float],
               seeds: Sequence[int], indices: Sequence[int]) -> List[int]:
        """logits: float32 [R, V]; one (temperature, top_p, seed, token index) per row."""
        return self.read(self.launch(logits, temperatures, top_ps, seeds, indices))

    @property
    def device_tokens(self) -> torch.Tensor:
        """int32 [max_rows] on the device: row r holds the token of row r of the last launch."""
        return self._out

    def read(self, ticket) -> List[int]:
        """The tokens of the launch that returned ``ticket``; waits for that launch only."""
        turn, R = ticket
        if R == 0:
            return []
        self._landed[turn].synchronize()
        return self._landing[turn][:R].tolist()

    def launch(self, logits: torch.Tensor, temperatures: Sequence[float], top_ps: Sequence[float],
               seeds: Sequence[int], indices: Sequence[int]):
        """Start sampling and the copy of the tokens to the host; returns a ticket for ``read``.
        At most two launches may be unread at a time."""
        R = logits.shape[0]
        if not (len(temperatures) == len(top_ps) == len(seeds) == len(indices) == R):
            raise ValueError("one set of sampling parameters per row of logits is needed")
        if R > self.max_rows:
            raise ValueError(f"{R} rows to sample, the sampler was made for {self.max_rows}")
        if R == 0:
            return (0, 0)
        if not any(temperatures):
            # all rows greedy: nothing to upload, and the argmax alone spreads a row over several workgroups
            kernels.argmax(logits, self._out, self._argmax_work)
        else:
            h = self._host_np[self._turn]
            h[0, :R] = temperatures
            h[1, :R] = top_ps
            h[2, :R] = [uniform(s, i) if t > 0 else 0.0 for s, i, t in zip(seeds, indices, temperatures)]
            self._dev.copy_(self._host[self._turn], non_blocking=True)
            kernels.sample(logits, self._dev[0], self._dev[1], self._dev[2], self._out, self._sample_work,
                           top_p_rows=any(t > 0 and p < 1 for t, p in zip(temperatures, top_ps)))
        turn = self._turn
        self._turn ^= 1
        self._landing[turn][:R].copy_(self._out[:R], non_blocking=True)
        self._landed[turn].record()
        return (turn, R)
