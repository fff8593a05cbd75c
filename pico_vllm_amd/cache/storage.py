"""Device tensors of the cache: pages of keys and values per layer, and the
per-request state of mixers that keep one.

Layout of one layer (one allocation each for K and V):
  K [pages, kv heads, page size, head size]     a token's key is contiguous
  V [pages, kv heads, head size, page size]     a head-dimension's values of a page are contiguous
The reference keeps one tensor [2, L, pages, kv heads, page, d] for all layers
(pico_vllm/blockmanager.py:39-42) with V laid out like K; V is transposed here
because the matrix-core kernels contract over keys.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict

import torch

from ..parts.spec import CacheSpec
from .manager import CacheManager


@dataclass
class PagedKVLayer:
    k: torch.Tensor
    v: torch.Tensor
    group: int
    page_size: int
    read_only: bool = False    # True for a run that reads another run's cache: it attends over it and stores nothing


@dataclass
class StateLayer:
    state: torch.Tensor        # [slots + 1, *state_shape]; the last slot belongs to padding rows
    group: int = -1


class CacheStorage:
    def __init__(self, manager: CacheManager, layer_specs: Dict[int, CacheSpec], dtype: torch.dtype,
                 device: torch.device):
        self.manager = manager
        self._layers: Dict[int, object] = {}
        P = manager.page_size
        for layer, spec in layer_specs.items():
            if spec.kind == "paged_kv":
                gi = manager.layer_group[layer]
                n = manager.groups[gi].pool.num_pages
                k = torch.zeros(n, spec.num_kv_heads, P, spec.head_dim, dtype=dtype, device=device)
                v = torch.zeros(n, spec.num_kv_heads, spec.head_dim, P, dtype=dtype, device=device)
                self._layers[layer] = PagedKVLayer(k, v, gi, P)
            elif spec.kind == "state":
                sdt = getattr(torch, spec.state_dtype)
                # one slot more than requests can hold: the padding rows of a recorded decode batch write there
                self._layers[layer] = StateLayer(
                    torch.zeros(manager.slots.num_slots + 1, *spec.state_shape, dtype=sdt, device=device))
            else:
                self._layers[layer] = None

    def layer(self, index: int, read_only: bool = False):
        """The cache of run entry ``index``; ``read_only`` for a run that was given another run's cache."""
        entry = self._layers.get(index)
        if read_only and isinstance(entry, PagedKVLayer):
            return PagedKVLayer(entry.k, entry.v, entry.group, entry.page_size, read_only=True)
        return entry

    def save_state(self):
        """Copies of every per-request state tensor (for ``restore_state``)."""
        return {i: l.state.clone() for i, l in self._layers.items() if isinstance(l, StateLayer)}

    def restore_state(self, saved) -> None:
        for i, t in saved.items():
            self._layers[i].state.copy_(t)

    def reset_state(self, slots) -> None:
        """Zero the state of these slots in every layer that keeps one (a new request took them)."""
        if not slots:
            return
        idx = None
        for l in self._layers.values():
            if isinstance(l, StateLayer):
                if idx is None:
                    idx = torch.tensor(sorted(set(slots)), dtype=torch.long, device=l.state.device)
                l.state.index_fill_(0, idx, 0)

    def num_bytes(self) -> int:
        total = 0
        for l in self._layers.values():
            if isinstance(l, PagedKVLayer):
                total += l.k.numel() * l.k.element_size() * 2
            elif isinstance(l, StateLayer):
                total += l.state.numel() * l.state.element_size()
        return total

    def bytes_per_token(self) -> int:
        """Cache bytes one token of context occupies over all layers."""
        total = 0
        for l in self._layers.values():
            if isinstance(l, PagedKVLayer):
                total += 2 * l.k.shape[1] * l.k.shape[3] * l.k.element_size()
        return total
