"""Device tensors of the cache: per layer the page tensors that its mixer's ``CacheSpec`` names, and the
per-request state of mixers that keep one.

A paged layer gets one allocation per tensor of its spec, [pages, *shape of one page] in the engine's dtype
(or the tensor's own); what the tensors hold and how a page is laid out is the mixer's business.  The
attention of this package asks for ``k`` and ``v`` (``parts.attention.kv_page_tensors``); the reference keeps
one tensor [2, L, pages, kv heads, page, d] for all layers (pico_vllm/blockmanager.py:39-42).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict

import torch

from ..parts.spec import CacheSpec
from .manager import CacheManager


@dataclass
class PagedKVLayer:
    """The page tensors of one layer by name (also as attributes: ``layer.k``)."""
    tensors: Dict[str, torch.Tensor]
    group: int
    page_size: int
    read_only: bool = False    # True for a run that reads another run's cache: it attends over it and stores nothing

    def __getattr__(self, name: str) -> torch.Tensor:
        try:
            return self.__dict__["tensors"][name]
        except KeyError:
            raise AttributeError(f"this layer's cache has no tensor {name!r}; it holds {sorted(self.__dict__.get('tensors', {}))}") from None


@dataclass
class StateLayer:
    state: torch.Tensor        # [slots + 1, *state_shape]; the last slot belongs to padding rows
    group: int = -1


def bytes_per_page(layer_specs: Dict[int, CacheSpec], page_size: int, dtype: torch.dtype) -> int:
    """Device bytes that one more page in every group's pool costs, over all paged layers."""
    total = 0
    for spec in layer_specs.values():
        if spec.kind == "paged_kv":
            for t in spec.page_tensors:
                n = 1
                for s in t.resolved(page_size):
                    n *= s
                total += n * torch.empty(0, dtype=getattr(torch, t.dtype) if t.dtype else dtype).element_size()
    return total


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
                self._layers[layer] = PagedKVLayer(
                    {t.name: torch.zeros(n, *t.resolved(P), dtype=getattr(torch, t.dtype) if t.dtype else dtype, device=device)
                     for t in spec.page_tensors}, gi, P)
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
            return PagedKVLayer(entry.tensors, entry.group, entry.page_size, read_only=True)
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
                total += sum(t.numel() * t.element_size() for t in l.tensors.values())
            elif isinstance(l, StateLayer):
                total += l.state.numel() * l.state.element_size()
        return total

    def bytes_per_token(self) -> int:
        """Cache bytes one token of context occupies over all layers."""
        total = 0
        for l in self._layers.values():
            if isinstance(l, PagedKVLayer):
                total += sum(t[0].numel() * t.element_size() for t in l.tensors.values()) // l.page_size
        return total
