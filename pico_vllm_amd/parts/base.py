"""Interfaces of the parts a layer is made of.

A part is built from the constants in its ``PartSpec`` (sizes, eps, theta,
flags); it never sees a model configuration and does not know which model it
is in.  Parts can be constructed without a GPU: ``param_specs`` only needs the
constants.  ``load`` receives the part's CPU tensors by name (relative to the
part's prefix) and puts what it needs on the device; ``forward`` runs on the
GPU.

Interfaces:
  Norm.add_norm(resid, delta, rows=None) -> normed;  Norm.deferred(resid, delta) -> DeferredNorm or None
  PositionEncoding.rotate_and_store(qkv, ctx, kv, block_table, nq, nkv, d)
  Mixer.cache_spec() -> CacheSpec;  Mixer.forward(x, ctx, cache) -> y
  FeedForward.forward(x, ctx) -> y
  Block.forward(resid, pending, ctx, cache) -> (resid, pending)
  StreamPart.forward(resid, ctx) -> resid
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

import torch

from .spec import CacheSpec, ParamSpec


@dataclass
class StepContext:
    """What one step gives every part: the flattened batch on the device.

    Tokens of all sequences lie one after the other ([T] arrays); sequence b
    owns tokens cu_seqlens[b] .. cu_seqlens[b+1]."""
    num_tokens: int
    num_seqs: int
    token_ids: torch.Tensor          # int32 [T]
    positions: torch.Tensor          # int32 [T]   absolute position of each token in its request
    token_seq: torch.Tensor          # int32 [T]   row of the token's sequence in the per-sequence arrays
    cu_seqlens: torch.Tensor         # int32 [B+1]
    context_lens: torch.Tensor       # int32 [B]   cached + new tokens
    state_slots: torch.Tensor        # int32 [B]   slot of fixed-size state (zeroed when a new request takes it; padding rows: the spare last slot)
    block_tables: List[torch.Tensor]  # per cache group: int32 [B, max_pages]
    slot_mapping: List[torch.Tensor]  # per cache group: int32 [T], page * page size + offset of each token (-1: none)
    want_rows: torch.Tensor          # int32 [R]   flat token indices whose logits are wanted
    act_dtype: torch.dtype
    # host-side facts for choosing kernels (fixed at capture time under a graph)
    max_new_tokens: int = 1          # longest portion in the batch
    max_context: int = 1             # longest context in the batch
    all_decode: bool = False         # every sequence brings exactly one token
    host: Dict[str, Any] = field(default_factory=dict)   # numpy copies of the arrays above
    shared: Dict[Any, Any] = field(default_factory=dict)  # what parts compute once per step and share between layers


class Part:
    """Common to all parts: declared tensors and loading.

    ``graph_safe``: whether the part's work in a decode step is fixed once the step's shape is (device work only,
    nothing decided from values on the host, no synchronisation), so that the step may be recorded into a HIP graph
    and replayed.  A part that reads ``ctx.host`` or copies values to the host per step sets it to False; a model
    with such a part anywhere never runs from a graph, whatever the engine's options say.

    ``graph_safe_prompts``: the same for a step that is one prompt portion, which is recorded padded: behind the
    portion's sequence stands a second one of filler tokens (slot -1, a block table of -1, outputs ignored) that
    brings the step to a recorded size; in front of the portion there may be sequences of one token each, the last
    of them empty rows as in a recorded decode step (context 0, a block table of -1, the spare state slot).  A part
    that says True does device work only in such a step, may take what it decides on the host from the step that
    was recorded (``ctx.host`` is that step's), and keeps nothing of the filler or the empty rows.  The default is
    False: prompt steps of a model with such a part run unrecorded.

    ``graph_variant(ctx)``: what such a part decides on the host for a prompt step (a kernel's shape, say), as
    something hashable.  Steps whose variants differ are recorded apart, so that a replayed step runs what the
    same step unrecorded would."""
    graph_safe = True
    graph_safe_prompts = False

    def graph_variant(self, ctx: "StepContext") -> tuple:
        """This part's and its parts' host-side choices for the step (empty: none)."""
        out = ()
        for p in self._sub_parts():
            out += p.graph_variant(ctx)
        return out

    def _sub_parts(self) -> List["Part"]:
        return [p for p in vars(self).values() if isinstance(p, Part)]

    def is_graph_safe(self, prompts: bool = False) -> bool:
        """This part and the parts it is built from."""
        own = self.graph_safe_prompts if prompts else self.graph_safe
        return own and all(p.is_graph_safe(prompts) for p in self._sub_parts())

    def param_specs(self) -> List[ParamSpec]:
        return []

    def load(self, tensors: Dict[str, torch.Tensor], device: torch.device, dtype: torch.dtype) -> None:
        pass

    # ---- sizes for reports (the benchmark's roofline) ---------------------
    def _members(self):
        """Sub-parts and matrices this part holds: its attributes, and what lists, tuples and dicts among
        them hold (experts in a list, say)."""
        from ..ops.linear import Linear

        def walk(v, depth=0):
            if isinstance(v, (Part, Linear)):
                yield v
            elif depth < 3 and isinstance(v, (list, tuple)):
                for x in v:
                    yield from walk(x, depth + 1)
            elif depth < 3 and isinstance(v, dict):
                for x in v.values():
                    yield from walk(x, depth + 1)
        for v in vars(self).values():
            yield from walk(v)

    def weight_bytes(self) -> int:
        """Bytes of the matrices a step streams through this part: its ``Linear``s and its sub-parts',
        wherever they are kept.  A part that reads only some of them per step (experts that no token of the
        step was routed to) still counts all: the figure is what a full batch reads."""
        from ..ops.linear import Linear
        return sum(m.weight.numel() * m.weight.element_size() if isinstance(m, Linear) else m.weight_bytes()
                   for m in self._members())

    def flops(self, tokens: int, pairs: int) -> float:
        """Floating-point operations of a step with ``tokens`` new tokens and ``pairs`` (query, key) pairs that
        attention looks at (a prompt of T tokens alone: T (T + 1) / 2): two per weight and token for the matrices
        of this part and its sub-parts; a part with other work (attention's scores) adds its own.  A part that
        runs only some of its matrices per token (routing) overrides this."""
        from ..ops.linear import Linear
        return sum(2.0 * tokens * m.weight.numel() if isinstance(m, Linear) else m.flops(tokens, pairs)
                   for m in self._members())


class DeferredNorm:
    """A norm whose operands are known but which has not run: ``resid_in + delta`` normed.  A block hands
    this, instead of the normed activations, to a consumer that says ``takes_deferred_norm`` and whose first
    kernel may do the norm itself (one launch less in a step of one token).  The consumer either
    does so and sets ``resid`` to the residual stream after the sum, or calls ``run()``, which is the
    norm's own kernel.  ``kind``, ``weight`` and ``eps`` say which norm it is ("rms": RMSNorm)."""

    def __init__(self, norm: "Norm", resid_in: torch.Tensor, delta: Optional[torch.Tensor], kind: str,
                 weight: torch.Tensor, eps: float):
        self.norm, self.resid_in, self.delta = norm, resid_in, delta
        self.kind, self.weight, self.eps = kind, weight, eps
        self.resid: Optional[torch.Tensor] = None

    def run(self) -> torch.Tensor:
        h = self.norm.add_norm(self.resid_in, self.delta)
        self.resid = self.resid_in          # summed in place
        return h


class Norm(Part):
    def deferred(self, resid: torch.Tensor, delta: Optional[torch.Tensor]) -> Optional[DeferredNorm]:
        """The norm of ``resid + delta`` as something a consumer may run inside its own first kernel, or
        None where that cannot pay (the default)."""
        return None

    def add_norm(self, resid: torch.Tensor, delta: Optional[torch.Tensor],
                 rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """resid (float32 [T, H]) += delta, returns the normed rows in the activation dtype;
        with ``rows`` only those rows are produced and resid is left unchanged.  delta is
        [T, H] in the activation dtype or float32, or a float32 stack [S, T, H] of partial
        sums (what ``ops.linear.Linear.partial`` returns), all of which are added."""
        raise NotImplementedError


class StreamPart(Part):
    """A part that works on the residual stream outside the layers (``ModelSpec.before_layers`` /
    ``after_layers``): learned absolute positions added to the embeddings, a norm of the embeddings."""

    def forward(self, resid: torch.Tensor, ctx: "StepContext") -> torch.Tensor:
        """resid: float32 [T, H], the residual stream (with nothing pending); returns it (changed in place or anew)."""
        raise NotImplementedError


class PositionEncoding(Part):
    def rotate_and_store(self, qkv: torch.Tensor, ctx: StepContext, kv, block_table: torch.Tensor,
                         nq: int, nkv: int, d: int) -> None:
        """Encode positions into q (in place) and k, and write k, v into the pages of ``kv``."""
        raise NotImplementedError

    def project_rotate_store(self, x: torch.Tensor, linear, ctx: StepContext, kv, block_table: torch.Tensor,
                             nq: int, nkv: int, d: int) -> torch.Tensor:
        """qkv = linear(x), then ``rotate_and_store``; returns a tensor whose first nq * d columns are
        the encoded queries.  An encoding may override this to fuse the three steps; one that sets
        ``takes_deferred_norm`` may be given a ``DeferredNorm`` as x."""
        if isinstance(x, DeferredNorm):
            x = x.run()
        qkv = linear(x)
        self.rotate_and_store(qkv, ctx, kv, block_table, nq, nkv, d)
        return qkv


class Mixer(Part):
    takes_deferred_norm = False      # True: forward may be given a DeferredNorm as x (and must run or fuse it)

    def cache_spec(self) -> CacheSpec:
        return CacheSpec("none")

    def forward(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        """x: normed activations [T, H]; cache: this run's cache entry
        (``cache.storage.PagedKVLayer`` or ``StateLayer`` or None); returns [T, H]."""
        raise NotImplementedError


class FeedForward(Part):
    takes_deferred_norm = False      # as for a mixer

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """An arrangement of parts.  ``slot_categories`` names its slots and the
    registry category each is built from."""
    slot_categories: Dict[str, str] = {}

    def __init__(self, parts: Dict[str, Part]):
        self.parts = parts

    def _sub_parts(self) -> List[Part]:
        return list(self.parts.values())

    @property
    def mixer(self) -> Mixer:
        return self.parts["mixer"]

    def forward(self, resid: torch.Tensor, pending: Optional[torch.Tensor], ctx: StepContext, cache):
        """resid: float32 residual stream; pending: a delta not yet added to it
        (or None).  Returns (resid, pending) for the next block."""
        raise NotImplementedError
