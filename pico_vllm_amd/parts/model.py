"""The decoder model put together from a ``ModelSpec``."""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from ..config.registry import load_model_description
from ..ops import kernels
from ..ops.linear import Linear
from ..weights.loader import load_checkpoint
from . import attention, block, mlp, norm, rotary  # noqa: F401  (register the parts)
from .base import Block, StepContext
from .registry import build_part, part_class
from .spec import CacheSpec, ModelSpec, ParamSpec

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def _build_layer(lspec, act_dtype) -> Tuple[Block, Dict[str, str]]:
    cls = part_class("block", lspec.block)
    missing = set(cls.slot_categories) - set(lspec.slots)
    if missing:
        raise ValueError(f"layer {lspec.prefix}: block {lspec.block!r} needs slots {sorted(missing)}")
    parts, sub = {}, {}
    for slot, cat in cls.slot_categories.items():
        name, pspec = lspec.slots[slot]
        parts[slot] = build_part(cat, pspec, act_dtype=act_dtype)
        sub[slot] = name
    return cls(parts), sub


def _layer_params(lspec, blk: Block, sub: Dict[str, str]) -> List[Tuple[str, str, ParamSpec]]:
    """(slot, full checkpoint name, spec) of every tensor of a layer."""
    out = []
    for slot, part in blk.parts.items():
        for p in part.param_specs():
            full = f"{lspec.prefix}.{sub[slot]}.{p.name}"
            out.append((slot, full, ParamSpec(full, p.shape, p.role, p.std)))
    return out


def model_param_specs(spec: ModelSpec) -> List[ParamSpec]:
    """Every tensor the model wants from a checkpoint (no device needed)."""
    out = [ParamSpec(spec.embed_name, (spec.vocab_size, spec.hidden_size))]
    for lspec in spec.layers:
        blk, sub = _build_layer(lspec, torch.float32)
        out += [p for _, _, p in _layer_params(lspec, blk, sub)]
    for prefix, pspec in tuple(spec.before_layers) + tuple(spec.after_layers):
        part = build_part("stream", pspec, act_dtype=torch.float32)
        out += [ParamSpec(f"{prefix}.{p.name}" if prefix else p.name, p.shape, p.role, p.std) for p in part.param_specs()]
    fn = build_part("norm", spec.final_norm, act_dtype=torch.float32)
    out += [ParamSpec(f"{spec.final_norm_name}.{p.name}", p.shape, p.role, p.std) for p in fn.param_specs()]
    if spec.head_name:
        out.append(ParamSpec(spec.head_name, (spec.vocab_size, spec.hidden_size)))
    if spec.head_bias_name:
        out.append(ParamSpec(spec.head_bias_name, (spec.vocab_size,), role="bias"))
    return out


class DecoderModel:
    """embedding (times ``spec.embed_scale``) -> ``spec.before_layers`` -> layers in ``run_order`` -> ``spec.after_layers`` -> final norm on the wanted rows ->
    output matrix (+ ``spec.head_bias_name``, soft cap ``spec.logit_softcap``) (pico_vllm/model.py:427-445; the
    reference's model has no multiplier, bias or cap: 1, none and 0 here).  Logits are float32 and exist
    only for the wanted rows (the reference computes all rows and keeps the
    last, engine.py:374).  An untied model multiplies by ``lm_head.weight``
    (the reference always uses the embedding matrix, model.py:445)."""

    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device: torch.device):
        self.spec, self.dtype, self.device = spec, dtype, torch.device(device)
        self.layers: List[Block] = []
        self._sub: List[Dict[str, str]] = []
        for lspec in spec.layers:
            blk, sub = _build_layer(lspec, dtype)
            self.layers.append(blk)
            self._sub.append(sub)
        self.final_norm = build_part("norm", spec.final_norm, act_dtype=dtype)
        # what stands around the layers on the residual stream: (prefix, part)
        self.before = [(pre, build_part("stream", ps, act_dtype=dtype)) for pre, ps in spec.before_layers]
        self.after = [(pre, build_part("stream", ps, act_dtype=dtype)) for pre, ps in spec.after_layers]
        self.embed: Optional[torch.Tensor] = None
        self.head: Optional[Linear] = None
        for i, e in enumerate(spec.run_order):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"run order names layer {e.layer}, the model has {len(self.layers)}")
            if e.cache_of is not None:
                if not 0 <= e.cache_of < i or spec.run_order[e.cache_of].cache_of is not None:
                    raise ValueError(f"run entry {i}: cache_of must name an earlier entry that owns its cache")
                owner = self.layers[spec.run_order[e.cache_of].layer].mixer.cache_spec()
                if self.layers[e.layer].mixer.cache_spec() != owner:
                    raise ValueError(f"run entry {i} cannot use the cache of entry {e.cache_of}: different cache needs")

    def cache_specs(self) -> Dict[int, CacheSpec]:
        """CacheSpec by cache id (the index of the run entry that owns the cache)."""
        return {i: self.layers[self.spec.run_order[i].layer].mixer.cache_spec() for i in self.spec.cache_owners()}

    def param_specs(self) -> List[ParamSpec]:
        return model_param_specs(self.spec)

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        dev, spec = self.device, self.spec
        self.embed = tensors[spec.embed_name].to(dev).contiguous()
        for lspec, blk, sub in zip(spec.layers, self.layers, self._sub):
            for slot, part in blk.parts.items():
                pre = f"{lspec.prefix}.{sub[slot]}."
                part.load({p.name: tensors[pre + p.name] for p in part.param_specs()}, dev, self.dtype)
        for prefix, part in self.before + self.after:
            pre = prefix + "." if prefix else ""
            part.load({p.name: tensors[pre + p.name] for p in part.param_specs()}, dev, self.dtype)
        pre = spec.final_norm_name + "."
        self.final_norm.load({p.name: tensors[pre + p.name] for p in self.final_norm.param_specs()}, dev, self.dtype)
        self.head = Linear(tensors[spec.head_name].to(dev) if spec.head_name else self.embed,
                           tensors[spec.head_bias_name].to(dev) if spec.head_bias_name else None)

    def is_graph_safe(self, prompts: bool = False) -> bool:
        """Whether a decode step (``prompts``: a padded prompt step) of this model may be recorded into a HIP
        graph: every part says so."""
        return all(p.is_graph_safe(prompts) for p in self._all_parts())

    def _all_parts(self):
        return self.layers + [self.final_norm] + [p for _, p in self.before + self.after]

    def graph_variant(self, ctx) -> tuple:
        """The host-side choices of all parts for this step, each distinct one once (layers of one kind choose
        alike): part of the key under which a prompt step is recorded."""
        seen = []
        for blk in self.layers:
            v = blk.graph_variant(ctx)
            if v and v not in seen:
                seen.append(v)
        return tuple(seen)

    def num_weight_bytes(self) -> int:
        """Bytes of matrices a decode step streams: what every part reports (``Part.weight_bytes``), a layer as often
        as the run order names it, and the output matrix (the embedding table only as that, when tied)."""
        total = self.head.weight.numel() * self.head.weight.element_size()
        total += sum(self.layers[e.layer].weight_bytes() for e in self.spec.run_order)
        return total + sum(p.weight_bytes() for _, p in self.before + self.after) + self.final_norm.weight_bytes()

    def flops(self, tokens: int, pairs: int, wanted_rows: int) -> float:
        """Floating-point operations of a step of ``tokens`` new tokens whose attention looks at ``pairs`` (query,
        key) pairs, with logits at ``wanted_rows`` rows: the sum of what the parts report (``Part.flops``)."""
        total = 2.0 * wanted_rows * self.head.weight.numel()
        total += sum(self.layers[e.layer].flops(tokens, pairs) for e in self.spec.run_order)
        return total + sum(p.flops(tokens, pairs) for _, p in self.before + self.after)

    def forward(self, ctx: StepContext, storage) -> torch.Tensor:
        """Logits float32 [R, V] at ctx.want_rows."""
        with kernels.stream_scope():
            return self._forward(ctx, storage)

    def _forward(self, ctx: StepContext, storage) -> torch.Tensor:
        ctx.shared.clear()      # what layers share belongs to this pass (a context may be run again, as at graph capture)
        resid = kernels.embedding(self.embed, ctx.token_ids[:ctx.num_tokens], scale=self.spec.embed_scale)
        for _, part in self.before:
            resid = part.forward(resid, ctx)
        pending = None
        for i, e in enumerate(self.spec.run_order):
            # a run that names another run's cache reads it and stores nothing of its own
            resid, pending = self.layers[e.layer].forward(resid, pending, ctx,
                                                          storage.layer(self.spec.cache_id(i), read_only=e.cache_of is not None))
        if ctx.want_rows.numel() == 0:
            return torch.empty(0, self.spec.vocab_size, dtype=torch.float32, device=self.device)
        if self.after:
            if pending is not None:            # these parts see the whole stream: the last layer's delta joins it first
                for delta in (pending if pending.dim() == 3 else (pending,)):       # a stack of partial sums: each in turn
                    kernels.residual_add(resid, delta)
                pending = None
            for _, part in self.after:
                resid = part.forward(resid, ctx)
        h = self.final_norm.add_norm(resid, pending, rows=ctx.want_rows)
        logits = self.head(h, out_dtype=torch.float32)
        if self.spec.logit_softcap > 0:
            kernels.softcap(logits, self.spec.logit_softcap)
        return logits


def load_model(model_dir: str, dtype: str = "bfloat16", device: str = "cuda:0") -> DecoderModel:
    """Build the model that config.json names and load its weights."""
    if dtype not in _DTYPES:
        raise ValueError(f"dtype must be one of {sorted(_DTYPES)}, got {dtype!r}")
    _, cfg, spec = load_model_description(model_dir)
    model = DecoderModel(spec, _DTYPES[dtype], torch.device(device))
    tensors = load_checkpoint(model_dir, model.param_specs(), _DTYPES[dtype], optional=spec.ignored_tensors)
    model.load(tensors)
    model.config = cfg
    return model
