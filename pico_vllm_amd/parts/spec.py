"""Descriptions of a model as data: which parts each layer is made of, with
which constants, in which order the layers run and whose cache each run reads.

Nothing here touches a device.  An architecture turns its typed configuration
into a ``ModelSpec``; ``parts.model.DecoderModel`` builds the runnable parts
from it through the part registries in ``parts.registry``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple, Union


@dataclass(frozen=True)
class PartSpec:
    """A part chosen by name with its sizes and constants."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class ParamSpec:
    """One tensor a part wants from the checkpoint.

    ``role`` decides the dtype it is kept in and how random weights draw it:
      matrix  - bfloat16 (float32 in the 32-bit engine, or if stored in 32 bit); N(0, std)
      bias    - like matrix; N(0, std)
      norm    - float32 always; 1 + U(-0.1, 0.1)
      table   - int32 integer table; zeros
    """
    name: str
    shape: Tuple[int, ...]
    role: str = "matrix"
    std: float = 0.02


@dataclass(frozen=True)
class PageTensor:
    """One tensor that a paged cache keeps for every page.  ``shape`` is that of ONE page; the string
    "page" in it stands for the number of tokens a page holds (an engine option, not the part's).
    ``dtype``: a torch dtype by name, or None for the engine's."""
    name: str
    shape: Tuple[Union[int, str], ...]
    dtype: Optional[str] = None

    def resolved(self, page_size: int) -> Tuple[int, ...]:
        out = []
        for s in self.shape:
            if s == "page":
                out.append(page_size)
            elif isinstance(s, int) and s > 0:
                out.append(s)
            else:
                raise ValueError(f"page tensor {self.name!r}: a dimension is a positive int or 'page', got {s!r}")
        return tuple(out)


@dataclass(frozen=True)
class CacheSpec:
    """What a mixer keeps per request between steps.

    kind "paged_kv": what ``page_tensors`` lists, per page of tokens (the mixer names the tensors
    and their layout inside a page; the cache only allocates them, one allocation a tensor and
    layer, and hands them to the mixer by name); ``window`` > 0 means only the last ``window``
    positions are ever read again, so older pages can be given back early.
    kind "state": a fixed-size tensor of ``state_shape`` per request.
    kind "none": nothing.
    Layers with equal specs share a pool of page ids and a block table per request.
    """
    kind: str = "none"
    window: int = 0
    page_tensors: Tuple[PageTensor, ...] = ()
    state_shape: Tuple[int, ...] = ()
    state_dtype: str = "float32"

    def __post_init__(self):
        if self.kind == "paged_kv":
            names = [t.name for t in self.page_tensors]
            if not names or len(set(names)) != len(names):
                raise ValueError("a paged cache needs page tensors with distinct names")


@dataclass(frozen=True)
class LayerSpec:
    """One layer: an arrangement (``block``) whose slots are filled with
    parts.  ``slots`` maps a slot name of the arrangement (for the pre-norm
    block: norm1, mixer, norm2, ff) to (sub-prefix of the part's tensors in
    the checkpoint, the part).  ``prefix`` is the layer's own prefix."""
    prefix: str
    block: str
    slots: Dict[str, Tuple[str, PartSpec]]


@dataclass(frozen=True)
class RunEntry:
    """One entry of the run order: run ``layer`` (an index into ``layers``; a
    layer may be named by several entries, which then share its weights).
    Every entry owns a cache of its own unless ``cache_of`` names an EARLIER
    entry of the run order, whose cache this run's mixer is then given."""
    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    hidden_size: int
    vocab_size: int
    embed_name: str
    layers: List[LayerSpec]
    run_order: List[RunEntry]
    final_norm: PartSpec
    final_norm_name: str
    head_name: Optional[str]          # None: output matrix is the embedding matrix
    eos_token_id: Optional[int] = None
    max_position: int = 131072
    # names (shell patterns allowed) of tensors a checkpoint may hold that the model does not use: a tied model's
    # stored output matrix, buffers that another implementation keeps in its files
    ignored_tensors: Tuple[str, ...] = ()
    # parts that run on the residual stream before the first and after the last layer (category "stream":
    # learned absolute positions, a norm of the embeddings): (prefix of the part's tensors, the part)
    before_layers: Tuple[Tuple[str, PartSpec], ...] = ()
    after_layers: Tuple[Tuple[str, PartSpec], ...] = ()
    embed_scale: float = 1.0          # the embedding rows are multiplied by this (1: as they are)
    logit_softcap: float = 0.0        # > 0: logits = cap * tanh(logits / cap)
    head_bias_name: Optional[str] = None   # a bias [vocab] added to the logits

    def cache_id(self, entry_index: int) -> int:
        """The run entry whose cache entry ``entry_index`` uses."""
        e = self.run_order[entry_index]
        return entry_index if e.cache_of is None else e.cache_of

    def cache_owners(self) -> List[int]:
        """Run entries that own a cache."""
        return [i for i, e in enumerate(self.run_order) if e.cache_of is None]
