"""Loading a checkpoint by tensor name.

The model says which tensors it wants (name, shape, role); the loader finds
them in the folder's safetensors files and reports everything that does not
fit in ONE error: missing names, unexpected names and wrong shapes.  The
reference assigns ``.data`` by name with a bare KeyError for a missing tensor
and no shape check at all (pico_vllm/weights.py:18-19,42,58,67-68).

Kept dtypes: floating tensors become bfloat16, except that a tensor stored in
32 bit stays float32, norm weights are always float32, and the 32-bit engine
keeps everything in float32.  Integer tables become int32.
"""
from __future__ import annotations

from fnmatch import fnmatchcase
from typing import Dict, Iterable, List

import torch

from ..parts.spec import ParamSpec
from .safetensors_io import SafetensorsError, SafetensorsFile, list_safetensors


class WeightsError(ValueError):
    """The checkpoint does not fit the model; ``missing``, ``unexpected`` and
    ``wrong_shape`` hold the details that the message lists."""

    def __init__(self, where: str, missing, unexpected, wrong_shape, other=()):
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.wrong_shape, self.other = list(wrong_shape), list(other)
        lines = [f"checkpoint {where} does not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{n}: expected {list(e)}, found {list(f)}" for n, e, f in self.wrong_shape))
        for o in self.other:
            lines.append("  " + o)
        super().__init__("\n".join(lines))


def kept_dtype(role: str, stored: torch.dtype, engine_dtype: torch.dtype) -> torch.dtype:
    if role == "table":
        return torch.int32
    if role == "norm" or engine_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32          # stored in 32 bit: stays so
    return torch.bfloat16


def load_checkpoint(model_dir: str, wanted: Iterable[ParamSpec], engine_dtype: torch.dtype,
                    optional: Iterable[str] = ()) -> Dict[str, torch.Tensor]:
    """CPU tensors for every wanted name, converted to their kept dtype.

    ``optional`` names (shell patterns allowed) may be present without being wanted (a tied
    model's stored ``lm_head.weight``, ``ModelSpec.ignored_tensors``); they are ignored."""
    want: Dict[str, ParamSpec] = {p.name: p for p in wanted}
    optional = tuple(optional)
    files: List[SafetensorsFile] = []
    try:
        paths = list_safetensors(model_dir)
        if not paths:
            raise WeightsError(model_dir, sorted(want), [], [], ["the folder holds no .safetensors file"])
        owner: Dict[str, SafetensorsFile] = {}
        other: List[str] = []
        for p in paths:
            try:
                sf = SafetensorsFile(p)
            except SafetensorsError as e:
                raise WeightsError(model_dir, [], [], [], [str(e)]) from None
            files.append(sf)
            for name in sf.entries:
                if name in owner:
                    other.append(f"tensor {name} is stored twice ({owner[name].path} and {p})")
                owner[name] = sf
        missing = sorted(n for n in want if n not in owner)
        unexpected = sorted(n for n in owner if n not in want and not any(fnmatchcase(n, pat) for pat in optional))
        wrong = []
        for n, spec in want.items():
            if n in owner:
                dt, shape = owner[n].entries[n]
                if tuple(shape) != tuple(spec.shape):
                    wrong.append((n, spec.shape, shape))
                is_int = dt.startswith(("I", "U", "BOOL"))
                if is_int != (spec.role == "table"):
                    other.append(f"tensor {n} is stored as {dt}, which does not suit its role {spec.role!r}")
        if missing or unexpected or wrong or other:
            raise WeightsError(model_dir, missing, unexpected, wrong, other)
        out: Dict[str, torch.Tensor] = {}
        for n, spec in want.items():
            t = owner[n].tensor(n)
            out[n] = t.to(kept_dtype(spec.role, t.dtype, engine_dtype))
        return out
    finally:
        for sf in files:
            sf.close()
