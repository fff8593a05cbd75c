"""Reading and writing the safetensors container.

Format: 8 bytes little-endian header length N, N bytes of JSON mapping each
tensor name to {"dtype", "shape", "data_offsets": [begin, end)} (offsets
relative to the end of the header; "__metadata__" is free-form), then the raw
little-endian tensor bytes.  The reference reads the same files through the
safetensors package (pico_vllm/weights.py:10-15).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import numpy as np
import torch

_DTYPES = {
    "F32": (torch.float32, 4, np.float32), "BF16": (torch.bfloat16, 2, np.uint16),
    "F16": (torch.float16, 2, np.float16), "F64": (torch.float64, 8, np.float64),
    "I32": (torch.int32, 4, np.int32), "I64": (torch.int64, 8, np.int64),
    "I16": (torch.int16, 2, np.int16), "I8": (torch.int8, 1, np.int8),
    "U8": (torch.uint8, 1, np.uint8), "BOOL": (torch.bool, 1, np.bool_),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """A memory-mapped safetensors file; ``entries`` maps name -> (dtype name, shape)."""

    def __init__(self, path: str):
        self.path = path
        self._mm = None
        self._f = open(path, "rb")
        try:
            self._read_header(path)
        except BaseException:
            self.close()
            raise

    def _read_header(self, path: str) -> None:
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: file is truncated (no header length)")
        (n,) = struct.unpack("<Q", self._f.read(8))
        if 8 + n > size:
            raise SafetensorsError(f"{path}: file is truncated (header of {n} bytes does not fit in {size})")
        try:
            header = json.loads(self._f.read(n).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON: {e}") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: header is not a JSON object")
        self.metadata = header.pop("__metadata__", {})
        self._base = 8 + n
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        self.entries: Dict[str, Tuple[str, Tuple[int, ...]]] = {}
        self._offsets: Dict[str, Tuple[int, int]] = {}
        for name, info in header.items():
            try:
                dt, shape = info["dtype"], tuple(int(s) for s in info["shape"])
                b, e = (int(x) for x in info["data_offsets"])
            except (KeyError, TypeError, ValueError):
                raise SafetensorsError(f"{path}: tensor {name!r}: entry needs dtype, shape and data_offsets") from None
            if dt not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {dt}")
            want = int(np.prod(shape, dtype=np.int64)) * _DTYPES[dt][1]
            if b < 0 or min(shape, default=0) < 0 or e - b != want:
                raise SafetensorsError(f"{path}: tensor {name!r}: bytes {b}..{e} stored, shape {shape} needs {want}")
            if self._base + e > size:
                raise SafetensorsError(f"{path}: file is truncated inside tensor {name!r}")
            self.entries[name] = (dt, shape)
            self._offsets[name] = (b, e)

    def tensor(self, name: str) -> torch.Tensor:
        """A fresh CPU tensor (a copy of the mapped bytes) in the stored dtype."""
        dt, shape = self.entries[name]
        tdt, _, ndt = _DTYPES[dt]
        b, e = self._offsets[name]
        arr = np.frombuffer(self._mm, dtype=ndt, count=(e - b) // np.dtype(ndt).itemsize, offset=self._base + b)
        t = torch.from_numpy(arr.copy())
        if tdt == torch.bfloat16:
            t = t.view(torch.bfloat16)
        return t.reshape(shape)

    def close(self) -> None:
        if self._mm is not None:
            self._mm.close()
            self._mm = None
        self._f.close()

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()


def write_safetensors(path: str, tensors: Iterable[Tuple[str, Tuple[int, ...], torch.dtype]],
                      produce, metadata: Dict[str, str] | None = None) -> None:
    """Write a file whose tensors are made one at a time.

    ``tensors``: (name, shape, dtype) in file order; ``produce(name)`` returns
    the tensor when its turn comes, so a large model never sits in memory whole.
    """
    entries: List[Tuple[str, Tuple[int, ...], torch.dtype]] = list(tensors)
    header: Dict[str, object] = {}
    off = 0
    for name, shape, dt in entries:
        if dt not in _NAMES:
            raise SafetensorsError(f"cannot store dtype {dt}")
        nbytes = int(np.prod(shape, dtype=np.int64)) * _DTYPES[_NAMES[dt]][1]
        header[name] = {"dtype": _NAMES[dt], "shape": list(shape), "data_offsets": [off, off + nbytes]}
        off += nbytes
    if metadata:
        header["__metadata__"] = metadata
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, shape, dt in entries:
            t = produce(name)
            if tuple(t.shape) != tuple(shape) or t.dtype != dt:
                raise SafetensorsError(f"tensor {name!r}: produced {tuple(t.shape)} {t.dtype}, declared {shape} {dt}")
            t = t.contiguous()
            if dt == torch.bfloat16:
                t = t.view(torch.int16)
            f.write(t.numpy().tobytes())


def list_safetensors(model_dir: str) -> List[str]:
    """All *.safetensors files of a folder, sorted (pico_vllm/weights.py:10)."""
    return sorted(os.path.join(model_dir, n) for n in os.listdir(model_dir) if n.endswith(".safetensors"))
