"""Building and loading the HIP kernel library.

The kernels are plain HIP sources under ``csrc/`` compiled by ``hipcc`` for
gfx950 into one shared object per (source set, defines), loaded with ctypes.
A built library is reused when the hash of its sources and flags matches;
otherwise it is compiled at the first call, which prints a line per file so a
first run is not silent.  There is no fallback: a missing compiler or a failed
build raises.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from typing import Dict, Iterable, List, Sequence

CSRC = os.path.normpath(os.path.join(os.path.dirname(__file__), "..", "csrc"))
ARCH = "gfx950"
# packed float32 instructions are switched off for all device code
HIP_FLAGS = ["-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument"]

CORE_SOURCES = ("errors.hip", "elementwise.hip", "gemm_f32.hip", "gemm_bf16.hip", "gemm_skinny.hip", "attention_ref.hip", "sampling.hip")

ATTN_SOURCES = ("errors.hip", "attention_mfma.hip")

PEAK_SOURCES = ("errors.hip", "peaks.hip")

_loaded: Dict[str, ctypes.CDLL] = {}


class KernelBuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise KernelBuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin); "
                           "the HIP kernels cannot be built and there is no other code path")


def build_root() -> str:
    """In-tree ``_build`` if it can be written, else a per-user folder under the temp dir."""
    tree = os.path.normpath(os.path.join(os.path.dirname(__file__), "..", "_build"))
    try:
        os.makedirs(tree, exist_ok=True)
        probe = os.path.join(tree, f".w{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return tree
    except OSError:
        alt = os.path.join(tempfile.gettempdir(), f"pico_vllm_amd_build_{os.getuid()}")
        os.makedirs(alt, exist_ok=True)
        return alt


def _digest(sources: Sequence[str], defines: Sequence[str]) -> str:
    h = hashlib.sha256()
    h.update(" ".join(HIP_FLAGS + list(defines)).encode())
    for name in sorted(set(list(sources) + [n for n in os.listdir(CSRC) if n.endswith(".h")])):
        h.update(name.encode())
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def _say(msg: str) -> None:
    print(f"[pico_vllm_amd] {msg}", file=sys.stderr, flush=True)


def build_library(name: str, sources: Sequence[str], defines: Sequence[str] = (), force: bool = False) -> str:
    """Compile ``sources`` (names under csrc/) into lib<name>.so and return its path."""
    root = build_root()
    so = os.path.join(root, f"lib{name}.so")
    stamp = so + ".hash"
    digest = _digest(sources, defines)
    if not force and os.path.isfile(so) and os.path.isfile(stamp):
        with open(stamp) as f:
            if f.read().strip() == digest:
                return so
    hipcc = _hipcc()
    _say(f"building {os.path.basename(so)} for {ARCH} ({len(sources)} files) ...")
    t0 = time.time()
    objdir = os.path.join(root, f"obj_{name}_{os.getpid()}")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src: str) -> str:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *HIP_FLAGS, *defines, "-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise KernelBuildError(f"hipcc failed on {src}:\n{' '.join(cmd)}\n{r.stderr[-4000:]}")
        _say(f"  compiled {src} ({time.time() - t0:.0f}s)")
        return obj

    try:
        with ThreadPoolExecutor(max_workers=min(8, len(sources))) as ex:
            objs = list(ex.map(compile_one, sources))
        tmp = so + f".tmp{os.getpid()}"
        cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", tmp]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise KernelBuildError(f"linking {so} failed:\n{r.stderr[-4000:]}")
        os.replace(tmp, so)
        with open(stamp, "w") as f:
            f.write(digest)
    finally:
        shutil.rmtree(objdir, ignore_errors=True)
    _say(f"built {os.path.basename(so)} in {time.time() - t0:.0f}s")
    return so


def load_library(name: str, sources: Sequence[str], defines: Sequence[str] = ()) -> ctypes.CDLL:
    key = name
    if key not in _loaded:
        path = build_library(name, sources, defines)
        try:
            _loaded[key] = ctypes.CDLL(path)
        except OSError as e:
            raise KernelBuildError(f"cannot load {path}: {e}") from None
    return _loaded[key]


def core() -> ctypes.CDLL:
    """The library every model needs."""
    return load_library("pico_core", CORE_SOURCES)


def attention_library(head_dim: int) -> ctypes.CDLL:
    """Matrix-core attention kernels specialised for one head size."""
    return load_library(f"pico_attn_d{head_dim}", ATTN_SOURCES, (f"-DPICO_HEAD_DIM={head_dim}",))


def peaks() -> ctypes.CDLL:
    """The two measuring kernels of the benchmark (a read stream, a matrix-core loop)."""
    return load_library("pico_peaks", PEAK_SOURCES)


def build_all(head_dims: Iterable[int] = tuple(range(16, 257, 16)), force: bool = True) -> List[str]:
    """Compile everything (used by the build check); returns the paths."""
    out = [build_library("pico_core", CORE_SOURCES, force=force), build_library("pico_peaks", PEAK_SOURCES, force=force)]
    if os.path.isfile(os.path.join(CSRC, "attention_mfma.hip")):
        for d in head_dims:
            out.append(build_library(f"pico_attn_d{d}", ATTN_SOURCES, (f"-DPICO_HEAD_DIM={d}",), force=force))
    return out
