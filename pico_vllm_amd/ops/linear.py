"""y = x W^T (+ b) with W stored [out, in] as in the checkpoint.

bfloat16 weights: with up to 64 rows of activations (decode, small mixed
steps; up to 256 for small matrices) the weight-streaming matrix-core kernel of this package, with bias,
SwiGLU or float32 output as its epilogue (for shapes it refuses, this package's plain matrix-core product); with more rows the library GEMM
(hipBLASLt through torch), as the reference uses the library for every
projection (pico_vllm/model.py:200,225,316,318).  float32 weights: this package's plain-FMA kernel, never a library
call, so the 32-bit engine has no reduced-precision matrix mode anywhere; if
the activations are bfloat16 (a tensor stored in 32 bit inside a bfloat16
engine) they are widened on load and the result is rounded once.
"""
from __future__ import annotations

import os
import tempfile
from typing import Optional

import torch

from . import kernels

# The library GEMM can be picked by the library's own tuner (PyTorch's TunableOp: it times the rocBLAS and
# hipBLASLt solutions for a shape once and keeps the fastest; on the 1.5B shapes with 2,048 rows that
# is 91 us against 122 us for the gate/up product).  Timing candidates stalls the first step of a shape for
# up to 30 s and switches a process-wide mode of torch on, so it is off unless ``set_library_tuning(True)``
# asks for it (``EngineArgs.tune_library_gemm``; the benchmark does).  A step's row count is arbitrary, so only
# row counts that are multiples of TUNE_ROWS (whole prompt portions) are tuned; every other count takes the
# library's default choice.  Results are kept in a per-user file under the temp dir and read back by the next process.
TUNE_ROWS = 512
_tuner_state = {"wanted": False, "ready": False, "tuning": None}


def set_library_tuning(on: bool) -> None:
    """Switch the tuner on or off for this process; off also hands torch's own mode back."""
    st = _tuner_state
    st["wanted"] = bool(on)
    if not on and st["ready"] is True:
        try:
            torch.cuda.tunable.tuning_enable(False)
            torch.cuda.tunable.enable(False)
        except Exception:
            pass
        st["ready"], st["tuning"] = False, None


def _library_tuning(rows: int) -> None:
    st = _tuner_state
    if not st["wanted"]:
        return
    tunable = torch.cuda.tunable
    if not st["ready"]:
        st["ready"] = True
        try:
            path = os.path.join(tempfile.gettempdir(), f"pico_vllm_amd_tunableop_{os.getuid()}.csv")
            tunable.enable(True)
            tunable.set_filename(path)
            tunable.set_max_tuning_duration(30)
            tunable.set_max_tuning_iterations(20)
            if os.path.exists(path):
                tunable.read_file(path)
        except Exception:                      # a build of torch without the tuner: the default choice serves
            st["ready"] = "off"
    if st["ready"] == "off":
        return
    # never while a graph is being recorded: timing candidates does not belong into a graph
    want = rows % TUNE_ROWS == 0 and not torch.cuda.is_current_stream_capturing()
    if st["tuning"] != want:
        tunable.tuning_enable(want)
        st["tuning"] = want


class Linear:
    def __init__(self, weight: torch.Tensor, bias: Optional[torch.Tensor] = None):
        if weight.dim() != 2:
            raise ValueError("a linear weight is a matrix")
        self.weight = weight.contiguous()
        self.bias = None if bias is None else bias.to(self.weight.dtype).contiguous()
        self.bias_f32 = None if bias is None else bias.float().contiguous()
        self.out_features, self.in_features = weight.shape

    def __call__(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        out_dtype = out_dtype or x.dtype
        if x.shape[-1] != self.in_features:
            raise ValueError(f"linear: input has {x.shape[-1]} features, the weight wants {self.in_features}")
        if self.weight.dtype == torch.float32:
            y = kernels.gemm_f32(x, self.weight, self.bias_f32)
            return y if out_dtype == torch.float32 else y.to(out_dtype)
        if x.dtype != torch.bfloat16:
            raise ValueError("linear: bfloat16 weights need bfloat16 activations")
        if kernels.skinny_ok(x, self.weight):
            epi = kernels.EPI_F32 if out_dtype == torch.float32 else kernels.EPI_BF16
            return kernels.gemm_skinny(x, self.weight, self.bias_f32, epi)
        if out_dtype == torch.float32:
            return kernels.gemm_bf16(x, self.weight, self.bias_f32, torch.float32)
        if kernels.skinny_rows(x, self.weight):
            # few rows of a shape that the weight-streaming kernel refuses (an inner size that is no multiple of 8):
            # this package's plain matrix-core product, in which a row's result does not depend on the other rows of
            # the step, as it does not in the weight-streaming kernel; the library's may
            return kernels.gemm_bf16(x, self.weight, self.bias_f32, torch.bfloat16)
        _library_tuning(x.shape[0])
        if self.bias is not None:
            return torch.addmm(self.bias, x, self.weight.t())
        return torch.mm(x, self.weight.t())

    def swiglu(self, x) -> torch.Tensor:
        """silu(gate) * up where [gate; up] = x W^T (W's first half of rows is the gate).  With few
        rows the activation is the epilogue of the weight-streaming kernel and [gate; up] never
        reaches memory.  x may be a norm that has not run (``parts.base.DeferredNorm``): with one
        row it becomes the same kernel's prologue."""
        if hasattr(x, "resid_in"):
            if (x.kind == "rms" and self.bias is None and kernels.skinny_norm_ok(x.resid_in, x.delta, self.weight)
                    and self.out_features % 2 == 0):
                out, x.resid = kernels.gemm_skinny_norm(x.resid_in, x.delta, x.weight, x.eps, self.weight, kernels.EPI_SWIGLU)
                return out
            x = x.run()
        if self.weight.dtype == torch.bfloat16 and self.bias is None and kernels.skinny_ok(x, self.weight):
            return kernels.gemm_skinny(x, self.weight, None, kernels.EPI_SWIGLU)
        return kernels.swiglu(self(x))

    def partial(self, x: torch.Tensor) -> torch.Tensor:
        """x W^T as something a norm's ``add_norm`` takes as delta: [T, N], or, when the matrix is
        too small to fill the chip with one workgroup per output tile, a float32 stack [S, T, N] of
        partial sums over S ranges of k, which the norm kernel adds up."""
        if self.weight.dtype == torch.bfloat16 and self.bias is None and kernels.skinny_ok(x, self.weight):
            splits = kernels.skinny_k_splits(self.out_features, self.in_features)
            if splits > 1:
                return kernels.gemm_skinny(x, self.weight, None, kernels.EPI_F32, splits)
        return self(x)
