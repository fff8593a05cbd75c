"""Python faces of the HIP kernels.

Every function checks on the host that shapes, dtypes and layouts are what the
kernel and its grid assume, then launches on torch's current stream.  Tensors
must live on the GPU; there is no CPU path.
"""
from __future__ import annotations

import ctypes
import functools
from typing import Optional

import torch

from . import library

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}
c_int, c_float, c_void_p, c_ll = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_longlong


class KernelError(RuntimeError):
    pass


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"dtype {t.dtype} is not supported by the kernels (float32 or bfloat16)") from None


def _gpu(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("the kernels run on the GPU only; got a CPU tensor")


def _ptr(t: Optional[torch.Tensor]):
    return c_void_p(t.data_ptr() if t is not None else 0)


_bound_stream = None


def _stream():
    if _bound_stream is not None:
        return _bound_stream
    return c_void_p(torch.cuda.current_stream().cuda_stream)


class stream_scope:
    """Look torch's current stream up once for all launches inside the scope (the lookup costs
    more than a launch).  The scope must not span a change of the current stream."""

    def __enter__(self):
        global _bound_stream
        self._outer = _bound_stream
        _bound_stream = c_void_p(torch.cuda.current_stream().cuda_stream)
        return self

    def __exit__(self, *exc):
        global _bound_stream
        _bound_stream = self._outer
        return False


def _check(lib, code: int) -> None:
    if code != 0:
        lib.pico_last_error.restype = ctypes.c_char_p
        raise KernelError(lib.pico_last_error().decode())


def _i32(t: torch.Tensor, name: str, n: Optional[int] = None) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{name} must be a contiguous int32 tensor")
    if n is not None and t.numel() < n:
        raise KernelError(f"{name} has {t.numel()} entries, {n} are needed")


def embedding(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """out[t] = table[ids[t]] * scale as float32 rows (the residual stream)."""
    _gpu(table, ids)
    V, H = table.shape
    T = ids.numel()
    _i32(ids, "ids")
    if not table.is_contiguous():
        raise KernelError("embedding table must be contiguous")
    if out is None:
        out = torch.empty(T, H, dtype=torch.float32, device=table.device)
    elif out.shape != (T, H) or out.dtype != torch.float32 or not out.is_contiguous():
        raise KernelError("embedding: out must be a contiguous float32 [T, H] tensor")
    lib = library.core()
    _check(lib, lib.pico_embedding(_ptr(table), _dt(table), _ptr(ids), _ptr(out), T, H, V, c_float(scale), _stream()))
    return out


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x = cap * tanh(x / cap) in place, float32."""
    _gpu(x)
    if x.dtype != torch.float32 or not x.is_contiguous() or not cap > 0:
        raise KernelError("softcap: a contiguous float32 tensor and a positive cap")
    lib = library.core()
    _check(lib, lib.pico_softcap(_ptr(x), c_ll(x.numel()), c_float(cap), _stream()))
    return x


def add_rmsnorm(resid: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """rows is None: resid += delta (if given), returns norm(resid).
    rows given: returns norm(resid[rows] + delta[rows]); resid is left alone.
    delta is [T, H], or a float32 stack [S, T, H] of partial sums that are all added."""
    _gpu(resid, delta, weight, rows)
    T, H = resid.shape
    if resid.dtype != torch.float32 or not resid.is_contiguous():
        raise KernelError("the residual stream must be contiguous float32")
    if weight.dtype != torch.float32 or weight.shape != (H,) or not weight.is_contiguous():
        raise KernelError(f"norm weight must be float32 of shape [{H}]")
    slabs = 1
    if delta is not None:
        if delta.dim() == 3:
            slabs = delta.shape[0]
            if delta.dtype != torch.float32:
                raise KernelError("a stack of partial sums must be float32")
        if tuple(delta.shape[-2:]) != (T, H) or not delta.is_contiguous():
            raise KernelError("delta must be contiguous and shaped like the residual stream")
    n = T
    if rows is not None:
        _i32(rows, "rows")
        n = rows.numel()
    if out is None:
        out = torch.empty(n, H, dtype=out_dtype, device=resid.device)
    elif out.shape != (n, H) or out.dtype != out_dtype or not out.is_contiguous():
        raise KernelError("add_rmsnorm: out has the wrong shape or dtype")
    lib = library.core()
    ddt = _dt(delta) if delta is not None else F32
    _check(lib, lib.pico_add_rmsnorm(_ptr(resid), _ptr(delta), ddt, slabs, c_ll(T * H), _ptr(weight), _ptr(out),
                                     _DT[out_dtype], _ptr(rows), n, H, c_float(eps), _stream()))
    return out


def residual_add(resid: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    _gpu(resid, delta)
    if resid.dtype != torch.float32 or not resid.is_contiguous() or delta.shape != resid.shape \
            or not delta.is_contiguous():
        raise KernelError("residual_add: float32 contiguous residual and an equally shaped contiguous delta")
    lib = library.core()
    _check(lib, lib.pico_residual_add(_ptr(resid), _ptr(delta), _dt(delta), c_ll(resid.numel()), _stream()))
    return resid


def swiglu(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _gpu(gate_up)
    T, I2 = gate_up.shape
    if I2 % 2 or not gate_up.is_contiguous():
        raise KernelError("swiglu: input must be contiguous [T, 2 I]")
    I = I2 // 2
    if out is None:
        out = torch.empty(T, I, dtype=gate_up.dtype, device=gate_up.device)
    elif out.shape != (T, I) or out.dtype != gate_up.dtype or not out.is_contiguous():
        raise KernelError("swiglu: out has the wrong shape or dtype")
    lib = library.core()
    _check(lib, lib.pico_swiglu(_ptr(gate_up), _ptr(out), _dt(gate_up), T, I, _stream()))
    return out


def gemm_f32(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
             out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 out = a @ w.T + bias with plain FMA.  a: [M, K] float32 or bfloat16 (rows may be
    strided), w: [N, K] float32."""
    _gpu(a, w, bias)
    M, K = a.shape
    N, K2 = w.shape
    if K != K2:
        raise KernelError(f"gemm: inner sizes differ ({K} and {K2})")
    if w.dtype != torch.float32 or w.stride(1) != 1 or a.stride(1) != 1:
        raise KernelError("gemm_f32: w must be float32 and both operands contiguous along K")
    if bias is not None and (bias.dtype != torch.float32 or bias.shape != (N,) or not bias.is_contiguous()):
        raise KernelError("gemm_f32: bias must be contiguous float32 [N]")
    if out is None:
        out = torch.empty(M, N, dtype=torch.float32, device=a.device)
    elif out.shape != (M, N) or out.dtype != torch.float32 or out.stride(1) != 1:
        raise KernelError("gemm_f32: out has the wrong shape or dtype")
    lib = library.core()
    _check(lib, lib.pico_gemm_f32(_ptr(a), _dt(a), _ptr(w), _ptr(bias), _ptr(out), M, N, K,
                                  a.stride(0) if M > 1 else K, w.stride(0), out.stride(0) if M > 1 else N, _stream()))
    return out


def gemm_bf16(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
              out_dtype: torch.dtype = torch.bfloat16, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = a @ w.T + bias on the matrix cores; a [M, K], w [N, K] bfloat16, bias float32,
    out float32 or bfloat16."""
    _gpu(a, w, bias)
    M, K = a.shape
    N, K2 = w.shape
    if K != K2:
        raise KernelError(f"gemm: inner sizes differ ({K} and {K2})")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or a.stride(1) != 1 or w.stride(1) != 1:
        raise KernelError("gemm_bf16: operands must be bfloat16 and contiguous along K")
    if bias is not None and (bias.dtype != torch.float32 or bias.shape != (N,) or not bias.is_contiguous()):
        raise KernelError("gemm_bf16: bias must be contiguous float32 [N]")
    if out is None:
        out = torch.empty(M, N, dtype=out_dtype, device=a.device)
    elif out.shape != (M, N) or out.dtype != out_dtype or out.stride(1) != 1:
        raise KernelError("gemm_bf16: out has the wrong shape or dtype")
    lib = library.core()
    _check(lib, lib.pico_gemm_bf16(_ptr(a), _ptr(w), _ptr(bias), _ptr(out), _DT[out_dtype], M, N, K,
                                   a.stride(0) if M > 1 else K, w.stride(0), out.stride(0) if M > 1 else N,
                                   _stream()))
    return out


EPI_BF16, EPI_F32, EPI_SWIGLU = 0, 1, 2
MAX_HEAD_DIM = 256          # the largest head size any attention kernel takes


# The weight-streaming kernel takes any number of rows in blocks of 64, each block reading the matrix
# again.  Up to 64 rows it always serves.  Up to SKINNY_MID_ROWS rows it serves matrices of at most
# SKINNY_MID_WEIGHT elements (the q/k/v and o projections of small models), which the caches hold
# between the blocks: a step of that size is bound by the host's launches, and this kernel costs the
# host less than half of a library call (8 against 19 us) and takes the GPU no longer (10.6 against
# 18.5 us at 128 rows of a 2,048 x 1,536 matrix, 19.5 against 18.9 us at 256).
SKINNY_ROWS, SKINNY_MID_ROWS, SKINNY_MID_WEIGHT = 64, 256, 1 << 22


def skinny_rows(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether a step of this many rows is one the weight-streaming kernel is meant for."""
    return a.dim() == 2 and (a.shape[0] <= SKINNY_ROWS or (a.shape[0] <= SKINNY_MID_ROWS and w.numel() <= SKINNY_MID_WEIGHT))


def skinny_ok(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the weight-streaming kernel takes these operands (few rows, 16-byte aligned rows)."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.dim() == 2
            and skinny_rows(a, w)
            and a.shape[1] % 8 == 0 and a.stride(1) == 1 and w.stride(1) == 1
            and (a.stride(0) % 8 == 0 or a.shape[0] == 1) and w.stride(0) % 8 == 0
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def gemm_skinny(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, epilogue: int = EPI_BF16,
                k_splits: int = 1) -> torch.Tensor:
    """a [M <= 64, K] x w [N, K]^T, both bfloat16.  EPI_BF16 -> bf16 [M, N]; EPI_F32 -> float32 [M, N], or with
    k_splits > 1 a stack [k_splits, M, N] of partial sums (bias in the first); EPI_SWIGLU (w = [gate; up])
    -> bf16 [M, N / 2] = silu(gate) * up."""
    _gpu(a, w, bias)
    M, K = a.shape
    N, K2 = w.shape
    if K != K2:
        raise KernelError(f"gemm: inner sizes differ ({K} and {K2})")
    if not skinny_ok(a, w):
        raise KernelError("gemm_skinny: operands must be bfloat16, few rows (skinny_ok), K a multiple of 8, rows 16-byte aligned")
    if bias is not None and (bias.dtype != torch.float32 or bias.shape != (N,) or not bias.is_contiguous()):
        raise KernelError("gemm_skinny: bias must be contiguous float32 [N]")
    if k_splits > 1 and epilogue != EPI_F32:
        raise KernelError("gemm_skinny: only the float32 epilogue can leave partial sums")
    if epilogue == EPI_F32:
        shape = (M, N) if k_splits == 1 else (k_splits, M, N)
        out = torch.empty(shape, dtype=torch.float32, device=a.device)
        ldo = N
    elif epilogue == EPI_SWIGLU:
        if N % 2:
            raise KernelError("gemm_skinny: SwiGLU needs an even number of weight rows")
        out = torch.empty(M, N // 2, dtype=torch.bfloat16, device=a.device)
        ldo = N // 2
    else:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=a.device)
        ldo = N
    lib = library.core()
    _check(lib, lib.pico_gemm_skinny(_ptr(a), a.stride(0) if M > 1 else K, _ptr(w), w.stride(0), _ptr(bias), _ptr(out),
                                     ldo, c_ll(M * N), epilogue, M, N, K, k_splits, _stream()))
    return out


@functools.lru_cache(maxsize=None)
def skinny_k_splits(N: int, K: int, max_splits: int = 8) -> int:
    """Into how many ranges of whole 256-wide steps the k of a small matrix is cut, each range a
    workgroup of its own that leaves a slab of partial sums: the cut with which the fullest compute
    unit reads least.  It depends on the matrix alone, never on the number of tokens."""
    return int(library.core().pico_gemm_skinny_k_splits(N, K, max_splits))


def _check_cache(k_cache: torch.Tensor, v_cache: torch.Tensor, nkv: int, d: int):
    """K pages [pages, nkv, P, d]; V pages [pages, nkv, d, P]."""
    if k_cache.dim() != 4 or v_cache.dim() != 4 or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("cache tensors must be contiguous and 4-dimensional")
    pages, h, P, dd = k_cache.shape
    if (h, dd) != (nkv, d) or tuple(v_cache.shape) != (pages, nkv, d, P) or v_cache.dtype != k_cache.dtype:
        raise KernelError(f"cache shapes {tuple(k_cache.shape)} / {tuple(v_cache.shape)} do not fit "
                          f"{nkv} kv heads of size {d}")
    return pages, P


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """cos and sin of position * inv_freq in float32: [T, len(inv_freq), 2].  Every layer of a step
    rotates by the same angles, so a step computes them once."""
    _gpu(positions, inv_freq)
    T = positions.numel()
    _i32(positions, "positions", T)
    if inv_freq.dtype != torch.float32 or inv_freq.dim() != 1 or not inv_freq.is_contiguous():
        raise KernelError("inv_freq must be contiguous float32")
    out = torch.empty(T, inv_freq.numel(), 2, dtype=torch.float32, device=positions.device)
    lib = library.core()
    _check(lib, lib.pico_rope_table(_ptr(positions), _ptr(inv_freq), _ptr(out), T, inv_freq.numel(), _stream()))
    return out


def _check_table(cos_sin: Optional[torch.Tensor], T: int, half: int) -> None:
    if half == 0:
        return
    if cos_sin is None or cos_sin.dtype != torch.float32 or cos_sin.shape != (T, half, 2) or not cos_sin.is_contiguous():
        raise KernelError(f"the table of cosines and sines must be contiguous float32 [{T}, {half}, 2]")


def rope_kv_store(qkv: torch.Tensor, cos_sin: Optional[torch.Tensor], slots: torch.Tensor,
                  k_cache: torch.Tensor, v_cache: torch.Tensor, nq: int, nkv: int, d: int, rotary_dim: int) -> None:
    """Rotate q (in place) and k by the angles of ``cos_sin`` (``rope_table``; None when rotary_dim
    is 0), write k and v of token t to slot ``slots[t]`` (page * page size + offset in the page;
    negative: nothing is stored)."""
    _gpu(qkv, cos_sin, slots, k_cache, v_cache)
    T = qkv.shape[0]
    if qkv.shape != (T, (nq + 2 * nkv) * d) or not qkv.is_contiguous():
        raise KernelError(f"qkv must be contiguous [T, {(nq + 2 * nkv) * d}], got {tuple(qkv.shape)}")
    pages, P = _check_cache(k_cache, v_cache, nkv, d)
    if k_cache.dtype != qkv.dtype:
        raise KernelError("cache and activations differ in dtype")
    _i32(slots, "slots", T)
    _check_table(cos_sin, T, rotary_dim // 2)
    lib = library.core()
    _check(lib, lib.pico_rope_kv_store(_ptr(qkv), _dt(qkv), _ptr(cos_sin) if rotary_dim else None, _ptr(slots),
                                       _ptr(k_cache), _ptr(v_cache), T, nq, nkv, d, rotary_dim, P, pages, _stream()))


def gemm_skinny_rope(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], cos_sin: torch.Tensor,
                     slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     nq: int, nkv: int, d: int) -> torch.Tensor:
    """The q/k/v projection of up to 64 tokens with bias, rotate-half encoding of q and k (over the
    whole head size) and the store of k and v at ``slots`` in one kernel; returns the encoded queries
    [M, nq * d].  w: [(nq + 2 nkv) * d, K] bfloat16, rows [q heads | k heads | v heads]."""
    _gpu(a, w, bias, cos_sin, slots, k_cache, v_cache)
    M, K = a.shape
    if w.shape != ((nq + 2 * nkv) * d, K):
        raise KernelError(f"gemm_skinny_rope: weight {tuple(w.shape)} is not [{(nq + 2 * nkv) * d}, {K}]")
    if not skinny_ok(a, w):
        raise KernelError("gemm_skinny_rope: operands must be bfloat16, few rows (skinny_ok), K a multiple of 8, rows 16-byte aligned")
    if bias is not None and (bias.dtype != torch.float32 or bias.shape != (w.shape[0],) or not bias.is_contiguous()):
        raise KernelError("gemm_skinny_rope: bias must be contiguous float32 [N]")
    pages, P = _check_cache(k_cache, v_cache, nkv, d)
    if k_cache.dtype != torch.bfloat16:
        raise KernelError("gemm_skinny_rope: the cache must be bfloat16")
    if d % 32 or P & (P - 1):
        raise KernelError("gemm_skinny_rope: head size must be a multiple of 32 and the page size a power of two")
    _i32(slots, "slots", M)
    _check_table(cos_sin, M, d // 2)
    q = torch.empty(M, nq * d, dtype=torch.bfloat16, device=a.device)
    lib = library.core()
    _check(lib, lib.pico_gemm_skinny_rope(_ptr(a), a.stride(0) if M > 1 else K, _ptr(w), w.stride(0), _ptr(bias), _ptr(q),
                                          nq * d, _ptr(cos_sin), _ptr(slots), _ptr(k_cache),
                                          _ptr(v_cache), M, K, nq, nkv, d, P, pages, _stream()))
    return q


# The norm in front of a projection inside the projection's launch: every workgroup norms the row itself, which
# pays for a single row (a decode step of one request: a launch of 4.5 us saved, some reading added).
SKINNY_NORM_ROWS, SKINNY_NORM_MAX_K, SKINNY_NORM_SLABS = 1, 4096, 8


def skinny_norm_ok(resid: torch.Tensor, delta: Optional[torch.Tensor], w: torch.Tensor) -> bool:
    """Whether ``gemm_skinny_norm`` / ``gemm_skinny_rope_norm`` take this residual stream [M, K], these partial
    sums (None, float32 [M, K] or float32 [S, M, K]) and this weight [N, K]."""
    if resid.dim() != 2 or resid.dtype != torch.float32 or not resid.is_contiguous():
        return False
    M, K = resid.shape
    if not (1 <= M <= SKINNY_NORM_ROWS and K % 64 == 0 and K <= SKINNY_NORM_MAX_K):
        return False
    if delta is not None and (delta.dtype != torch.float32 or not delta.is_contiguous() or tuple(delta.shape[-2:]) != (M, K)
                              or delta.dim() not in (2, 3) or (delta.dim() == 3 and delta.shape[0] > SKINNY_NORM_SLABS)):
        return False
    return (w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] == K and w.stride(1) == 1 and w.stride(0) % 8 == 0
            and w.data_ptr() % 16 == 0)


def _norm_args(resid, delta, norm_w, who):
    M, K = resid.shape
    if norm_w.dtype != torch.float32 or norm_w.shape != (K,) or not norm_w.is_contiguous():
        raise KernelError(f"{who}: norm weight must be float32 of shape [{K}]")
    slabs = 0 if delta is None else (delta.shape[0] if delta.dim() == 3 else 1)
    resid_out = torch.empty_like(resid)
    return M, K, slabs, resid_out


def gemm_skinny_norm(resid: torch.Tensor, delta: Optional[torch.Tensor], norm_w: torch.Tensor, eps: float,
                     w: torch.Tensor, epilogue: int = EPI_BF16):
    """epilogue(norm(resid + delta) w^T) for one row in one kernel; returns (out, resid + delta).
    The norm is RMSNorm with weight ``norm_w``; epilogues as ``gemm_skinny`` (EPI_F32: one slab)."""
    _gpu(resid, delta, norm_w, w)
    if not skinny_norm_ok(resid, delta, w):
        raise KernelError("gemm_skinny_norm: operands outside what the kernel takes (skinny_norm_ok)")
    M, K, slabs, resid_out = _norm_args(resid, delta, norm_w, "gemm_skinny_norm")
    N = w.shape[0]
    if epilogue == EPI_SWIGLU and N % 2:
        raise KernelError("gemm_skinny_norm: SwiGLU needs an even number of weight rows")
    n_out = N // 2 if epilogue == EPI_SWIGLU else N
    out = torch.empty(M, n_out, dtype=torch.float32 if epilogue == EPI_F32 else torch.bfloat16, device=resid.device)
    lib = library.core()
    _check(lib, lib.pico_gemm_skinny_norm(_ptr(resid), _ptr(delta), slabs, c_ll(M * K), _ptr(norm_w), c_float(eps),
                                          _ptr(resid_out), _ptr(w), w.stride(0), _ptr(out), n_out, epilogue, M, N, K,
                                          _stream()))
    return out, resid_out


def gemm_skinny_rope_norm(resid: torch.Tensor, delta: Optional[torch.Tensor], norm_w: torch.Tensor, eps: float,
                          w: torch.Tensor, bias: Optional[torch.Tensor], cos_sin: torch.Tensor, slots: torch.Tensor,
                          k_cache: torch.Tensor, v_cache: torch.Tensor, nq: int, nkv: int, d: int):
    """``gemm_skinny_rope`` on norm(resid + delta) for one row in one kernel; returns (encoded queries
    [M, nq * d], resid + delta)."""
    _gpu(resid, delta, norm_w, w, bias, cos_sin, slots, k_cache, v_cache)
    if not skinny_norm_ok(resid, delta, w):
        raise KernelError("gemm_skinny_rope_norm: operands outside what the kernel takes (skinny_norm_ok)")
    M, K, slabs, resid_out = _norm_args(resid, delta, norm_w, "gemm_skinny_rope_norm")
    if w.shape != ((nq + 2 * nkv) * d, K):
        raise KernelError(f"gemm_skinny_rope_norm: weight {tuple(w.shape)} is not [{(nq + 2 * nkv) * d}, {K}]")
    if bias is not None and (bias.dtype != torch.float32 or bias.shape != (w.shape[0],) or not bias.is_contiguous()):
        raise KernelError("gemm_skinny_rope_norm: bias must be contiguous float32 [N]")
    pages, P = _check_cache(k_cache, v_cache, nkv, d)
    if k_cache.dtype != torch.bfloat16:
        raise KernelError("gemm_skinny_rope_norm: the cache must be bfloat16")
    if d % 32 or P & (P - 1):
        raise KernelError("gemm_skinny_rope_norm: head size must be a multiple of 32 and the page size a power of two")
    _i32(slots, "slots", M)
    _check_table(cos_sin, M, d // 2)
    q = torch.empty(M, nq * d, dtype=torch.bfloat16, device=resid.device)
    lib = library.core()
    _check(lib, lib.pico_gemm_skinny_rope_norm(_ptr(resid), _ptr(delta), slabs, c_ll(M * K), _ptr(norm_w), c_float(eps),
                                               _ptr(resid_out), _ptr(w), w.stride(0), _ptr(bias), _ptr(q), nq * d,
                                               _ptr(cos_sin), _ptr(slots), _ptr(k_cache), _ptr(v_cache), M, K, nq, nkv, d,
                                               P, pages, _stream()))
    return q, resid_out


def paged_attention_ref(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                        positions: torch.Tensor, token_seq: torch.Tensor, nq: int, nkv: int, d: int,
                        scale: float, window: int = 0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q: [T, >= nq*d] (row stride free, heads first in the row); returns [T, nq*d]."""
    _gpu(q, k_cache, v_cache, block_table, positions, token_seq)
    T = q.shape[0]
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < nq * d:
        raise KernelError("q must be [T, >= nq*d] with unit stride along the row")
    pages, P = _check_cache(k_cache, v_cache, nkv, d)
    if k_cache.dtype != q.dtype:
        raise KernelError("cache and activations differ in dtype")
    _i32(positions, "positions", T)
    _i32(token_seq, "token_seq", T)
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous():
        raise KernelError("block_table must be contiguous int32 [sequences, pages]")
    if out is None:
        out = torch.empty(T, nq * d, dtype=q.dtype, device=q.device)
    elif out.shape != (T, nq * d) or out.dtype != q.dtype or not out.is_contiguous():
        raise KernelError("attention: out has the wrong shape or dtype")
    lib = library.core()
    _check(lib, lib.pico_paged_attention_ref(_ptr(q), q.stride(0) if T > 1 else q.shape[1], _dt(q), _ptr(k_cache),
                                             _ptr(v_cache), _ptr(block_table), block_table.shape[1],
                                             _ptr(positions), _ptr(token_seq), _ptr(out), T, nq, nkv, d, P, window,
                                             c_float(scale), pages, _stream()))
    return out


def sample_workspace(rows: int, device) -> torch.Tensor:
    """What ``sample`` needs beside its output for up to ``rows`` rows (partial results of its chain of launches)."""
    lib = library.core()
    lib.pico_sample_workspace_words.restype = ctypes.c_longlong
    return torch.empty(max(2, int(lib.pico_sample_workspace_words(rows))), dtype=torch.int32, device=device)


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor, u: torch.Tensor,
           out: Optional[torch.Tensor] = None, work: Optional[torch.Tensor] = None, top_p_rows: bool = True) -> torch.Tensor:
    """One token id per row of float32 logits; per-row temperature (0 = greedy), top_p and
    uniform number.  ``work``: ``sample_workspace`` for at least as many rows (made here if not given).
    ``top_p_rows=False``: the caller knows that no row has top_p < 1, and the launches that look for the
    threshold of such rows are left out (a top_p below 1 is then taken as 1)."""
    _gpu(logits, temperature, top_p, u, work)
    R, V = logits.shape
    if logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise KernelError("sample: logits must be float32 with unit stride along the vocabulary")
    for name, t in (("temperature", temperature), ("top_p", top_p), ("u", u)):
        if t.dtype != torch.float32 or t.numel() < R or not t.is_contiguous():
            raise KernelError(f"sample: {name} must be contiguous float32 with one entry per row")
    if out is None:
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
    elif out.dtype != torch.int32 or out.numel() < R or not out.is_contiguous():
        raise KernelError("sample: out must be contiguous int32 with one entry per row")
    lib = library.core()
    if work is None:
        work = sample_workspace(R, logits.device)
    else:
        lib.pico_sample_workspace_words.restype = ctypes.c_longlong
        if work.dtype != torch.int32 or not work.is_contiguous() or work.numel() < int(lib.pico_sample_workspace_words(R)) \
                or work.data_ptr() % 16:
            raise KernelError("sample: the workspace must come from sample_workspace for at least as many rows")
    _check(lib, lib.pico_sample(_ptr(logits), logits.stride(0) if R > 1 else V, R, V, _ptr(temperature),
                                _ptr(top_p), _ptr(u), _ptr(out), _ptr(work), int(bool(top_p_rows)), _stream()))
    return out


def argmax_workspace(rows: int, device) -> tuple:
    """What ``argmax`` needs beside its output: the maxima of the chunks of every row and where they are."""
    n = rows * int(library.core().pico_argmax_chunks())
    return torch.empty(n, dtype=torch.float32, device=device), torch.empty(n, dtype=torch.int32, device=device)


def argmax(logits: torch.Tensor, out: torch.Tensor, work: tuple) -> torch.Tensor:
    """The index of the first maximum of every row of float32 logits (what ``sample`` gives for
    temperature 0), several workgroups a row."""
    _gpu(logits, out, *work)
    R, V = logits.shape
    if logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise KernelError("argmax: logits must be float32 with unit stride along the vocabulary")
    if out.dtype != torch.int32 or out.numel() < R or not out.is_contiguous():
        raise KernelError("argmax: out must be contiguous int32 with one entry per row")
    lib = library.core()
    need = R * int(lib.pico_argmax_chunks())
    val, idx = work
    if val.dtype != torch.float32 or idx.dtype != torch.int32 or val.numel() < need or idx.numel() < need \
            or not val.is_contiguous() or not idx.is_contiguous():
        raise KernelError("argmax: the workspace must come from argmax_workspace for at least as many rows")
    _check(lib, lib.pico_argmax(_ptr(logits), logits.stride(0) if R > 1 else V, R, V, _ptr(val), _ptr(idx), _ptr(out), _stream()))
    return out
