"""The entry point that allocates nothing (csrc/no_alloc.h), called through ctypes as a caller outside this
package would: its output against that of the entry point with a workspace, on two calls in a row, the second
with a smaller input, so that what the first call left in the library's own memory must not matter."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _lib():
    from pico_vllm_amd.ops import library
    lib = ctypes.CDLL(library.build_library("pico_core", library.CORE_SOURCES))
    lib.pico_last_error.restype = ctypes.c_char_p
    return lib


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _both(lib, logits, rows, V):
    """(with the library's own memory, with a workspace) for the first ``rows`` rows and ``V`` columns."""
    ld = logits.stride(0)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = torch.full((rows,), -7, dtype=torch.int32, device=DEV)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = lib.pico_argmax_noalloc(_ptr(logits), ld, rows, V, _ptr(out), stream)
    assert rc == 0, lib.pico_last_error().decode()
    assert torch.cuda.memory_allocated() == before
    chunks = lib.pico_argmax_chunks()
    val = torch.empty(rows * chunks, dtype=torch.float32, device=DEV)
    idx = torch.empty(rows * chunks, dtype=torch.int32, device=DEV)
    want = torch.full((rows,), -9, dtype=torch.int32, device=DEV)
    rc = lib.pico_argmax(_ptr(logits), ld, rows, V, _ptr(val), _ptr(idx), _ptr(want), stream)
    assert rc == 0, lib.pico_last_error().decode()
    torch.cuda.synchronize()
    return out.cpu(), want.cpu()


def test_argmax_without_allocation_twice_in_a_row_the_second_smaller():
    lib = _lib()
    assert lib.pico_noalloc_init() == 0, lib.pico_last_error().decode()
    g = torch.Generator().manual_seed(3)
    big = torch.randn(37, 5003, generator=g)
    big[5, 4999] = 9.0
    big[6, 0] = 9.0
    big[7, 100] = big[7, 3000] = 11.0           # a tie: the lowest index wins
    logits = big.to(DEV)
    out, want = _both(lib, logits, 37, 5003)
    assert torch.equal(out, want)
    others = [r for r in range(37) if r != 7]           # (row 7 holds a tie, which torch's argmax need not break alike)
    assert torch.equal(out.long()[others], big.argmax(dim=1)[others])
    assert int(out[5]) == 4999 and int(out[6]) == 0 and int(out[7]) == 100
    # a smaller input straight after: fewer rows, fewer columns, so that every chunk boundary moves and the
    # entries of rows 5 .. 36 in the library's memory are stale
    small = torch.randn(5, 611, generator=g)
    small[2, 610] = 8.0
    logits2 = small.to(DEV)
    out2, want2 = _both(lib, logits2, 5, 611)
    assert torch.equal(out2, want2)
    assert torch.equal(out2.long(), small.argmax(dim=1))
    # and the first input again, a row stride wider than the row
    out3, want3 = _both(lib, logits, 20, 4000)
    assert torch.equal(out3, want3)
    others = [r for r in range(20) if r != 7]
    assert torch.equal(out3.long()[others], big[:20, :4000].argmax(dim=1)[others]) and int(out3[7]) == 100


def test_more_rows_than_the_library_holds_are_refused():
    lib = _lib()
    most = lib.pico_noalloc_max_rows()
    logits = torch.zeros(most + 1, 8, device=DEV)
    out = torch.zeros(most + 1, dtype=torch.int32, device=DEV)
    rc = lib.pico_argmax_noalloc(_ptr(logits), 8, most + 1, 8, _ptr(out), ctypes.c_void_p(0))
    assert rc != 0 and "holds" in lib.pico_last_error().decode()
    rc = lib.pico_argmax_noalloc(_ptr(logits), 8, most, 8, _ptr(out), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, lib.pico_last_error().decode()
    torch.cuda.synchronize()
    assert int(out[:most].abs().sum()) == 0
