"""Choice of the matrix-core attention kernels for the bfloat16 engine."""
from __future__ import annotations


def choose(nq: int, nkv: int, head_dim: int, window: int):
    """A callable (qkv, cache, block_table, ctx, scale) -> [T, nq*d], or None when the
    sizes are outside what the fast kernels take (the plain kernel serves them)."""
    return None
