"""The host's choices for the bfloat16 attention kernels (shape of the prefill workgroups, chunks of keys, splits of a
decode step): pure arithmetic on the shape of a batch, checked here without a GPU against the cases they were
measured on."""
import pytest

from pico_vllm_amd.ops.attention_fast import FastAttention


def plan(nq, nkv=2, d=128, window=0, cus=256):
    fa = FastAttention.__new__(FastAttention)            # no library: only the arithmetic
    fa.nq, fa.nkv, fa.d, fa.window, fa.cus = nq, nkv, d, window, cus
    return fa


def test_the_shape_of_the_prefill_workgroups():
    fa = plan(12)
    assert fa.prefill_teams([2048], [2048]) == 3            # a causal triangle: the longest tile decides
    assert fa.prefill_teams([512], [4096]) == 3             # few tiles
    assert fa.prefill_teams([1] * 8, [4000] * 8) == 3       # decode tokens inside a mixed step
    assert fa.prefill_teams([2048], [16384]) == 4           # many long, equal tiles that fill 128 queries
    assert fa.prefill_teams([32] * 64, [2032] * 64) == 1    # much work in short portions
    assert fa.prefill_teams([2048] * 2, [2048] * 2) == 6    # between few tiles and much work
    assert fa.prefill_teams([2048] * 4, [2048] * 4) == 4
    assert plan(28, 4).prefill_teams([2048], [2048]) == 6 and plan(40, 8).prefill_teams([2048], [2048]) == 4
    # a chip with fewer compute units has "much work" sooner
    assert plan(12, cus=64).prefill_teams([2048], [2048]) == 4


def test_when_the_keys_are_cut_into_chunks():
    fa = plan(12)
    assert fa.prefill_chunks([2048], [2048]) is None                    # no prefix: short tiles
    assert fa.prefill_chunks([2048] * 8, [4096] * 8) is None            # work for every compute unit
    assert fa.prefill_chunks([2048], [4096]) == (4, 2048, 2)
    assert fa.prefill_chunks([2048], [16384]) == (4, 8192, 2)           # 192 workgroups on 512 places
    assert fa.prefill_chunks([2048], [32768]) == (4, 4096, 8)
    assert fa.prefill_chunks([64], [8064]) == (1, 2048, 4)              # one 64-query tile per head
    assert fa.prefill_chunks([300], [1500]) is None                     # a short context
    assert plan(28, 4).prefill_chunks([2048], [16384]) is None          # 448 workgroups on 512 places
    assert plan(40, 8).prefill_chunks([2048], [32768]) == (4, 8192, 4)  # 640 workgroups: a second round nearly empty
    assert plan(12, window=100).prefill_chunks([64], [8064]) is None    # windows keep whole tiles
    assert plan(5, 5, 48).prefill_chunks([64], [8064]) is None          # head sizes that the 16-query kernel does not serve
    for new, ctx in (([2048], [16384]), ([64], [8064]), ([512, 300], [8192, 5000])):
        shape, chunk_len, most = fa.prefill_chunks(new, ctx)
        assert chunk_len % 128 == 0 and chunk_len & (chunk_len - 1) == 0      # whole LDS tiles; few recorded steps
        assert 2 <= -(-max(ctx) // chunk_len) <= most <= 16                   # room for the longest context's chunks


@pytest.mark.parametrize("num_seqs,context,want", [(1, 4096, 64), (8, 4096, 32), (64, 4096, 4), (1, 32768, 256), (8, 100, 2),
                                                   (3, 4096, 64)])
def test_the_splits_of_a_decode_step(num_seqs, context, want):
    # two workgroups a compute unit, no split shorter than a 64-key tile (two beyond 64 splits), at most 256; the
    # number of sequences counts as the power of two that a recorded step is padded to
    assert plan(12).num_splits(num_seqs, context) == want


def test_a_window_bounds_the_splits():
    assert plan(12, window=100).num_splits(1, 32768) == 3                # 131 keys at most


def test_the_filler_of_a_recorded_step_takes_no_part_in_the_plan():
    # a recorded step has a sequence of filler behind its portion (and single tokens, some of them empty rows, in front):
    # the plan is that of the real sequences, so that the step gets the shapes it would get unrecorded
    import numpy as np
    from types import SimpleNamespace
    fa = plan(12)

    def step(lens, contexts, filler):
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        return SimpleNamespace(num_seqs=len(lens), shared={},
                               host={"cu_seqlens": cu, "context_lens": np.asarray(contexts, dtype=np.int32), "filler": filler})

    for lens, contexts in (([2048], [16384]), ([300], [300]), ([1, 1, 1, 700], [50, 900, 0, 5000]), ([1, 1, 100], [4000, 4000, 2100])):
        alone = fa.plan(step(lens, contexts, 0))
        for fill in (0, 1, 13, 1900):
            assert fa.plan(step(lens + [fill], contexts + [fill], 1)) == alone, (lens, fill)
        assert alone[1] == sum(n == 1 for n in lens)                 # the single tokens that stand first
    # counted as a sequence, a long filler would change the shapes: that is what leaving it out avoids
    assert fa.plan(step([2048, 2048], [16384, 2048], 0)) != fa.plan(step([2048, 2048], [16384, 2048], 1))
