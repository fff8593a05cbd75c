"""The step's flat arrays, built on the host from (request, tokens, wanted places): no GPU."""
import numpy as np
import pytest
import torch

from pico_vllm_amd.cache.manager import CacheManager
from pico_vllm_amd.engine.batch import BatchBuffers, BatchError, SeqStep, build_context
from pico_vllm_amd.parts.attention import kv_page_tensors
from pico_vllm_amd.parts.spec import CacheSpec

FULL = CacheSpec("paged_kv", page_tensors=kv_page_tensors(1, 16))
WIN = CacheSpec("paged_kv", window=12, page_tensors=kv_page_tensors(1, 16))
P, VOCAB = 8, 100


def setup(cached, new, max_seqs=6):
    """Requests r0, r1, ... with ``cached[i]`` tokens in the cache and room for ``new[i]`` more."""
    m = CacheManager({0: FULL, 1: WIN}, P, 64, max_seqs)
    for i, (c, n) in enumerate(zip(cached, new)):
        m.add_request(f"r{i}")
        if c:
            assert m.grow(f"r{i}", c)
            m.advance(f"r{i}", c)
        assert m.grow(f"r{i}", c + n)
    buf = BatchBuffers(torch.device("cpu"), max_tokens=64, max_seqs=max_seqs + 2, max_pages=8, num_groups=2)
    return m, buf


def test_a_mixed_step_is_laid_out_token_by_token():
    cached, new = [0, 21, 37, 5], [9, 1, 1, 4]
    m, buf = setup(cached, new)
    rng = np.random.default_rng(0)
    toks = [rng.integers(0, VOCAB, n).tolist() for n in new]
    seqs = [SeqStep("r0", toks[0], [0, 8]), SeqStep("r1", toks[1], [0]), SeqStep("r2", toks[2], []), SeqStep("r3", toks[3], [3])]
    ctx = build_context(seqs, m, buf, torch.bfloat16, VOCAB)
    T = sum(new)
    assert (ctx.num_tokens, ctx.num_seqs, ctx.max_new_tokens, ctx.max_context, ctx.all_decode) == (T, 4, 9, 38, False)
    assert ctx.token_ids.tolist() == sum(toks, [])
    assert ctx.positions.tolist() == [c + j for c, n in zip(cached, new) for j in range(n)]
    assert ctx.token_seq.tolist() == [b for b, n in enumerate(new) for _ in range(n)]
    assert ctx.cu_seqlens.tolist() == [0, 9, 10, 11, 15]
    assert ctx.context_lens.tolist() == [c + n for c, n in zip(cached, new)]
    assert ctx.want_rows.tolist() == [0, 8, 9, 14]
    assert ctx.state_slots.tolist() == [m.slot(f"r{i}") for i in range(4)] and len(set(ctx.state_slots.tolist())) == 4
    assert ctx.host["cu_seqlens"].tolist() == ctx.cu_seqlens.tolist()
    assert ctx.host["context_lens"].tolist() == ctx.context_lens.tolist()
    for g in range(2):
        width = ctx.block_tables[g].shape[1]
        assert width == -(-38 // P)                                   # as wide as the longest context needs
        for b in range(4):
            table = m.block_table(f"r{b}", g)
            need = -(-(cached[b] + new[b]) // P)
            assert ctx.block_tables[g][b].tolist() == table[:need] + [-1] * (width - need)
        # every new token's place: page * page size + offset (pico_vllm/cache.py:132-141)
        want = [m.token_slot(f"r{b}", cached[b] + j, g) for b in range(4) for j in range(new[b])]
        assert ctx.slot_mapping[g].tolist() == want
    # the window's group has given pages back (request r2 is at position 37, its window reaches back to 26)
    assert ctx.block_tables[1][2].tolist()[:3] == [-1, -1, -1] and min(ctx.block_tables[0][2].tolist()) >= 0


def test_rows_of_padding_and_a_sequence_of_filler():
    m, buf = setup([10, 3, 30], [1, 1, 1])
    seqs = [SeqStep(f"r{i}", [i + 1], [0]) for i in range(3)]
    ctx = build_context(seqs, m, buf, torch.bfloat16, VOCAB, pad_to=4)
    assert (ctx.num_tokens, ctx.num_seqs, ctx.all_decode) == (4, 4, True)
    assert ctx.context_lens.tolist() == [11, 4, 31, 0] and ctx.cu_seqlens.tolist() == [0, 1, 2, 3, 4]
    assert ctx.want_rows.tolist() == [0, 1, 2, 3]
    assert ctx.state_slots.tolist()[3] == m.slots.num_slots           # the spare slot that no request holds
    assert ctx.block_tables[0].shape == (4, buf.max_pages)            # a recorded step: the widest table
    assert ctx.block_tables[0][3].tolist() == [-1] * buf.max_pages and ctx.slot_mapping[0].tolist()[3] == -1
    # a prompt portion brought to 16 tokens by a second sequence of filler: positions from 0, nothing stored or wanted
    m, buf = setup([24], [5])
    ctx = build_context([SeqStep("r0", [1, 2, 3, 4, 5], [4])], m, buf, torch.bfloat16, VOCAB, pad_tokens_to=16)
    assert (ctx.num_tokens, ctx.num_seqs, ctx.all_decode) == (16, 2, False)
    assert ctx.positions.tolist() == [24, 25, 26, 27, 28] + list(range(11))
    assert ctx.token_seq.tolist() == [0] * 5 + [1] * 11 and ctx.cu_seqlens.tolist() == [0, 5, 16]
    assert ctx.context_lens.tolist() == [29, 11] and ctx.want_rows.tolist() == [4]
    assert ctx.slot_mapping[0].tolist()[5:] == [-1] * 11 and ctx.block_tables[0][1].tolist() == [-1] * buf.max_pages
    assert ctx.state_slots.tolist()[1] == m.slots.num_slots
    assert build_context([SeqStep("r0", [1] * 5, [])], m, buf, torch.bfloat16, VOCAB, pad_tokens_to=5).num_tokens == 5


def test_single_tokens_and_one_portion_padded_both_ways():
    # three requests with one token each, padded to four rows, in front of a portion of 5 tokens padded to 16
    m, buf = setup([10, 3, 30, 24], [1, 1, 1, 5])
    seqs = [SeqStep(f"r{i}", [i + 1], [0]) for i in range(3)] + [SeqStep("r3", [1, 2, 3, 4, 5], [4])]
    ctx = build_context(seqs, m, buf, torch.bfloat16, VOCAB, pad_to=4, pad_tokens_to=16)
    assert (ctx.num_tokens, ctx.num_seqs, ctx.all_decode, ctx.max_new_tokens) == (20, 6, False, 5)
    assert ctx.token_ids.tolist() == [1, 2, 3, 0, 1, 2, 3, 4, 5] + [0] * 11
    assert ctx.positions.tolist() == [10, 3, 30, 0, 24, 25, 26, 27, 28] + list(range(11))
    assert ctx.token_seq.tolist() == [0, 1, 2, 3] + [4] * 5 + [5] * 11
    assert ctx.cu_seqlens.tolist() == [0, 1, 2, 3, 4, 9, 20]
    assert ctx.context_lens.tolist() == [11, 4, 31, 0, 29, 11]
    assert ctx.want_rows.tolist() == [0, 1, 2, 3, 8]                  # the empty row is wanted like the real ones
    spare = m.slots.num_slots
    assert ctx.state_slots.tolist() == [m.slot("r0"), m.slot("r1"), m.slot("r2"), spare, m.slot("r3"), spare]
    for g in range(2):
        assert ctx.block_tables[g].shape == (6, buf.max_pages)
        assert ctx.block_tables[g][3].tolist() == [-1] * buf.max_pages == ctx.block_tables[g][5].tolist()
        want = [m.token_slot(f"r{i}", c, g) for i, c in enumerate([10, 3, 30])] + [-1] \
            + [m.token_slot("r3", 24 + j, g) for j in range(5)] + [-1] * 11
        assert ctx.slot_mapping[g].tolist() == want
        assert ctx.block_tables[g][4].tolist()[:4] == m.block_table("r3", g)[:4]
    assert ctx.host["cu_seqlens"].tolist() == ctx.cu_seqlens.tolist() and ctx.host["context_lens"].tolist() == ctx.context_lens.tolist()
    # no single token at all is allowed too (rows of padding only), and so is a full house
    ctx = build_context(seqs[3:], m, buf, torch.bfloat16, VOCAB, pad_to=2, pad_tokens_to=8)
    assert ctx.cu_seqlens.tolist() == [0, 1, 2, 7, 10] and ctx.context_lens.tolist() == [0, 0, 29, 3] and ctx.want_rows.tolist() == [0, 1, 6]
    ctx = build_context(seqs, m, buf, torch.bfloat16, VOCAB, pad_to=3, pad_tokens_to=5)
    assert ctx.cu_seqlens.tolist() == [0, 1, 2, 3, 8, 8] and ctx.want_rows.tolist() == [0, 1, 2, 7]
    # a step after it that is not padded leaves nothing of it behind
    ctx = build_context(seqs, m, buf, torch.bfloat16, VOCAB)
    assert ctx.cu_seqlens.tolist() == [0, 1, 2, 3, 8] and ctx.slot_mapping[0].tolist()[3:] == [m.token_slot("r3", 24 + j, 0) for j in range(5)]


def test_what_a_step_refuses():
    m, buf = setup([10, 3], [4, 1])
    a, b = SeqStep("r0", [1, 2, 3, 4], [3]), SeqStep("r1", [5], [0])

    def refused(seqs, message, **pad):
        with pytest.raises(BatchError, match=message):
            build_context(seqs, m, buf, torch.bfloat16, VOCAB, **pad)

    refused([], "at least one sequence")
    refused([a, b], "followed by one prompt portion", pad_to=4, pad_tokens_to=16)        # the portion stands last
    m.add_request("r2"); m.grow("r2", 1)
    refused([b, SeqStep("r2", [1], [0]), a], "followed by one prompt portion", pad_to=1, pad_tokens_to=16)   # more single tokens than rows
    refused([b, a], "more than the 2", pad_to=2, pad_tokens_to=2)
    refused([a, SeqStep("r1", [], [])], "at least one token")
    refused([a, SeqStep("r0", [9], [0])], "stands twice")
    refused([a], "more than the 2", pad_tokens_to=2)
    refused([SeqStep("r0", [1, 2, VOCAB, 4], [])], "token id outside")
    refused([SeqStep("r0", [1, -1, 3, 4], [])], "token id outside")
    refused([SeqStep("r1", [VOCAB], [0])], "token id outside")
    refused([SeqStep("r0", [1, 2, 3, 4], [4])], "wanted place 4 is outside its 4 tokens")
    refused([SeqStep("r1", [5], [1])], "wanted place 1 is outside its 1 tokens")
    refused([a, b], "exceeds the buffers", pad_to=buf.max_seqs + 1)
    small = BatchBuffers(torch.device("cpu"), max_tokens=64, max_seqs=4, max_pages=1, num_groups=2)
    with pytest.raises(BatchError, match="needs 2 pages, the buffers hold 1"):
        build_context([a], m, small, torch.bfloat16, VOCAB)
    build_context([a, b], m, buf, torch.bfloat16, VOCAB)              # and the step itself is fine


def test_the_sizes_at_which_prompt_steps_are_recorded():
    from pico_vllm_amd.engine.step import prompt_sizes
    assert prompt_sizes(2048) == [16, 32, 64, 128, 192, 256, 320, 384, 448, 512, 640, 768, 896, 1024, 1280, 1536, 1792, 2048]
    assert prompt_sizes(24) == [16, 24] and prompt_sizes(300) == [16, 32, 64, 128, 192, 256, 300] and prompt_sizes(8) == [8]
    assert prompt_sizes(1) == [] and prompt_sizes(16) == [16] and prompt_sizes(64) == [16, 32, 64]
    for most in (24, 300, 2048, 5000):
        sizes = prompt_sizes(most)
        assert sizes == sorted(set(sizes)) and sizes[-1] == most
        for n in range(2, most + 1):                     # every portion finds a size, with little filler
            size = next(s for s in sizes if s >= n)
            filler = size - n
            assert filler < 16 if n < 16 else 2 * filler < size if n < 128 else 3 * filler <= size if n < 512 else 5 * filler <= size
