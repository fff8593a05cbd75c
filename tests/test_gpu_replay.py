"""Trace replay against the plain implementation: the same requests whole, with the last 32
tokens one by one, in portions of changing size, and mixed with other requests in a pool so small
that pages are used again; in 32-bit and in bfloat16."""
import functools
import json
import os
import random
import subprocess
import tempfile

import numpy as np
import pytest
import torch

import plain_qwen2 as P
from tiny_configs import CONFIGS, PAGE_SIZE, model_dir

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# What rounding does to a logit depends on the position: in float32 about 1e-6 of the logits' spread at most positions,
# ten times that at an ill-conditioned one (a residual stream that nearly cancels in front of a norm), for every
# arithmetic alike; in bfloat16 the same a few thousand times larger.  The yardstick is therefore taken per position, from
# DRAWS independent runs of the plain implementation with the rounding in question, against the plain implementation in
# float64:
#   float32   the plain implementation in float32 with its hidden and intermediate dimensions permuted
#             (plain_qwen2.permute_inner_dimensions: the same function, other orders of summation);
#   bfloat16  the plain implementation with every activation between the parts, and the probabilities in front of P.V,
#             rounded to bfloat16 with a subtractive dither (plain_qwen2.dithered_bf16: the error of each rounding is that
#             of a bfloat16 rounding, uniform within half a unit in the last place, but drawn anew in every run).
# Each run is a draw of that rounding's effect on every position; the engine's error is one more.  Where the error of a
# position is essentially one direction (the worst case for tails), the engine's rms error over the position's logits
# divided by the rms of the K draws there is Student's |t| with K degrees of freedom, and its largest error over the
# largest of the K draws' is |a| / max |b_k| of K + 1 normal numbers: FALSE_ALARM is the probability per position that an
# arithmetic exactly as noisy as the draws' would exceed the bounds (noise_bounds).  NOISIER says how much noisier than
# the draws the engine may be: it bounds the engine's rms error at the median position of a request of 16 tokens or
# more in units of the draws' (a statistic that no single position decides), and scales the two bounds per position.  float32: 1 (the CPU
# library's sums are longer runs than the engine's trees of radix 16; the engine measures 0.6 at the median position).
# bfloat16: 1.5 (the engine does not round exactly where the draws do: it rounds the unnormalised probabilities of an
# online softmax, and fused kernels skip roundings; it measures 0.9).
# No fixed fraction of the spread is asserted, and no ratio to one single draw: at an ill-conditioned position the ratio of
# two draws has no useful bound (3.8 was seen in float32 among 340 configurations, where the plain float32 run itself was
# 2.3e-5 of the spread off).
FALSE_ALARM = 1e-5
NOISIER = {"float32": 1.0, "bfloat16": 1.5}


def noise_draws(name, longest: int = 0) -> int:
    """How many runs make the yardstick: 32 for the tiny models, fewer where one run takes seconds (a large model, or
    a request of thousands of tokens)."""
    c = CONFIGS[name]
    params = c["num_hidden_layers"] * c["hidden_size"] * (3 * c["intermediate_size"] + 4 * c["hidden_size"]) + c["vocab_size"] * c["hidden_size"]
    return 32 if params <= 20e6 and longest <= 2048 else 16 if params <= 100e6 else 8


@functools.lru_cache(maxsize=None)
def noise_bounds(K: int):
    """(bound on a position's rms error in units of the K draws' rms there, bound on its largest error in units of the
    K draws' largest there) at FALSE_ALARM, for an arithmetic as noisy as the draws'."""
    from scipy import integrate, optimize, stats
    t_rms = float(stats.t.isf(FALSE_ALARM / 2, K))

    def exceed(T):       # P(|a| > T max_k |b_k|), a and the K b_k standard normal
        f = lambda m: K * (2 * stats.norm.cdf(m) - 1) ** (K - 1) * 2 * stats.norm.pdf(m) * 2 * stats.norm.sf(T * m)
        return integrate.quad(f, 0, 12, limit=200)[0]
    t_max = float(optimize.brentq(lambda T: exceed(T) - FALSE_ALARM, 0.5, 500))
    return t_rms, t_max


def make_requests(name, lengths, seed=0):
    V = CONFIGS[name]["vocab_size"]
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(V) for _ in range(n)] for i, n in enumerate(lengths)}


_plain_cache = {}


def plain_logits(name, tokens):
    """The plain implementation with every sum in float64: in float32 its own rounding is as large as the
    engine's (1.8e-5 of the spread at one position of one drawn configuration, measured against float64),
    and a comparison of the two could not tell whose error it sees."""
    key = (name, tuple(tokens))
    if key not in _plain_cache:
        if name not in _plain_cache:
            _plain_cache[name] = P.PlainModel(model_dir(name))
            _plain_cache[name, "float64"] = P.PlainModel(model_dir(name), torch.float64)
        _plain_cache[key] = _plain_cache[name, "float64"].logits(tokens).numpy()
    return _plain_cache[key]


def roundup(n, m=64):
    return -(-n // m) * m


class Trace:
    """Steps plus the bookkeeping of which (request, position) each output row is."""

    def __init__(self):
        self.steps, self.rows, self.fed, self.live_peak = [], {}, {}, 0

    def add(self, entries, end=()):
        """entries: list of (id, tokens, want)."""
        k = len(self.steps)
        rows = []
        for rid, toks, want in entries:
            base = self.fed.get(rid, 0)
            rows += [(rid, base + w) for w in want]
            self.fed[rid] = base + len(toks)
        self.live_peak = max(self.live_peak, sum(roundup(n) for n in self.fed.values()))
        self.steps.append({"step": k, "entries": [{"id": r, "tokens": t, "want": list(w)} for r, t, w in entries],
                           "end": list(end)})
        self.rows[k] = rows
        for rid in end:
            del self.fed[rid]


def whole(reqs):
    t = Trace()
    for rid, toks in reqs.items():
        t.add([(rid, toks, range(len(toks)))], end=[rid])
    return t


def tail_one_by_one(reqs, tail=32):
    t = Trace()
    for rid, toks in reqs.items():
        n = max(1, len(toks) - tail)
        t.add([(rid, toks[:n], range(n))])
        for i in range(n, len(toks)):
            t.add([(rid, toks[i:i + 1], [0])], end=[rid] if i == len(toks) - 1 else [])
        if n == len(toks):
            t.add([], end=[rid])
    return t


def portions(reqs, sizes=(13, 2, 7, 2, 5, 3, 16, 2, 17, 4, 31, 2, 8)):
    t = Trace()
    for rid, toks in reqs.items():
        i, k = 0, 0
        while i < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - i)
            k += 1
            t.add([(rid, toks[i:i + n], range(n))], end=[rid] if i + n == len(toks) else [])
            i += n
    return t


def mixed(reqs, seed=0, max_live=4, tail=32):
    """Up to four live requests; prompt portions of some beside single tokens of others; a request
    may sit a step out; finished requests end and later ones take their pages."""
    rng = random.Random(seed)
    t = Trace()
    waiting = list(reqs.items())
    live = {}                                   # id -> [tokens, fed]
    while waiting or live:
        while waiting and len(live) < max_live and rng.random() < 0.7:
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0]
        entries, end = [], []
        for rid, (toks, fed) in list(live.items()):
            if rng.random() < 0.2 and len(live) > 1:
                continue                        # left out of this step
            left = len(toks) - fed
            n = 1 if left <= tail else min(left - tail, rng.choice([2, 3, 5, 8, 13, 16, 17, 29]))
            if left - n == 1 and left > tail:
                n += 1
            entries.append((rid, toks[fed:fed + n], range(n)))
            live[rid][1] += n
            if live[rid][1] == len(toks):
                end.append(rid)
                del live[rid]
        if entries:
            t.add(entries, end)
    return t


def replay(name, dtype, trace, max_tokens=None):
    from pico_vllm_amd.engine.replay import TraceReplayer
    rp = TraceReplayer(model_dir(name), dtype, max_tokens or trace.live_peak, PAGE_SIZE[name])
    got = {}
    for step in trace.steps:
        out = rp.run_step(step)
        rows = trace.rows[step["step"]]
        assert (out is None) == (len(rows) == 0)
        if out is not None:
            assert out.shape == (len(rows), CONFIGS[name]["vocab_size"]) and out.dtype == np.float32
            for row, key in zip(out, rows):
                assert key not in got
                got[key] = row
    rp.runner.manager.check()
    pool = rp.runner.manager.groups[0].pool
    assert pool.num_free == pool.num_pages and not rp.live
    return got, pool


_noise_cache = {}


def rounding_noise(name, dtype, reqs):
    """For every request: (rms [positions], largest [positions], the number of runs) of the logit errors of ``noise_draws`` runs of
    the plain implementation with the rounding of ``dtype`` (see the top of the file) against the plain float64 run,
    over the draws and the vocabulary."""
    missing = [toks for toks in reqs.values() if (name, dtype, tuple(toks)) not in _noise_cache]
    if missing:
        plain_logits(name, missing[0])                                   # the models are read
        m32 = _plain_cache[name]
        gen = torch.Generator().manual_seed(1234)
        sq = {tuple(t): 0.0 for t in missing}
        mx = {tuple(t): 0.0 for t in missing}
        K = noise_draws(name, max(len(t) for t in reqs.values()))
        for _ in range(K):
            # float32: one permuted model at a time (it may be large); bfloat16: the model as it is, rounding drawn anew
            w = P.permute_inner_dimensions(m32.w, m32.cfg, gen) if dtype == "float32" else m32.w
            rnd = P._same if dtype == "float32" else P.dithered_bf16(gen)
            for toks in missing:
                with torch.no_grad():
                    e = P.forward(toks, w, m32.cfg, rnd=rnd).numpy().astype(np.float64) - plain_logits(name, toks)
                sq[tuple(toks)] = sq[tuple(toks)] + (e ** 2).mean(axis=1)
                mx[tuple(toks)] = np.maximum(mx[tuple(toks)], np.abs(e).max(axis=1))
            del w
        for toks in missing:
            _noise_cache[name, dtype, tuple(toks)] = (np.sqrt(sq[tuple(toks)] / K), mx[tuple(toks)], K)
    return {rid: _noise_cache[name, dtype, tuple(toks)] for rid, toks in reqs.items()}


def compare(name, dtype, reqs, got, label):
    noise = rounding_noise(name, dtype, reqs)
    f = NOISIER[dtype]
    worst = 0.0
    for rid, toks in reqs.items():
        ref = plain_logits(name, toks)
        spread = float(ref.std())
        mine = np.stack([got[(rid, p)] for p in range(len(toks))])
        assert np.isfinite(mine).all()
        err = np.abs(mine - ref).astype(np.float64)
        n_rms, n_max, draws = noise[rid]
        t_rms, t_max = noise_bounds(draws)
        pos_rms = np.sqrt((err ** 2).mean(axis=1))
        a, b = pos_rms / n_rms, err.max(axis=1) / n_max
        g = float(np.sqrt((pos_rms ** 2).mean() / (n_rms ** 2).mean()))
        worst = max(worst, float(a.max()))
        at = int(err.max(axis=1).argmax())
        print(f"[replay] {label} {name} {dtype} {rid}: of the draws' own error: a position's rms {np.median(a):.2f}x (median, bound {f:.2f}) "
              f"{a.max():.2f}x (worst, bound {f * t_rms:.2f}), a position's largest {b.max():.2f}x (bound {f * t_max:.2f}), rms over the "
              f"request {g:.2f}x; worst {err.max() / spread:.2e} of the spread, where the draws reach {n_max[at] / spread:.2e}")
        # no single position stands out: a fault at a page edge or at the start of a portion would
        assert a.max() <= f * t_rms, (f"{label} {name} {dtype}: request {rid}: the rms error of position {int(a.argmax())} is {a.max():.2f}x that "
                                      f"of the draws there (first position above {f * t_rms:.2f}: {int(np.argmax(a > f * t_rms))})")
        assert b.max() <= f * t_max, (f"{label} {name} {dtype}: request {rid}: the largest error of position {int(b.argmax())} is {b.max():.2f}x "
                                      f"the largest of the draws there (bound {f * t_max:.2f})")
        # and the engine is no noisier than it may be where nothing is special (of fewer than 16 positions the median is
        # hardly more than one position's draw, which the bounds above cover)
        assert len(toks) < 16 or np.median(a) <= f, (f"{label} {name} {dtype}: request {rid}: the median position's rms error is "
                                                     f"{np.median(a):.2f}x that of the draws (bound {f:.2f})")
    print(f"[replay] {label} {name} {dtype}: worst position {worst:.2f}x the draws' rms there")


LENGTHS = {"A": [70, 45, 100, 33, 64, 90], "B": [41, 97, 34, 80, 65, 50], "C": [50, 36, 81],
           # head sizes 24 and 40: no multiple of 16, so both precisions take the plain attention kernel
           "G": [70, 41, 97, 33, 64, 50], "H": [45, 100, 34, 80]}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "G", "H"])
def test_whole(name, dtype):
    reqs = make_requests(name, LENGTHS[name])
    got, _ = replay(name, dtype, whole(reqs))
    compare(name, dtype, reqs, got, "whole")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "G", "H"])
def test_last_32_tokens_one_by_one(name, dtype):
    reqs = make_requests(name, LENGTHS[name][:3], seed=1)
    got, _ = replay(name, dtype, tail_one_by_one(reqs))
    compare(name, dtype, reqs, got, "tail")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "G", "H"])
def test_portions_of_changing_size(name, dtype):
    reqs = make_requests(name, LENGTHS[name][:4], seed=2)
    got, _ = replay(name, dtype, portions(reqs))
    compare(name, dtype, reqs, got, "portions")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "G"])
def test_mixed_with_pages_used_again(name, dtype):
    reqs = make_requests(name, LENGTHS[name] + [57, 38], seed=3)
    trace = mixed(reqs, seed=4)
    assert max(len(s["entries"]) for s in trace.steps) >= 3
    got, pool = replay(name, dtype, trace)
    assert pool.reuse_count > 0 and pool.peak_used > pool.num_pages // 2      # pages were used again
    compare(name, dtype, reqs, got, "mixed")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", [f"R{i}" for i in range(10)] + ["D", "H"])
def test_configurations_drawn_at_random_whole_and_mixed(name, dtype):
    # sizes nobody picked by hand: whole requests, and the same requests mixed in a small pool
    reqs = make_requests(name, [40, 77, 33, 60], seed=7)
    got, _ = replay(name, dtype, whole(reqs))
    compare(name, dtype, reqs, got, "whole")
    t = mixed(reqs, seed=3, max_live=3)
    got, pool = replay(name, dtype, t)
    compare(name, dtype, reqs, got, "mixed")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompts_of_several_whole_key_tiles_at_head_size_96(dtype):
    # contexts beyond three whole 64-key tiles at a head size whose rows no workgroup's threads divide evenly:
    # whole, in portions (large ones after a long prefix) and with the tail decoded token by token
    reqs = make_requests("E", [260, 213], seed=11)
    got, _ = replay("E", dtype, whole(reqs))
    compare("E", dtype, reqs, got, "whole")
    got, _ = replay("E", dtype, portions(reqs, sizes=(70, 2, 130, 3, 40)))
    compare("E", dtype, reqs, got, "portions")
    got, _ = replay("E", dtype, tail_one_by_one(reqs, tail=8))
    compare("E", dtype, reqs, got, "tail")


def test_a_context_of_thousands_of_tokens_in_portions_of_2048(monkeypatch):
    # 6,200 tokens: whole in one step, and in portions of 2,048, 2,048, 2,048 and 52 with the last tokens one by
    # one.  Behind 4,096 tokens and more the bfloat16 attention cuts a portion's keys into chunks that run as workgroups
    # of their own (ops/attention_fast.py, prefill_chunks); a chunk lost or joined wrongly would move a row by a
    # quarter of its weight.
    from pico_vllm_amd.ops.attention_fast import FastAttention
    cuts = []
    chosen = FastAttention.prefill_chunks
    monkeypatch.setattr(FastAttention, "prefill_chunks", lambda self, n, c: cuts.append(chosen(self, n, c)) or cuts[-1])
    reqs = make_requests("F", [6200], seed=31)
    for dtype in ("bfloat16", "float32"):
        got, _ = replay("F", dtype, whole(reqs))
        compare("F", dtype, reqs, got, "long whole")
        del cuts[:]
        got, _ = replay("F", dtype, portions(reqs, sizes=(2048, 2048, 2048, 52, 1, 1, 1, 1)))
        compare("F", dtype, reqs, got, "long portions")
        if dtype == "bfloat16":
            assert any(c is not None for c in cuts), cuts          # the portions behind a long prefix were cut
    for key in [k for k in _plain_cache if k == "F" or (isinstance(k, tuple) and k[0] == "F")]:
        del _plain_cache[key]


@pytest.mark.parametrize("name", ["B", "C", "E"])
def test_twenty_requests_decoding_at_once(name, monkeypatch):
    # 20 requests of 33 to 200 tokens live at once, their last 32 tokens one by one in steps of 20 single tokens: from 17
    # sequences on a decode step cuts the contexts of all of them into pieces of one length (head sizes 32 and 96: the
    # kernel that reads the pages directly; 48: the one that stages tiles); the logits are the plain implementation's
    # within rounding, as with four live requests
    from pico_vllm_amd.engine.replay import TraceReplayer
    from pico_vllm_amd.ops.attention_fast import FastAttention
    cuts = []
    real = FastAttention.decode_cut
    monkeypatch.setattr(FastAttention, "decode_cut", lambda self, n, ns, dev: cuts.append(real(self, n, ns, dev)) or cuts[-1])
    lengths = [40, 150, 65, 97, 33, 180, 70, 129, 45, 200, 64, 90, 36, 160, 110, 50, 77, 140, 34, 100]
    reqs = make_requests(name, lengths, seed=9)
    tail = 32
    t = Trace()
    t.add([(rid, toks[:len(toks) - tail], range(len(toks) - tail)) for rid, toks in reqs.items()])
    for i in range(tail):
        t.add([(rid, toks[len(toks) - tail + i:len(toks) - tail + i + 1], [0]) for rid, toks in reqs.items()],
              end=list(reqs) if i == tail - 1 else [])
    rp = TraceReplayer(model_dir(name), "bfloat16", t.live_peak, PAGE_SIZE[name], max_live=24)
    got = {}
    for step in t.steps:
        out = rp.run_step(step)
        for row, key in zip(out, t.rows[step["step"]]):
            got[key] = row
    rp.runner.manager.check()
    assert sum(c is not None for c in cuts) >= tail, "the decode steps did not cut their contexts over all sequences"
    compare(name, "bfloat16", reqs, got, "twenty at once")


def test_forty_more_drawn_configurations_in_every_way_of_cutting():
    # a sweep over sizes nobody looked at, in both precisions, whole, with the tail token by token and mixed in a
    # small pool; it stops at the first configuration that fails and names it
    import tiny_configs as TC
    for seed in range(10, 50):
        name = f"S{seed}"
        TC.CONFIGS[name], TC.PAGE_SIZE[name] = TC.drawn(seed)
        for dtype in ("bfloat16", "float32"):
            reqs = make_requests(name, [40, 77, 33, 60], seed=seed)
            for label, trace in (("whole", whole(reqs)), ("tail", tail_one_by_one(reqs)),
                                 ("mixed", mixed(reqs, seed=seed, max_live=3))):
                got, _ = replay(name, dtype, trace)
                compare(name, dtype, reqs, got, f"sweep {label}")
        for key in [k for k in _plain_cache if k == name or (isinstance(k, tuple) and k[0] == name)]:
            del _plain_cache[key]           # the weights of forty models need not stay in memory


def test_float32_does_not_depend_on_the_cut_at_all():
    # every reduction of the 32-bit path has a fixed order per output element: bitwise equal
    reqs = make_requests("B", [77, 40], seed=5)
    a, _ = replay("B", "float32", whole(reqs))
    b, _ = replay("B", "float32", portions(reqs))
    c, _ = replay("B", "float32", mixed(reqs, seed=6))
    for key in a:
        assert np.array_equal(a[key], b[key]) and np.array_equal(a[key], c[key]), key


def test_long_decoding_and_first_tokens():
    # 300 tokens one by one from the very first token (position 0, a cache of one key) on
    reqs = make_requests("A", [300], seed=7)
    toks = reqs["r0"]
    t = Trace()
    for i in range(len(toks)):
        t.add([("r0", toks[i:i + 1], [0])], end=["r0"] if i == len(toks) - 1 else [])
    for dtype in ("float32", "bfloat16"):
        got, _ = replay("A", dtype, t)
        compare("A", dtype, reqs, got, "long decode")
        first = np.stack([got[("r0", p)] for p in range(4)])
        ref = plain_logits("A", toks)[:4]
        # (the first positions are among those that compare() has looked at one by one)
        _, n_max, draws = rounding_noise("A", dtype, reqs)["r0"]
        assert (np.abs(first - ref).max(axis=1) <= NOISIER[dtype] * noise_bounds(draws)[1] * n_max[:4]).all()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_model_without_layers_is_norm_times_output_matrix(dtype):
    # num_hidden_layers = 0 is a configuration the reader accepts: no cache group, no page, the final norm straight on
    # the embedding rows and the untied output matrix (the formula of test_plain.py's test of the same name)
    from pico_vllm_amd.engine.replay import TraceReplayer
    reqs = make_requests("Z", [40, 3, 21], seed=12)
    w = {k: v.double() for k, v in P.read_weights(model_dir("Z")).items()}
    E, g, W = w["model.embed_tokens.weight"], w["model.norm.weight"], w["lm_head.weight"]
    for trace in (whole(reqs), mixed(reqs, seed=2, tail=4)):
        rp = TraceReplayer(model_dir("Z"), dtype, trace.live_peak, PAGE_SIZE["Z"])
        assert not rp.runner.manager.groups
        for step in trace.steps:
            out = rp.run_step(step)
            for row, (rid, pos) in zip(out if out is not None else [], trace.rows[step["step"]]):
                x = E[reqs[rid][pos]]
                want = (x / torch.sqrt((x * x).mean() + CONFIGS["Z"]["rms_norm_eps"]) * g) @ W.T
                err = float((torch.from_numpy(row).double() - want).abs().max())
                assert err <= (2e-6 if dtype == "float32" else 2e-2) * float(want.abs().max()), (rid, pos, err)
        rp.runner.manager.check()
        assert not rp.live
    compare("Z", dtype, reqs, replay_rows(TraceReplayer(model_dir("Z"), dtype, 256, PAGE_SIZE["Z"]), whole(reqs)), "no layers")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_two_requests_that_share_the_pages_of_a_prefix_in_one_step(name, dtype):
    # ``fork_prefix`` lets a second request hold the whole pages of a first one's prefix (what an index of shared
    # prefixes would do; the reference adopts matched blocks, pico_vllm/cache.py:170-192).  Two block tables then name
    # the same pages in one step: a portion of one request beside single tokens and portions of the other.
    from pico_vllm_amd.engine.batch import SeqStep
    from pico_vllm_amd.engine.replay import TraceReplayer
    page = PAGE_SIZE[name]
    V = CONFIGS[name]["vocab_size"]
    rng = random.Random(21)
    shared = 5 * page
    first = [rng.randrange(V) for _ in range(shared + 30)]
    second = first[:shared] + [rng.randrange(V) for _ in range(41)]           # the same prefix, another continuation
    reqs = {"a": first, "b": second}
    rp = TraceReplayer(model_dir(name), dtype, 4 * 64 + 64, page)
    run, m = rp.runner, rp.runner.manager
    got = {}

    def step(entries):
        seqs = []
        for rid, lo, hi in entries:
            assert m.grow(rid, hi)
            seqs.append(SeqStep(rid, reqs[rid][lo:hi], list(range(hi - lo))))
        out = run.step(seqs).float().cpu().numpy()
        run.advance(seqs)
        at = 0
        for rid, lo, hi in entries:
            for p in range(lo, hi):
                got[rid, p] = out[at]
                at += 1

    assert m.add_request("a") and m.add_request("b")
    step([("a", 0, shared + 3)])                               # the prefix and a little more, alone
    m.fork_prefix("a", "b", shared)
    assert m.block_table("b")[:5] == m.block_table("a")[:5] and m.num_computed("b") == shared
    pool = m.groups[0].pool
    assert all(pool.ref_count(p) == 2 for p in m.block_table("a")[:5])
    step([("a", shared + 3, shared + 4), ("b", shared, shared + 17)])           # a single token beside a portion
    step([("b", shared + 17, shared + 19), ("a", shared + 4, shared + 20)])     # portions of both, the other way round
    step([("a", shared + 20, shared + 21), ("b", shared + 19, shared + 20)])    # two single tokens
    m.check()
    step([("a", shared + 21, shared + 30)])
    m.free_request("a")                                        # the shared pages stay: b still holds them
    assert all(pool.ref_count(p) == 1 for p in m.block_table("b")[:5])
    step([("b", shared + 20, shared + 41)])
    m.check()
    m.free_request("b")
    assert pool.num_free == pool.num_pages
    for rid in reqs:                                           # b's prefix positions were never run: a's rows stand for them
        for p in range(shared):
            got.setdefault((rid, p), got["a", p])
    compare(name, dtype, reqs, got, "shared prefix")


def replay_rows(rp, trace):
    """The rows a replayer gives for a trace, by (request, position)."""
    got = {}
    for step in trace.steps:
        out = rp.run_step(step)
        for row, key in zip(out if out is not None else [], trace.rows[step["step"]]):
            got[key] = row
    return got


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_program_itself_in_a_subprocess(dtype):
    reqs = make_requests("A", [40, 23, 50, 31, 36], seed=8)
    trace = mixed(reqs, seed=9, max_live=2)
    with tempfile.TemporaryDirectory() as out:
        inp = "\n".join(json.dumps(s) for s in trace.steps) + "\n"
        r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir("A"), "--dtype", dtype,
                            "--out", out, "--max-tokens", str(trace.live_peak)],
                           input=inp, capture_output=True, text=True, timeout=600)
        assert r.returncode == 0, r.stderr[-2000:]
        assert r.stdout.split("\n")[:-1] == [f"done {s['step']}" for s in trace.steps]
        got = {}
        for s in trace.steps:
            rows = trace.rows[s["step"]]
            path = os.path.join(out, f"{s['step']}.f32")
            assert os.path.exists(path) == bool(rows)
            if rows:
                a = np.fromfile(path, dtype="<f4").reshape(len(rows), -1)
                for row, key in zip(a, rows):
                    got[key] = row
        compare("A", dtype, reqs, got, "program")
        # from what the program wrote alone: every token landed on a page its request held, no page under two live
        # requests at once, and pages that ended requests gave back were used again by later ones
        with open(os.path.join(out, "pages.jsonl")) as f:
            log = [json.loads(line) for line in f]
        assert [e["step"] for e in log] == [s["step"] for s in trace.steps]
        owner, owners_ever, fed = {}, {}, {}
        for e, s in zip(log, trace.steps):
            assert [x["id"] for x in e["entries"]] == [x["id"] for x in s["entries"]]
            for x, y in zip(e["entries"], s["entries"]):
                assert x["first_position"] == fed.get(x["id"], 0)
                fed[x["id"]] = x["first_position"] + len(y["tokens"])
                (pages,) = x["pages"]                       # one group of layers
                lo, hi = x["first_position"] // PAGE_SIZE["A"], -(-fed[x["id"]] // PAGE_SIZE["A"])
                assert len(pages) == hi - lo and all(p >= 0 for p in pages)
                for p in pages:
                    assert owner.setdefault(p, x["id"]) == x["id"], f"page {p} under two live requests"
                    owners_ever.setdefault(p, set()).add(x["id"])
            for rid in e["end"]:
                owner = {p: o for p, o in owner.items() if o != rid}
        assert any(len(o) > 1 for o in owners_ever.values()), "no page was used again"
        assert len(owners_ever) <= trace.live_peak // PAGE_SIZE["A"]


def test_the_program_says_what_is_wrong_with_a_trace(tmp_path):
    import io
    from pico_vllm_amd.engine.batch import BatchError
    from pico_vllm_amd.engine.replay import TraceReplayer, main
    V = CONFIGS["A"]["vocab_size"]
    rp = TraceReplayer(model_dir("A"), "float32", max_tokens=64, page_size=PAGE_SIZE["A"])
    pool = rp.runner.manager.groups[0].pool
    out = rp.run_step({"step": 0, "entries": [{"id": "a", "tokens": [1, 2, 3], "want": [2]}], "end": []})
    assert out.shape == (1, V) and out.dtype == np.float32
    assert rp.run_step({"step": 1, "entries": [{"id": "a", "tokens": [4, 5]}]}) is None          # nothing wanted: no file
    with pytest.raises(RuntimeError, match="step 2: out of cache pages for request b"):
        rp.run_step({"step": 2, "entries": [{"id": "b", "tokens": [1] * 80, "want": []}], "end": []})
    with pytest.raises(BatchError, match="token id outside"):
        rp.run_step({"step": 3, "entries": [{"id": "a", "tokens": [V], "want": [0]}], "end": []})
    with pytest.raises(BatchError, match="wanted place 5"):
        rp.run_step({"step": 4, "entries": [{"id": "a", "tokens": [1, 2], "want": [5]}], "end": []})
    with pytest.raises(BatchError, match="stands twice"):
        rp.run_step({"step": 5, "entries": [{"id": "a", "tokens": [1], "want": [0]}, {"id": "a", "tokens": [2], "want": [0]}]})
    assert rp.run_step({"step": 6, "entries": [], "end": ["a", "b", "never seen"]}) is None
    rp.runner.manager.check()
    assert pool.num_free == pool.num_pages and not rp.live
    with pytest.raises(json.JSONDecodeError):
        main(["--model", model_dir("A"), "--dtype", "float32", "--out", str(tmp_path), "--max-tokens", "64"],
             stdin=io.StringIO("{\"step\": 0, \"entries\": [\n"), stdout=io.StringIO())
