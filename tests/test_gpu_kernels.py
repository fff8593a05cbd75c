"""Each HIP kernel alone against a plain float32 reference of the same op, at sizes other than
the engine's (odd widths, head sizes in steps of 16, page sizes 8..64)."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_qwen2 as P
from gpu_util import DEV, DTYPES, flat_batch, paged_cache, tol
from test_plain import REFERENCE_CASES

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    from pico_vllm_amd.ops import kernels
    return kernels


def close(a, b, dtype, scale=1.0):
    rtol, atol = tol(dtype)
    a, b = a.float().cpu(), b.float().cpu()
    assert a.shape == b.shape
    err = (a - b).abs()
    bound = atol * scale + rtol * b.abs()
    assert bool((err <= bound).all()), f"max err {float(err.max()):.3e} (bound {float(bound.min()):.3e}..)"


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding(K, dtype):
    table = torch.randn(301, 136).to(dtype)
    ids = torch.tensor([0, 300, 5, 5, 17], dtype=torch.int32)
    out = K.embedding(table.to(DEV), ids.to(DEV))
    assert out.dtype == torch.float32
    assert torch.equal(out.cpu(), table.float()[ids.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [64, 136, 1536, 5000])
def test_add_rmsnorm(K, dtype, H):
    T, eps = 7, 1e-5
    resid = torch.randn(T, H) * 3
    delta = (torch.randn(T, H)).to(dtype)
    w = 1 + 0.1 * torch.randn(H)
    want_sum = resid + delta.float()
    r = resid.clone().to(DEV)
    out = K.add_rmsnorm(r, delta.to(DEV), w.to(DEV), eps, dtype)
    close(r, want_sum, torch.float32)                                   # the residual stream is float32
    close(out, P.rms_norm(want_sum, w, eps), dtype)
    # no delta: the stream is untouched
    r2 = resid.clone().to(DEV)
    out = K.add_rmsnorm(r2, None, w.to(DEV), eps, dtype)
    assert torch.equal(r2.cpu(), resid)
    close(out, P.rms_norm(resid, w, eps), dtype)
    # wanted rows only: the stream is untouched, rows are gathered
    rows = torch.tensor([6, 0, 3], dtype=torch.int32)
    r3 = resid.clone().to(DEV)
    out = K.add_rmsnorm(r3, delta.to(DEV), w.to(DEV), eps, dtype, rows=rows.to(DEV))
    assert torch.equal(r3.cpu(), resid)
    close(out, P.rms_norm(want_sum[rows.long()], w, eps), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_residual_add(K, dtype):
    # the add without a norm, for an arrangement of parts that ends on an add
    resid, delta = torch.randn(7, 136) * 3, torch.randn(7, 136).to(dtype)
    r = resid.clone().to(DEV)
    assert K.residual_add(r, delta.to(DEV)) is r
    assert torch.equal(r.cpu(), resid + delta.float())


def test_rmsnorm_eps_is_inside_the_root(K):
    x = torch.full((1, 64), 1e-4)
    out = K.add_rmsnorm(x.to(DEV), None, torch.ones(64, device=DEV), 1e-2, torch.float32)
    close(out, x / math.sqrt(1e-8 + 1e-2), torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu(K, dtype):
    gu = (torch.randn(5, 2 * 172) * 2).to(dtype)
    close(K.swiglu(gu.to(DEV)), P.swiglu(gu), dtype)
    g = gu[:, :172].float()
    close(K.swiglu(torch.cat([gu[:, :172], torch.ones(5, 172).to(dtype)], -1).to(DEV)), F.silu(g), dtype)
    # halves that are multiples of 8 take the kernel with 16-byte loads in bfloat16
    for T, I in ((3, 8), (70, 320), (33, 8960)):
        gu = (torch.randn(T, 2 * I) * 2).to(dtype)
        close(K.swiglu(gu.to(DEV)), P.swiglu(gu), dtype)


@pytest.mark.parametrize("M,N,K_", [(1, 301, 136), (5, 64, 172), (70, 130, 64), (130, 17, 33)])
def test_gemm_f32(K, M, N, K_):
    a, w, b = torch.randn(M, K_), torch.randn(N, K_), torch.randn(N)
    out = K.gemm_f32(a.to(DEV), w.to(DEV), b.to(DEV))
    want = a.double() @ w.double().T + b.double()
    assert torch.allclose(out.cpu().double(), want, rtol=1e-5, atol=1e-4)
    # a row's result does not depend on the other rows of the call: bitwise
    one = K.gemm_f32(a[M // 2:M // 2 + 1].to(DEV), w.to(DEV), b.to(DEV))
    assert torch.equal(one.cpu()[0], out.cpu()[M // 2])
    # strided rows (a view into a wider buffer), bfloat16 activations
    wide = torch.randn(M, K_ + 24).to(DEV)
    out2 = K.gemm_f32(wide[:, 8:8 + K_], w.to(DEV))
    assert torch.allclose(out2.cpu().double(), wide[:, 8:8 + K_].cpu().double() @ w.double().T, rtol=1e-5, atol=1e-4)
    ab = a.to(torch.bfloat16)
    out3 = K.gemm_f32(ab.to(DEV), w.to(DEV))
    assert torch.allclose(out3.cpu().double(), ab.double() @ w.double().T, rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("K_", [64, 1000, 1536, 3584, 5120, 8960, 18944, 27648])
def test_gemm_f32_rounding_does_not_grow_with_the_inner_size(K, K_):
    # The sums are trees of radix 16 with L = ceil(log16 K) levels (at most 4).  An addition rounds its partial sum
    # by up to eps = 2^-24 of it, 0.58 eps rms; the partial sums of a group of 16 have on average 8.5 / 16 of the
    # group's mean square, and the groups' mean squares add up to the result's (random signs): every level adds
    # (0.58 eps)^2 * 8.5 to the relative mean square error, so rms error <= 0.58 sqrt(8.5 L) eps = 1.69 sqrt(L) eps
    # of the result's rms at ANY inner size.  One running sum over K terms would give 0.2 sqrt(K) eps: 19 eps at 8,960.
    g = torch.Generator().manual_seed(K_)
    a, w = torch.randn(8, K_, generator=g), torch.randn(96, K_, generator=g)
    want = a.double() @ w.double().T
    err = K.gemm_f32(a.to(DEV), w.to(DEV)).cpu().double() - want
    eps, levels = 2.0 ** -24, min(4, math.ceil(math.log(K_, 16)))
    rms = float(err.pow(2).mean().sqrt() / want.pow(2).mean().sqrt())
    print(f"[gemm_f32] K={K_}: rms error {rms / eps:.2f} eps, bound {1.69 * math.sqrt(levels):.2f} eps")
    assert rms <= 1.69 * math.sqrt(levels) * eps
    assert float(err.abs().max() / want.pow(2).mean().sqrt()) <= 5 * 1.69 * math.sqrt(levels) * eps     # 768 outputs: five sigma


@pytest.mark.parametrize("M,N,K_", [(1, 301, 136), (3, 256, 64), (8, 384, 192), (33, 130, 172), (64, 1000, 1536),
                                   (100, 77, 40)])
@pytest.mark.parametrize("out_dtype", DTYPES)
def test_gemm_bf16(K, M, N, K_, out_dtype):
    a, w, b = torch.randn(M, K_).bfloat16(), torch.randn(N, K_).bfloat16(), torch.randn(N)
    out = K.gemm_bf16(a.to(DEV), w.to(DEV), b.to(DEV), out_dtype)
    want = a.double() @ w.double().T + b.double()
    assert out.dtype == out_dtype
    if out_dtype == torch.float32:       # exact products, float32 accumulation
        assert torch.allclose(out.cpu().double(), want, rtol=1e-4, atol=1e-3 * math.sqrt(K_))
    else:
        assert torch.allclose(out.cpu().double(), want, rtol=1e-2, atol=1e-2 * math.sqrt(K_))
    out_nb = K.gemm_bf16(a.to(DEV), w.to(DEV), None, torch.float32)
    assert torch.allclose(out_nb.cpu().double(), a.double() @ w.double().T, rtol=1e-4, atol=1e-3 * math.sqrt(K_))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,rot,Pg", [(4, 1, 16, 16, 16), (6, 3, 32, 32, 8), (5, 5, 48, 48, 16), (2, 2, 64, 32, 32),
                                            (12, 2, 128, 128, 16), (3, 1, 24, 8, 16), (28, 4, 128, 128, 16),
                                            (6, 2, 24, 24, 8), (5, 1, 40, 40, 16), (4, 4, 72, 72, 8), (2, 1, 250, 250, 16)])
def test_rope_and_cache_store(K, dtype, nq, nkv, d, rot, Pg):
    theta = 10000.0
    new_lens, prefix_lens = [5, 1, 9], [14, 33, 0]          # 14..18 crosses a page edge of 16 (store_kvcache.py:107-118)
    pos, seq = flat_batch(new_lens, prefix_lens)
    T = int(pos.numel())
    qkv = torch.randn(T, (nq + 2 * nkv) * d).to(dtype)
    num_pages = 12 * 16 // Pg
    kc = torch.full((num_pages, nkv, Pg, d), 7.0, dtype=dtype, device=DEV)
    vc = torch.full((num_pages, nkv, d, Pg), 7.0, dtype=dtype, device=DEV)
    g = torch.Generator().manual_seed(0)
    perm = torch.randperm(num_pages, generator=g).tolist()
    maxp = max(-(-(n + p) // Pg) for n, p in zip(new_lens, prefix_lens))
    bt = torch.full((3, maxp), -1, dtype=torch.int32)
    for b, (n, p) in enumerate(zip(new_lens, prefix_lens)):
        for j in range(-(-(n + p) // Pg)):
            bt[b, j] = perm.pop()
    inv = (1.0 / (theta ** (torch.arange(0, rot, 2).float() / rot))).to(DEV)
    x = qkv.clone().to(DEV)
    slots = torch.tensor([int(bt[int(b), int(p) // Pg]) * Pg + int(p) % Pg for b, p in zip(seq, pos)],
                         dtype=torch.int32, device=DEV)
    slots[3] = -1                                           # a padding row: rotated, but nothing of it is stored
    table = K.rope_table(pos.to(DEV), inv)
    want_cos, want_sin = P.rope_tables(pos.cpu(), rot, theta)
    assert torch.allclose(table[..., 0].cpu(), want_cos[:, :rot // 2], atol=2e-6)
    assert torch.allclose(table[..., 1].cpu(), want_sin[:, :rot // 2], atol=2e-6)
    K.rope_kv_store(x, table, slots, kc, vc, nq, nkv, d, rot)
    # reference
    q, k, v = P.split_qkv(qkv.float(), nq, nkv, d)
    cos, sin = P.rope_tables(pos.cpu(), rot, theta)

    def rot_part(t):
        return torch.cat([P.apply_rope(t[..., :rot], cos, sin), t[..., rot:]], dim=-1)
    qr, kr = rot_part(q), rot_part(k)
    close(x[:, :nq * d].reshape(T, nq, d), qr, dtype, scale=3)
    assert torch.equal(x[:, nq * d:].cpu(), qkv[:, nq * d:])          # k and v in the activation buffer are untouched
    want_k = torch.full((num_pages, nkv, Pg, d), 7.0)
    want_v = torch.full((num_pages, nkv, d, Pg), 7.0)
    for t in range(T):
        if t == 3:
            continue
        b, p = int(seq[t]), int(pos[t])
        page, off = int(bt[b, p // Pg]), p % Pg
        want_k[page, :, off, :] = kr[t]
        want_v[page, :, :, off] = v[t]
    close(kc, want_k, dtype, scale=3)          # also: every slot that no token owns still holds 7
    close(vc, want_v, dtype, scale=3)


def _attn_case(K, dtype, new_lens, prefix_lens, nq, nkv, d, Pg, window=0, seed=0, boost=None):
    g = torch.Generator().manual_seed(seed)
    totals = [n + p for n, p in zip(new_lens, prefix_lens)]
    ks = [(torch.randn(N, nkv, d, generator=g)).to(dtype).float() for N in totals]
    vs = [(torch.randn(N, nkv, d, generator=g)).to(dtype).float() for N in totals]
    qs = [(torch.randn(n, nq, d, generator=g)).to(dtype).float() for n in new_lens]
    if boost is not None:
        boost(qs, ks, vs)
    num_pages = sum(-(-N // Pg) for N in totals) + 3
    kc, vc, bt = paged_cache(ks, vs, Pg, num_pages, dtype, seed)
    pos, seq = flat_batch(new_lens, prefix_lens)
    q = torch.cat(qs, 0).reshape(-1, nq * d).to(DEV, dtype)
    out = K.paged_attention_ref(q, kc, vc, bt, pos, seq, nq, nkv, d, 1.0 / math.sqrt(d), window)
    want = torch.cat([P.causal_attention(qb, kb, vb, q_positions=torch.arange(p, p + n), window=window)
                      for qb, kb, vb, n, p in zip(qs, ks, vs, new_lens, prefix_lens)], 0)
    return out.reshape(-1, nq, d), want


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", range(len(REFERENCE_CASES)))
def test_plain_attention_kernel_on_the_reference_cases(K, dtype, case):
    new_lens, prefix_lens = REFERENCE_CASES[case]
    out, want = _attn_case(K, dtype, new_lens, prefix_lens, 12, 2, 128, 16, seed=case)
    close(out, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,Pg", [(4, 1, 16, 16), (6, 3, 32, 8), (5, 5, 48, 16), (3, 1, 80, 32), (8, 2, 256, 64),
                                        (2, 2, 112, 8)])
def test_plain_attention_kernel_other_sizes(K, dtype, nq, nkv, d, Pg):
    out, want = _attn_case(K, dtype, [7, 1, 30, 2], [0, 70, 45, 129], nq, nkv, d, Pg, seed=3)
    close(out, want, dtype)


# Head sizes that are no multiple of 16 (the configuration allows any even one): the matrix-core kernels do not take
# them, so both engine precisions go through this kernel there.
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Pg", [8, 16])
@pytest.mark.parametrize("nq,nkv,d", [(6, 2, 24), (5, 1, 40), (4, 4, 72), (3, 1, 2), (2, 1, 250)])
@pytest.mark.parametrize("case", range(len(REFERENCE_CASES)))
def test_plain_attention_kernel_at_head_sizes_between_the_steps_of_16(K, dtype, Pg, nq, nkv, d, case):
    # the reference's own (new, prefix) cases (tests/test_prefill_paged_attn.py:183-260), with grouped heads
    new_lens, prefix_lens = REFERENCE_CASES[case]
    out, want = _attn_case(K, dtype, new_lens, prefix_lens, nq, nkv, d, Pg, seed=case + d)
    close(out, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("d", [24, 40, 72])
def test_attention_finds_one_far_key_at_head_sizes_between_the_steps_of_16(K, dtype, d):
    # as below: a dropped key, page or tail of the head dimension would show
    for far in (0, 7, 8, 63, 64, 301):
        def boost(qs, ks, vs, far=far):
            ks[0][far] = qs[0][-1, 0:1, :] * 8.0          # (a short head: a large factor makes the score stand out)
            vs[0][far] = 100.0
            vs[0][far][..., d - 1] = -100.0          # the last head dimension carries a value of its own
        out, want = _attn_case(K, dtype, [3], [330], 3, 1, d, 8, seed=far, boost=boost)
        assert float(want[-1, 0, :d - 1].mean()) > 50 and float(want[-1, 0, d - 1]) < -50
        close(out, want, dtype, scale=100)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_finds_one_far_key_among_hundreds(K, dtype):
    # one key far back gets a large score; its value dominates the output.  A kernel that drops a
    # block of keys, a page or a boundary position fails here, whereas with random scores the loss
    # of one key among 600 would hide under the tolerance.
    for far in (0, 15, 16, 63, 64, 200, 511):
        def boost(qs, ks, vs, far=far):
            ks[0][far] = qs[0][-1, 0:1, :] * 2.0          # same direction as the last query of head 0
            vs[0][far] = 100.0
        out, want = _attn_case(K, dtype, [3], [597], 2, 1, 64, 16, seed=far, boost=boost)
        assert float(want[-1, 0].mean()) > 50
        close(out, want, dtype, scale=100)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 5, 16, 17, 64, 100])
def test_attention_window_edge(K, dtype, window):
    # the key just outside the window carries a huge value: reading it would show at once
    def boost(qs, ks, vs):
        n = ks[0].shape[0]
        last = n - 1
        if last - window >= 0:
            vs[0][last - window] = 1000.0
    out, want = _attn_case(K, dtype, [4, 1], [126, 40], 4, 2, 32, 16, window=window, seed=window, boost=boost)
    assert float(want[3].abs().max()) < 50
    close(out, want, dtype)


@pytest.mark.parametrize("nq,nkv,d,rot", [(8, 1, 16, 16), (12, 2, 128, 128), (2, 2, 64, 32)])
def test_rotation_gives_a_token_the_same_bits_whatever_stands_beside_it(K, nq, nkv, d, rot):
    # seven tokens alone take the kernel for few tokens, the same seven among twenty the one with 16-byte accesses: the
    # same rotated queries and the same keys and values in the cache, bit for bit (a step padded for a recorded graph
    # must not differ from the step unpadded)
    g = torch.Generator().manual_seed(d)
    T, n, Pg = 20, 7, 16
    qkv = (torch.randn(T, (nq + 2 * nkv) * d, generator=g) * 2).bfloat16()
    pos = torch.randint(0, 3000, (T,), generator=g, dtype=torch.int32)
    slots = torch.randperm(4 * Pg, generator=g)[:T].to(torch.int32)
    inv = (1.0 / (10000.0 ** (torch.arange(0, rot, 2).float() / rot))).to(DEV)
    got = []
    for rows in (T, n):
        x = qkv[:rows].clone().to(DEV)
        kc = torch.zeros(4, nkv, Pg, d, dtype=torch.bfloat16, device=DEV)
        vc = torch.zeros(4, nkv, d, Pg, dtype=torch.bfloat16, device=DEV)
        K.rope_kv_store(x, K.rope_table(pos[:rows].to(DEV), inv), slots[:rows].to(DEV), kc, vc, nq, nkv, d, rot)
        got.append((x[:n].cpu(), [(kc[int(s) // Pg, :, int(s) % Pg].cpu(), vc[int(s) // Pg, :, :, int(s) % Pg].cpu()) for s in slots[:n]]))
    assert torch.equal(got[0][0], got[1][0])
    for (k1, v1), (k2, v2) in zip(got[0][1], got[1][1]):
        assert torch.equal(k1, k2) and torch.equal(v1, v2)


def test_sampling_greedy_and_ties(K):
    logits = torch.randn(5, 1000)
    logits[1, 7] = logits[1, 900] = 50.0            # tie: the lower index wins
    logits[2, 999] = 60.0
    z = torch.zeros(5)
    out = K.sample(logits.to(DEV), z.to(DEV), torch.ones(5, device=DEV), z.to(DEV))
    want = [P.sample_greedy(l) for l in logits]
    assert out.tolist() == want and want[1] == 7 and want[2] == 999


@pytest.mark.parametrize("R,V", [(1, 17), (5, 1000), (8, 151936), (64, 4099)])
def test_argmax_in_two_launches_is_the_greedy_sample(K, R, V):
    g = torch.Generator().manual_seed(V)
    logits = torch.randn(R, V, generator=g)
    logits[0, V // 3] = logits[0, V - 1] = 40.0                  # a tie across chunks: the lower index wins
    if R > 1:
        logits[1, V - 1] = 50.0                                  # the last element of the last chunk
        logits[R - 1, 0] = 50.0
    dev = logits.to(DEV)
    out = torch.full((R,), -1, dtype=torch.int32, device=DEV)
    K.argmax(dev, out, K.argmax_workspace(R, DEV))
    z = torch.zeros(R, device=DEV)
    assert out.tolist() == [P.sample_greedy(l) for l in logits] == K.sample(dev, z, z + 1, z).tolist()
    assert out[0] == V // 3
    wide = torch.randn(R, V + 5, generator=g).to(DEV)            # rows with a stride of their own
    K.argmax(wide[:, :V], out, K.argmax_workspace(R + 3, DEV))
    assert out.tolist() == wide[:, :V].argmax(1).tolist()
    with pytest.raises(K.KernelError):
        K.argmax(dev, out, K.argmax_workspace(max(R - 1, 0), DEV))


@pytest.mark.parametrize("V", [301, 5000, 151936, 300007])      # (the last: a thread's piece of a chunk is beyond what it holds in registers)
def test_sampling_temperature_follows_the_inverse_cdf(K, V):
    g = torch.Generator().manual_seed(V)
    R = 64
    logits = torch.randn(R, V, generator=g) * 3
    temps = torch.rand(R, generator=g) * 1.5 + 0.2
    us = torch.rand(R, generator=g)
    out = K.sample(logits.to(DEV), temps.to(DEV), torch.ones(R, device=DEV), us.to(DEV)).tolist()
    agree = 0
    for r in range(R):
        p = P.temperature_probs(logits[r], float(temps[r]))
        want = P.inverse_cdf(p, float(us[r]))
        cum = torch.cumsum(p, 0)
        # equal, or u falls within float32 rounding of a boundary of the CDF
        if out[r] == want:
            agree += 1
        else:
            lo, hi = sorted((out[r], want))
            assert hi - lo <= 2 and abs(float(cum[lo]) - float(us[r])) < 1e-5, (r, out[r], want)
    assert agree >= R - 3


def test_sampling_top_p_keeps_a_prefix_of_tied_tokens(K):
    # tokens of equal probability at the threshold: the sorted rule keeps as many of them as it takes to reach
    # top_p, not all (pico_vllm/sampler.py:25-32); which ones is the sort's choice, here the lowest indices
    cases = [(torch.tensor([0.2, 0.4, 0.2, 0.2]), 0.5, {1, 0}), (torch.tensor([0.2, 0.4, 0.2, 0.2]), 0.7, {1, 0, 2}),
             (torch.tensor([0.2, 0.4, 0.2, 0.2]), 0.95, {0, 1, 2, 3}), (torch.full((100,), 0.01), 0.305, set(range(31))),
             (torch.tensor([0.25, 0.25, 0.25, 0.25]), 0.1, {0})]
    for probs, top_p, kept in cases:
        logits = probs.log()[None, :].contiguous()
        assert set(torch.nonzero(P.top_p_probs(logits[0], 1.0, top_p)).flatten().tolist()) == kept
        seen = set()
        for u in torch.linspace(0.001, 0.999, 97):
            tok = K.sample(logits.to(DEV), torch.ones(1, device=DEV), torch.tensor([top_p], device=DEV), u.reshape(1).to(DEV))
            seen.add(int(tok[0]))
        assert seen == kept, (probs.tolist()[:5], top_p, sorted(seen))


def test_sampling_at_the_real_vocabulary_row_by_row(K):
    # 151,936 logits a row, rows of every kind side by side: greedy, plain temperature, wide and narrow nuclei, flat and
    # peaked distributions.  Every row against the plain rule, and the same token when the row is sampled alone.
    g = torch.Generator().manual_seed(21)
    R, V = 14, 151936
    logits = torch.randn(R, V, generator=g) * torch.tensor([1, 1, 3, 3, 3, 8, 8, 0.1, 0.1, 20, 20, 3, 3, 3.0])[:, None]
    temps = torch.tensor([0.0, 1.0, 0.7, 0.7, 1.3, 1.0, 0.5, 1.0, 1.0, 1.0, 2.0, 0.0, 0.9, 1.1])
    top_ps = torch.tensor([1.0, 1.0, 0.9, 0.5, 0.05, 0.95, 0.3, 0.9, 0.999, 0.8, 0.6, 0.5, 1.0, 0.99])
    us = torch.rand(R, generator=g)
    dev = logits.to(DEV)
    work = K.sample_workspace(R, DEV)
    out = K.sample(dev, temps.to(DEV), top_ps.to(DEV), us.to(DEV), work=work).tolist()
    assert out == K.sample(dev, temps.to(DEV), top_ps.to(DEV), us.to(DEV), work=work).tolist()      # and again: the same
    exact = 0
    for r in range(R):
        alone = K.sample(dev[r:r + 1], temps[r:r + 1].to(DEV), top_ps[r:r + 1].to(DEV), us[r:r + 1].to(DEV))
        assert int(alone[0]) == out[r], (r, int(alone[0]), out[r])
        if temps[r] == 0:
            assert out[r] == P.sample_greedy(logits[r])
            continue
        p = P.top_p_probs(logits[r].double(), float(temps[r]), float(top_ps[r]))
        assert float(p[out[r]]) > 0, (r, "a token outside the kept set")
        want = P.inverse_cdf(p, float(us[r]))
        cum = torch.cumsum(p, 0)
        exact += out[r] == want
        # equal, or u falls within rounding of a boundary of the CDF (float32 exponentials against float64 ones)
        assert out[r] == want or abs(float(cum[min(out[r], want)]) - float(us[r])) < 1e-4, (r, out[r], want)
    assert exact >= R - 3
    # rows that are known to have no nucleus skip the search for it
    plain_rows = torch.ones(R, device=DEV)
    assert K.sample(dev, temps.to(DEV), plain_rows, us.to(DEV), top_p_rows=False).tolist() \
        == K.sample(dev, temps.to(DEV), plain_rows, us.to(DEV)).tolist()
    with pytest.raises(K.KernelError, match="workspace"):
        K.sample(dev, temps.to(DEV), top_ps.to(DEV), us.to(DEV), work=K.sample_workspace(R - 1, DEV))


def test_sampling_at_the_edges_of_its_options(K):
    # a nucleus so small that only the likeliest token fits, a temperature so low that it holds all the mass, one so high
    # that the distribution is flat, and a vocabulary smaller than the number of chunks a row is read in
    g = torch.Generator().manual_seed(3)
    for V in (5, 31, 33, 1000, 151936):
        logits = torch.randn(6, V, generator=g) * 2
        best = logits.argmax(1).tolist()
        temps = torch.tensor([1.0, 1e-4, 1.0, 50.0, 50.0, 0.3])
        top_ps = torch.tensor([1e-6, 1.0, 1e-6, 1.0, 0.999999, 1e-3])
        for u in (0.0, 0.37, 0.999999):
            us = torch.full((6,), u)
            out = K.sample(logits.to(DEV), temps.to(DEV), top_ps.to(DEV), us.to(DEV)).tolist()
            assert [out[0], out[1], out[2], out[5]] == [best[0], best[1], best[2], best[5]], (V, u, out, best)
            for r in (3, 4):                                   # nearly flat: the token at which the CDF passes u
                p = P.top_p_probs(logits[r].double(), 50.0, float(top_ps[r]))
                want = P.inverse_cdf(p, u)
                assert 0 <= out[r] < V and (out[r] == want or abs(float(torch.cumsum(p, 0)[min(out[r], want)]) - u) < 1e-4), (V, u, r, out[r], want)


def test_sampling_never_returns_a_token_whose_probability_underflowed(K):
    # a low temperature leaves a handful of tokens with a probability above zero; with u just below 1 the running sum
    # of a thread may stop short of the target by rounding, and the fallback must then be the last token that has
    # any probability, never one of the thousands behind it whose exp() is 0
    g = torch.Generator().manual_seed(5)
    for V in (1000, 151936):
        logits = torch.randn(4, V, generator=g)
        alive = [sorted(torch.randperm(V, generator=g)[:3].tolist()) for _ in range(4)]
        for r, idx in enumerate(alive):
            logits[r, idx] = torch.tensor([30.0, 30.5, 29.5])
        temps = torch.full((4,), 0.05)                       # exp((x - 30.5) / 0.05) is 0 for every other token
        for u in (0.0, 0.5, 0.9999999, 1.0 - 2.0 ** -24):
            out = K.sample(logits.to(DEV), temps.to(DEV), torch.ones(4, device=DEV), torch.full((4,), u).to(DEV),
                           top_p_rows=False).tolist()
            assert all(out[r] in alive[r] for r in range(4)), (V, u, out, alive)
            out = K.sample(logits.to(DEV), temps.to(DEV), torch.tensor([1.0, 0.9, 0.5, 1.0]).to(DEV),
                           torch.full((4,), u).to(DEV)).tolist()
            assert all(out[r] in alive[r] for r in range(4)), (V, u, out, alive)


def test_sampling_refuses_a_workspace_that_is_not_16_byte_aligned(K):
    logits = torch.randn(2, 100).to(DEV)
    ones = torch.ones(2, device=DEV)
    work = K.sample_workspace(3, DEV)
    with pytest.raises(K.KernelError, match="workspace"):
        K.sample(logits, ones, ones, ones * 0.5, work=work[2:])          # 8 bytes off


def test_sampling_top_p(K):
    probs = torch.tensor([[0.05, 0.5, 0.15, 0.3]])
    logits = torch.log(probs)
    for top_p, kept in ((0.81, {1, 3, 2}), (0.79, {1, 3}), (0.2, {1})):
        seen = set()
        for i in range(200):
            u = torch.tensor([(i + 0.5) / 200])
            tok = K.sample(logits.to(DEV), torch.ones(1, device=DEV), torch.tensor([top_p], device=DEV), u.to(DEV))
            seen.add(int(tok[0]))
            want = P.inverse_cdf(P.top_p_probs(logits[0], 1.0, top_p), float(u))
            p_kept = P.top_p_probs(logits[0], 1.0, top_p)
            cum = torch.cumsum(p_kept, 0)
            assert int(tok[0]) == want or min(abs(float(c) - float(u)) for c in cum) < 1e-5
        assert seen == kept
    # a large vocabulary with random logits: every draw lies in the kept set of the plain rule
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(16, 5000, generator=g) * 4
    us = torch.rand(16, generator=g)
    out = K.sample(logits.to(DEV), torch.full((16,), 0.7, device=DEV), torch.full((16,), 0.9, device=DEV), us.to(DEV))
    for r in range(16):
        p = P.top_p_probs(logits[r], 0.7, 0.9)
        assert float(p[int(out[r])]) > 0
        want = P.inverse_cdf(p, float(us[r]))
        assert abs(int(out[r]) - want) <= 0 or abs(float(torch.cumsum(p, 0)[min(int(out[r]), want)]) - float(us[r])) < 1e-4


# ---- matrix-core attention (bfloat16) ----------------------------------------------------------
def _fast_case(new_lens, prefix_lens, nq, nkv, d, Pg, seed=0, boost=None, decode=False, nsplit=1, teams=0, as_step=False,
               window=0, chunk_len=0, max_chunks=0, order=None, cut=None):
    from pico_vllm_amd.ops.attention_fast import FastAttention
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(seed)
    totals = [n + p for n, p in zip(new_lens, prefix_lens)]
    ks = [torch.randn(N, nkv, d, generator=g).to(dtype).float() for N in totals]
    vs = [torch.randn(N, nkv, d, generator=g).to(dtype).float() for N in totals]
    qs = [torch.randn(n, nq, d, generator=g).to(dtype).float() for n in new_lens]
    if boost is not None:
        boost(qs, ks, vs)
    num_pages = sum(-(-N // Pg) for N in totals) + 3
    kc, vc, bt = paged_cache(ks, vs, Pg, num_pages, dtype, seed)
    B = len(new_lens)
    cu = torch.tensor([0] + list(torch.tensor(new_lens).cumsum(0)), dtype=torch.int32, device=DEV)
    ctxl = torch.tensor(totals, dtype=torch.int32, device=DEV)
    # queries live inside a wider buffer, as q does inside the qkv activations
    T = sum(new_lens)
    wide = torch.zeros(T, (nq + 2 * nkv) * d, dtype=dtype, device=DEV)
    wide[:, :nq * d] = torch.cat(qs, 0).reshape(T, nq * d).to(DEV, dtype)
    fa = FastAttention(nq, nkv, d, window)
    scale = 1.0 / math.sqrt(d)
    if as_step:          # the way the attention part calls it: the kernels are chosen from the shape of the batch
        from types import SimpleNamespace
        step = SimpleNamespace(num_seqs=B, all_decode=max(new_lens) == 1, max_context=max(totals), cu_seqlens=cu,
                               context_lens=ctxl, host={"cu_seqlens": cu.cpu().numpy(), "context_lens": ctxl.cpu().numpy()}, shared={})
        out = fa(wide, SimpleNamespace(k=kc, v=vc), bt, step, scale)
    elif decode:
        if cut is not None:             # a cut to fill: the contexts of all sequences in pieces of one length
            cut.append(fa.decode_cut(B, nsplit, DEV))
        out = fa.decode(wide, kc, vc, bt, ctxl, B, scale, nsplit, cut=cut[0] if cut is not None else None)
    else:
        if order is not None:           # a list to fill: the query tiles of all sequences longest first
            order.append(fa.order_list(T, B, DEV))
        out = fa.prefill(wide, kc, vc, bt, cu, ctxl, B, scale, teams=teams, chunk_len=chunk_len,
                         max_chunks=max_chunks or (-(-max(totals) // chunk_len) if chunk_len else 0),
                         order=order[0] if order is not None else None)
    want = torch.cat([P.causal_attention(qb, kb, vb, q_positions=torch.arange(p, p + n), window=window)
                      for qb, kb, vb, n, p in zip(qs, ks, vs, new_lens, prefix_lens)], 0)
    return out.reshape(-1, nq, d), want


@pytest.mark.parametrize("window", [1, 20, 64, 100, 129, 1000])
@pytest.mark.parametrize("nq,nkv,d,Pg", [(12, 2, 128, 16), (6, 3, 32, 8), (4, 1, 64, 16), (5, 5, 48, 16), (4, 1, 16, 16), (4, 2, 256, 32),
                                        (4, 1, 96, 16)])
def test_fast_attention_with_a_window(K, nq, nkv, d, Pg, window):
    # only the last `window` keys count: prompt portions (the window's edge inside a key tile, at a tile's end, beyond the
    # prefix), decode tokens with every split, a mixed step; keys before the window are made large so that one that is
    # let in shows (their pages are what a cache manager gives back)
    def boost(qs, ks, vs):
        for q in qs:
            q *= 2.0
    new_lens, prefix_lens = [70, 1, 200, 2, 1, 130], [0, 300, 131, 63, 17, 500]
    for teams in (1, 2, 3, 4, 6):
        out, want = _fast_case(new_lens, prefix_lens, nq, nkv, d, Pg, seed=window, boost=boost, teams=teams, window=window)
        close(out, want, torch.bfloat16)
    for nsplit in (1, 3, 8):
        out, want = _fast_case([1, 1, 1, 1], [300, 17, 0, 1000], nq, nkv, d, Pg, seed=window + 1, boost=boost, decode=True,
                               nsplit=nsplit, window=window)
        close(out, want, torch.bfloat16)
    out, want = _fast_case([1, 1, 40, 9], [300, 64, 100, 0], nq, nkv, d, Pg, seed=window + 2, boost=boost, as_step=True, window=window)
    close(out, want, torch.bfloat16)


def test_a_window_reads_nothing_before_it(K):
    # pages before the window hold not-a-number: a kernel that let one of their keys or values into a sum would show it
    from pico_vllm_amd.ops.attention_fast import FastAttention
    nq, nkv, d, Pg, window = 4, 2, 64, 16, 40
    g = torch.Generator().manual_seed(3)
    N = 400
    k = torch.randn(N, nkv, d, generator=g).bfloat16().float()
    v = torch.randn(N, nkv, d, generator=g).bfloat16().float()
    dead = N - window                                     # the one query, at position N - 1, sees keys dead .. N - 1
    k[:dead], v[:dead] = float("nan"), float("nan")
    kc, vc, bt = paged_cache([k], [v], Pg, N // Pg + 2, torch.bfloat16, 1, garbage=False)
    q = torch.randn(1, nq, d, generator=g).bfloat16()
    fa = FastAttention(nq, nkv, d, window)
    ctxl = torch.tensor([N], dtype=torch.int32, device=DEV)
    want = P.causal_attention(q.float(), k[dead:], v[dead:], window=window)
    for nsplit in (1, 4):
        out = fa.decode(q.reshape(1, -1).to(DEV), kc, vc, bt, ctxl, 1, d ** -0.5, nsplit)
        close(out.reshape(1, nq, d), want, torch.bfloat16)
    cu = torch.tensor([0, 1], dtype=torch.int32, device=DEV)
    out = fa.prefill(q.reshape(1, -1).to(DEV), kc, vc, bt, cu, ctxl, 1, d ** -0.5)
    close(out.reshape(1, nq, d), want, torch.bfloat16)


@pytest.mark.parametrize("case", range(len(REFERENCE_CASES)))
def test_fast_prefill_on_the_reference_cases(K, case):
    new_lens, prefix_lens = REFERENCE_CASES[case]
    out, want = _fast_case(new_lens, prefix_lens, 12, 2, 128, 16, seed=case)
    close(out, want, torch.bfloat16)


@pytest.mark.parametrize("nq,nkv,d,Pg", [(4, 1, 16, 16), (6, 3, 32, 8), (5, 5, 48, 16), (3, 1, 80, 32), (8, 2, 256, 64),
                                        (2, 2, 64, 8), (12, 2, 128, 16)])
def test_fast_prefill_other_sizes_and_long_portions(K, nq, nkv, d, Pg):
    # portions longer than one 128-query tile, a decode token, a 2-token portion, long prefixes
    out, want = _fast_case([7, 1, 300, 2, 129], [0, 70, 45, 129, 500], nq, nkv, d, Pg, seed=3)
    close(out, want, torch.bfloat16)


@pytest.mark.parametrize("teams", [1, 2, 3, 4, 6])
@pytest.mark.parametrize("nq,nkv,d,Pg", [(6, 3, 32, 8), (2, 2, 64, 8), (12, 2, 128, 16), (8, 2, 256, 64), (4, 1, 96, 32),
                                        (4, 1, 96, 16), (4, 1, 96, 8), (8, 2, 256, 16), (2, 1, 160, 8)])
def test_fast_prefill_with_every_shape_of_workgroup(K, nq, nkv, d, Pg, teams):
    # the shape of the workgroups (1 to 3 teams on a 64-query tile, 4: two query blocks a wave, 128-query tiles, 6: two teams of those)
    # is a hint: every value gives the same attention; lengths around the 64- and 128-query tiles and the
    # 64-, 128- and 192-key tiles of one to three teams; pages of 8 and 16 keys take the short way in whole tiles
    out, want = _fast_case([63, 1, 65, 130, 2, 200, 193, 127, 257], [0, 127, 1, 62, 191, 129, 383, 1, 64], nq, nkv, d, Pg, seed=5,
                           teams=teams)
    close(out, want, torch.bfloat16)


@pytest.mark.parametrize("teams,chunk_len", [(1, 0), (2, 0), (3, 0), (4, 0), (6, 0), (1, 256), (4, 128)])
@pytest.mark.parametrize("nq,nkv,d,Pg", [(12, 2, 128, 16), (6, 3, 32, 8), (4, 1, 96, 32), (2, 1, 160, 8)])
def test_fast_prefill_takes_the_tiles_of_several_sequences_longest_first(K, nq, nkv, d, Pg, teams, chunk_len):
    # with a list to fill, the workgroups take the query tiles of all sequences by the keys they read, most first: the
    # list is a permutation of the tiles in that order, and the attention is the same bits as sequence by sequence
    new_lens, prefix_lens = [63, 1, 65, 130, 2, 200, 193, 127, 257], [0, 127, 1, 62, 191, 129, 383, 1, 64]
    plain, want = _fast_case(new_lens, prefix_lens, nq, nkv, d, Pg, seed=5, teams=teams, chunk_len=chunk_len)
    order = []
    out, _ = _fast_case(new_lens, prefix_lens, nq, nkv, d, Pg, seed=5, teams=teams, chunk_len=chunk_len, order=order)
    close(out, want, torch.bfloat16)
    assert torch.equal(out, plain)
    bmq = 128 if teams in (4, 6) and d <= 128 else 64
    tiles = [(b, t) for b, n in enumerate(new_lens) for t in range(-(-n // bmq))]
    grid = sum(new_lens) // bmq + len(new_lens)                 # tiles the launch has room for; the list may be longer
    got = order[0].cpu().tolist()[:grid]
    assert got[len(tiles):] == [-1] * (grid - len(tiles)) and order[0].numel() >= grid
    listed = [(e >> 16, e & 0xffff) for e in got[:len(tiles)]]
    assert sorted(listed) == tiles
    keys = [min(prefix_lens[b] + new_lens[b], prefix_lens[b] + (t + 1) * bmq) for b, t in listed]
    assert keys == sorted(keys, reverse=True)
    if nq == 12 and teams == 1 and not chunk_len:
        # a list that was never written names no tile the kernel accepts: nothing is read through it, nothing is written
        from pico_vllm_amd.ops.attention_fast import FastAttention
        fa, B, T = FastAttention(nq, nkv, d), len(new_lens), sum(new_lens)
        g = torch.Generator().manual_seed(1)
        ks = [torch.randn(n + p, nkv, d, generator=g).bfloat16().float() for n, p in zip(new_lens, prefix_lens)]
        kc, vc, bt = paged_cache(ks, ks, Pg, sum(-(-k.shape[0] // Pg) for k in ks) + 3, torch.bfloat16, 1)
        cu = torch.tensor([0] + list(torch.tensor(new_lens).cumsum(0)), dtype=torch.int32, device=DEV)
        ctxl = torch.tensor([n + p for n, p in zip(new_lens, prefix_lens)], dtype=torch.int32, device=DEV)
        q = torch.randn(T, (nq + 2 * nkv) * d, generator=g).bfloat16().to(DEV)
        for junk in (1 << 30, (3 << 16) | 40, 0x7fff0000):
            lst = fa.order_list(T, B, DEV).fill_(junk)
            res = fa.prefill(q, kc, vc, bt, cu, ctxl, B, d ** -0.5, out=torch.zeros(T, nq * d, dtype=torch.bfloat16, device=DEV),
                             teams=teams, order=lst, order_build=False)
            assert not res.float().abs().sum().item()


@pytest.mark.parametrize("Pg", [8, 16, 32])
@pytest.mark.parametrize("d", list(range(16, 257, 16)))
def test_fast_prefill_whole_key_tiles_at_every_head_size_and_page_size(K, d, Pg):
    # contexts of three and more whole key tiles: where a thread's chunks of K are a whole number of pages
    # apart the kernel prepares its addresses once per tile, elsewhere it must not; queries are scaled up so
    # that a few keys carry each row's weight and a wrong key or row part shows
    def boost(qs, ks, vs):
        for q in qs:
            q *= 4.0            # a power of two: the scaled queries are bfloat16 numbers still
    out, want = _fast_case([200, 70, 3], [0, 330, 400], 2, 1, d, Pg, seed=17 + d + Pg, boost=boost)
    assert float(want.abs().mean()) > 0.3
    close(out, want, torch.bfloat16)
    # and the decode kernels of that head size, whole and split
    for nsplit in (1, 5):
        out, want = _fast_case([1, 1], [330, 65], 2, 1, d, Pg, seed=d + Pg, boost=boost, decode=True, nsplit=nsplit)
        close(out, want, torch.bfloat16)


@pytest.mark.parametrize("window", [0, 100])
@pytest.mark.parametrize("nq,nkv,d,Pg,nsplit", [(12, 2, 128, 16, 8), (6, 3, 32, 8, 2), (5, 5, 48, 16, 3), (4, 1, 256, 32, 4), (8, 2, 96, 16, 16)])
def test_fast_decode_with_the_contexts_cut_into_pieces_of_one_length(K, nq, nkv, d, Pg, nsplit, window):
    # from 17 sequences on (32, counted as a recorded step is padded) the contexts of a decode step are cut into pieces of one length over all sequences (the pieces of
    # a long context are as long as a short context's): the cut covers every sequence's keys once, in order, in whole units
    # of 32 keys (of an LDS tile where the kernel stages tiles), in no more pieces than nsplit splits of 32 sequences
    # would be and with the smallest length that allows that; the attention is the plain one; and sequences without a context
    # behind the others (the padding of a recorded step) change no bit of the others
    from pico_vllm_amd.ops.attention_fast import FastAttention
    def boost(qs, ks, vs):
        for q in qs:
            q *= 2.0
    prefix_lens = [3000, 17, 0, 1000, 64, 129, 2047, 5, 700, 31, 32, 33, 1500, 95, 96, 2, 260, 511, 4100, 1]
    new_lens = [1] * len(prefix_lens)
    cut = []
    out, want = _fast_case(new_lens, prefix_lens, nq, nkv, d, Pg, seed=nsplit + window, boost=boost, decode=True, nsplit=nsplit,
                           window=window, cut=cut)
    close(out, want, torch.bfloat16)
    plan, slots = cut[0]
    B = len(prefix_lens)
    assert slots == 32 * nsplit
    pieces = plan[:4 * slots].reshape(slots, 4).cpu().tolist()
    rows = plan[4 * slots:4 * slots + 2 * B].reshape(B, 2).cpu().tolist()
    unit = 32 if (d % 32 == 0 and d <= 128 and nq // nkv <= 16) else (64 if d <= 128 else 32)
    used = sum(n for _, n in rows)
    assert used <= slots and all(p[0] == -1 for p in pieces[used:])
    lengths = set()
    for b, (first, n) in enumerate(rows):
        ctx = prefix_lens[b] + 1
        low = max(0, ctx - window) // unit * unit if window else 0
        mine = pieces[first:first + n]
        assert [p[0] for p in mine] == [b] * n and all(p[3] == ctx for p in mine) and 1 <= n <= 256
        assert mine[0][1] == low and mine[-1][2] == ctx and all(x[2] == y[1] for x, y in zip(mine, mine[1:]))
        lengths |= {p[2] - p[1] for p in mine[:-1]}
        T = mine[0][2] - mine[0][1] if n > 1 else None
        assert all(p[2] - p[1] == T for p in mine[:-1])
    assert len(lengths) <= 1 and all(t % unit == 0 for t in lengths)
    if lengths:                                            # a unit shorter, the pieces would not fit the launch
        T = lengths.pop()
        spans = [prefix_lens[b] + 1 - (max(0, prefix_lens[b] + 1 - window) // unit * unit if window else 0) for b in range(B)]
        assert all(-(-x // T) == n for x, (_, n) in zip(spans, rows))
        assert T == unit or sum(-(-x // (T - unit)) for x in spans) > slots or -(-max(spans) // (T - unit)) > 256
    # the same sequences with three rows without a context behind them: the same bits
    fa = FastAttention(nq, nkv, d, window)
    g = torch.Generator().manual_seed(7)
    totals = [p + 1 for p in prefix_lens]
    ks = [torch.randn(N, nkv, d, generator=g).bfloat16().float() for N in totals]
    vs = [torch.randn(N, nkv, d, generator=g).bfloat16().float() for N in totals]
    kc, vc, bt = paged_cache(ks, vs, Pg, sum(-(-N // Pg) for N in totals) + 3, torch.bfloat16, 1)
    q = torch.randn(B + 3, (nq + 2 * nkv) * d, generator=g).bfloat16().to(DEV)
    ctxl = torch.tensor(totals + [0, 0, 0], dtype=torch.int32, device=DEV)
    bt16 = torch.full((B + 3, bt.shape[1]), -1, dtype=torch.int32, device=DEV)
    bt16[:B] = bt
    real = fa.decode(q[:B], kc, vc, bt, ctxl[:B], B, d ** -0.5, nsplit, cut=fa.decode_cut(B, nsplit, DEV))
    padded = fa.decode(q, kc, vc, bt16, ctxl, B + 3, d ** -0.5, nsplit, cut=fa.decode_cut(B + 3, nsplit, DEV))
    assert torch.equal(real, padded[:B]) and not padded[B:].float().abs().sum().item()
    # a cut that was never written names no piece of this step: nothing is read through it, every row comes out empty
    plan, slots = fa.decode_cut(B, nsplit, DEV)
    for junk in (1 << 30, -7):
        plan.fill_(junk)
        out = fa.decode(q[:B], kc, vc, bt, ctxl[:B], B, d ** -0.5, nsplit, cut=(plan, slots), cut_build=False)
        assert not out.float().abs().sum().item()


@pytest.mark.parametrize("nq,nkv,d,Pg", [(12, 2, 128, 16), (6, 3, 32, 8), (5, 5, 48, 16), (4, 1, 16, 16)])
@pytest.mark.parametrize("new_lens,prefix_lens", [([1, 1, 1, 70, 2, 1], [300, 17, 64, 33, 129, 5]),     # decode rows first, as the scheduler orders them
                                                  ([1, 1, 1, 1], [300, 17, 64, 0]),                      # decode only
                                                  ([1, 40], [1000, 0]), ([9, 1, 1], [0, 20, 30])])      # no decode row in front
def test_fast_attention_of_a_mixed_step(K, nq, nkv, d, Pg, new_lens, prefix_lens):
    # leading single-token sequences go through the decode kernel, the rest through the prefill kernel
    out, want = _fast_case(new_lens, prefix_lens, nq, nkv, d, Pg, seed=9, as_step=True)
    close(out, want, torch.bfloat16)


def test_fast_attention_of_a_step_with_much_work(K):
    # eight portions of 256 tokens after 2,048 with 16 heads: the step is served by the workgroups of 128 queries
    from pico_vllm_amd.ops.attention_fast import FastAttention
    fa = FastAttention.__new__(FastAttention)
    fa.nq = 16
    assert fa.prefill_teams([256] * 8, [2304] * 8) == 4
    out, want = _fast_case([256] * 8, [2048] * 8, 16, 4, 32, 16, seed=13, as_step=True)
    close(out, want, torch.bfloat16)


@pytest.mark.parametrize("teams", [0, 1, 2, 4, 6])
@pytest.mark.parametrize("nq,nkv,d,Pg,chunk_len", [(12, 2, 128, 16, 256), (6, 3, 32, 8, 128), (2, 2, 64, 8, 384), (4, 1, 96, 32, 128),
                                                  (4, 2, 256, 16, 512), (2, 1, 160, 8, 256)])
def test_fast_prefill_with_the_keys_cut_into_chunks(K, nq, nkv, d, Pg, chunk_len, teams):
    # every chunk of a tile's keys is a workgroup of its own and a second launch joins them: tiles of one chunk and of
    # many in one batch, a chunk's edge inside a tile's own positions (its first queries see no key of the last
    # chunk), portions of one and two tokens, a context that ends one key into a chunk, more room for chunks than needed;
    # queries are scaled up so that few keys carry a row's weight and a chunk that is lost or joined wrongly shows
    def boost(qs, ks, vs):
        for q in qs:
            q *= 2.0
    new_lens, prefix_lens = [300, 77, 1, 130, 2, 64], [1000, 0, 555, 2 * chunk_len - 129, chunk_len - 1, 3 * chunk_len]
    out, want = _fast_case(new_lens, prefix_lens, nq, nkv, d, Pg, seed=chunk_len + d, boost=boost, teams=teams, chunk_len=chunk_len)
    close(out, want, torch.bfloat16)
    more, _ = _fast_case(new_lens, prefix_lens, nq, nkv, d, Pg, seed=chunk_len + d, boost=boost, teams=teams, chunk_len=chunk_len,
                         max_chunks=-(-max(n + p for n, p in zip(new_lens, prefix_lens)) // chunk_len) + 3)
    assert torch.equal(out, more)


def test_fast_prefill_refuses_chunks_it_cannot_cut(K):
    from pico_vllm_amd.ops.kernels import KernelError
    for kw in (dict(teams=3, chunk_len=256), dict(teams=1, chunk_len=200), dict(teams=1, chunk_len=256, window=50),
               dict(teams=1, chunk_len=256, max_chunks=65)):
        with pytest.raises(KernelError):
            _fast_case([70], [300], 4, 2, 64, 16, **kw)
    with pytest.raises(KernelError):            # a head size that the 16-query kernel does not serve
        _fast_case([70], [300], 4, 2, 48, 16, teams=1, chunk_len=256)


def test_a_step_behind_a_long_prefix_cuts_its_keys_into_chunks(K):
    # the host's choice (FastAttention.prefill_chunks) and the step that it serves
    from pico_vllm_amd.ops.attention_fast import FastAttention
    fa = FastAttention.__new__(FastAttention)
    fa.nq, fa.nkv, fa.d, fa.window, fa.cus = 12, 2, 128, 0, 256
    assert fa.prefill_chunks([2048], [2048]) is None                    # no prefix: short tiles
    assert fa.prefill_chunks([2048] * 8, [4096] * 8) is None            # work for every compute unit
    assert fa.prefill_chunks([2048], [16384]) == (4, 8192, 2)           # 192 workgroups of 256 key tiles each on 512 places
    assert fa.prefill_chunks([2048], [32768]) == (4, 4096, 8)
    assert fa.prefill_chunks([64], [8064]) == (1, 2048, 4)              # one tile per head
    fa.nq = 28
    assert fa.prefill_chunks([2048], [16384]) is None                   # 448 workgroups on 512 places
    fa.window = 100
    assert fa.prefill_chunks([64], [8064]) is None
    fa.nq, fa.nkv, fa.d, fa.window = 4, 2, 64, 0
    assert fa.prefill_chunks([64, 70], [8064, 7070]) == (1, 2048, 4)
    out, want = _fast_case([1, 64, 70], [300, 8000, 7000], 4, 2, 64, 16, seed=21, as_step=True)      # behind a decode row
    close(out, want, torch.bfloat16)


def test_fast_prefill_chooses_teams_by_the_shape_of_the_batch():
    from pico_vllm_amd.ops.attention_fast import FastAttention
    fa = FastAttention.__new__(FastAttention)
    fa.nq = 12
    assert fa.prefill_teams([2048], [2048]) == 3            # a causal triangle: the longest tile decides
    assert fa.prefill_teams([512], [4096]) == 3             # few tiles
    assert fa.prefill_teams([1] * 8, [4000] * 8) == 3       # decode tokens inside a mixed step
    assert fa.prefill_teams([2048], [16384]) == 4           # many long, equal tiles that fill 128 queries
    assert fa.prefill_teams([32] * 64, [2032] * 64) == 1    # much work in short portions
    assert fa.prefill_teams([2048] * 2, [2048] * 2) == 6    # more than the longest tile's worth for every unit, not much more
    assert fa.prefill_teams([512] * 4, [1024] * 4) == 6
    assert fa.prefill_teams([2048] * 4, [2048] * 4) == 4    # much work


def test_fast_prefill_with_a_cache_of_4_gib(K):
    # offsets into such a cache do not fit 32 bits: the kernel with 64-bit addresses serves it;
    # the pages used lie at both ends of the cache
    from pico_vllm_amd.ops.attention_fast import FastAttention
    nq, nkv, d, Pg = 2, 1, 64, 16
    pages = (1 << 32) // (nkv * Pg * d * 2) + 7
    g = torch.Generator().manual_seed(11)
    n, prefix = 70, 90
    N = n + prefix
    k = torch.randn(N, nkv, d, generator=g).bfloat16().float()
    v = torch.randn(N, nkv, d, generator=g).bfloat16().float()
    q = torch.randn(n, nq, d, generator=g).bfloat16().float()
    kc = torch.zeros(pages, nkv, Pg, d, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros(pages, nkv, d, Pg, dtype=torch.bfloat16, device=DEV)
    need = -(-N // Pg)
    ids = [pages - 1 - 3 * j if j % 2 else 5 * j for j in range(need)]
    for j, page in enumerate(ids):
        m = min(Pg, N - j * Pg)
        kc[page, :, :m, :] = k[j * Pg:j * Pg + m].transpose(0, 1).to(DEV, torch.bfloat16)
        vc[page, :, :, :m] = v[j * Pg:j * Pg + m].permute(1, 2, 0).to(DEV, torch.bfloat16)
    bt = torch.tensor([ids], dtype=torch.int32, device=DEV)
    cu = torch.tensor([0, n], dtype=torch.int32, device=DEV)
    ctxl = torch.tensor([N], dtype=torch.int32, device=DEV)
    fa = FastAttention(nq, nkv, d)
    out = fa.prefill(q.reshape(n, nq * d).to(DEV, torch.bfloat16), kc, vc, bt, cu, ctxl, 1, 1.0 / math.sqrt(d))
    want = P.causal_attention(q, k, v, q_positions=torch.arange(prefix, N))
    close(out.reshape(n, nq, d), want, torch.bfloat16)
    del kc, vc
    torch.cuda.empty_cache()


@pytest.mark.parametrize("nq,nkv,d,Pg", [(4, 1, 16, 16), (6, 3, 32, 8), (5, 5, 48, 16), (3, 1, 80, 32), (8, 2, 256, 64),
                                        (12, 2, 128, 16), (32, 1, 64, 16)])
@pytest.mark.parametrize("nsplit", [1, 3, 8, 65, 256])
def test_fast_decode(K, nq, nkv, d, Pg, nsplit):
    out, want = _fast_case([1, 1, 1, 1, 1], [0, 70, 45, 129, 1000], nq, nkv, d, Pg, seed=4, decode=True, nsplit=nsplit)
    close(out, want, torch.bfloat16)


def test_fast_kernels_find_one_far_key_among_hundreds(K):
    for far in (0, 15, 16, 31, 32, 63, 64, 127, 128, 200, 511, 596):
        def boost(qs, ks, vs, far=far):
            ks[0][far] = qs[0][-1, 0:1, :] * 2.0
            vs[0][far] = 100.0
        out, want = _fast_case([3], [597], 2, 1, 64, 16, seed=far, boost=boost)
        assert float(want[-1, 0].mean()) > 50
        close(out, want, torch.bfloat16, scale=100)
        for nsplit in (1, 4):
            out, want = _fast_case([1], [599], 2, 1, 64, 16, seed=far, boost=boost, decode=True, nsplit=nsplit)
            assert float(want[-1, 0].mean()) > 50
            close(out, want, torch.bfloat16, scale=100)


@pytest.mark.parametrize("far", [2, 9000, 20470])
def test_fast_attention_finds_a_far_key_among_twenty_thousand(K, far):
    # 20,480 cached keys (1,280 pages) and one key that matters: every split of decode, and a portion of a
    # prompt after that prefix, reach it through the block table
    def boost(qs, ks, vs, far=far):
        for q in qs:
            ks[0][far] = q[-1, 0:1, :] * 3.0
        vs[0][far] = 100.0
    for nsplit in (1, 7, 32, 100, 256):
        out, want = _fast_case([1], [20480], 4, 2, 64, 16, seed=far, boost=boost, decode=True, nsplit=nsplit)
        assert float(want[-1, 0].mean()) > 50
        close(out, want, torch.bfloat16, scale=100)
    out, want = _fast_case([1], [20480], 4, 2, 64, 16, seed=far, boost=boost, as_step=True)
    close(out, want, torch.bfloat16, scale=100)
    for teams in (0, 1, 3):
        out, want = _fast_case([70], [20411], 4, 2, 64, 16, seed=far, boost=boost, teams=teams)
        assert float(want[-1, 0].mean()) > 50
        close(out, want, torch.bfloat16, scale=100)


def test_fast_kernels_refuse_what_they_cannot_do(K):
    from pico_vllm_amd.ops.attention_fast import choose, supported
    assert choose(4, 2, 24, 0) is None and choose(4, 2, 512, 0) is None and choose(4, 2, 64, -1) is None
    assert supported(12, 2, 128, 0) and supported(12, 2, 128, 4096)


# ---- weight-streaming GEMM --------------------------------------------------------------------
@pytest.mark.parametrize("M,N,K_", [(1, 2048, 1536), (8, 1536, 1536), (64, 1536, 8960), (33, 301, 136), (5, 384, 192),
                                   (2, 64, 320), (17, 1000, 264), (12, 1536, 1536), (16, 90, 64), (24, 512, 1024),
                                   (32, 301, 256), (9, 1000, 8960),
                                   # more than 32 tokens and many tiles: two tiles a workgroup (an odd number of tiles,
                                   # an odd number of slices, a single slice)
                                   (50, 10270, 192), (40, 10400, 64), (64, 10240, 320),
                                   # more than 64 tokens of a small matrix: blocks of 64 tokens, the last one partial
                                   # (with 1 to 32 and with more than 32 tokens)
                                   (65, 301, 136), (100, 1536, 1536), (130, 2048, 1536), (256, 1000, 264), (200, 90, 8960),
                                   # the four projections at the 7B sizes (hidden 3584, 28 + 2 * 4 heads of 128, 18944) ...
                                   (1, 4608, 3584), (64, 3584, 3584), (40, 37888, 3584), (8, 3584, 18944),
                                   # ... and at the 32B sizes (hidden 5120, 40 + 2 * 8 heads of 128, 27648)
                                   (3, 7168, 5120), (1, 5120, 5120), (64, 55296, 5120), (17, 5120, 27648)])
def test_gemm_skinny_epilogues(K, M, N, K_):
    g = torch.Generator().manual_seed(M * N)
    a = torch.randn(M, K_, generator=g).bfloat16()
    w = (torch.randn(N, K_, generator=g) / math.sqrt(K_)).bfloat16()
    b = torch.randn(N, generator=g)
    want = a.double() @ w.double().T
    out = K.gemm_skinny(a.to(DEV), w.to(DEV), b.to(DEV), K.EPI_F32)
    assert torch.allclose(out.cpu().double(), want + b.double(), rtol=1e-4, atol=1e-4)
    out = K.gemm_skinny(a.to(DEV), w.to(DEV), b.to(DEV), K.EPI_BF16)
    assert out.dtype == torch.bfloat16 and torch.allclose(out.cpu().double(), want + b.double(), rtol=1e-2, atol=1e-2)
    # partial sums over ranges of k add up to the product; the bias is in the first slab only
    for splits in range(2, 9):
        per = -(-(-(-K_ // splits)) // 256) * 256
        if -(-K_ // per) != splits:
            continue
        slabs = K.gemm_skinny(a.to(DEV), w.to(DEV), b.to(DEV), K.EPI_F32, splits)
        assert slabs.shape == (splits, M, N)
        assert torch.allclose(slabs.cpu().double().sum(0), want + b.double(), rtol=1e-4, atol=1e-4)
        assert torch.allclose(slabs[1:].cpu().double().sum(0) + slabs[0].cpu().double(), want + b.double(), rtol=1e-4, atol=1e-4)
    # the stack goes into the norm kernel as delta
    if N >= 64:
        splits = K.skinny_k_splits(N, K_)
        delta = K.gemm_skinny(a.to(DEV), w.to(DEV), None, K.EPI_F32, splits)
        resid = torch.randn(M, N, generator=g)
        r = resid.clone().to(DEV)
        out = K.add_rmsnorm(r, delta, torch.ones(N, device=DEV), 1e-6, torch.float32)
        assert torch.allclose(r.cpu().double(), resid.double() + want, rtol=1e-4, atol=1e-4)
        close(out, P.rms_norm((resid.double() + want).float(), torch.ones(N), 1e-6), torch.float32, scale=10)
    # SwiGLU epilogue: w = [gate rows; up rows]
    if N % 2 == 0:
        out = K.gemm_skinny(a.to(DEV), w.to(DEV), None, K.EPI_SWIGLU)
        close(out, P.swiglu(want.float()), torch.bfloat16, scale=2)
    # a row's result does not depend on the other rows of the call
    one = K.gemm_skinny(a[M // 2:M // 2 + 1].to(DEV), w.to(DEV), b.to(DEV), K.EPI_F32)
    full = K.gemm_skinny(a.to(DEV), w.to(DEV), b.to(DEV), K.EPI_F32)
    assert torch.equal(one.cpu()[0], full.cpu()[M // 2])


@pytest.mark.parametrize("M,nq,nkv,d,H,Pg,bias", [(1, 12, 2, 128, 1536, 16, True), (8, 12, 2, 128, 1536, 16, True),
                                                  (64, 6, 3, 32, 192, 8, True), (37, 3, 1, 64, 136, 32, False),
                                                  (5, 2, 2, 96, 264, 16, True), (13, 4, 2, 64, 320, 16, True),
                                                  (29, 2, 1, 128, 128, 8, False),
                                                  # several blocks of 64 tokens
                                                  (70, 12, 2, 128, 1536, 16, True), (256, 6, 3, 32, 192, 8, True),
                                                  (150, 3, 1, 64, 136, 32, False)])
def test_gemm_skinny_with_rotation_and_cache_store(K, M, nq, nkv, d, H, Pg, bias):
    # projection + bias + rotate-half + store in one kernel against the plain steps one after the other
    theta = 1e6
    g = torch.Generator().manual_seed(M + d)
    x = torch.randn(M, H, generator=g).bfloat16()
    N = (nq + 2 * nkv) * d
    w = (torch.randn(N, H, generator=g) / math.sqrt(H)).bfloat16()
    b = torch.randn(N, generator=g) if bias else None
    pos = torch.randint(0, 5000, (M,), generator=g, dtype=torch.int32)
    num_pages = M + 4
    pages = torch.randperm(num_pages, generator=g)[:M]
    offs = torch.randint(0, Pg, (M,), generator=g)
    slots = (pages * Pg + offs).to(torch.int32)
    if M > 2:
        slots[M // 2] = -1                                  # a padding row stores nothing
    kc = torch.full((num_pages, nkv, Pg, d), 7.0, dtype=torch.bfloat16, device=DEV)
    vc = torch.full((num_pages, nkv, d, Pg), 7.0, dtype=torch.bfloat16, device=DEV)
    inv = (1.0 / (theta ** (torch.arange(0, d, 2).float() / d))).to(DEV)
    q_out = K.gemm_skinny_rope(x.to(DEV), w.to(DEV), None if b is None else b.to(DEV), K.rope_table(pos.to(DEV), inv),
                               slots.to(DEV), kc, vc, nq, nkv, d)
    qkv = (x.double() @ w.double().T + (0 if b is None else b.double())).float()
    q, k, v = P.split_qkv(qkv, nq, nkv, d)
    cos, sin = P.rope_tables(pos, d, theta)
    qr, kr = P.apply_rope(q, cos, sin), P.apply_rope(k, cos, sin)
    close(q_out.reshape(M, nq, d), qr, torch.bfloat16, scale=4)
    want_k = torch.full((num_pages, nkv, Pg, d), 7.0)
    want_v = torch.full((num_pages, nkv, d, Pg), 7.0)
    for t in range(M):
        if int(slots[t]) < 0:
            continue
        want_k[int(pages[t]), :, int(offs[t]), :] = kr[t]
        want_v[int(pages[t]), :, :, int(offs[t])] = v[t]
    close(kc, want_k, torch.bfloat16, scale=4)             # also: every slot that no token owns still holds 7
    close(vc, want_v, torch.bfloat16, scale=4)


@pytest.mark.parametrize("N,K_,slabs", [(2048, 1536, 5), (17920, 1536, 3), (1000, 320, 1), (90, 64, 0), (640, 2048, 8),
                                        (2 * 323, 512, -1), (1000, 3584, 6), (512, 4096, 8), (384, 2112, 0),
                                        (4608, 3584, 7), (37888, 3584, 5)])
def test_gemm_skinny_with_the_norm_in_front(K, N, K_, slabs):
    # norm(resid + partial sums) W^T of one row in one kernel against the norm kernel followed by the product;
    # slabs: 0 = nothing to add, -1 = one sum [1, K], else a stack [slabs, 1, K]
    g = torch.Generator().manual_seed(N + K_)
    resid = torch.randn(1, K_, generator=g)
    delta = None if slabs == 0 else torch.randn((1, K_) if slabs < 0 else (slabs, 1, K_), generator=g)
    nw = 1 + 0.1 * torch.randn(K_, generator=g)
    w = (torch.randn(N, K_, generator=g) / math.sqrt(K_)).bfloat16().to(DEV)
    eps = 1e-5
    d_dev = None if delta is None else delta.to(DEV)
    assert K.skinny_norm_ok(resid.to(DEV), d_dev, w)
    assert not K.skinny_norm_ok(torch.randn(2, K_).to(DEV), None, w)
    r2 = resid.clone().to(DEV)
    h = K.add_rmsnorm(r2, d_dev, nw.to(DEV), eps, torch.bfloat16)              # the two kernels: r2 is summed in place
    total = resid.double() + (0 if delta is None else delta.double().reshape(-1, 1, K_).sum(0))
    for epi in (K.EPI_F32, K.EPI_BF16, K.EPI_SWIGLU):
        out, r_out = K.gemm_skinny_norm(resid.to(DEV), d_dev, nw.to(DEV), eps, w, epi)
        assert torch.equal(r_out, r2)                                            # the same sums in the same order
        want = K.gemm_skinny(h, w, None, epi)
        scale = float(want.float().abs().max())
        # the sum of squares is formed by other threads: the normed row may differ in a last bfloat16 bit
        assert float((out.float() - want.float()).abs().max()) <= 2e-2 * scale, epi
        assert float((out.float() - want.float()).abs().mean()) <= 1e-3 * scale, epi
        if epi == K.EPI_F32:
            close(out, (P.rms_norm(total.float(), nw, eps).bfloat16().double() @ w.cpu().double().T).float(), torch.bfloat16, scale=4)
    assert torch.allclose(r_out.cpu().double(), total, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("nq,nkv,d,H,Pg,bias,slabs", [(12, 2, 128, 1536, 16, True, 5), (6, 3, 32, 192, 8, True, 0),
                                                      (3, 1, 64, 128, 32, False, 1), (4, 2, 64, 320, 16, True, 3),
                                                      (28, 4, 128, 3584, 16, True, 5)])
def test_gemm_skinny_with_the_norm_in_front_and_rotation_and_cache_store(K, nq, nkv, d, H, Pg, bias, slabs):
    theta = 1e6
    g = torch.Generator().manual_seed(d + H)
    resid = torch.randn(1, H, generator=g)
    delta = None if slabs == 0 else torch.randn(slabs, 1, H, generator=g)
    nw = 1 + 0.1 * torch.randn(H, generator=g)
    N = (nq + 2 * nkv) * d
    w = (torch.randn(N, H, generator=g) / math.sqrt(H)).bfloat16().to(DEV)
    b = torch.randn(N, generator=g).to(DEV) if bias else None
    pos = torch.randint(0, 5000, (1,), generator=g, dtype=torch.int32)
    slots = torch.tensor([3 * Pg + 5], dtype=torch.int32, device=DEV)
    inv = (1.0 / (theta ** (torch.arange(0, d, 2).float() / d))).to(DEV)
    table = K.rope_table(pos.to(DEV), inv)
    d_dev = None if delta is None else delta.to(DEV)
    caches = []
    for fused in (False, True):
        kc = torch.full((6, nkv, Pg, d), 7.0, dtype=torch.bfloat16, device=DEV)
        vc = torch.full((6, nkv, d, Pg), 7.0, dtype=torch.bfloat16, device=DEV)
        if fused:
            q, r_out = K.gemm_skinny_rope_norm(resid.to(DEV), d_dev, nw.to(DEV), 1e-6, w, b, table, slots, kc, vc, nq, nkv, d)
        else:
            r_out = resid.clone().to(DEV)
            h = K.add_rmsnorm(r_out, d_dev, nw.to(DEV), 1e-6, torch.bfloat16)
            q = K.gemm_skinny_rope(h, w, b, table, slots, kc, vc, nq, nkv, d)
        caches.append((q.float(), r_out, kc.float(), vc.float()))
    (q0, r0, k0, v0), (q1, r1, k1, v1) = caches
    assert torch.equal(r0, r1)
    for a, c in ((q0, q1), (k0, k1), (v0, v1)):
        scale = float(a.abs().max())
        assert float((a - c).abs().max()) <= 2e-2 * scale and float((a - c).abs().mean()) <= 1e-3 * scale
    assert float((k0 == 7.0).float().mean()) > 0.5 and torch.equal(k0 == 7.0, k1 == 7.0)     # only the token's slot was written


def test_the_norm_in_front_is_refused_beyond_its_widest_row(K):
    # a width of 5,120 (the 32B size) does not fit the kernel's row buffer: the caller is told so and runs the norm itself
    w = torch.zeros(256, 5120, dtype=torch.bfloat16, device=DEV)
    resid = torch.zeros(1, 5120, device=DEV)
    assert not K.skinny_norm_ok(resid, None, w)
    with pytest.raises(K.KernelError):
        K.gemm_skinny_norm(resid, None, torch.ones(5120, device=DEV), 1e-6, w)


def test_gemm_skinny_refuses_misaligned_operands(K):
    a = torch.randn(4, 172).bfloat16().to(DEV)          # K = 172 is no multiple of 8
    w = torch.randn(64, 172).bfloat16().to(DEV)
    assert not K.skinny_ok(a, w)
    with pytest.raises(K.KernelError):
        K.gemm_skinny(a, w)
    # more than 64 rows: small matrices only, and never more than 256
    small, large = torch.randn(64, 64).bfloat16().to(DEV), torch.zeros(4104, 1024, dtype=torch.bfloat16, device=DEV)
    assert K.skinny_ok(torch.randn(65, 64).bfloat16().to(DEV), small)
    assert K.skinny_ok(torch.randn(64, 1024).bfloat16().to(DEV), large)
    assert not K.skinny_ok(torch.randn(65, 1024).bfloat16().to(DEV), large)
    assert not K.skinny_ok(torch.randn(257, 64).bfloat16().to(DEV), small)
    with pytest.raises(K.KernelError):
        K.gemm_skinny(torch.randn(257, 64).bfloat16().to(DEV), small)


def test_the_wrappers_refuse_operands_that_do_not_fit_before_anything_is_launched(K):
    # a kernel trusts the sizes it is given; what does not fit them is refused on the host, by name
    from pico_vllm_amd.ops.attention_fast import FastAttention
    bf, f32, i32 = torch.bfloat16, torch.float32, torch.int32

    def dev(*shape, dtype=f32):
        return torch.zeros(*shape, dtype=dtype, device=DEV)

    def refused(message, fn, *args, **kw):
        with pytest.raises(K.KernelError, match=message):
            fn(*args, **kw)

    T, H, V = 5, 64, 30
    ids, table = dev(T, dtype=i32), dev(V, H)
    refused("GPU only", K.embedding, table.cpu(), ids)
    refused("not supported", K.embedding, table.half(), ids)
    refused("contiguous int32", K.embedding, table, ids.long())
    refused("table must be contiguous", K.embedding, dev(V, 2 * H)[:, ::2], ids)
    refused("out must be", K.embedding, table, ids, out=dev(T, H, dtype=bf))
    refused("softcap", K.softcap, dev(4, 4, dtype=bf), 2.0)
    refused("softcap", K.softcap, dev(4, 4), 0.0)
    resid, w = dev(T, H), dev(H)
    refused("residual stream", K.add_rmsnorm, resid.to(bf), None, w, 1e-6, bf)
    refused("norm weight", K.add_rmsnorm, resid, None, dev(H + 1), 1e-6, bf)
    refused("partial sums must be float32", K.add_rmsnorm, resid, dev(2, T, H, dtype=bf), w, 1e-6, bf)
    refused("shaped like the residual", K.add_rmsnorm, resid, dev(T, H + 8), w, 1e-6, bf)
    refused("rows must be a contiguous int32", K.add_rmsnorm, resid, None, w, 1e-6, bf, rows=dev(2, dtype=torch.int64))
    refused("out has the wrong shape", K.add_rmsnorm, resid, None, w, 1e-6, bf, out=dev(T, H))
    refused("residual_add", K.residual_add, resid, dev(T, H + 8))
    refused("swiglu: input", K.swiglu, dev(T, 7))
    refused("swiglu: out", K.swiglu, dev(T, 8), out=dev(T, 8))
    a, wf = dev(T, H), dev(9, H)
    refused("inner sizes differ", K.gemm_f32, a, dev(9, H + 1))
    refused("w must be float32", K.gemm_f32, a, wf.to(bf))
    refused("bias must be", K.gemm_f32, a, wf, dev(8))
    refused("out has the wrong", K.gemm_f32, a, wf, None, dev(T, 9, dtype=bf))
    ab, wb = dev(T, H, dtype=bf), dev(16, H, dtype=bf)
    refused("inner sizes differ", K.gemm_bf16, ab, dev(16, H + 8, dtype=bf))
    refused("must be bfloat16", K.gemm_bf16, a, wb)
    refused("bias must be", K.gemm_bf16, ab, wb, dev(16, dtype=bf))
    refused("out has the wrong", K.gemm_bf16, ab, wb, None, bf, dev(T, 16))
    refused("inner sizes differ", K.gemm_skinny, ab, dev(16, H + 8, dtype=bf))
    refused("skinny_ok", K.gemm_skinny, dev(65, H, dtype=bf), dev((1 << 16) + 8, H, dtype=bf))   # many rows, a large matrix
    refused("skinny_ok", K.gemm_skinny, dev(T, 60, dtype=bf), dev(16, 60, dtype=bf))       # K no multiple of 8
    refused("bias must be", K.gemm_skinny, ab, wb, dev(15))
    refused("partial sums", K.gemm_skinny, ab, wb, None, K.EPI_BF16, 2)
    refused("even number", K.gemm_skinny, ab, dev(15, H, dtype=bf), None, K.EPI_SWIGLU)
    assert not K.skinny_norm_ok(dev(2, H), None, wb) and not K.skinny_norm_ok(dev(1, H), dev(9, 1, H), wb)
    assert K.skinny_norm_ok(dev(1, H), dev(3, 1, H), wb)
    refused("skinny_norm_ok", K.gemm_skinny_norm, dev(2, H), None, w, 1e-6, wb)
    refused("norm weight", K.gemm_skinny_norm, dev(1, H), None, dev(H + 1), 1e-6, wb)
    refused("even number", K.gemm_skinny_norm, dev(1, H), None, w, 1e-6, dev(15, H, dtype=bf), K.EPI_SWIGLU)
    # rotation and the cache: 2 query heads, 1 kv head of size 32, pages of 8
    nq, nkv, d, Pg = 2, 1, 32, 8
    kc, vc = dev(4, nkv, Pg, d, dtype=bf), dev(4, nkv, d, Pg, dtype=bf)
    qkv, slots, cs = dev(T, (nq + 2 * nkv) * d, dtype=bf), dev(T, dtype=i32), dev(T, d // 2, 2)
    K.rope_kv_store(qkv, cs, slots, kc, vc, nq, nkv, d, d)
    refused("qkv must be contiguous", K.rope_kv_store, dev(T, 100, dtype=bf), cs, slots, kc, vc, nq, nkv, d, d)
    refused("4-dimensional", K.rope_kv_store, qkv, cs, slots, kc[0], vc, nq, nkv, d, d)
    refused("do not fit", K.rope_kv_store, qkv, cs, slots, kc, dev(4, nkv, Pg, d, dtype=bf), nq, nkv, d, d)
    refused("differ in dtype", K.rope_kv_store, qkv, cs, slots, kc.float(), vc.float(), nq, nkv, d, d)
    refused("slots has 5 entries, 6 are needed", K.rope_kv_store, dev(6, (nq + 2 * nkv) * d, dtype=bf), cs, slots, kc, vc, nq, nkv, d, d)
    refused("table of cosines", K.rope_kv_store, qkv, dev(T, d // 2), slots, kc, vc, nq, nkv, d, d)
    refused("table of cosines", K.rope_kv_store, qkv, None, slots, kc, vc, nq, nkv, d, d)
    refused("inv_freq", K.rope_table, slots, dev(4, dtype=bf))
    wq, bq = dev((nq + 2 * nkv) * d, H, dtype=bf), dev((nq + 2 * nkv) * d)
    K.gemm_skinny_rope(ab, wq, bq, cs, slots, kc, vc, nq, nkv, d)
    refused("weight .* is not", K.gemm_skinny_rope, ab, wb, None, cs, slots, kc, vc, nq, nkv, d)
    refused("skinny_ok", K.gemm_skinny_rope, a, wq.float(), bq, cs, slots, kc, vc, nq, nkv, d)
    refused("bias must be", K.gemm_skinny_rope, ab, wq, bq[:-1], cs, slots, kc, vc, nq, nkv, d)
    refused("cache must be bfloat16", K.gemm_skinny_rope, ab, wq, bq, cs, slots, kc.float(), vc.float(), nq, nkv, d)
    refused("multiple of 32", K.gemm_skinny_rope, ab, dev(4 * 16, H, dtype=bf), None, dev(T, 8, 2), slots,
            dev(4, 1, Pg, 16, dtype=bf), dev(4, 1, 16, Pg, dtype=bf), 2, 1, 16)
    r1, cs1 = dev(1, H), dev(1, d // 2, 2)
    K.gemm_skinny_rope_norm(r1, None, w, 1e-6, wq, bq, cs1, slots, kc, vc, nq, nkv, d)
    refused("skinny_norm_ok", K.gemm_skinny_rope_norm, dev(2, H), None, w, 1e-6, wq, bq, cs1, slots, kc, vc, nq, nkv, d)
    refused("weight .* is not", K.gemm_skinny_rope_norm, r1, None, w, 1e-6, wb, None, cs1, slots, kc, vc, nq, nkv, d)
    refused("bias must be", K.gemm_skinny_rope_norm, r1, None, w, 1e-6, wq, bq[:-1], cs1, slots, kc, vc, nq, nkv, d)
    refused("cache must be bfloat16", K.gemm_skinny_rope_norm, r1, None, w, 1e-6, wq, bq, cs1, slots, kc.float(), vc.float(), nq, nkv, d)
    refused("multiple of 32", K.gemm_skinny_rope_norm, r1, None, w, 1e-6, dev(4 * 16, H, dtype=bf), None, dev(1, 8, 2), slots,
            dev(4, 1, Pg, 16, dtype=bf), dev(4, 1, 16, Pg, dtype=bf), 2, 1, 16)
    # attention
    q, bt, pos, seq = dev(T, nq * d, dtype=bf), dev(1, 4, dtype=i32), dev(T, dtype=i32), dev(T, dtype=i32)
    K.paged_attention_ref(q, kc, vc, bt, pos, seq, nq, nkv, d, 0.1)
    refused("unit stride", K.paged_attention_ref, q[:, :d], kc, vc, bt, pos, seq, nq, nkv, d, 0.1)
    refused("differ in dtype", K.paged_attention_ref, q.float(), kc, vc, bt, pos, seq, nq, nkv, d, 0.1)
    refused("block_table", K.paged_attention_ref, q, kc, vc, bt.long(), pos, seq, nq, nkv, d, 0.1)
    refused("out has the wrong", K.paged_attention_ref, q, kc, vc, bt, pos, seq, nq, nkv, d, 0.1, out=dev(T, nq * d))
    fa = FastAttention(nq, nkv, d)
    ctxl, cu = torch.ones(T, dtype=i32, device=DEV), torch.arange(T + 1, dtype=i32, device=DEV)
    bt5 = dev(T, 4, dtype=i32)
    fa.decode(q, kc, vc, bt5, ctxl, T, 0.1, 1)
    refused("one query token per sequence", fa.decode, q, kc, vc, bt5, ctxl, T - 1, 0.1, 1)
    refused("at most 32 query heads", FastAttention(33, 1, d).decode, dev(T, 33 * d, dtype=bf), kc, vc, bt5, ctxl, T, 0.1, 1)
    refused("bfloat16 tensors", fa.decode, q.float(), kc, vc, bt5, ctxl, T, 0.1, 1)
    refused("unit stride", fa.prefill, q[:, :d], kc, vc, bt5, cu, ctxl, T, 0.1)
    refused("block_table", fa.prefill, q, kc, vc, bt, cu, ctxl, T, 0.1)              # a table for one sequence, five given
    refused("sequence metadata", fa.prefill, q, kc, vc, bt5, cu.long(), ctxl, T, 0.1)
    refused("sequence metadata", fa.decode, q, kc, vc, bt5, ctxl[:2], T, 0.1, 1)
    # sampling
    logits, t1 = dev(3, V), dev(3)
    K.sample(logits, t1, t1 + 1, t1)
    refused("logits must be float32", K.sample, logits.to(bf), t1, t1, t1)
    refused("top_p must be", K.sample, logits, t1, dev(2), t1)
    refused("out must be", K.sample, logits, t1, t1, t1, dev(3))
    work = K.argmax_workspace(3, DEV)
    K.argmax(logits, dev(3, dtype=i32), work)
    refused("logits must be float32", K.argmax, logits.to(bf), dev(3, dtype=i32), work)
    refused("out must be", K.argmax, logits, dev(2, dtype=i32), work)
    refused("workspace", K.argmax, logits, dev(3, dtype=i32), K.argmax_workspace(2, DEV))
    torch.cuda.synchronize()


def test_the_library_product_with_its_tuner_on_gives_the_same_and_hands_the_mode_back():
    # rows in multiples of 512 are timed by the library's tuner when asked; other counts take its default; off again
    # torch's own mode is as it was
    from pico_vllm_amd.ops import linear as L
    g = torch.Generator().manual_seed(0)
    x, w, b = torch.randn(1024, 320, generator=g).bfloat16(), torch.randn(200, 320, generator=g).bfloat16(), torch.randn(200, generator=g)
    lin = L.Linear(w.to(DEV), b.to(DEV))
    want = x.double() @ w.double().T + b.bfloat16().double()
    before = lin(x.to(DEV))
    assert not torch.cuda.tunable.is_enabled()
    L.set_library_tuning(True)
    try:
        tuned = lin(x.to(DEV))                    # 1,024 rows: tuned
        assert torch.cuda.tunable.is_enabled() and torch.cuda.tunable.tuning_is_enabled()
        other = lin(x[:300].to(DEV))              # 300 rows: the library's default choice, nothing is timed
        assert not torch.cuda.tunable.tuning_is_enabled()
        no_bias = L.Linear(w.to(DEV))(x[:512].to(DEV))
    finally:
        L.set_library_tuning(False)
    assert not torch.cuda.tunable.is_enabled() and not torch.cuda.tunable.tuning_is_enabled()
    for got, ref in ((before, want), (tuned, want), (other, want[:300]), (no_bias, want[:512] - b.bfloat16().double())):
        assert got.dtype == torch.bfloat16
        assert torch.allclose(got.cpu().double(), ref, rtol=1e-2, atol=1e-2 * math.sqrt(320))
