"""Helpers shared by the GPU tests."""
import torch

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    """(rtol, atol) for one kernel's output against a float32 reference of the same op:
    float32 differs by summation order only; bfloat16 rounds inputs and output to 8 bits."""
    return (1e-5, 1e-5) if dtype == torch.float32 else (2e-2, 2e-2)


def paged_cache(k_seqs, v_seqs, P, num_pages, dtype, seed=0, garbage=True):
    """Scatter whole sequences of keys/values ([N, nkv, d] each) into pages in random physical
    order.  Returns K [pages, nkv, P, d], V [pages, nkv, d, P], block_table int32 [B, maxp].
    Unused pages and the tails of last pages hold garbage, which nothing may read."""
    nkv, d = k_seqs[0].shape[1:]
    g = torch.Generator().manual_seed(seed)
    if garbage:
        K = torch.randn(num_pages, nkv, P, d, generator=g) * 50
        V = torch.randn(num_pages, nkv, d, P, generator=g) * 50
    else:
        K, V = torch.zeros(num_pages, nkv, P, d), torch.zeros(num_pages, nkv, d, P)
    perm = torch.randperm(num_pages, generator=g).tolist()
    need = [-(-k.shape[0] // P) for k in k_seqs]
    assert sum(need) <= num_pages
    bt = torch.full((len(k_seqs), max(need)), -1, dtype=torch.int32)
    for b, (k, v) in enumerate(zip(k_seqs, v_seqs)):
        for j in range(need[b]):
            page = perm.pop()
            bt[b, j] = page
            n = min(P, k.shape[0] - j * P)
            K[page, :, :n, :] = k[j * P:j * P + n].transpose(0, 1)
            V[page, :, :, :n] = v[j * P:j * P + n].permute(1, 2, 0)
    return K.to(DEV, dtype), V.to(DEV, dtype), bt.to(DEV)


def flat_batch(new_lens, prefix_lens):
    """positions and token_seq (int32 on the GPU) of a batch whose sequence b brings new_lens[b]
    tokens after prefix_lens[b] cached ones."""
    pos, seq = [], []
    for b, (n, p) in enumerate(zip(new_lens, prefix_lens)):
        pos += list(range(p, p + n))
        seq += [b] * n
    return (torch.tensor(pos, dtype=torch.int32, device=DEV), torch.tensor(seq, dtype=torch.int32, device=DEV))
