"""Builds paged-KV test cases: a shared pool whose pages are handed out from a seeded random permutation
(raw pages, then compressed-row pages, per request), as the serving engine upstream does with its block manager
(upstream inference.ipynb cell 1 `get_tabels` uses sequential pages; the permutation is the harder case)."""
import torch

from oracle import nsa_oracle as O


def build_pool(ctx_lens, KH, D, VD, page=128, seed=0, kernel=32, stride=16, extra_pages=3, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    n_raw = [(L + page - 1) // page for L in ctx_lens]
    ys = [max((L - kernel) // stride + 1, 0) for L in ctx_lens]
    n_cmp = [max((y + page - 1) // page, 1) for y in ys]
    P = sum(n_raw) + sum(n_cmp) + extra_pages
    perm = torch.randperm(P, generator=g)
    B = len(ctx_lens)
    bt = torch.full((B, max(max(n_raw), 1)), -1, dtype=torch.int32)
    cbt = torch.full((B, max(n_cmp)), -1, dtype=torch.int32)
    pos = 0
    for b in range(B):
        bt[b, :n_raw[b]] = perm[pos:pos + n_raw[b]].to(torch.int32)
        pos += n_raw[b]
        cbt[b, :n_cmp[b]] = perm[pos:pos + n_cmp[b]].to(torch.int32)
        pos += n_cmp[b]
    kc = torch.randn(P, page, KH, D, generator=g).to(dtype)
    vc = torch.randn(P, page, KH, VD, generator=g).to(dtype)
    return dict(k=kc, v=vc, bt=bt, cbt=cbt, ys=ys, page=page, ctx=list(ctx_lens))


def cmp_row_slot(case, b, i):
    page = case["page"]
    return int(case["cbt"][b, i // page]) * page + i % page


def prepool(case, upto_lens, kernel=32, stride=16):
    """Pools (on the CPU, fp32 mean rounded to the cache dtype) the compressed rows that lie entirely inside the
    first upto_lens[b] tokens of each request and writes them to their pool rows."""
    for name in ("k", "v"):
        cache = case[name]
        flat = cache.view(-1, cache.shape[2], cache.shape[3])
        for b, L in enumerate(upto_lens):
            y = max((L - kernel) // stride + 1, 0)
            if y == 0:
                continue
            xs = O.gather_rows(cache, case["bt"][b], case["ctx"][b]).float()
            for i in range(y):
                flat[cmp_row_slot(case, b, i)] = xs[i * stride:i * stride + kernel].mean(0).to(cache.dtype)


def prefill_slot_mapping(case, cached_lens, kernel=32, stride=16):
    """One entry per compressed row of every request (y_cu order): destination row, or -1 for rows that were
    already pooled from the cached prefix."""
    slots = []
    for b, L in enumerate(case["ctx"]):
        y_old = max((cached_lens[b] - kernel) // stride + 1, 0)
        for i in range(case["ys"][b]):
            slots.append(-1 if i < y_old else cmp_row_slot(case, b, i))
    ycu = [0]
    for y in case["ys"]:
        ycu.append(ycu[-1] + y)
    return torch.tensor(slots, dtype=torch.int32), torch.tensor(ycu, dtype=torch.int32)


def decode_slot_mapping(case, kernel=32, stride=16):
    """-1 unless the newest token completes a compressed row (context_len % stride == 0 and len >= kernel)."""
    out = []
    for b, L in enumerate(case["ctx"]):
        if L >= kernel and (L - kernel) % stride == 0:
            out.append(cmp_row_slot(case, b, case["ys"][b] - 1))
        else:
            out.append(-1)
    return torch.tensor(out, dtype=torch.int32)
