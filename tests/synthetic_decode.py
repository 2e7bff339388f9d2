"""Synthetic paged-KV batches for the decode benchmark and the full-size tests (test and benchmark scaffolding, not
part of the flash_nsa package): a pool whose pages are handed out from a seeded
random permutation (raw pages, then compressed-row pages, per request), random K/V/q/gates, and the slot of the
compressed row that the newest token completes."""
import torch


def build_decode_case(dev, B=64, QH=64, KH=4, D=128, page=256, lo=4096, hi=32768, seed=3, staggered_pools=True):
    """staggered_pools: the pools come from allocate_kv_pools (V pool staggered against the K pool, what a serving
    engine built on this package allocates); False: two separate tensors whose bases coincide modulo 1 KB, which is
    what an allocation of one pool right after the other gives."""
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(lo, hi + 1, (B,), generator=g).tolist()
    ys = [max((L - 32) // 16 + 1, 0) for L in lens]
    n_raw = [(L + page - 1) // page for L in lens]
    n_cmp = [max((y + page - 1) // page, 1) for y in ys]
    P = sum(n_raw) + sum(n_cmp)
    perm = torch.randperm(P, generator=g)
    bt = torch.full((B, max(n_raw)), -1, dtype=torch.int32)
    cbt = torch.full((B, max(n_cmp)), -1, dtype=torch.int32)
    pos = 0
    for b in range(B):
        bt[b, :n_raw[b]] = perm[pos:pos + n_raw[b]].to(torch.int32)
        pos += n_raw[b]
        cbt[b, :n_cmp[b]] = perm[pos:pos + n_cmp[b]].to(torch.int32)
        pos += n_cmp[b]
    gd = torch.Generator(device=dev).manual_seed(seed)
    k = torch.randn(P, page, KH, D, device=dev, generator=gd, dtype=torch.float32).to(torch.bfloat16)
    v = torch.randn(P, page, KH, D, device=dev, generator=gd, dtype=torch.float32).to(torch.bfloat16)
    if staggered_pools:
        from flash_nsa.inference import allocate_kv_pools
        (ks, vs), = allocate_kv_pools(P, page, KH, D, device=dev)
        ks.copy_(k)
        vs.copy_(v)
        k, v = ks, vs
    q = torch.randn(B, QH, D, device=dev, generator=gd, dtype=torch.float32).to(torch.bfloat16)
    w = torch.randn(B, QH, 3, device=dev, generator=gd, dtype=torch.float32).to(torch.bfloat16)
    slots = []
    for b, L in enumerate(lens):
        if L >= 32 and (L - 32) % 16 == 0:
            i = ys[b] - 1
            slots.append(int(cbt[b, i // page]) * page + i % page)
        else:
            slots.append(-1)
    ctx = torch.tensor(lens, dtype=torch.int32, device=dev)
    return dict(q=q, k=k, v=v, w=w, ctx=ctx, bt=bt.to(dev), cbt=cbt.to(dev),
                slots=torch.tensor(slots, dtype=torch.int32, device=dev), lens=lens, ys=ys, page=page)


def pool_all_rows(c, dev):
    """Pools every compressed row of the cached contexts of a build_case() dict (what earlier steps left behind)."""
    from flash_nsa.inference import mean_pooling_prefill
    B, page = len(c["lens"]), c["page"]
    ycu = torch.zeros(B + 1, dtype=torch.int32)
    ycu[1:] = torch.cumsum(torch.tensor(c["ys"]), 0)
    slots = torch.cat([(c["cbt"][b].cpu()[torch.arange(y) // page].to(torch.int64) * page + torch.arange(y) % page)
                       for b, y in enumerate(c["ys"])]).to(torch.int32).to(dev)
    for cache in (c["k"], c["v"]):
        mean_pooling_prefill(cache, ycu.to(dev), max(c["ys"]), c["bt"], slots)
