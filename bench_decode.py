"""Paged-KV NSA decode benchmark (one query token per request), timed as HIP-graph replays.

Workload (BASELINE.json configs[4]): batch 64, context lengths uniform in [4096, 32768] from seed 3, page size 256,
block tables = slices of a random permutation of the pool, 64 q / 4 kv heads, d=128, bf16 N(0,1), top-16 of
64-token blocks + window 512.  Algorithmic bytes per request of length L: compressed K and V rows once (y*KH*(D+VD)*2; the second read of the
compressed K for the importance pass is an implementation choice and is not counted), 16 selected blocks, the
513 window rows, q + w + o.
"""
import torch

PEAK_HBM_GBS = 8000.0
# bytes per step crossing the L2 <-> memory-side boundary (rocprofv3 --pmc FETCH_SIZE x2.000 + WRITE_SIZE x1.000, the
# factors being what the counters read for a 1 GiB copy), measured for the default case of build_case()
MEASURED_TRAFFIC_DEFAULT_CASE = 334.2e6


def build_case(dev, B=64, QH=64, KH=4, D=128, page=256, lo=4096, hi=32768, seed=3):
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


# Decode attention of one layer with a 4 GiB KV pool, batch = 4 GiB / (S * 4 kv heads * 2 (K,V) * 2 bytes * 128), every
# request at context S, graph replay: microseconds the reference reports on one H800 (upstream README.md:291-300)
REFERENCE_H800_DECODE_US = {4096: 689, 8192: 421, 16384: 279, 32768: 206, 65536: 172, 131072: 160}


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


def decode_sweep(dev, lengths=(4096, 8192, 16384, 32768, 65536, 131072), reps=100):
    """The reference's decode table: fixed 4 GiB KV pool, so the batch shrinks as the context grows (512 requests of
    4K tokens ... 16 requests of 128K tokens).  nsa_decode picks its path itself: one launch per step while the
    batch fills the GPU, the compressed branch cut into parts (two launches) for small batches of long contexts.
    Prints one JSON line per context length."""
    import json
    from flash_nsa import nsa_decode
    from flash_nsa.inference import auto_cmp_splits
    for S in lengths:
        B = (4 << 30) // (S * 4 * 2 * 2 * 128)
        c = build_case(dev, B=B, lo=S, hi=S, seed=5)
        pool_all_rows(c, dev)
        args = (c["q"], c["k"], c["v"], c["w"], c["ctx"], c["bt"], c["slots"], c["cbt"])
        kw = dict(fixed_y_maxlen=max(2048, (S // 16 + 255) // 256 * 256), fixed_num_slc_blocks=max(512, S // 64))
        nsa_decode(*args, **kw)
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            nsa_decode(*args, **kw)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            nsa_decode(*args, **kw)
        for _ in range(10):
            graph.replay()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(reps):
            graph.replay()
        e.record()
        torch.cuda.synchronize()
        us = s.elapsed_time(e) * 1e3 / reps
        nbytes = algorithmic_bytes(c["lens"])
        print(json.dumps({"context": S, "batch": B, "us_per_step": round(us, 1),
                          "cmp_parts": auto_cmp_splits(B, 4, kw["fixed_y_maxlen"]),
                          "algorithmic_gbs": round(nbytes / us / 1e3, 1),
                          "reference_h800_us": REFERENCE_H800_DECODE_US.get(S)}), flush=True)
        del c, args, graph


def algorithmic_bytes(lens, KH=4, D=128, VD=128, QH=64, top_n=16, block=64, window=512):
    tot = 0
    for L in lens:
        y = max((L - 32) // 16 + 1, 0)
        tot += y * KH * (D + VD) * 2
        tot += min(top_n, (L - 1) // block + 1) * block * KH * (D + VD) * 2
        tot += min(L, window + 1) * KH * (D + VD) * 2
        tot += QH * D * 2 + QH * 3 * 2 + QH * VD * 2
    return tot


def decode_bench(dev, reps=200, warmup=20):
    from flash_nsa import nsa_decode
    from flash_nsa.inference import kv_mean_pooling_decode
    c = build_case(dev)
    args = (c["q"], c["k"], c["v"], c["w"], c["ctx"], c["bt"], c["slots"], c["cbt"])
    kw = dict(fixed_y_maxlen=2048, fixed_num_slc_blocks=512)
    # the compressed rows of the cached context are pooled once up front (every row, through the prefill pooling)
    from flash_nsa.inference import mean_pooling_prefill
    ycu = torch.zeros(len(c["lens"]) + 1, dtype=torch.int32)
    ycu[1:] = torch.cumsum(torch.tensor(c["ys"]), 0)
    page = c["page"]
    all_slots = torch.cat([(c["cbt"][b].cpu()[torch.arange(y) // page].to(torch.int64) * page + torch.arange(y) % page)
                           for b, y in enumerate(c["ys"])]).to(torch.int32).to(dev)
    for cache in (c["k"], c["v"]):
        mean_pooling_prefill(cache, ycu.to(dev), max(c["ys"]), c["bt"], all_slots)
    eager = nsa_decode(*args, **kw)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            nsa_decode(*args, **kw)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = nsa_decode(*args, **kw)
    for _ in range(warmup):
        graph.replay()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(reps):
        graph.replay()
    e.record()
    torch.cuda.synchronize()
    us = s.elapsed_time(e) * 1e3 / reps
    same = bool(torch.equal(out, eager))
    # eager (no graph) for comparison
    s.record()
    for _ in range(20):
        nsa_decode(*args, **kw)
    e.record()
    torch.cuda.synchronize()
    eager_us = s.elapsed_time(e) * 1e3 / 20
    nbytes = algorithmic_bytes(c["lens"])
    gbs = nbytes / (us * 1e-6) / 1e9
    res = {"workload": "paged NSA decode, batch 64, ctx uniform [4096,32768] (seed 3), page 256, 64q/4kv heads, "
                       "d=128, bf16, hipGraph replay", "us_per_step": us, "eager_us_per_step": eager_us,
           "graph_equals_eager": same, "algorithmic_bytes": nbytes,
           "roofline": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                        "frac": gbs / PEAK_HBM_GBS, "traffic": MEASURED_TRAFFIC_DEFAULT_CASE}}
    # the same step with the cache write of the newest token's K/V inside the launch (KV-cache writer fused)
    page = c["page"]
    B, KH, D = len(c["lens"]), c["k"].size(2), c["k"].size(3)
    new_k = c["k"].view(-1, KH, D)[[int(c["bt"][b, (L - 1) // page]) * page + (L - 1) % page
                                     for b, L in enumerate(c["lens"])]].clone()
    new_v = c["v"].view(-1, KH, D)[[int(c["bt"][b, (L - 1) // page]) * page + (L - 1) % page
                                     for b, L in enumerate(c["lens"])]].clone()
    raw_slots = torch.tensor([int(c["bt"][b, (L - 1) // page]) * page + (L - 1) % page
                              for b, L in enumerate(c["lens"])], dtype=torch.int32, device=dev)
    kw2 = dict(kw, new_k=new_k, new_v=new_v, slot_mapping=raw_slots)
    out2 = nsa_decode(*args, **kw2)
    torch.cuda.synchronize()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        nsa_decode(*args, **kw2)
    torch.cuda.current_stream().wait_stream(side)
    graph2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph2):
        out2 = nsa_decode(*args, **kw2)
    for _ in range(warmup):
        graph2.replay()
    torch.cuda.synchronize()
    s.record()
    for _ in range(reps):
        graph2.replay()
    e.record()
    torch.cuda.synchronize()
    res["us_per_step_with_cache_write"] = s.elapsed_time(e) * 1e3 / reps
    res["cache_write_equals_plain"] = bool(torch.equal(out2, eager))
    return res


def cache_writer_bench(dev, reps=50):
    """KV-cache writer on the chunked-prefill configuration (16 requests, cached prefix uniform in [0,16384] from
    seed 2, 2048 new tokens each, page 256, 4 kv heads, d=128): plain scatter, and the scatter fused with the pooling
    of the compressed rows the chunk completes, against the three separate launches."""
    from flash_nsa.inference import (PageTableBuilder, allocate_kv_pools, store_kvcache,
                                     store_kvcache_and_pool_prefill, mean_pooling_prefill)
    KH, D, page, chunk = 4, 128, 256, 2048
    g = torch.Generator().manual_seed(2)
    cached = torch.randint(0, 16385, (16,), generator=g).tolist()
    (kc, vc), = allocate_kv_pools(2000, page, KH, D, device=dev)
    kc.normal_()
    vc.normal_()
    b = PageTableBuilder(2000, page)
    ids = list(range(16))
    b.prefill(ids, [max(c, 1) for c in cached], device=dev)
    st = b.prefill(ids, [chunk] * 16, device=dev)
    t = 16 * chunk
    gd = torch.Generator(device=dev).manual_seed(2)
    key = torch.randn(t, KH, D, device=dev, generator=gd, dtype=torch.float32).to(torch.bfloat16)
    val = torch.randn(t, KH, D, device=dev, generator=gd, dtype=torch.float32).to(torch.bfloat16)

    def timeit(fn):
        fn()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(reps):
            fn()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) * 1e3 / reps

    pool_args = (st["y_cu_seqlens"], st["y_maxlen"], st["block_tables"], st["cmp_slot_mapping"])
    store_us = timeit(lambda: store_kvcache(key, val, kc, vc, st["slot_mapping"]))
    pool_us = timeit(lambda: (mean_pooling_prefill(kc, *pool_args), mean_pooling_prefill(vc, *pool_args)))
    fused_us = timeit(lambda: store_kvcache_and_pool_prefill(
        key, val, kc, vc, st["x_cu_seqlens"], st["x_maxlen"], st["context_lens"], st["slot_mapping"],
        st["y_cu_seqlens"], st["y_maxlen"], st["cmp_slot_mapping"], st["block_tables"]))
    nbytes = 2 * 2 * t * KH * D * 2  # K and V rows, read once and written once
    return {"workload": "store_kvcache of 16 x 2048 new tokens, 4 kv heads, d=128, bf16, page 256",
            "store_us": store_us, "algorithmic_bytes": nbytes,
            "roofline": {"bound": "hbm", "achieved": nbytes / (store_us * 1e-6) / 1e9, "peak": PEAK_HBM_GBS,
                         "unit": "GB/s", "frac": nbytes / (store_us * 1e-6) / 1e9 / PEAK_HBM_GBS, "traffic": None},
            "store_then_pool_us": store_us + pool_us, "fused_store_pool_us": fused_us}


if __name__ == "__main__":
    import json
    import os
    import sys
    root = os.path.dirname(os.path.abspath(__file__))
    sys.path.insert(0, os.path.join(root, "scalable-flash-native-sparse-attention_amd"))
    print(json.dumps({"decode": decode_bench(torch.device("cuda:0")),
                      "cache_writer": cache_writer_bench(torch.device("cuda:0"))}))


if __name__ == "__main__":
    import argparse
    import json
    import os
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)),
                                    "scalable-flash-native-sparse-attention_amd"))
    ap = argparse.ArgumentParser()
    ap.add_argument("--sweep", action="store_true", help="context-length sweep with a fixed 4 GiB KV pool")
    a = ap.parse_args()
    device = torch.device("cuda:0")
    if a.sweep:
        decode_sweep(device)
    else:
        print(json.dumps(decode_bench(device)))
