"""Paged-KV NSA decode benchmark (one query token per request), timed as HIP-graph replays.

Workload (BASELINE.json configs[4]): batch 64, context lengths uniform in [4096, 32768] from seed 3, page size 256,
block tables = slices of a random permutation of the pool, 64 q / 4 kv heads, d=128, bf16 N(0,1), top-16 of
64-token blocks + window 512.  Algorithmic bytes per request of length L: compressed K and V rows once (y*KH*(D+VD)*2; the second read of the
compressed K for the importance pass is an implementation choice and is not counted), 16 selected blocks, the
513 window rows, q + w + o.
"""
import os
import sys

import torch

# the synthetic batches are test / benchmark scaffolding and live beside the tests
sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "tests"))

PEAK_HBM_GBS = 8000.0
# bytes per step crossing the L2 <-> memory-side boundary (rocprofv3 --pmc FETCH_SIZE x2.000 + WRITE_SIZE x1.000, the
# factors being what the counters read for a 1 GiB copy), measured for the default case of build_decode_case()
MEASURED_TRAFFIC_DEFAULT_CASE = 331.9e6


# Decode attention of one layer with a 4 GiB KV pool, batch = 4 GiB / (S * 4 kv heads * 2 (K,V) * 2 bytes * 128), every
# request at context S, graph replay: microseconds the reference reports on one H800 (upstream README.md:291-300)
REFERENCE_H800_DECODE_US = {4096: 689, 8192: 421, 16384: 279, 32768: 206, 65536: 172, 131072: 160}


def decode_sweep(dev, lengths=(4096, 8192, 16384, 32768, 65536, 131072), reps=100):
    """The reference's decode table: fixed 4 GiB KV pool, so the batch shrinks as the context grows (512 requests of
    4K tokens ... 16 requests of 128K tokens).  nsa_decode picks its path itself: one launch per step while the
    batch fills the GPU, the compressed branch cut into parts (two launches) for small batches of long contexts.
    Prints one JSON line per context length."""
    import json
    from flash_nsa import nsa_decode
    from flash_nsa.inference import auto_cmp_splits
    from synthetic_decode import build_decode_case, pool_all_rows
    for S in lengths:
        B = (4 << 30) // (S * 4 * 2 * 2 * 128)
        c = build_decode_case(dev, B=B, lo=S, hi=S, seed=5)
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


def _capture(fn):
    """Runs fn on a side stream (so that lazily created state exists), then captures it in a graph."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fn()
    return graph, out


def _time_replays(graphs, reps, warmup):
    """Microseconds per replay, the graphs taken round-robin (one graph: every replay re-reads the same memory)."""
    for i in range(warmup):
        graphs[i % len(graphs)].replay()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for i in range(reps):
        graphs[i % len(graphs)].replay()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) * 1e3 / reps


def decode_bench(dev, reps=500, warmup=100, cold_copies=6, leg="all"):
    """leg: "all", or one of "hot", "cold", "unstaggered", "cache-write" to run that leg alone (a kernel trace of the
    command then holds the launches of one reported figure only).
    Hot: one graph replayed over one batch (its 342 MB of K/V can stay partly in the 256 MB memory-side cache between
    replays).  Cold: `cold_copies` copies of the batch in disjoint memory, one graph each, replayed round-robin, so
    that (cold_copies - 1) x 342 MB of other K/V pass through the caches before a copy is read again: every replay
    streams its K/V from HBM."""
    from flash_nsa import nsa_decode
    from synthetic_decode import build_decode_case, pool_all_rows
    c = build_decode_case(dev)
    pool_all_rows(c, dev)  # the compressed rows of the cached context, as earlier steps left them
    kw = dict(fixed_y_maxlen=2048, fixed_num_slc_blocks=512)

    def args_of(case):
        return (case["q"], case["k"], case["v"], case["w"], case["ctx"], case["bt"], case["slots"], case["cbt"])

    args = args_of(c)
    eager = nsa_decode(*args, **kw)
    torch.cuda.synchronize()
    graph, out = _capture(lambda: nsa_decode(*args, **kw))
    want = lambda name: leg in ("all", name)
    if not want("hot"):
        res = {"workload": "paged NSA decode, batch 64, ctx uniform [4096,32768] (seed 3), page 256, leg " + leg,
               "algorithmic_bytes": algorithmic_bytes(c["lens"])}
        if want("cold"):
            _decode_cold_leg(res, c, graph, out, eager, args_of, kw, reps, cold_copies)
        if want("unstaggered"):
            _decode_unstaggered_leg(res, dev, eager, args_of, kw, reps, warmup)
        if want("cache-write"):
            _decode_cache_write_leg(res, c, dev, args, eager, kw, reps, warmup)
        return res
    us = _time_replays([graph], reps, warmup)
    same = bool(torch.equal(out, eager))
    # eager (no graph) for comparison
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(20):
        nsa_decode(*args, **kw)
    e.record()
    torch.cuda.synchronize()
    eager_us = s.elapsed_time(e) * 1e3 / 20
    nbytes = algorithmic_bytes(c["lens"])
    gbs = nbytes / (us * 1e-6) / 1e9
    res = {"workload": "paged NSA decode, batch 64, ctx uniform [4096,32768] (seed 3), page 256, 64q/4kv heads, "
                       "d=128, bf16, hipGraph replay; K/V pools from allocate_kv_pools (V pool staggered by 256 B)",
           "us_per_step": us, "eager_us_per_step": eager_us,
           "graph_equals_eager": same, "algorithmic_bytes": nbytes,
           "roofline": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                        "frac": gbs / PEAK_HBM_GBS, "traffic": MEASURED_TRAFFIC_DEFAULT_CASE}}
    # A serving engine captures the decode step of ALL its layers in one graph (nano-vllm does), so consecutive attention
    # launches are nodes of one graph and not separate graph launches: 8 steps of this batch per graph, time per step.
    # The difference to us_per_step is the gap between two graph launches (about 5 us), which is not kernel time.
    steps_per_graph = 8
    gm, outm = _capture(lambda: [nsa_decode(*args, **kw) for _ in range(steps_per_graph)][-1])
    us_m = _time_replays([gm], max(reps // steps_per_graph, 20), max(warmup // steps_per_graph, 5)) / steps_per_graph
    res["us_per_step_8_steps_per_graph"] = us_m
    res["roofline_8_steps_per_graph"] = {"bound": "hbm", "achieved": nbytes / (us_m * 1e-6) / 1e9, "peak": PEAK_HBM_GBS,
                                         "unit": "GB/s", "frac": nbytes / (us_m * 1e-6) / 1e9 / PEAK_HBM_GBS,
                                         "traffic": MEASURED_TRAFFIC_DEFAULT_CASE}
    res["multi_step_graph_equals_eager"] = bool(torch.equal(outm, eager))
    del gm, outm
    if leg == "hot":
        return res
    _decode_cold_leg(res, c, graph, out, eager, args_of, kw, reps, cold_copies)
    _decode_unstaggered_leg(res, dev, eager, args_of, kw, reps, warmup)
    _decode_cache_write_leg(res, c, dev, args, eager, kw, reps, warmup)
    return res


def _decode_cold_leg(res, c, graph, out, eager, args_of, kw, reps, cold_copies):
    """copies of the pool, tables and inputs at other addresses, one graph each, replayed in turn"""
    from flash_nsa import nsa_decode
    nbytes = res["algorithmic_bytes"]
    copies = [c] + [dict(c, **{n: c[n].clone() for n in ("q", "k", "v", "w", "ctx", "bt", "slots", "cbt")})
                    for _ in range(cold_copies - 1)]
    graphs, outs = [graph], [out]
    for cc in copies[1:]:
        a = args_of(cc)
        g, o = _capture(lambda a=a: nsa_decode(*a, **kw))
        graphs.append(g)
        outs.append(o)
    cold_us = _time_replays(graphs, reps // len(graphs) * len(graphs), len(graphs) * 8)
    cold_gbs = nbytes / (cold_us * 1e-6) / 1e9
    res["us_per_step_cold"] = cold_us
    res["cold_copies"] = len(graphs)
    res["cold_equals_hot"] = all(bool(torch.equal(o, eager)) for o in outs)
    res["roofline_cold"] = {"bound": "hbm", "achieved": cold_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                            "frac": cold_gbs / PEAK_HBM_GBS, "traffic": None}


def _decode_unstaggered_leg(res, dev, eager, args_of, kw, reps, warmup):
    """the same batch in pools whose K and V bases coincide modulo 1 KB (one pool allocated right behind the other, as
    upstream's engine does): both streams of a workgroup then share a quarter of the memory channels"""
    from flash_nsa import nsa_decode
    from synthetic_decode import build_decode_case, pool_all_rows
    ca = build_decode_case(dev, staggered_pools=False)
    pool_all_rows(ca, dev)
    aa = args_of(ca)
    nsa_decode(*aa, **kw)
    ga, oa = _capture(lambda: nsa_decode(*aa, **kw))
    res["us_per_step_unstaggered_pools"] = _time_replays([ga], reps, warmup)
    res["unstaggered_equals_staggered"] = bool(torch.equal(oa, eager))


def _decode_cache_write_leg(res, c, dev, args, eager, kw, reps, warmup):
    """the same step with the cache write of the newest token's K/V inside the launch (KV-cache writer fused)"""
    from flash_nsa import nsa_decode
    page = c["page"]
    KH, D = c["k"].size(2), c["k"].size(3)
    newest = [int(c["bt"][b, (L - 1) // page]) * page + (L - 1) % page for b, L in enumerate(c["lens"])]
    new_k = c["k"].view(-1, KH, D)[newest].clone()
    new_v = c["v"].view(-1, KH, D)[newest].clone()
    raw_slots = torch.tensor(newest, dtype=torch.int32, device=dev)
    kw2 = dict(kw, new_k=new_k, new_v=new_v, slot_mapping=raw_slots)
    nsa_decode(*args, **kw2)
    torch.cuda.synchronize()
    graph2, out2 = _capture(lambda: nsa_decode(*args, **kw2))
    res["us_per_step_with_cache_write"] = _time_replays([graph2], reps, warmup)
    res["cache_write_equals_plain"] = bool(torch.equal(out2, eager))


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
        print(json.dumps({"decode": decode_bench(device), "cache_writer": cache_writer_bench(device)}))
