"""Benchmark of the NSA hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--seq-len T] [--no-cpu] [--no-decode] [--single-stream]
    python bench.py --sweep 4096,8192,16384,32768,65536,131072,262144,524288,1048576

A step is one forward+backward of the NSA core (NSACore: mean K-compression, sigmoid-mul V-compression,
kernel 32 / stride 16 / block 64 / top-16 / window 512) on one causal sequence of T=65536 tokens,
64 q-heads / 4 kv-heads / head dim 128, bf16, synthetic N(0,1) inputs resident in HBM.
Prints ONE JSON line: whole-step throughput in algorithmic TFLOP/s, per-stage milliseconds measured with HIP
events on the launch stream, the roofline of the dominant kernel, and the CPU oracle timed on the host.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "scalable-flash-native-sparse-attention_amd"))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
# Bytes per launch crossing the L2 <-> memory-side boundary (rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE, each scaled by
# what the same counter reads for a 1 GiB copy: x2.000 and x1.000), measured on the T=65536 workload of this file;
# reported as roofline.traffic for that workload only.
MEASURED_TRAFFIC_T64K = {
    "cmp_dkdv": 34.26e9, "slc_dq": 75.58e9, "slc_fwd": 73.54e9, "slc_dkdv": 36.38e9, "cmp_dq": 7.21e9,
    "topk": 2.30e9, "cmp_fwd": 2.25e9, "swa_dkdv": 11.39e9, "swa_dq": 6.54e9, "swa_fwd": 3.24e9,
}
PEAK_HBM_GBS = 8000.0


def branch_counts(lens, kernel=32, stride=16, block=64, top_n=16, window=512):
    """(N_c, N_s, N_w): visible (query, key) pairs per q-head of the three branches, summed over sequences."""
    import numpy as np
    nc = ns = nw = 0
    for L in lens:
        t = np.arange(L, dtype=np.int64)
        y = max((L - kernel) // stride + 1, 0)
        nc += int(np.clip((t - (kernel - 1)) // stride + 1, 0, y).sum())
        ns += int((block * np.minimum(top_n, t // block + 1)).sum())
        nw += int(np.minimum(t + 1, window + 1).sum())
    return nc, ns, nw


def stage_flops(lens, QH, D, VD, **kw):
    nc, ns, nw = branch_counts(lens, **kw)
    f = dict(cmp_fwd=QH * 2 * (D + VD) * nc, topk=QH * 2 * D * nc, slc_fwd=QH * 2 * (D + VD) * ns,
             swa_fwd=QH * 2 * (D + VD) * nw)
    # backward: S, dP, dV, dK (2.0x forward) are attributed to the dk/dv kernel, dQ (0.5x) to the dq kernel;
    # the dq kernel's own recomputation of S and dP is overhead and not counted
    for br in ("cmp", "slc", "swa"):
        f[br + "_dkdv"] = 2.0 * f[br + "_fwd"]
        f[br + "_dq"] = 0.5 * f[br + "_fwd"]
    f["fwd_total"] = f["cmp_fwd"] + f["topk"] + f["slc_fwd"] + f["swa_fwd"]
    f["bwd_total"] = 2.5 * (f["cmp_fwd"] + f["slc_fwd"] + f["swa_fwd"])
    return f


class StageTimer:
    """HIP-event timing of named stages on the current stream."""

    def __init__(self):
        self.events = []

    def run(self, name, fn):
        import torch
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        out = fn()
        e.record()
        self.events.append((name, s, e))
        return out

    def summary(self):
        import torch
        torch.cuda.synchronize()
        acc = {}
        for name, s, e in self.events:
            acc.setdefault(name, []).append(s.elapsed_time(e))
        return {k: sum(v) / len(v) for k, v in acc.items()}


def staged_step(timer, q, k, v, w, wv, do, sm_scale):
    """The same launches as NSAFunction.forward/backward, stage by stage under event timers."""
    import torch
    from flash_nsa.ops.compress_kv import mean_pooling_fwd, construct_block_fwd, construct_block_bwd, mean_pooling_bwd
    from flash_nsa.ops.act import sigmoid_mul_fwd, sigmoid_mul_bwd
    from flash_nsa.ops.compress_attn import cmp_attn_fwd, cmp_attn_bwd
    from flash_nsa.ops.topk import slc_topk_indices, get_bind_from_find
    from flash_nsa.ops.select_attn import slc_attn_fwd, slc_attn_bwd
    from flash_nsa.ops.sliding_window_attention import swa_fwd, swa_bwd
    from flash_nsa.ops.combine import combine_fwd, combine_bwd
    from flash_nsa import _lib
    from flash_nsa.utils import NSAHelper as H
    from flash_nsa.modules.megatron_level_nsa import _store_into

    R = timer.run
    cmp_k = R("pool_k", lambda: mean_pooling_fwd(k))
    win_v = R("im2col_v", lambda: construct_block_fwd(v))
    hid_v = R("gemm_cmp_v", lambda: torch.matmul(win_v.flatten(-2, -1), wv.t()))
    cmp_v = R("sigmoid_mul", lambda: sigmoid_mul_fwd(hid_v))
    cmp_o, cmp_lse = R("cmp_fwd", lambda: cmp_attn_fwd(q, cmp_k, cmp_v, sm_scale=sm_scale))
    topk, _ = R("topk", lambda: slc_topk_indices(q, cmp_k, cmp_lse, sm_scale=sm_scale))
    slc_o, slc_lse = R("slc_fwd", lambda: slc_attn_fwd(q, k, v, topk, sm_scale=sm_scale))
    swa_o, swa_lse = R("swa_fwd", lambda: swa_fwd(q, k, v, sm_scale=sm_scale))
    R("combine_fwd", lambda: combine_fwd(cmp_o, slc_o, swa_o, w))

    dcmp_o, dslc_o, dswa_o, dw, delta = R("combine_bwd", lambda: combine_bwd(cmp_o, slc_o, swa_o, w, do, True))
    dq = torch.zeros(q.shape, device=q.device, dtype=torch.float32)
    T, QH, D = q.shape
    _, KH, VD = v.shape

    def common(kk, vv, lse, lse_st, lse_sh, dlt, dout):
        return (q.data_ptr(), q.stride(0), q.stride(1), kk.data_ptr(), kk.stride(0), kk.stride(1), vv.data_ptr(),
                vv.stride(0), vv.stride(1), dout.data_ptr(), dout.stride(0), dout.stride(1), lse.data_ptr(), lse_st,
                lse_sh, dlt.data_ptr(), dlt.stride(0), dlt.stride(1))

    dk = torch.empty(T, KH, D, device=q.device, dtype=torch.float32)
    dv = torch.empty(T, KH, VD, device=q.device, dtype=torch.float32)
    cs = common(k, v, swa_lse, swa_lse.stride(0), swa_lse.stride(1), delta[2], dswa_o)
    # dq modes as in the fused backward: the selected branch stores (1), the window branch adds (2)
    R("swa_dq", lambda: _lib.call("nsa_swa_bwd_dq", *cs, dq.data_ptr(), dq.stride(0), dq.stride(1), 2,
                                  H.x_cu_seqlens.data_ptr(), H.batch, H.x_maxlen, QH, KH, D, VD, H.window_size,
                                  sm_scale, _lib.stream_ptr()))
    R("swa_dkdv", lambda: _lib.call("nsa_swa_bwd_dkdv", *cs, dk.data_ptr(), dk.stride(0), dk.stride(1),
                                    dv.data_ptr(), dv.stride(0), dv.stride(1), 1, H.x_cu_seqlens.data_ptr(), H.batch,
                                    H.x_maxlen, QH, KH, D, VD, H.window_size, sm_scale, _lib.stream_ptr()))
    cl = common(k, v, slc_lse, slc_lse.stride(0), slc_lse.stride(1), delta[1], dslc_o)
    R("slc_dq", lambda: _lib.call("nsa_slc_attn_bwd_dq", *cl, topk.data_ptr(), topk.stride(0), topk.stride(1),
                                  dq.data_ptr(), dq.stride(0), dq.stride(1), 1, H.x_cu_seqlens.data_ptr(), H.batch,
                                  H.x_maxlen, QH, KH, D, VD, H.block_size, topk.size(-1), sm_scale, _lib.stream_ptr()))
    bind = R("inverse_index", lambda: get_bind_from_find(topk))
    R("slc_dkdv", lambda: _lib.call("nsa_slc_attn_bwd_dkdv", *cl, dk.data_ptr(), dk.stride(0), dk.stride(1),
                                    dv.data_ptr(), dv.stride(0), dv.stride(1), H.x_cu_seqlens.data_ptr(),
                                    H.k_cu_seqlens.data_ptr(), H.blk_seq.data_ptr(), bind["csr_off"].data_ptr(),
                                    bind["csr_tok"].data_ptr(), bind["item_off"].data_ptr(), bind["nblk"],
                                    bind["chunk_tokens"], bind["n_items_bound"], H.batch, QH, KH, D, VD,
                                    H.block_size, sm_scale, _lib.stream_ptr()))
    cc = common(cmp_k, cmp_v, cmp_lse, cmp_lse.stride(1), cmp_lse.stride(0), delta[0], dcmp_o)
    dq_out = torch.empty_like(q)  # the last dq kernel adds the fp32 partial sum and stores q's dtype
    R("cmp_dq", lambda: _lib.call("nsa_cmp_attn_bwd_dq_final", *cc, dq.data_ptr(), dq.stride(0), dq.stride(1),
                                  dq_out.data_ptr(), dq_out.stride(0), dq_out.stride(1), H.x_cu_seqlens.data_ptr(),
                                  H.y_cu_seqlens.data_ptr(), H.batch, H.x_maxlen, QH, KH, D, VD, H.kernel_size,
                                  H.stride, sm_scale, _lib.stream_ptr()))
    dck = torch.zeros(cmp_k.shape, device=q.device, dtype=torch.float32)
    dcv = torch.zeros(cmp_v.shape, device=q.device, dtype=torch.float32)
    R("cmp_dkdv", lambda: _lib.call("nsa_cmp_attn_bwd_dkdv", *cc, dck.data_ptr(), dck.stride(0), dck.stride(1),
                                    dcv.data_ptr(), dcv.stride(0), dcv.stride(1), H.x_cu_seqlens.data_ptr(),
                                    H.y_cu_seqlens.data_ptr(), H.batch, H.x_maxlen, H.y_maxlen, QH, KH, D, VD,
                                    H.kernel_size, H.stride, 0, sm_scale, _lib.stream_ptr()))
    R("pool_k_bwd", lambda: mean_pooling_bwd(k, dck.to(k.dtype), dk))

    def cmp_v_bwd():
        dhid = sigmoid_mul_bwd(hid_v, dcv.to(v.dtype), inplace=False)
        dwin = torch.matmul(dhid, wv).view(*win_v.shape)
        construct_block_bwd(v, dwin, dv)
        return torch.matmul(dhid.flatten(0, 1).t(), win_v.flatten(-2, -1).flatten(0, 1))

    R("cmp_v_bwd", cmp_v_bwd)


def selected_attention_floor(q, k, v, do, KH, reps=3):
    """Extra, not part of `value`: the selected-attention forward and dQ kernels on two synthetic selection patterns
    of the benchmark shape -- `random` (3 forced blocks + 13 uniformly random earlier blocks per token and kv head:
    what random q / k select, bound by the L2-miss path) and `clustered` (the 13 free blocks drawn from the 64
    nearest: K/V stay in cache, which shows the kernels' own floor).  Milliseconds per launch."""
    import torch
    from flash_nsa.ops.select_attn import slc_attn_fwd, slc_attn_bwd
    T, QH, D = q.shape
    dev = q.device
    g = torch.Generator(device=dev).manual_seed(7)
    cur = torch.arange(T, device=dev) // 64
    forced = torch.stack([torch.zeros_like(cur), cur, cur - 1], -1)[None].expand(KH, T, 3)

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(reps):
            fn()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / reps

    out = {}
    for name in ("random", "clustered"):
        u = torch.rand(KH, T, 13, generator=g, device=dev)
        free = (u * (cur + 1)[None, :, None]).long() if name == "random" else cur[None, :, None] - (u * 64).long()
        topk = torch.cat([forced, free], -1).clamp_(min=0).to(torch.int32).contiguous()
        o, lse = slc_attn_fwd(q, k, v, topk)
        dq = torch.zeros(T, QH, D, device=dev, dtype=torch.float32)
        out[name] = {"slc_fwd_ms": round(timed(lambda: slc_attn_fwd(q, k, v, topk)), 3),
                     "slc_dq_ms": round(timed(lambda: slc_attn_bwd(q, k, v, topk, o, lse, do, dq=dq, parts="dq")), 3)}
    return out


def layer_bench(dev, T, QH, KH, D, reps=20):
    """The step either side of the core: the fused rotary embedding of q and k at the headline shape (an HBM-bound
    kernel: q and k read and written once, the fp32 tables read once), and, for scale, forward+backward of the whole
    attention layer (library GEMM projections with hidden = QH*D, RoPE, core, output projection)."""
    import torch
    from flash_nsa import HFNSA, NSAConfig, fused_apply_rope
    q = torch.randn(1, T, QH, D, device=dev, dtype=torch.bfloat16)
    k = torch.randn(1, T, KH, D, device=dev, dtype=torch.bfloat16)
    ang = torch.arange(T, device=dev, dtype=torch.float32)[:, None] / (
        10000 ** (torch.arange(0, D, 2, device=dev, dtype=torch.float32) / D))[None]
    cos, sin = torch.cat([ang.cos(), ang.cos()], -1)[None], torch.cat([ang.sin(), ang.sin()], -1)[None]

    def timeit(fn, n):
        fn()
        torch.cuda.synchronize()
        s_, e_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s_.record()
        for _ in range(n):
            fn()
        e_.record()
        torch.cuda.synchronize()
        return s_.elapsed_time(e_) / n

    rope_ms = timeit(lambda: fused_apply_rope(q, k, cos, sin, inplace=True), reps)
    nbytes = 2 * (q.numel() + k.numel()) * 2 + 2 * cos.numel() * 4
    out = {"rope_us": rope_ms * 1e3, "rope_algorithmic_bytes": nbytes,
           "rope_roofline": {"bound": "hbm", "achieved": nbytes / (rope_ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                             "unit": "GB/s", "frac": nbytes / (rope_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, "traffic": None}}
    del q, k
    hidden = QH * D
    torch.manual_seed(0)
    layer = HFNSA(NSAConfig(hidden_size=hidden, head_dim=D, num_heads=QH, num_kv_heads=KH)).to(
        device=dev, dtype=torch.bfloat16)
    x = (torch.randn(1, T, hidden, device=dev, dtype=torch.bfloat16) * 0.1).requires_grad_()
    dy = torch.randn(1, T, hidden, device=dev, dtype=torch.bfloat16)

    def step():
        layer(x, (cos, sin)).backward(dy)
        x.grad = None
        for p_ in layer.parameters():
            p_.grad = None

    out["layer_fwd_bwd_ms"] = timeit(step, 3)
    out["layer_workload"] = f"HFNSA layer, hidden {hidden}, one sequence T={T}, mean compression"
    return out


# forward / backward ms the reference reports on one H800 for one causal sequence of this length, 64q/4kv heads,
# d=128, mean compression (upstream README.md:213-237)
REFERENCE_H800_MS = {4096: (1.370, 2.772), 8192: (2.630, 5.571), 16384: (5.660, 12.322), 32768: (13.237, 28.960),
                     65536: (34.162, 73.689), 131072: (101.123, 213.904)}


def length_sweep(lengths, QH=64, KH=4, D=128):
    """Forward and backward time of NSACore (mean compression, as the reference's table) per sequence length; prints
    one JSON line per length.  Lengths of 2^18 and more show that one GPU's memory holds what the reference shards
    over eight (its 1M-token run: 575.6 / 1509.2 ms on 8 GPUs with context parallelism, upstream README.md:275-283)."""
    import torch
    from flash_nsa import NSAConfig, NSACore
    dev = torch.device("cuda:0")
    core = NSACore(NSAConfig(head_dim=D, num_heads=QH, num_kv_heads=KH))
    for T in lengths:
        g = torch.Generator(device=dev).manual_seed(0)
        rnd = lambda *s_: torch.randn(*s_, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
        q, k, v, w, do = rnd(T, QH, D), rnd(T, KH, D), rnd(T, KH, D), rnd(T, QH, 3), rnd(T, QH, D)
        cu = torch.tensor([0, T], device=dev, dtype=torch.int32)
        for t in (q, k, v, w):
            t.requires_grad_()
        reps = 5 if T <= 131072 else 2
        ev = lambda: torch.cuda.Event(enable_timing=True)
        fwd_ms = bwd_ms = 0.0
        torch.cuda.reset_peak_memory_stats()
        for it in range(reps + 1):  # the first pass is a warm-up
            e0, e1, e2 = ev(), ev(), ev()
            e0.record()
            out = core(q, k, v, w, cu)
            e1.record()
            out.backward(do)
            e2.record()
            torch.cuda.synchronize()
            if it:
                fwd_ms += e0.elapsed_time(e1) / reps
                bwd_ms += e1.elapsed_time(e2) / reps
            for t in (q, k, v, w):
                t.grad = None
        fl = stage_flops([T], QH, D, D)
        ref = REFERENCE_H800_MS.get(T)
        print(json.dumps({"seq_len": T, "fwd_ms": round(fwd_ms, 3), "bwd_ms": round(bwd_ms, 3),
                          "fwd_tflops": round(fl["fwd_total"] / fwd_ms / 1e9, 1),
                          "bwd_tflops": round(fl["bwd_total"] / bwd_ms / 1e9, 1),
                          "peak_mem_gib": round(torch.cuda.max_memory_allocated() / 2**30, 2),
                          "reference_h800_fwd_bwd_ms": ref}), flush=True)
        del q, k, v, w, do, out


def cpu_baseline(min_seconds=12.0):
    """Oracle forward+backward of the reference's CPU-runnable case (T=4096, 16 q / 1 kv heads, fp32),
    repeated until `min_seconds` of CPU work have been timed."""
    import torch
    from oracle import nsa_oracle as O
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    T, QH, KH, D = 4096, 16, 1, 128
    g = torch.Generator().manual_seed(0)
    q, k, v, w = [torch.randn(*s, generator=g).requires_grad_() for s in
                  ((T, QH, D), (T, KH, D), (T, KH, D), (T, QH, 3))]
    fwd_s = bwd_s = 0.0
    reps = 0
    while fwd_s + bwd_s < min_seconds and reps < 64:
        for t in (q, k, v, w):
            t.grad = None
        t0 = time.perf_counter()
        o = O.nsa_forward(q, k, v, w, [0, T])
        t1 = time.perf_counter()
        o.backward(torch.ones_like(o))
        t2 = time.perf_counter()
        fwd_s += t1 - t0
        bwd_s += t2 - t1
        reps += 1
    # one more forward, stage by stage: the breakdown upstream prints with HFNSACore(bench=True)
    # (flash_nsa/modules/hf_level_nsa.py:145-158): cmp_k, cmp_v, cmp_o, top_k, slc_o, swa_o, combine
    stage_s = {}

    def timed(name, fn):
        t0 = time.perf_counter()
        out = fn()
        stage_s[name] = round(time.perf_counter() - t0, 4)
        return out

    with torch.no_grad():
        cu, cfg = [0, T], O.OracleConfig()
        ck = timed("cmp_k", lambda: O.mean_pooling(k, cu))
        cv = timed("cmp_v", lambda: O.mean_pooling(v, cu))
        cmp_o, cmp_lse = timed("cmp_o", lambda: O.cmp_attn(q, ck, cv, cu))
        topk = timed("top_k", lambda: O.slc_topk(q, ck, cmp_lse, cu, cfg))
        slc_o, _ = timed("slc_o", lambda: O.slc_attn(q, k, v, topk, cu))
        swa_o, _ = timed("swa_o", lambda: O.swa(q, k, v, cu))
        timed("combine", lambda: O.combine(cmp_o, slc_o, swa_o, w))
    fl = stage_flops([T], QH, D, D)
    total = (fl["fwd_total"] + fl["bwd_total"]) * reps
    return {"value": total / (fwd_s + bwd_s) / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"{reps} forward+backward passes of the CPU oracle, T={T}, {QH}q/{KH}kv heads, d={D}, fp32, "
                      f"torch {torch.__version__} with {torch.get_num_threads()} threads",
            "fwd_s": fwd_s / reps, "bwd_s": bwd_s / reps, "fwd_stage_s": stage_s}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--seq-len", type=int, default=65536)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-decode", action="store_true")
    ap.add_argument("--single-stream", action="store_true",
                    help="keep the backward on one stream (for kernel traces: with the default two streams the dq and "
                         "dk/dv kernels overlap and each one's traced duration is stretched by the other)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one plain 1 GiB device-to-device copy kernel, so that a counter run of this "
                         "command holds a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE with")
    ap.add_argument("--decode-leg", type=str, default="all", choices=["all", "hot", "cold", "unstaggered", "cache-write"],
                    help="run only this leg of the decode benchmark (for kernel traces that should reproduce one "
                         "reported figure)")
    ap.add_argument("--decode-only", action="store_true", help="skip the training step (with --decode-leg)")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the labelled extras that launch the step's kernels on other inputs (for kernel traces "
                         "and counter runs, whose per-kernel averages should cover the benchmark step only)")
    ap.add_argument("--sweep", type=str, default=None,
                    help="comma-separated sequence lengths: print forward / backward times per length and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (--gpus 1); multi-GPU sharding is a design note only",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from flash_nsa import NSAConfig, NSACore
    from flash_nsa import _lib
    _lib.LIB.load()  # fail loudly if the HIP library is missing
    if args.single_stream:
        from flash_nsa.modules import megatron_level_nsa
        megatron_level_nsa.OVERLAP_STREAMS = False
    if args.sweep:
        length_sweep([int(x) for x in args.sweep.split(",")])
        return
    dev = torch.device("cuda:0")
    if args.decode_only:
        from bench_decode import decode_bench
        print(json.dumps({"decode": decode_bench(dev, leg=args.decode_leg)}))
        return
    T, QH, KH, D = args.seq_len, 64, 4, 128
    g = torch.Generator(device=dev).manual_seed(0)
    rnd = lambda *s: torch.randn(*s, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    q, k, v, w, do = rnd(T, QH, D), rnd(T, KH, D), rnd(T, KH, D), rnd(T, QH, 3), rnd(T, QH, D)
    cu = torch.tensor([0, T], device=dev, dtype=torch.int32)
    cfg = NSAConfig(head_dim=D, num_heads=QH, num_kv_heads=KH, cmp_k_method="mean", cmp_v_method="sigmoid-mul")
    torch.manual_seed(0)
    core = NSACore(cfg).to(device=dev, dtype=torch.bfloat16)
    for t in (q, k, v, w):
        t.requires_grad_()

    def step():
        for t in (q, k, v, w):
            t.grad = None
        core.cmp_v_weight.grad = None
        out = core(q, k, v, w, cu)
        out.backward(do)
        return out

    if args.calibrate_copy:
        src = torch.ones(1 << 29, device=dev, dtype=torch.bfloat16)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # forward-only and per-stage times (HIP events on the launch stream)
    with torch.no_grad():
        core(q, k, v, w, cu)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            core(q, k, v, w, cu)
        torch.cuda.synchronize()
        fwd_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        timer = StageTimer()
        qd, kd, vd, wd = q.detach(), k.detach(), v.detach(), w.detach()
        staged_step(StageTimer(), qd, kd, vd, wd, core.cmp_v_weight.detach(), do, core.sm_scale)  # warm
        for _ in range(max(args.steps, 3)):
            staged_step(timer, qd, kd, vd, wd, core.cmp_v_weight.detach(), do, core.sm_scale)
        stages = timer.summary()

    fl = stage_flops([T], QH, D, D)
    total_flops = fl["fwd_total"] + fl["bwd_total"]
    mfma_stages = {s: stages[s] for s in stages if s in fl}
    dom = max(mfma_stages, key=mfma_stages.get)
    achieved = fl[dom] / (stages[dom] * 1e-3) / 1e12
    traffic = MEASURED_TRAFFIC_T64K.get(dom) if T == 65536 else None
    result = {
        "metric": "NSA fwd+bwd ms & TFLOP/s @T=64K bf16; paged decode us/step bs64 ctx<=32K",
        "value": total_flops / (ms_per_step * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"NSA forward+backward, one causal sequence T={T}, 64q/4kv heads, d=128, mean K / "
                               "sigmoid-mul V compression (kernel 32, stride 16), block 64, top-16, window 512",
                   "seq_len": T, "q_heads": QH, "kv_heads": KH, "head_dim": D},
        "fwd_ms": fwd_ms, "bwd_ms": ms_per_step - fwd_ms,
        "fwd_tflops": fl["fwd_total"] / (fwd_ms * 1e-3) / 1e12,
        "algorithmic_tflop": {"fwd": fl["fwd_total"] / 1e12, "bwd": fl["bwd_total"] / 1e12},
        "stage_ms": {k_: round(v_, 4) for k_, v_ in stages.items()},
        "stage_tflops": {s: round(fl[s] / (stages[s] * 1e-3) / 1e12, 1) for s in mfma_stages},
        # fraction of the bf16 MFMA peak of every matrix-bound stage kernel (the worst kernel, not only the longest)
        "stage_frac": {s: round(fl[s] / (stages[s] * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4) for s in mfma_stages},
        "roofline": {"bound": "mfma", "kernel": dom, "achieved": achieved, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / PEAK_BF16_TFLOPS, "traffic": traffic,
                     # the whole step against the same peak
                     "step_frac": total_flops / (ms_per_step * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
                     "fwd_frac": fl["fwd_total"] / (fwd_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS},
    }
    # the same step with dK / dV summed in a run-independent order (NSAHelper.set_deterministic)
    from flash_nsa import NSAHelper
    NSAHelper.set_deterministic(True)
    try:
        step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        result["ms_per_step_deterministic"] = (time.perf_counter() - t0) * 1e3 / args.steps
    finally:
        NSAHelper.set_deterministic(False)
    if not args.no_extras:
        with torch.no_grad():
            result["selected_attention_by_selection_pattern"] = selected_attention_floor(q.detach(), k.detach(),
                                                                                         v.detach(), do, KH)
    if traffic is not None:
        # the selected-block kernels re-read K/V blocks that fall out of the 4 MB L2 slices: their launch time is
        # set by this memory-side rate rather than by the MFMA work
        result["roofline"]["memory_side_gbs"] = traffic / (stages[dom] * 1e-3) / 1e9
        result["roofline"]["memory_side_frac_of_hbm_peak"] = result["roofline"]["memory_side_gbs"] / PEAK_HBM_GBS
    if not args.no_decode:
        from bench_decode import decode_bench, cache_writer_bench
        result["decode"] = decode_bench(dev, leg=args.decode_leg)
        result["cache_writer"] = cache_writer_bench(dev)
        result["layer"] = layer_bench(dev, T, QH, KH, D)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
