"""Full-size runs of the benchmark configurations, checked through properties that do not need the (dense, CPU)
oracle at that size:
  * causality / prefix consistency: the first rows of a long run equal a run on the prefix alone;
  * packing invariance: a packed variable-length batch equals its sequences run one by one;
  * decode: the fused decode step equals the stage-by-stage path and a single-request prefill of the last token;
  * a slice of the full-size run (first tokens, where the oracle is affordable) against the oracle."""
import pytest
import torch

from oracle import nsa_oracle as O
from gpu_util import assert_close, bar_violations, make_cu

pytestmark = pytest.mark.gpu


def dev_randn(shape, seed, device):
    g = torch.Generator(device=device).manual_seed(seed)
    return torch.randn(*shape, generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)


def test_c1_exact(device):
    """The reference's own CPU-runnable configuration at its own shape: one causal sequence of 4096 tokens, 16
    q-heads on 1 kv head, d = 128, i.i.d. N(0,1) from seed 0, mean compression 32/16, blocks of 64, top-16 with 1
    initial + 2 local forced blocks, window 512.  The device's selection is compared with the oracle's own (sets
    identical except at score ties within 1e-3), the forward with the fp32 oracle, the backward with the oracle
    that keeps the pipeline's rounding points; every element at 2e-2 + 1e-2 |ref| (dk / dv, sums over up to 4096 x 16
    query rows: relative to max(|ref|, rms of the row))."""
    from flash_nsa import NSAConfig, NSACore
    from flash_nsa.ops.compress_kv import mean_pooling_fwd
    from flash_nsa.ops.compress_attn import cmp_attn_fwd
    from flash_nsa.ops.topk import slc_topk_indices
    T, QH, KH, D = 4096, 16, 1, 128
    g = torch.Generator().manual_seed(0)
    q, k, v, w = [torch.randn(*s, generator=g).to(torch.bfloat16) for s in
                  ((T, QH, D), (T, KH, D), (T, KH, D), (T, QH, 3))]
    do = torch.randn(T, QH, D, generator=g).to(torch.bfloat16)
    cu = torch.tensor([0, T], dtype=torch.int32)
    core = NSACore(NSAConfig(head_dim=D, num_heads=QH, num_kv_heads=KH))
    qd, kd, vd, wd = [t.to(device).requires_grad_() for t in (q, k, v, w)]
    out = core(qd, kd, vd, wd, cu.to(device))
    out.backward(do.to(device))
    with torch.no_grad():
        ck, cv = mean_pooling_fwd(kd.detach()), mean_pooling_fwd(vd.detach())
        _, lse = cmp_attn_fwd(qd.detach(), ck, cv)
        topk, _ = slc_topk_indices(qd.detach(), ck, lse)
    cfg = O.OracleConfig()
    rt, imps = O.slc_topk(q.float(), ck.float().cpu(), None, cu, cfg, return_importance=True)
    n_rows, n_diff, n_bad = O.topk_mismatch_report(topk.cpu(), rt, imps, cu, 64, 16, tie_tol=1e-3)
    assert n_rows == T and n_bad == 0 and n_diff <= 4, (n_rows, n_diff, n_bad)
    # at 4096 tokens most rows have more than 16 blocks to choose from: the selection is a real choice
    assert int((torch.arange(T) // 64 + 1 > 16).sum()) > T // 2
    ref_o = O.nsa_forward(q.float(), k.float(), v.float(), w.float(), cu, cfg, topk=topk.cpu())
    assert_close(out, ref_o, "o against the fp32 oracle")
    ref = O.nsa_forward_backward(q.float(), k.float(), v.float(), w.float(), do.float(), cu, cfg, topk=topk.cpu(),
                                 round_dtype=torch.bfloat16, round_mma=True)
    assert_close(out, ref["o"], "o")
    assert_close(qd.grad, ref["dq"], "dq")
    assert_close(kd.grad, ref["dk"], "dk", row_scale=True)
    assert_close(vd.grad, ref["dv"], "dv", row_scale=True)
    assert_close(wd.grad, ref["dw"], "dw")
    # The reference the acceptance bar names: autograd through the plain fp32 oracle, nothing rounded anywhere.  o, dq
    # and dw at the plain bar; dk / dv (sums over up to 4096 x 16 query rows of products that the device rounds to bf16
    # between its kernels) relative to max(|ref|, rms of the row), and the number of their elements that miss the
    # plain, un-scaled bar is stated: at most 1 in 10 000.
    qr, kr, vr, wr = [t.float().requires_grad_() for t in (q, k, v, w)]
    O.nsa_forward(qr, kr, vr, wr, cu, cfg, topk=topk.cpu()).backward(do.float())
    assert_close(qd.grad, qr.grad, "dq against autograd through the fp32 oracle")
    assert_close(wd.grad, wr.grad, "dw against autograd through the fp32 oracle")
    for name, got, want in (("dk", kd.grad, kr.grad), ("dv", vd.grad, vr.grad)):
        assert_close(got, want, f"{name} against autograd through the fp32 oracle", row_scale=True)
        n_out, n_all, worst = bar_violations(got, want)
        print(f"c1 {name} vs fp32 autograd: {n_out}/{n_all} elements outside the un-scaled bar, max |err| {worst:.4g}")
        assert n_out <= 1e-4 * n_all, (name, n_out, n_all, worst)


def test_long_context_packed_batch_beyond_4gib_offsets(device):
    """Upstream documents a single-GPU limit of 256K tokens from 32-bit pointer offsets (README.md:99).  A packed
    batch of 3 x 131072 tokens (64q/4kv, d = 128) puts the third sequence beyond 2^32 bytes and 2^31 elements of q,
    o, dO and dq: its output and dq must equal, bit for bit, the same sequence run alone; dk / dv to the order of
    the fp32 atomic additions."""
    from flash_nsa import NSAConfig, NSACore
    L, QH, KH, D = 131072, 64, 4, 128
    T = 3 * L
    assert 2 * L * QH * D * 2 >= 2 ** 32 and 2 * L * QH * D >= 2 ** 31
    core = NSACore(NSAConfig(head_dim=D, num_heads=QH, num_kv_heads=KH))
    q, k, v, w, do = [dev_randn(s, 30 + i, device) for i, s in
                      enumerate([(T, QH, D), (T, KH, D), (T, KH, D), (T, QH, 3), (T, QH, D)])]

    def run(sl, cu):
        ts = [t[sl].clone().requires_grad_() for t in (q, k, v, w)]
        o = core(*ts, torch.tensor(cu, dtype=torch.int32, device=device))
        o.backward(do[sl])
        return [o.detach()] + [t.grad for t in ts]

    packed = run(slice(0, T), [0, L, 2 * L, T])
    assert all(torch.isfinite(t[2 * L:]).all() for t in packed)
    third = [t[2 * L:].clone() for t in packed]
    first = [t[:L].clone() for t in packed]
    del packed
    torch.cuda.empty_cache()
    for name, got, sl in (("third", third, slice(2 * L, T)), ("first", first, slice(0, L))):
        single = run(sl, [0, L])
        assert torch.equal(got[0], single[0]), f"{name} sequence: forward differs from the sequence run alone"
        assert torch.equal(got[1], single[1]), f"{name} sequence: dq differs"
        assert_close(got[2], single[2], f"{name} sequence: dk", atol=2e-3, rtol=8e-3, row_scale=True)
        assert_close(got[3], single[3], f"{name} sequence: dv", atol=2e-3, rtol=8e-3, row_scale=True)
        assert torch.equal(got[4], single[4]), f"{name} sequence: dw differs"
        del single
        torch.cuda.empty_cache()


def test_long_context_262144_tokens(device):
    """One sequence of 262144 tokens (64q/4kv, d = 128) forward + backward: gradients finite, the first 4096 rows of
    o and dq bit-equal to a 4096-token run (causality), the last 64 rows of kv group 0 against the oracle (their
    selection compared with the oracle's own, their output with the device's selection), and the block selector
    forced to work in short segments returns the same indices as the default at this length."""
    from flash_nsa import NSAConfig, NSACore, NSAHelper, _lib
    from flash_nsa.ops.compress_kv import mean_pooling_fwd
    from flash_nsa.ops.compress_attn import cmp_attn_fwd
    from flash_nsa.ops.topk import slc_topk_indices
    T, QH, KH, D, P, n = 262144, 64, 4, 128, 4096, 64
    q, k, v, w, do = [dev_randn(s, 40 + i, device) for i, s in
                      enumerate([(T, QH, D), (T, KH, D), (T, KH, D), (T, QH, 3), (T, QH, D)])]
    core = NSACore(NSAConfig(head_dim=D, num_heads=QH, num_kv_heads=KH))
    cu = torch.tensor([0, T], dtype=torch.int32, device=device)
    ts = [t.clone().requires_grad_() for t in (q, k, v, w)]
    out = core(*ts, cu)
    out.backward(do)
    for t in ts:
        assert torch.isfinite(t.grad).all()
    ps = [t[:P].clone().requires_grad_() for t in (q, k, v, w)]
    short = core(*ps, torch.tensor([0, P], dtype=torch.int32, device=device))
    short.backward(do[:P])
    assert torch.equal(out[:P], short) and torch.equal(ts[0].grad[:P], ps[0].grad)
    out = out.detach()
    del ts, ps, short
    torch.cuda.empty_cache()
    # selection: default segmenting against forced short segments
    NSAHelper.init_cu_seqlens(cu)
    with torch.no_grad():
        ck, cv = mean_pooling_fwd(k), mean_pooling_fwd(v)
        _, lse = cmp_attn_fwd(q, ck, cv)
        topk, _ = slc_topk_indices(q, ck, lse)
        try:
            _lib.call("nsa_set_tuning", b"topk_seg_blocks", 512)
            topk_seg, _ = slc_topk_indices(q, ck, lse)
        finally:
            _lib.call("nsa_reset_tuning")
    assert torch.equal(topk, topk_seg), "segment length changed the selection"
    # the last n rows of kv group 0 against the oracle: the sequence laid out as a paged pool with identity tables
    page = 256
    y = ck.shape[0]
    ypad = (y + page - 1) // page * page
    kh0 = lambda t: t[:, :1].float().cpu()
    pad = lambda t: torch.cat([t, t.new_zeros(ypad - y, 1, D)], 0)
    kc = torch.cat([kh0(k), pad(kh0(ck))], 0).view(-1, page, 1, D)
    vc = torch.cat([kh0(v), pad(kh0(cv))], 0).view(-1, page, 1, D)
    bt = torch.arange(T // page, dtype=torch.int32)[None]
    cbt = (T // page + torch.arange(ypad // page, dtype=torch.int32))[None]
    qs, ws = q[T - n:, :16].float().cpu(), w[T - n:, :16].float().cpu()
    tk_dev = topk[:1, T - n:].cpu()
    xcu, ctx = torch.tensor([0, n]), torch.tensor([T])
    ref_o, parts = O.nsa_paged_forward(qs, kc, vc, ws, xcu, ctx, bt, cbt, topk=tk_dev, round_dtype=torch.bfloat16,
                                       return_parts=True)
    assert_close(out[T - n:, :16], ref_o, "o (last rows of the 262144-token run)")
    own = O.select_blocks(parts[0]["imp"], torch.arange(T - n, T), 64, 16, 1, 2, -1)
    n_rows, n_diff, n_bad = O.topk_mismatch_report(tk_dev, own, [parts[0]["imp"]], [0, n], 64, 16, tie_tol=1e-3,
                                                   t_offsets=[T - n])
    assert n_rows == n and n_bad == 0, (n_rows, n_diff, n_bad)


def test_c2_prefix_consistency_and_oracle_slice(device):
    """T = 65536, 64q/4kv heads, d = 128, mean K compression and sigmoid-mul V compression (the benchmark
    configuration with its own compression pair): forward + backward run; the first 4096 rows of the forward equal a
    4096-token run (causality), and the first 1024 rows of kv group 0 match the oracle run with the same pair and the
    same compression weight."""
    from flash_nsa import NSAConfig, NSACore
    T, QH, KH, D, P = 65536, 64, 4, 128, 4096
    q, k, v, w = [dev_randn(s, i, device) for i, s in enumerate([(T, QH, D), (T, KH, D), (T, KH, D), (T, QH, 3)])]
    torch.manual_seed(0)
    core = NSACore(NSAConfig(head_dim=D, num_heads=QH, num_kv_heads=KH, cmp_v_method="sigmoid-mul")).to(
        device=device, dtype=torch.bfloat16)
    qg = q.clone().requires_grad_()
    cu = torch.tensor([0, T], dtype=torch.int32, device=device)
    out = core(qg, k, v, w, cu)
    do = dev_randn((T, QH, D), 9, device)
    out.backward(do)
    assert torch.isfinite(out).all() and torch.isfinite(qg.grad).all()
    qs_ = q[:P].clone().requires_grad_()
    short = core(qs_, k[:P].contiguous(), v[:P].contiguous(), w[:P].contiguous(),
                 torch.tensor([0, P], dtype=torch.int32, device=device))
    assert torch.equal(out[:P], short), "rows of the prefix changed when later tokens were appended"
    # dq of a row depends on the keys at or before it only: the same property for the backward
    short.backward(do[:P].contiguous())
    assert torch.equal(qg.grad[:P], qs_.grad), "dq of the prefix changed when later tokens were appended"
    short = short.detach()
    # oracle on a slice: first 1024 tokens, the 16 q-heads of kv head 0, device's own block selection
    n = 1024
    from flash_nsa.modules.megatron_level_nsa import compress_kv_fwd
    from flash_nsa import NSAHelper
    from flash_nsa.ops.compress_kv import mean_pooling_fwd
    from flash_nsa.ops.compress_attn import cmp_attn_fwd
    from flash_nsa.ops.topk import slc_topk_indices
    cun = torch.tensor([0, n], dtype=torch.int32, device=device)
    qs, ks, vs, ws = q[:n, :16].contiguous(), k[:n, :1].contiguous(), v[:n, :1].contiguous(), w[:n, :16].contiguous()
    with torch.no_grad():
        core16 = NSACore(NSAConfig(head_dim=D, num_heads=16, num_kv_heads=1, cmp_v_method="sigmoid-mul")).to(
            device=device, dtype=torch.bfloat16)
        core16.cmp_v_weight.copy_(core.cmp_v_weight)
        o16 = core16(qs, ks, vs, ws, cun)
        ck = mean_pooling_fwd(ks)
        cv = compress_kv_fwd(vs, core16.cmp_v_weight, "sigmoid-mul", NSAHelper)[2]
        _, lse = cmp_attn_fwd(qs, ck, cv)
        topk, _ = slc_topk_indices(qs, ck, lse)
    # not bit-equal: the compression GEMM of 63 windows and the one of 4 x 4095 windows take different library
    # kernels, whose V rows differ in the last bf16 bit
    assert_close(o16, out[:n, :16], "a kv group computed alone against the same group inside 4 groups", atol=4e-3,
                 rtol=8e-3)
    qr = qs.float().cpu().requires_grad_()
    ocfg = O.OracleConfig(cmp_v_method="sigmoid-mul")
    ref = O.nsa_forward(qr, ks.float().cpu(), vs.float().cpu(), ws.float().cpu(), [0, n], ocfg,
                        wv=core.cmp_v_weight.detach().float().cpu(), topk=topk.cpu(), round_dtype=torch.bfloat16)
    assert_close(o16, ref, "o (slice of the 64K run)")
    ref.backward(do[:n, :16].float().cpu())
    assert_close(qg.grad[:n, :16], qr.grad, "dq (slice of the 64K run)")


def test_c2_recompute_and_learned_compression_full_size(device):
    """T = 65536 with the benchmark's learned V compression (sigmoid-mul) and a learned K compression: the run that
    recomputes every intermediate in the backward returns the output and dq of the run that keeps them, bit for bit,
    and the weight gradients agree to the order of the fp32 atomic additions feeding them."""
    from flash_nsa import NSAConfig, NSACore, NSAHelper
    T, QH, KH, D = 65536, 64, 4, 128
    q, k, v, w, do = [dev_randn(s, 20 + i, device) for i, s in
                      enumerate([(T, QH, D), (T, KH, D), (T, KH, D), (T, QH, 3), (T, QH, D)])]
    cu = torch.tensor([0, T], dtype=torch.int32, device=device)
    res = {}
    for rec in (False, True):
        cfg = NSAConfig(head_dim=D, num_heads=QH, num_kv_heads=KH, cmp_k_method="linear", cmp_v_method="sigmoid-mul",
                        recompute_cmp_kv=rec, recompute_cmp_o=rec, recompute_slc_o=rec, recompute_swa_o=rec)
        torch.manual_seed(0)
        core = NSACore(cfg).to(device=device, dtype=torch.bfloat16)
        qg = q.clone().requires_grad_()
        out = core(qg, k, v, w, cu)
        out.backward(do)
        res[rec] = (out.detach(), qg.grad, core.cmp_k_weight.grad, core.cmp_v_weight.grad)
    NSAHelper.set_recompute()
    assert torch.isfinite(res[True][1]).all()
    assert torch.equal(res[False][0], res[True][0]) and torch.equal(res[False][1], res[True][1])
    for a, b, name in zip(res[False][2:], res[True][2:], ("dWk", "dWv")):
        assert torch.isfinite(a).all()
        assert_close(b, a.float(), name, atol=2e-2, rtol=1e-2, row_scale=True)


def test_c3_packed_batch_equals_single_sequences(device):
    """8 sequences with lengths uniform in [4096, 8192] (seed 1), forward + backward: packed == one by one."""
    from flash_nsa import NSAConfig, NSACore
    g = torch.Generator().manual_seed(1)
    lens = torch.randint(4096, 8193, (8,), generator=g).tolist()
    cu = make_cu(lens)
    T, QH, KH, D = int(cu[-1]), 64, 4, 128
    q, k, v, w, do = [dev_randn(s, 10 + i, device) for i, s in
                      enumerate([(T, QH, D), (T, KH, D), (T, KH, D), (T, QH, 3), (T, QH, D)])]
    core = NSACore(NSAConfig(head_dim=D, num_heads=QH, num_kv_heads=KH))

    def run(qq, kk, vv, ww, dd, cuu):
        ts = [t.clone().requires_grad_() for t in (qq, kk, vv, ww)]
        o = core(*ts, cuu.to(device))
        o.backward(dd)
        return [o.detach()] + [t.grad for t in ts]

    packed = run(q, k, v, w, do, cu)
    for b in (0, 3, 7):
        a, e = int(cu[b]), int(cu[b + 1])
        single = run(q[a:e], k[a:e], v[a:e], w[a:e], do[a:e], make_cu([e - a]))
        assert torch.equal(packed[0][a:e], single[0]), f"sequence {b}: forward differs"
        assert torch.equal(packed[1][a:e], single[1]), f"sequence {b}: dq differs"
        # dk/dv are accumulated with fp32 atomics in a data-dependent order: equal up to fp32 summation order, i.e. one bf16 ulp (2^-7 relative) after the final rounding
        assert_close(packed[2][a:e], single[2], f"sequence {b}: dk", atol=2e-3, rtol=8e-3, row_scale=True)
        assert_close(packed[3][a:e], single[3], f"sequence {b}: dv", atol=2e-3, rtol=8e-3, row_scale=True)
        assert_close(packed[4][a:e], single[4], f"sequence {b}: dw", atol=1e-6, rtol=0)


def _decode_block_scores(c, kh, b, device, G=16, D=128, block=64, kernel=32, stride=16):
    """fp64 selection-block scores of one (request, kv head) of the decode benchmark case: softmax over the
    compressed keys, summed over the q-heads of the group, folded by the overlap of every compressed key with the
    block (flash_nsa/ops/topk.py:101-118 upstream)."""
    page, L, y = c["page"], c["lens"][b], c["ys"][b]
    i = torch.arange(y, device=device)
    rows = c["cbt"][b][i // page].long() * page + i % page
    kc = c["k"].view(-1, c["k"].shape[-2], D)[rows, kh].double()
    qg = c["q"][b, kh * G:(kh + 1) * G].double()
    p = torch.softmax(qg @ kc.t() * D ** -0.5, -1).sum(0)
    nb = (L - 1) // block + 1
    imp = torch.zeros(nb, dtype=torch.float64, device=device)
    for j in range(nb):
        i0, cs = (j * block - kernel) // stride + 1, stride - kernel
        for r in range((block + kernel - stride) // stride):
            if 0 <= i0 + r < y:
                imp[j] += p[i0 + r] * (min(cs + kernel, block) - max(cs, 0)) / stride
            cs += stride
    return imp


def test_c5_decode_full_batch(device):
    """Batch 64, contexts uniform in [4096, 32768], page 256, random page permutation (benchmark configuration):
    fused decode == stage-by-stage decode; one request re-checked as a one-token paged prefill; graph replay."""
    from flash_nsa import nsa_decode, nsa_prefill
    from flash_nsa.inference import nsa_decode_staged, mean_pooling_prefill
    from synthetic_decode import build_decode_case
    c = build_decode_case(device)
    page = c["page"]
    ycu = torch.zeros(65, dtype=torch.int32)
    ycu[1:] = torch.cumsum(torch.tensor(c["ys"]), 0)
    slots_all = torch.cat([(c["cbt"][b].cpu()[torch.arange(y) // page].to(torch.int64) * page + torch.arange(y) % page)
                           for b, y in enumerate(c["ys"])]).to(torch.int32).to(device)
    for cache in (c["k"], c["v"]):
        mean_pooling_prefill(cache, ycu.to(device), max(c["ys"]), c["bt"], slots_all)
    kw = dict(fixed_y_maxlen=2048, fixed_num_slc_blocks=512)
    fused = nsa_decode(c["q"], c["k"], c["v"], c["w"], c["ctx"], c["bt"], c["slots"], c["cbt"], **kw)
    staged = nsa_decode_staged(c["q"], c["k"], c["v"], c["w"], c["ctx"], c["bt"], c["cbt"], **kw)
    assert torch.isfinite(fused).all()
    # The fused kernel keeps the probabilities of the compressed keys as fp16 between its two phases, the staged
    # path recomputes them in fp32: the selections may differ where two block scores tie.  Such rows are checked
    # to be ties (fp64 scores closer than 1e-3) and left out of the output comparison.
    from flash_nsa.inference import decode_cmp_topk, cmp_attn_decode, topk_decode
    _, tk_f = decode_cmp_topk(c["q"], c["k"], c["v"], c["cbt"], c["ctx"], 2048, 512)
    _, lse = cmp_attn_decode(c["q"], c["k"], c["v"], block_tables=c["cbt"], context_lens=c["ctx"])
    tk_s = topk_decode(c["q"], c["k"], lse, fixed_y_maxlen=2048, fixed_num_slc_blocks=512, block_tables=c["cbt"],
                       context_lens=c["ctx"])
    def rows_without_ties(tk, name):
        """[B, QH] mask of the rows whose selection equals the staged one; the others must be score ties"""
        differ = (tk.sort(-1).values != tk_s.sort(-1).values).any(-1)       # [KH, B]
        assert int(differ.sum()) <= 8, f"{name}: {int(differ.sum())} of {differ.numel()} selections differ"
        for kh, b in differ.nonzero().tolist():
            imp = _decode_block_scores(c, kh, b, device)
            only_a = sorted(set(tk[kh, b].tolist()) - set(tk_s[kh, b].tolist()))
            only_s = sorted(set(tk_s[kh, b].tolist()) - set(tk[kh, b].tolist()))
            assert len(only_a) == len(only_s)
            lo = min(float(imp[j]) for j in only_a + only_s)
            hi = max(float(imp[j]) for j in only_a + only_s)
            assert hi - lo < 1e-3, f"{name}: request {b}, kv head {kh} differs beyond a tie: {only_a} vs {only_s}"
        return (~differ).t().repeat_interleave(16, dim=1)

    keep = rows_without_ties(tk_f, "fused")
    assert_close(fused[keep], staged[keep], "fused vs staged decode", atol=8e-3, rtol=1e-2)
    # the path for small batches of long contexts (compressed branch in 4 parts, fp16 probabilities spilled)
    from flash_nsa.inference import decode_split
    split = nsa_decode(c["q"], c["k"], c["v"], c["w"], c["ctx"], c["bt"], c["slots"], c["cbt"], cmp_num_splits=4, **kw)
    parts = decode_split(c["q"], c["k"], c["v"], c["w"], c["bt"], c["cbt"], c["ctx"], nsplit=4, return_parts=True, **kw)
    assert torch.equal(split, parts[0])
    keep = rows_without_ties(parts[4], "split")
    assert_close(split[keep], staged[keep], "split vs staged decode", atol=8e-3, rtol=1e-2)
    # request 5 as a single-token prefill through nsa_prefill (all compressed rows already pooled: slots -1)
    b = 5
    L, y = c["lens"][b], c["ys"][b]
    o1 = nsa_prefill(c["q"][b:b + 1], c["k"], c["v"], c["w"][b:b + 1], torch.tensor([0, 1], dtype=torch.int32, device=device),
                     torch.tensor([0, y], dtype=torch.int32, device=device), 1, y, c["ctx"][b:b + 1], c["bt"][b:b + 1],
                     torch.full((y,), -1, dtype=torch.int32, device=device), c["cbt"][b:b + 1], **kw)
    assert_close(fused[b:b + 1], o1, "decode vs one-token prefill", atol=8e-3, rtol=1e-2)


def test_c4_chunked_prefill_full_size(device):
    """16 requests, cached prefix uniform in [0, 16384] + a new chunk of 2048 tokens, page 256, random page
    permutation (benchmark configuration): the chunk's output equals the training forward on the gathered
    contiguous sequence (rows of the chunk), and the pooled rows equal the contiguous pooling bit for bit."""
    from flash_nsa import NSAConfig, NSACore, nsa_prefill, NSAHelper
    from flash_nsa.inference import mean_pooling_prefill
    from flash_nsa.ops.compress_kv import mean_pooling_fwd
    from paged_util import build_pool, prefill_slot_mapping
    QH, KH, D, page, chunk = 64, 4, 128, 256, 2048
    g = torch.Generator().manual_seed(2)
    cached = torch.randint(0, 16385, (16,), generator=g).tolist()
    ctx = [c + chunk for c in cached]
    case = build_pool(ctx, KH, D, D, page=page, seed=2)
    d = {k_: (v_.to(device) if isinstance(v_, torch.Tensor) else v_) for k_, v_ in case.items()}
    # an earlier step pooled the rows that lie inside the cached prefix
    pre = dict(case)
    pre["ctx"] = cached
    pre["ys"] = [max((L - 32) // 16 + 1, 0) for L in cached]
    slots0, ycu0 = prefill_slot_mapping(pre, [0] * 16)
    cached_t = torch.tensor(cached, dtype=torch.int32, device=device)
    if int(ycu0[-1]) > 0:
        for cache in (d["k"], d["v"]):
            mean_pooling_prefill(cache, ycu0.to(device), max(pre["ys"]), d["bt"], slots0.to(device))
    slots, ycu = prefill_slot_mapping(case, cached)
    xcu = make_cu([chunk] * 16)
    t = 16 * chunk
    q, w = dev_randn((t, QH, D), 31, device), dev_randn((t, QH, 3), 32, device)
    ctx_t = torch.tensor(ctx, dtype=torch.int32, device=device)
    o = nsa_prefill(q, d["k"], d["v"], w, xcu.to(device), ycu.to(device), chunk, max(case["ys"]), ctx_t, d["bt"],
                    slots.to(device), d["cbt"], fixed_y_maxlen=2048, fixed_num_slc_blocks=512)
    assert torch.isfinite(o).all()
    core = NSACore(NSAConfig(head_dim=D, num_heads=QH, num_kv_heads=KH))
    kc, vc = d["k"].cpu(), d["v"].cpu()
    for b in (0, 7, 15):
        L = ctx[b]
        ks = O.gather_rows(kc, case["bt"][b], L).to(device)
        vs = O.gather_rows(vc, case["bt"][b], L).to(device)
        qf = dev_randn((L, QH, D), 40 + b, device)
        wf = dev_randn((L, QH, 3), 50 + b, device)
        qf[-chunk:] = q[b * chunk:(b + 1) * chunk]
        wf[-chunk:] = w[b * chunk:(b + 1) * chunk]
        cu1 = torch.tensor([0, L], dtype=torch.int32, device=device)
        with torch.no_grad():
            full = core(qf, ks, vs, wf, cu1)
            ck = mean_pooling_fwd(ks)
        assert_close(o[b * chunk:(b + 1) * chunk], full[-chunk:], f"request {b}: chunk vs contiguous forward",
                     atol=4e-3, rtol=1e-2)
        pooled = O.gather_rows(kc * 0 + d["k"].cpu(), case["cbt"][b], case["ys"][b])
        assert torch.equal(pooled, ck.cpu()), f"request {b}: pooled rows differ from contiguous pooling"
