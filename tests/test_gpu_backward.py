"""GPU parity of the backward operators and of the composed modules against torch.autograd through the CPU
oracle (same seeded bf16 inputs, fp32 oracle arithmetic).  Mirrors upstream test.py --func cmp/slc/combine/nsa
(test.py:131-353) with asserted tolerances."""
import pytest
import torch

from oracle import nsa_oracle as O
from gpu_util import make_cu, make_qkvw, randn_bf16, assert_close

pytestmark = pytest.mark.gpu

LENS_CASES = [[1000], [5, 31, 32, 47, 48, 100, 333, 700], [64, 0, 129, 513]]
HEAD_CASES = [(16, 1, 128), (8, 2, 128), (4, 4, 64), (16, 2, 128), (32, 1, 128)]


def setup_helper(cu_dev, **kw):
    from flash_nsa import NSAHelper
    NSAHelper.set_hyperparameters(**kw)
    NSAHelper.init_cu_seqlens(cu_dev)
    return NSAHelper


def leaf(x):
    return x.float().clone().requires_grad_()


@pytest.mark.parametrize("lens", LENS_CASES)
def test_mean_pooling_bwd(device, lens):
    from flash_nsa.ops.compress_kv import mean_pooling_bwd, construct_block_bwd
    cu = make_cu(lens)
    T = int(cu[-1])
    x = randn_bf16(T, 2, 128, seed=1)
    setup_helper(cu.to(device))
    xr = leaf(x)
    y = O.mean_pooling(xr, cu)
    dy = randn_bf16(*y.shape, seed=2)
    y.backward(dy.float())
    dx = mean_pooling_bwd(x.to(device), dy.to(device))
    assert_close(dx, xr.grad, "pool dx", atol=2e-3, rtol=1e-2)
    acc = torch.ones(T, 2, 128, device=device, dtype=torch.float32)
    mean_pooling_bwd(x.to(device), dy.to(device), acc)
    assert_close(acc, xr.grad + 1, "pool dx accumulate", atol=1e-5, rtol=1e-5)
    xb = leaf(x)
    blk = O.construct_block(xb, cu)
    dblk = randn_bf16(*blk.shape, seed=3)
    blk.backward(dblk.float())
    dxb = construct_block_bwd(x.to(device), dblk.to(device))
    assert_close(dxb, xb.grad, "construct_block dx", atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("lens", LENS_CASES)
@pytest.mark.parametrize("QH,KH,D", HEAD_CASES)
def test_cmp_attn_bwd(device, lens, QH, KH, D):
    from flash_nsa.ops.compress_kv import mean_pooling_fwd
    from flash_nsa.ops.compress_attn import cmp_attn_fwd, cmp_attn_bwd
    cu = make_cu(lens)
    T = int(cu[-1])
    q, k, v, _ = make_qkvw(T, QH, KH, D, seed=40)
    do = randn_bf16(T, QH, D, seed=44)
    setup_helper(cu.to(device))
    qd = q.to(device)
    ck, cv = mean_pooling_fwd(k.to(device)), mean_pooling_fwd(v.to(device))
    o, lse = cmp_attn_fwd(qd, ck, cv)
    dq, dck, dcv = cmp_attn_bwd(qd, ck, cv, o, lse, do.to(device), q_chunk_tokens=256)
    ref = O.branch_forward_backward("cmp", q.float(), ck.float().cpu(), cv.float().cpu(), do.float(), cu,
                                    round_dtype=torch.bfloat16, round_mma=True)
    assert_close(dq, ref["dq"], "cmp dq")
    if ck.numel():
        assert_close(dck, ref["dk"], "cmp dk", row_scale=True)
        assert_close(dcv, ref["dv"], "cmp dv", row_scale=True)


@pytest.mark.parametrize("lens", LENS_CASES)
@pytest.mark.parametrize("QH,KH,D", HEAD_CASES)
def test_swa_bwd(device, lens, QH, KH, D):
    from flash_nsa.ops.sliding_window_attention import swa_fwd, swa_bwd
    cu = make_cu(lens)
    T = int(cu[-1])
    q, k, v, _ = make_qkvw(T, QH, KH, D, seed=50)
    do = randn_bf16(T, QH, D, seed=54)
    setup_helper(cu.to(device), window_size=200)
    qd, kd, vd = q.to(device), k.to(device), v.to(device)
    o, lse = swa_fwd(qd, kd, vd)
    dq, dk, dv = swa_bwd(qd, kd, vd, o, lse, do.to(device), dkv_fp32=True)
    ref = O.branch_forward_backward("swa", q.float(), k.float(), v.float(), do.float(), cu,
                                    O.OracleConfig(window_size=200), round_dtype=torch.bfloat16, round_mma=True)
    assert_close(dq, ref["dq"], "swa dq")
    assert_close(dk, ref["dk"], "swa dk", row_scale=True)
    assert_close(dv, ref["dv"], "swa dv", row_scale=True)
    setup_helper(cu.to(device))


@pytest.mark.parametrize("lens", LENS_CASES)
@pytest.mark.parametrize("QH,KH,D", HEAD_CASES)
def test_slc_attn_bwd(device, lens, QH, KH, D):
    from flash_nsa.ops.compress_kv import mean_pooling_fwd
    from flash_nsa.ops.compress_attn import cmp_attn_fwd
    from flash_nsa.ops.topk import slc_topk_indices, get_bind_from_find
    from flash_nsa.ops.select_attn import slc_attn_fwd, slc_attn_bwd
    from flash_nsa import NSAHelper
    cu = make_cu(lens)
    T = int(cu[-1])
    q, k, v, _ = make_qkvw(T, QH, KH, D, seed=60)
    do = randn_bf16(T, QH, D, seed=64)
    top_n = 6
    setup_helper(cu.to(device), top_n=top_n)
    qd, kd, vd = q.to(device), k.to(device), v.to(device)
    ck = mean_pooling_fwd(kd)
    _, lse_c = cmp_attn_fwd(qd, ck, ck)
    topk, _ = slc_topk_indices(qd, ck, lse_c)
    # inverse index: every (token, valid slot) appears exactly once, lists ascending
    bind = get_bind_from_find(topk, chunk_tokens=64)
    off = bind["csr_off"].cpu()
    tok = bind["csr_tok"].cpu()
    tk = topk.cpu()
    kcu = NSAHelper.k_cu_seqlens.cpu()
    for kh in range(KH):
        exp = {}
        for b in range(len(lens)):
            for n in range(lens[b]):
                for s in range(min(top_n, n // 64 + 1)):
                    exp.setdefault(int(kcu[b]) + int(tk[kh, int(cu[b]) + n, s]), []).append(n)
        for jb in range(int(kcu[-1])):
            got = tok[int(off[kh, jb]):int(off[kh, jb + 1])].tolist()
            assert got == sorted(exp.get(jb, [])), (kh, jb)
    o, lse = slc_attn_fwd(qd, kd, vd, topk)
    dq, dk, dv = slc_attn_bwd(qd, kd, vd, topk, o, lse, do.to(device), bind=bind)
    ref = O.branch_forward_backward("slc", q.float(), k.float(), v.float(), do.float(), cu,
                                    O.OracleConfig(top_n=top_n), topk=tk, round_dtype=torch.bfloat16, round_mma=True)
    assert_close(dq, ref["dq"], "slc dq")
    assert_close(dk, ref["dk"], "slc dk", row_scale=True)
    assert_close(dv, ref["dv"], "slc dv", row_scale=True)
    setup_helper(cu.to(device))


def test_combine_bwd(device):
    from flash_nsa.ops.combine import combine_bwd
    a, b, c = [randn_bf16(300, 8, 128, seed=s) for s in (1, 2, 3)]
    w = randn_bf16(300, 8, 3, seed=4)
    do = randn_bf16(300, 8, 128, seed=5)
    ar, br, cr, wr = leaf(a), leaf(b), leaf(c), leaf(w)
    O.combine(ar, br, cr, wr).backward(do.float())
    da, db, dc, dw, delta = combine_bwd(a.to(device), b.to(device), c.to(device), w.to(device), do.to(device),
                                        return_delta=True)
    assert_close(da, ar.grad, "da")
    assert_close(db, br.grad, "db")
    assert_close(dc, cr.grad, "dc")
    assert_close(dw, wr.grad, "dw")
    # the correction term is the row sum over the STORED (bf16) branch gradient, the one the attention backward reads
    for i, (x, g) in enumerate(((a, ar), (b, br), (c, cr))):
        stored = g.grad.to(torch.bfloat16).float()
        assert_close(delta[i], (x.float() * stored).sum(-1), f"delta{i}")


@pytest.mark.parametrize("core", ["hf", "megatron"])
@pytest.mark.parametrize("lens,QH,KH,D,methods", [
    ([1500], 16, 1, 128, ("mean", "mean")),
    ([5, 31, 48, 333, 700, 900], 8, 2, 128, ("mean", "sigmoid-mul")),
    ([300, 800], 4, 2, 64, ("linear", "swiglu")),
    ([700, 260], 32, 1, 128, ("mean", "mean")),       # 32 q-heads per kv head
    ([515], 64, 1, 64, ("mean", "mean")),             # 64 q-heads per kv head (two head chunks in the selector)
    ([400, 330], 16, 2, 128, ("mean", "mean")),       # groups of 8
    ([400, 330], 6, 3, 64, ("mean", "mean")),         # groups of 2
    ([400, 330], 12, 4, 64, ("mean", "mean")),        # groups of 3 (not a power of two)
    # 48 ragged sequences, some empty or shorter than one compression window
    ([(37 * i * i + 11 * i) % 257 for i in range(48)], 16, 2, 128, ("mean", "sigmoid-mul")),
])
def test_nsa_core_fwd_bwd(device, core, lens, QH, KH, D, methods):
    """HFNSACore and NSACore against the composed oracle (upstream only compares them with each other)."""
    from flash_nsa import NSAConfig, HFNSACore, NSACore
    from flash_nsa.ops.compress_attn import cmp_attn_fwd
    from flash_nsa.ops.topk import slc_topk_indices
    cu = make_cu(lens)
    T = int(cu[-1])
    q, k, v, w = make_qkvw(T, QH, KH, D, seed=70)
    do = randn_bf16(T, QH, D, seed=75)
    cfg = NSAConfig(head_dim=D, num_heads=QH, num_kv_heads=KH, top_n=8, window_size=128, cmp_k_method=methods[0],
                    cmp_v_method=methods[1])
    torch.manual_seed(0)
    mod = (HFNSACore(cfg) if core == "hf" else NSACore(cfg)).to(device=device, dtype=torch.bfloat16)
    if core == "hf":
        wk = mod.compress_k.fc.weight if methods[0] != "mean" else None
        wv = mod.compress_v.fc.weight if methods[1] != "mean" else None
    else:
        wk, wv = mod.cmp_k_weight, mod.cmp_v_weight
    qd, kd, vd, wd = [t.to(device).requires_grad_() for t in (q, k, v, w)]
    out = mod(qd, kd, vd, wd, cu.to(device))
    out.backward(do.to(device))

    ocfg = O.OracleConfig(top_n=8, window_size=128, cmp_k_method=methods[0], cmp_v_method=methods[1])
    # indices: take the device's selection (checked against the oracle's in the forward tests) so that a
    # near-tie cannot change which keys the two sides attend
    with torch.no_grad():
        from flash_nsa.modules.megatron_level_nsa import compress_kv_fwd
        ck = compress_kv_fwd(kd.detach(), wk, methods[0])[2]
        cv = compress_kv_fwd(vd.detach(), wv, methods[1])[2]
        _, lse = cmp_attn_fwd(qd.detach(), ck, cv)
        topk, _ = slc_topk_indices(qd.detach(), ck, lse)
    # The reference keeps the rounding points of the pipeline (the tensors that upstream, too, stores in bf16
    # between kernels: compressed rows, branch outputs and their gradients, the correction term formed from them,
    # P and dS as matrix operands);
    # tests/test_oracle_pinning.py shows that without rounding it is torch.autograd through the fp32 oracle, and how
    # far the two references are apart.  Every element is held to the same bar.
    ref = O.nsa_forward_backward(q.float(), k.float(), v.float(), w.float(), do.float(), cu, ocfg, topk=topk.cpu(),
                                 wk=None if wk is None else wk.detach().float().cpu(),
                                 wv=None if wv is None else wv.detach().float().cpu(), round_dtype=torch.bfloat16,
                                 round_mma=True)
    assert_close(out, ref["o"], "o")
    assert_close(qd.grad, ref["dq"], "dq")
    assert_close(kd.grad, ref["dk"], "dk", row_scale=True)
    assert_close(vd.grad, ref["dv"], "dv", row_scale=True)
    assert_close(wd.grad, ref["dw"], "dw")
    # dk / dv (sums over every later query row and the q-heads of the group) and the compression-weight gradients
    # (sums over every compressed row of the batch) use max(|ref|, rms of the row) in the relative term: the rounding
    # error of such a sum scales with the magnitude of its row, not with the element's own, possibly cancelled, value
    if wk is not None:
        assert_close(wk.grad, ref["dwk"], "dWk", row_scale=True)
    if wv is not None:
        assert_close(wv.grad, ref["dwv"], "dWv", row_scale=True)


@pytest.mark.parametrize("hp", [
    dict(kernel_size=64, stride=32, block_size=128, top_n=4, window_size=256),
    dict(kernel_size=64, stride=16, block_size=64, top_n=5, window_size=100),
    dict(kernel_size=32, stride=8, block_size=64, top_n=16, window_size=512),
    dict(kernel_size=16, stride=16, block_size=64, top_n=3, window_size=1, num_init_blocks=0, num_local_blocks=1),
    dict(kernel_size=32, stride=16, block_size=64, top_n=8, window_size=64, num_init_blocks=2, num_local_blocks=3),
    dict(top_n=64, window_size=64),                                   # more slots than most tokens have blocks
    dict(top_n=1, num_init_blocks=0, num_local_blocks=1),             # the token's own block only
    dict(top_n=2, num_init_blocks=1, num_local_blocks=1, window_size=0),  # window = the token itself
    # selection blocks other than 64 / 128 (upstream accepts every block >= kernel that is a multiple of the stride;
    # this build: every multiple of 32)
    dict(kernel_size=32, stride=16, block_size=32, top_n=12, window_size=64),
    dict(kernel_size=32, stride=8, block_size=32, top_n=6, window_size=100),
    dict(kernel_size=32, stride=16, block_size=96, top_n=5, window_size=64),
    dict(kernel_size=64, stride=16, block_size=256, top_n=3, window_size=128),
    dict(kernel_size=32, stride=32, block_size=160, top_n=4, num_local_blocks=1, window_size=32),
    # head dims other than 128 (upstream accepts every power of two, flash_nsa/ops/compress_attn.py:542)
    dict(head_dim=32, top_n=6, window_size=100),
    dict(head_dim=256, top_n=6, window_size=100),
    dict(head_dim=64, top_n=6, window_size=100),
])
def test_nsa_core_other_hyperparameters(device, hp):
    """Compression window / stride, selection block, top-n, forced blocks and window other than the defaults
    (upstream NSAHelper.set_hyperparameters, flash_nsa/utils.py:180-214): selection identical to the oracle's on the
    device's compressed keys, forward and backward against the composed oracle."""
    from flash_nsa import NSAConfig, NSACore, NSAHelper
    from flash_nsa.ops.compress_attn import cmp_attn_fwd
    from flash_nsa.ops.topk import slc_topk_indices
    from flash_nsa.modules.megatron_level_nsa import compress_kv_fwd
    hp = dict(hp)
    lens, QH, KH, D = [1500, 700, 90], 8, 2, hp.pop("head_dim", 128)
    cu = make_cu(lens)
    T = int(cu[-1])
    q, k, v, w = make_qkvw(T, QH, KH, D, seed=71)
    do = randn_bf16(T, QH, D, seed=76)
    try:
        mod = NSACore(NSAConfig(head_dim=D, num_heads=QH, num_kv_heads=KH, **hp)).to(device=device, dtype=torch.bfloat16)
        qd, kd, vd, wd = [t.to(device).requires_grad_() for t in (q, k, v, w)]
        out = mod(qd, kd, vd, wd, cu.to(device))
        out.backward(do.to(device))
        with torch.no_grad():
            ck = compress_kv_fwd(kd.detach(), None, "mean")[2]
            cv = compress_kv_fwd(vd.detach(), None, "mean")[2]
            _, lse = cmp_attn_fwd(qd.detach(), ck, cv)
            topk, _ = slc_topk_indices(qd.detach(), ck, lse)
    finally:
        NSAHelper.set_hyperparameters()
    ocfg = O.OracleConfig(**hp)
    rt, imps = O.slc_topk(q.float(), ck.float().cpu(), None, cu, ocfg, return_importance=True)
    n_rows, n_diff, n_bad = O.topk_mismatch_report(topk.cpu(), rt, imps, cu, ocfg.block_size, ocfg.top_n, tie_tol=1e-3)
    assert n_bad == 0 and n_diff <= max(1, n_rows // 200), (n_rows, n_diff, n_bad)
    ref = O.nsa_forward_backward(q.float(), k.float(), v.float(), w.float(), do.float(), cu, ocfg, topk=topk.cpu(),
                                 round_dtype=torch.bfloat16, round_mma=True)  # see test_nsa_core_fwd_bwd
    assert_close(out, ref["o"], "o")
    assert_close(qd.grad, ref["dq"], "dq")
    assert_close(kd.grad, ref["dk"], "dk", row_scale=True)
    assert_close(vd.grad, ref["dv"], "dv", row_scale=True)
    assert_close(wd.grad, ref["dw"], "dw")


@pytest.mark.parametrize("QH,KH,block_size", [(8, 2, 64), (16, 2, 64), (32, 2, 64), (16, 2, 128), (16, 1, 96)])
def test_nsa_core_qk192_v128(device, QH, KH, block_size):
    """Dqk = 192, Dv = 128 (the head shape upstream's inference notebook exercises), forward + backward, with 4, 8
    and 16 q-heads per kv head: a row of 192 channels is 24 sixteen-byte pieces, which do not divide the thread count
    of the selected dK/dV kernel, so its load steps straddle tokens and take the general addressing path."""
    from flash_nsa import NSAConfig, NSACore
    from flash_nsa.ops.compress_kv import mean_pooling_fwd
    from flash_nsa.ops.compress_attn import cmp_attn_fwd
    from flash_nsa.ops.topk import slc_topk_indices
    lens, D, VD = [700, 333], 192, 128
    cu = make_cu(lens)
    T = int(cu[-1])
    q, k, v, w = make_qkvw(T, QH, KH, D, VD, seed=80)
    do = randn_bf16(T, QH, VD, seed=85)
    cfg = NSAConfig(qk_head_dim=D, v_head_dim=VD, num_heads=QH, num_kv_heads=KH, top_n=6, window_size=100,
                    block_size=block_size)
    mod = NSACore(cfg)
    qd, kd, vd, wd = [t.to(device).requires_grad_() for t in (q, k, v, w)]
    out = mod(qd, kd, vd, wd, cu.to(device))
    out.backward(do.to(device))
    with torch.no_grad():
        ck, cv = mean_pooling_fwd(kd.detach()), mean_pooling_fwd(vd.detach())
        _, lse = cmp_attn_fwd(qd.detach(), ck, cv)
        topk, _ = slc_topk_indices(qd.detach(), ck, lse)
    ref = O.nsa_forward_backward(q.float(), k.float(), v.float(), w.float(), do.float(), cu,
                                 O.OracleConfig(top_n=6, window_size=100, block_size=block_size), topk=topk.cpu(),
                                 round_dtype=torch.bfloat16, round_mma=True)
    assert_close(out, ref["o"], "o")
    assert_close(qd.grad, ref["dq"], "dq")
    assert_close(kd.grad, ref["dk"], "dk", row_scale=True)
    assert_close(vd.grad, ref["dv"], "dv", row_scale=True)
    assert_close(wd.grad, ref["dw"], "dw")


def test_two_stream_backward_equals_single_stream(device):
    """The fused backward puts its dq chain on a second stream next to the dk/dv kernels: same results as with
    everything on one stream (dq bit-equal; dk/dv up to the order of the fp32 atomics)."""
    from flash_nsa import NSAConfig, NSACore
    from flash_nsa.modules import megatron_level_nsa as M
    lens, QH, KH, D = [1500, 700, 333], 32, 2, 128
    cu = make_cu(lens)
    T = int(cu[-1])
    q, k, v, w = make_qkvw(T, QH, KH, D, D, seed=90)
    do = randn_bf16(T, QH, D, seed=91).to(device)
    core = NSACore(NSAConfig(head_dim=D, num_heads=QH, num_kv_heads=KH, cmp_v_method="sigmoid-mul"))
    core = core.to(device=device, dtype=torch.bfloat16)

    def run(overlap):
        old = M.OVERLAP_STREAMS
        M.OVERLAP_STREAMS = overlap
        try:
            ts = [t.to(device).requires_grad_() for t in (q, k, v, w)]
            core.zero_grad()
            out = core(*ts, cu.to(device))
            out.backward(do)
            torch.cuda.synchronize()
            return [out.detach()] + [t.grad for t in ts] + [core.cmp_v_weight.grad.clone()]
        finally:
            M.OVERLAP_STREAMS = old

    a, b = run(True), run(False)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]) and torch.equal(a[4], b[4])
    assert_close(a[2], b[2], "dk", atol=2e-3, rtol=8e-3, row_scale=True)
    assert_close(a[3], b[3], "dv", atol=2e-3, rtol=8e-3, row_scale=True)
    assert_close(a[5], b[5], "d cmp_v_weight", atol=2e-3, rtol=2e-2, row_scale=True)


@pytest.mark.parametrize("methods", [("mean", "mean"), ("sigmoid-mul", "swiglu"), ("linear", "mean")])
def test_recompute_flags_change_memory_not_results(device, methods):
    """Every recompute_* flag on (upstream flash_nsa/modules/megatron_level_nsa.py:107-147): the forward keeps fewer
    bytes alive, the backward rebuilds them with the same kernels, so output and gradients are those of the run that
    saved everything (dq / dWk / dWv bit for bit; dk / dv / dw up to the order of their fp32 atomic additions)."""
    from flash_nsa import NSAConfig, NSACore, NSAHelper
    lens, QH, KH, D = [900, 420], 8, 2, 128
    cu = make_cu(lens).to(device)
    T = sum(lens)
    q, k, v, w = make_qkvw(T, QH, KH, D, seed=90)
    do = randn_bf16(T, QH, D, seed=95).to(device)
    flags = ("recompute_cmp_kv", "recompute_cmp_o", "recompute_slc_o", "recompute_swa_o")
    runs = {}
    for on in (False, True):
        cfg = NSAConfig(head_dim=D, num_heads=QH, num_kv_heads=KH, top_n=8, window_size=128, cmp_k_method=methods[0],
                        cmp_v_method=methods[1], **{f: on for f in flags})
        torch.manual_seed(0)
        mod = NSACore(cfg).to(device=device, dtype=torch.bfloat16)
        leaves = [t.to(device).requires_grad_() for t in (q, k, v, w)]
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        out = mod(*leaves, cu)
        torch.cuda.synchronize()
        held = torch.cuda.memory_allocated() - before
        out.backward(do)
        grads = [t.grad for t in leaves] + [p.grad for p in (mod.cmp_k_weight, mod.cmp_v_weight) if p is not None]
        runs[on] = (out.detach(), grads, held)
        assert all(getattr(NSAHelper, f) == on for f in flags)
    NSAHelper.set_recompute()
    (o0, g0, held0), (o1, g1, held1) = runs[False], runs[True]
    assert torch.equal(o0, o1)
    assert torch.equal(g0[0], g1[0]), "dq"
    for a, b, name in zip(g0[1:4], g1[1:4], ("dk", "dv", "dw")):
        assert_close(a, b.float(), name, atol=1e-5, rtol=8e-3)
    for a, b in zip(g0[4:], g1[4:]):
        assert_close(a, b.float(), "dW", atol=1e-5, rtol=8e-3)
    # three branch outputs [T,QH,D] bf16 + their lse are no longer kept
    assert held0 - held1 >= 3 * T * QH * D * 2, (held0, held1)


def test_weight_gradient_accumulates_into_main_grad(device):
    """A compression weight with an fp32 `main_grad` (the mixed-precision optimizers of Megatron keep one, upstream
    flash_nsa/modules/megatron_level_nsa.py:20-44): the backward adds dW to it without rounding to bf16 first and,
    when the parameter carries `grad_added_to_main_grad`, sets it and returns a placeholder gradient."""
    from flash_nsa import NSAConfig, NSACore
    lens, QH, KH, D = [700, 300], 4, 2, 64
    cu = make_cu(lens).to(device)
    T = sum(lens)
    q, k, v, w = make_qkvw(T, QH, KH, D, seed=100)
    do = randn_bf16(T, QH, D, seed=105).to(device)
    cfg = NSAConfig(head_dim=D, num_heads=QH, num_kv_heads=KH, top_n=8, window_size=128, cmp_k_method="linear",
                    cmp_v_method="sigmoid-mul")

    def run(with_main_grad):
        torch.manual_seed(0)
        mod = NSACore(cfg).to(device=device, dtype=torch.bfloat16)
        if with_main_grad:
            for i, p in enumerate((mod.cmp_k_weight, mod.cmp_v_weight)):
                p.main_grad = torch.full(p.shape, 0.5 + i, device=device, dtype=torch.float32)
            mod.cmp_v_weight.grad_added_to_main_grad = False
        leaves = [t.to(device).requires_grad_() for t in (q, k, v, w)]
        mod(*leaves, cu).backward(do)
        return mod

    plain, mixed = run(False), run(True)
    for i, name in enumerate(("cmp_k_weight", "cmp_v_weight")):
        want = getattr(plain, name).grad.float() + (0.5 + i)
        got = getattr(mixed, name).main_grad
        # the plain gradient went through one rounding to bf16, the accumulated one did not
        assert_close(got, want, name, atol=2e-2, rtol=1e-2, row_scale=True)
    assert mixed.cmp_k_weight.grad is None
    assert mixed.cmp_v_weight.grad_added_to_main_grad is True
    assert mixed.cmp_v_weight.grad is not None and mixed.cmp_v_weight.grad.shape == mixed.cmp_v_weight.shape


@pytest.mark.parametrize("block_size,lens,QH,KH", [(64, [5000, 700, 333, 64, 0, 1500], 32, 2),
                                                   (128, [3000, 129], 16, 2), (32, [2500, 77], 8, 4)])
def test_deterministic_dk_dv(device, block_size, lens, QH, KH):
    """dkdv_repeat=True / NSAHelper.set_deterministic: the work items of the dk/dv kernels store into their own slots
    and a second launch sums them in a fixed order.  Two runs are bit-identical in every gradient, and the results
    agree with the default (atomic) mode to the order of fp32 summation.  The sequences are long enough for several
    query chunks per key tile and several list chunks per selection block (forced small chunk sizes)."""
    from flash_nsa import NSAConfig, NSACore, NSAHelper
    from flash_nsa.ops.compress_kv import mean_pooling_fwd
    from flash_nsa.ops.compress_attn import cmp_attn_fwd, cmp_attn_bwd
    from flash_nsa.ops.select_attn import slc_attn_fwd, slc_attn_bwd
    from flash_nsa.ops.topk import slc_topk_indices, get_bind_from_find
    D = 128
    cu = make_cu(lens)
    T = int(cu[-1])
    q, k, v, w = [t.to(device) for t in make_qkvw(T, QH, KH, D, seed=120)]
    do = randn_bf16(T, QH, D, seed=125).to(device)
    # the operators, with chunk sizes that give every key several work items
    H = setup_helper(cu.to(device), block_size=block_size, top_n=6)
    ck, cv = mean_pooling_fwd(k), mean_pooling_fwd(v)
    o, lse = cmp_attn_fwd(q, ck, cv)
    runs = [cmp_attn_bwd(q, ck, cv, o, lse, do, dkdv_repeat=True, q_chunk_tokens=256, parts="dkdv")[1:] for _ in range(3)]
    for r in runs[1:]:
        assert torch.equal(r[0], runs[0][0]) and torch.equal(r[1], runs[0][1]), "compressed dk/dv differ between runs"
    _, dk_a, dv_a = cmp_attn_bwd(q, ck, cv, o, lse, do, q_chunk_tokens=256, parts="dkdv")
    assert_close(runs[0][0], dk_a, "compressed dk: ordered sum vs atomics", atol=1e-3, rtol=1e-4)
    assert_close(runs[0][1], dv_a, "compressed dv: ordered sum vs atomics", atol=1e-3, rtol=1e-4)
    topk, _ = slc_topk_indices(q, ck, lse)
    so, slse = slc_attn_fwd(q, k, v, topk)
    bind = get_bind_from_find(topk, chunk_tokens=64)
    base = torch.full((T, KH, D), 0.5, device=device, dtype=torch.float32)   # dk / dv are added into
    sruns = []
    for _ in range(3):
        dk, dv = base.clone(), base.clone()
        slc_attn_bwd(q, k, v, topk, so, slse, do, None, dk, dv, bind=bind, parts="dkdv", dkdv_repeat=True)
        sruns.append((dk, dv))
    for r in sruns[1:]:
        assert torch.equal(r[0], sruns[0][0]) and torch.equal(r[1], sruns[0][1]), "selected dk/dv differ between runs"
    dk, dv = base.clone(), base.clone()
    slc_attn_bwd(q, k, v, topk, so, slse, do, None, dk, dv, bind=bind, parts="dkdv")
    assert_close(sruns[0][0], dk, "selected dk: ordered sum vs atomics", atol=1e-3, rtol=1e-4)
    assert_close(sruns[0][1], dv, "selected dv: ordered sum vs atomics", atol=1e-3, rtol=1e-4)
    # the fused core: every gradient bit-identical across runs, and equal to the default mode up to summation order
    core = NSACore(NSAConfig(head_dim=D, num_heads=QH, num_kv_heads=KH, block_size=block_size, top_n=6))

    def run():
        ts = [t.clone().requires_grad_() for t in (q, k, v, w)]
        core(*ts, cu.to(device)).backward(do)
        return [t.grad for t in ts]

    try:
        NSAHelper.set_deterministic(True)
        a, b = run(), run()
    finally:
        NSAHelper.set_deterministic(False)
    for name, x, y in zip(("dq", "dk", "dv", "dw"), a, b):
        assert torch.equal(x, y), f"{name} differs between two deterministic runs"
    c = run()
    for name, x, y in zip(("dq", "dk", "dv", "dw"), a, c):
        assert_close(x, y.float(), f"{name}: deterministic vs default mode", atol=2e-3, rtol=8e-3, row_scale=True)
