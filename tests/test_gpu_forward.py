"""GPU parity of the forward operators against the CPU oracle (same seeded bf16 inputs).
Mirrors upstream test.py --func mean/construct/cmp/topk/slc/combine (test.py:74-318), with asserted tolerances."""
import pytest
import torch

from oracle import nsa_oracle as O
from gpu_util import make_cu, make_qkvw, randn_bf16, assert_close

pytestmark = pytest.mark.gpu

LENS_CASES = [
    [1000],
    [5, 31, 32, 47, 48, 100, 333, 700],
    [64, 0, 129, 513],
]
HEAD_CASES = [(16, 1, 128), (8, 2, 128), (4, 4, 64)]


def setup_helper(cu_dev, **kw):
    from flash_nsa import NSAHelper
    NSAHelper.set_hyperparameters(**kw)
    NSAHelper.init_cu_seqlens(cu_dev)
    return NSAHelper


@pytest.mark.parametrize("lens", LENS_CASES)
def test_mean_pooling_and_construct_block(device, lens):
    from flash_nsa.ops.compress_kv import mean_pooling_fwd, construct_block_fwd
    cu = make_cu(lens)
    T = int(cu[-1])
    x = randn_bf16(T, 4, 128, seed=1)
    setup_helper(cu.to(device))
    y = mean_pooling_fwd(x.to(device))
    ref = O.mean_pooling(x.float(), cu)
    assert y.shape == ref.shape
    # fp32 mean rounded to bf16: allow one bf16 ulp of slack for summation order
    assert_close(y, ref, "mean_pooling", atol=2e-3, rtol=8e-3)
    blk = construct_block_fwd(x.to(device))
    refb = O.construct_block(x.float(), cu)
    assert torch.equal(blk.float().cpu(), refb)


@pytest.mark.parametrize("lens", LENS_CASES)
@pytest.mark.parametrize("QH,KH,D", HEAD_CASES)
def test_cmp_attn_fwd(device, lens, QH, KH, D):
    from flash_nsa.ops.compress_kv import mean_pooling_fwd
    from flash_nsa.ops.compress_attn import cmp_attn_fwd
    cu = make_cu(lens)
    T = int(cu[-1])
    q, k, v, _ = make_qkvw(T, QH, KH, D, seed=10)
    setup_helper(cu.to(device))
    ck = mean_pooling_fwd(k.to(device))
    cv = mean_pooling_fwd(v.to(device))
    o, lse = cmp_attn_fwd(q.to(device), ck, cv)
    ro, rl = O.cmp_attn(q.float(), ck.float().cpu(), cv.float().cpu(), cu)
    assert_close(o, ro, "cmp_o")
    assert_close(lse, rl, "cmp_lse", atol=1e-3, rtol=1e-4)


@pytest.mark.parametrize("lens", LENS_CASES)
@pytest.mark.parametrize("QH,KH,D", HEAD_CASES)
def test_swa_fwd(device, lens, QH, KH, D):
    from flash_nsa.ops.sliding_window_attention import swa_fwd
    cu = make_cu(lens)
    T = int(cu[-1])
    q, k, v, _ = make_qkvw(T, QH, KH, D, seed=20)
    setup_helper(cu.to(device), window_size=200)
    o, lse = swa_fwd(q.to(device), k.to(device), v.to(device))
    ro, rl = O.swa(q.float(), k.float(), v.float(), cu, 200)
    assert_close(o, ro, "swa_o")
    assert_close(lse, rl, "swa_lse", atol=1e-3, rtol=1e-4)
    setup_helper(cu.to(device))


GROUP_CASES = [(32, 1, 128), (64, 1, 64), (16, 2, 128), (6, 3, 64), (12, 4, 64)]  # groups of 32, 64, 8, 2, 3


@pytest.mark.parametrize("lens,QH,KH,D", [(l, *h) for l in LENS_CASES for h in HEAD_CASES] +
                         [(LENS_CASES[1], *h) for h in GROUP_CASES])
def test_topk_and_slc_fwd(device, lens, QH, KH, D):
    from flash_nsa.ops.compress_kv import mean_pooling_fwd
    from flash_nsa.ops.compress_attn import cmp_attn_fwd
    from flash_nsa.ops.topk import slc_topk_indices
    from flash_nsa.ops.select_attn import slc_attn_fwd
    cu = make_cu(lens)
    T = int(cu[-1])
    q, k, v, _ = make_qkvw(T, QH, KH, D, seed=30)
    top_n = 6
    setup_helper(cu.to(device), top_n=top_n)
    cfg = O.OracleConfig(top_n=top_n)
    qd, kd, vd = q.to(device), k.to(device), v.to(device)
    ck = mean_pooling_fwd(kd)
    cv = mean_pooling_fwd(vd)
    _, lse = cmp_attn_fwd(qd, ck, cv)
    topk, probs = slc_topk_indices(qd, ck, lse, return_slc_prob=True)
    rt, imps = O.slc_topk(q.float(), ck.float().cpu(), None, cu, cfg, return_importance=True)
    assert topk.dtype == torch.int32 and topk.shape == (KH, T, top_n)
    n_rows, n_diff, n_bad = O.topk_mismatch_report(topk.cpu(), rt, imps, cu, 64, top_n, tie_tol=1e-3)
    assert n_bad == 0, f"{n_bad} rows differ beyond score ties ({n_diff} differing of {n_rows})"
    assert n_diff <= max(1, n_rows // 200)
    # slot order and ignore value: rows identical to the oracle wherever the sets agree
    same = (topk.cpu() == rt).all(-1)
    assert same.float().mean() > 0.99
    # block scores returned on request match the oracle's
    for b in range(len(lens)):
        a, e = int(cu[b]), int(cu[b + 1])
        nb = imps[b].shape[-1]
        if e > a:
            assert_close(probs[:, a:e, :nb], imps[b], "block scores", atol=2e-3, rtol=2e-3)
    # selected attention with the device's own indices fed to the oracle
    o, l2 = slc_attn_fwd(qd, kd, vd, topk)
    ro, rl = O.slc_attn(q.float(), k.float(), v.float(), topk.cpu(), cu, 64)
    assert_close(o, ro, "slc_o")
    assert_close(l2, rl, "slc_lse", atol=1e-3, rtol=1e-4)
    setup_helper(cu.to(device))


@pytest.mark.parametrize("lens,QH,KH,D", [([9000, 2500, 700], 32, 2, 128), ([6000, 100], 4, 4, 64),
                                          ([5000, 3000], 4, 2, 128), ([4500], 64, 1, 64)])
def test_topk_segmented_selection_equals_one_pass(device, lens, QH, KH, D):
    """Three forms of the block selector must return bit-identical indices and scores: the one-launch kernel with the
    scores of all blocks in LDS, the same kernel working segment by segment (long contexts; the segment length is a
    tuning value), and the two-launch form with the scores in a workspace -- in one pass over all tokens and in chunks
    of as many tokens as a small workspace holds.  All of them match the oracle."""
    from flash_nsa import _lib
    from flash_nsa.ops import topk as topk_mod
    from flash_nsa.ops.compress_kv import mean_pooling_fwd
    from flash_nsa.ops.compress_attn import cmp_attn_fwd
    from flash_nsa.ops.topk import slc_topk_indices
    cu = make_cu(lens)
    T = int(cu[-1])
    q, k, _, _ = make_qkvw(T, QH, KH, D, seed=33)
    setup_helper(cu.to(device))
    qd, kd = q.to(device), k.to(device)
    ck = mean_pooling_fwd(kd)
    _, lse = cmp_attn_fwd(qd, ck, ck)
    G = QH // KH
    results = {}
    try:
        _lib.call("nsa_set_tuning", b"topk_two_pass", 0)
        for seg in (0, 32, 64, 96):
            if seg == 0 and G <= 2:
                continue  # the score rows of 64 / 32 tokens per workgroup do not fit in one pass at this length
            _lib.call("nsa_set_tuning", b"topk_seg_blocks", seg)
            results[seg] = slc_topk_indices(qd, ck, lse, return_slc_prob=True)
    finally:
        _lib.call("nsa_reset_tuning")
    results["auto"] = slc_topk_indices(qd, ck, lse, return_slc_prob=True)
    limit = topk_mod.TOPK_WORKSPACE_LIMIT
    try:
        for small in (1 << 20, 300 << 10):   # a few hundred tokens per chunk, chunk edges inside sequences
            topk_mod.TOPK_WORKSPACE_LIMIT = small
            results[f"workspace {small}"] = slc_topk_indices(qd, ck, lse, return_slc_prob=True)
    finally:
        topk_mod.TOPK_WORKSPACE_LIMIT = limit
    keys = list(results)
    for key in keys[1:]:
        assert torch.equal(results[key][0], results[keys[0]][0]), f"indices differ: segment {key} vs {keys[0]}"
        assert torch.equal(results[key][1], results[keys[0]][1]), f"scores differ: segment {key} vs {keys[0]}"
    topk, probs = results["auto"]
    cfg = O.OracleConfig()
    rt, imps = O.slc_topk(q.float(), ck.float().cpu(), None, cu, cfg, return_importance=True)
    n_rows, n_diff, n_bad = O.topk_mismatch_report(topk.cpu(), rt, imps, cu, 64, 16, tie_tol=1e-3)
    assert n_bad == 0, f"{n_bad} rows differ beyond score ties ({n_diff} differing of {n_rows})"
    assert n_diff <= max(1, n_rows // 200)
    for b in range(len(lens)):
        a, e = int(cu[b]), int(cu[b + 1])
        assert_close(probs[:, a:e, :imps[b].shape[-1]], imps[b], "block scores", atol=2e-3, rtol=2e-3)


def test_combine_fwd(device):
    from flash_nsa.ops.combine import combine_fwd
    a, b, c = [randn_bf16(300, 8, 128, seed=s) for s in (1, 2, 3)]
    w = randn_bf16(300, 8, 3, seed=4)
    o = combine_fwd(a.to(device), b.to(device), c.to(device), w.to(device))
    assert_close(o, O.combine(a.float(), b.float(), c.float(), w.float()), "combine")
