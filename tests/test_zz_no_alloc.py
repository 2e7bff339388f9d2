"""nsa_decode_split_static (the entry point that allocates nothing: its scratch is a static device array) against
nsa_decode_split with caller-allocated scratch, through the C ABI: same kernels, same arithmetic, so every output is
bit-identical -- on two calls in a row, the second with a smaller batch and shorter contexts, so that the second
call runs over what the first left in the shared array."""
import pytest
import torch

from gpu_util import randn_bf16
from paged_util import build_pool, decode_slot_mapping, prepool

pytestmark = pytest.mark.gpu

QH, KH, D = 64, 4, 128


def _to_dev(case, device):
    return {k: (v.to(device) if torch.is_tensor(v) else v) for k, v in case.items()}


def _run_both(device, ctx, nsplit, y_cap, nb_cap, seed, pool_new_row):
    from flash_nsa.inference import decode_split
    case = build_pool(ctx, KH, D, D, page=128, seed=seed)
    prepool(case, [L - 1 for L in ctx] if pool_new_row else ctx)
    slots = decode_slot_mapping(case).to(device) if pool_new_row else None
    B = len(ctx)
    q, w = randn_bf16(B, QH, D, seed=seed + 1).to(device), randn_bf16(B, QH, 3, seed=seed + 2).to(device)
    ctx_t = torch.tensor(ctx, dtype=torch.int32, device=device)
    d1, d2 = _to_dev(case, device), _to_dev(case, device)
    d2["k"], d2["v"] = d2["k"].clone(), d2["v"].clone()
    kw = dict(nsplit=nsplit, fixed_y_maxlen=y_cap, fixed_num_slc_blocks=nb_cap, return_parts=True,
              cmp_slot_mapping=slots)
    ref = decode_split(q, d1["k"], d1["v"], w, d1["bt"], d1["cbt"], ctx_t, **kw)
    got = decode_split(q, d2["k"], d2["v"], w, d2["bt"], d2["cbt"], ctx_t, static_scratch=True, **kw)
    torch.cuda.synchronize()
    names = ("out", "cmp_o", "slc_o", "swa_o", "topk", "lse")
    live = ctx_t > 0
    for name, a, r in zip(names, got, ref):
        if name == "topk":
            a, r = a[:, live], r[:, live]
        else:
            a, r = a[live], r[live]
        assert torch.equal(a, r), f"{name}: static-scratch call differs from the caller-scratch call"
    assert torch.equal(d1["k"], d2["k"]) and torch.equal(d1["v"], d2["v"]), "pooled rows differ"
    assert torch.isfinite(got[0][live].float()).all()


def test_static_scratch_decode_equals_caller_scratch_two_calls_in_a_row(device):
    from flash_nsa import _lib
    cap = _lib.value("nsa_decode_split_static_capacity")
    assert cap == 32 << 20
    # first call: 9 requests up to 8K tokens in 4 parts; second: 3 shorter requests in 2 parts
    assert _lib.value("nsa_decode_split_static_bytes", 9, KH, D, 4, 512) <= cap
    _run_both(device, [8192, 4099, 333, 48, 31, 2064, 1, 777, 6000], nsplit=4, y_cap=512, nb_cap=128, seed=71,
              pool_new_row=True)
    _run_both(device, [1500, 640, 96], nsplit=2, y_cap=512, nb_cap=128, seed=75, pool_new_row=True)
    # and once more at the first size, now over the second call's leftovers
    _run_both(device, [8192, 4099, 333, 48, 31, 2064, 1, 777, 6000], nsplit=4, y_cap=512, nb_cap=128, seed=79,
              pool_new_row=False)


def test_static_scratch_decode_refuses_sizes_beyond_its_buffer(device):
    from flash_nsa import _lib
    from flash_nsa.inference import decode_split
    ctx = [64] * 40
    assert _lib.value("nsa_decode_split_static_bytes", len(ctx), KH, D, 8, 8192) > (32 << 20)
    case = build_pool(ctx, KH, D, D, page=128, seed=81)
    prepool(case, ctx)
    d = _to_dev(case, device)
    q, w = randn_bf16(len(ctx), QH, D, seed=82).to(device), randn_bf16(len(ctx), QH, 3, seed=83).to(device)
    ctx_t = torch.tensor(ctx, dtype=torch.int32, device=device)
    with pytest.raises(RuntimeError, match="static buffer holds"):
        decode_split(q, d["k"], d["v"], w, d["bt"], d["cbt"], ctx_t, nsplit=8, fixed_y_maxlen=8192,
                     fixed_num_slc_blocks=2048, static_scratch=True)


def test_static_scratch_decode_under_graph_capture(device):
    """What the entry point is for: the step recorded into a HIP graph (its outputs come from the graph's own pool, the
    scratch from the static array) replays bit-equal to the eager call, several times, with the program's own eager
    work and synchronisations between the replays and with new inputs through the same buffers."""
    from flash_nsa.inference import decode_split
    ctx = [8192, 4099, 333, 2064, 777, 6000]
    case = build_pool(ctx, KH, D, D, page=128, seed=85)
    prepool(case, ctx)
    d = _to_dev(case, device)
    B = len(ctx)
    q, w = randn_bf16(B, QH, D, seed=86).to(device), randn_bf16(B, QH, 3, seed=87).to(device)
    ctx_t = torch.tensor(ctx, dtype=torch.int32, device=device)
    kw = dict(nsplit=4, fixed_y_maxlen=512, fixed_num_slc_blocks=128, static_scratch=True)
    args = (q, d["k"], d["v"], w, d["bt"], d["cbt"], ctx_t)
    eager = decode_split(*args, **kw).clone()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = decode_split(*args, **kw)
    for it in range(3):
        out.zero_()
        junk = torch.randn(1 << 20, device=device).sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {it} differs from the eager call"
    q.copy_(randn_bf16(B, QH, D, seed=88).to(device))
    eager2 = decode_split(*args, **kw).clone()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, eager2) and not torch.equal(eager, eager2)
