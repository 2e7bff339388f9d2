"""KV-cache writer, its fusion with the pooling (prefill chunk) and with the decode launch, and the page-table
builder driving nsa_prefill / nsa_decode end to end."""
import pytest
import torch

from oracle import nsa_oracle as O
from gpu_util import assert_close, randn_bf16

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("KH,D,VD", [(4, 128, 128), (2, 192, 128), (1, 64, 64)])
def test_store_kvcache_is_bit_exact(device, KH, D, VD):
    from flash_nsa.inference import store_kvcache
    pages, page, N = 7, 64, 300
    kc, vc = randn_bf16(pages, page, KH, D, seed=1), randn_bf16(pages, page, KH, VD, seed=2)
    key, val = randn_bf16(N, KH, D, seed=3), randn_bf16(N, KH, VD, seed=4)
    g = torch.Generator().manual_seed(5)
    slots = torch.randperm(pages * page, generator=g)[:N].to(torch.int32)
    slots[::7] = -1
    rk, rv = kc.clone(), vc.clone()
    O.store_kvcache(key, val, rk, rv, slots)
    dk, dv = kc.to(device), vc.to(device)
    # a view with a row stride larger than the row (the new K/V are usually slices of a fused projection output)
    wide = torch.empty(N, KH * D + KH * VD + 24, dtype=torch.bfloat16, device=device)
    wide[:, :KH * D] = key.view(N, -1).to(device)
    wide[:, KH * D:KH * (D + VD)] = val.view(N, -1).to(device)
    store_kvcache(wide[:, :KH * D].view(N, KH, D), wide[:, KH * D:KH * (D + VD)].view(N, KH, VD), dk, dv,
                  slots.to(device))
    assert torch.equal(dk.cpu(), rk) and torch.equal(dv.cpu(), rv)


def test_fused_store_and_pool_prefill_equals_store_then_pool(device):
    from flash_nsa.inference import (PageTableBuilder, allocate_kv_pools, store_kvcache,
                                     store_kvcache_and_pool_prefill, mean_pooling_prefill)
    KH, D, page = 4, 128, 64
    (k1, v1), (k2, v2) = allocate_kv_pools(120, page, KH, D, num_layers=2, device=device)
    for t in (k1, v1, k2, v2):
        t.zero_()
    b = PageTableBuilder(120, page)
    ids = [0, 1, 2, 3]
    for chunk, new in enumerate(([100, 31, 700, 64], [333, 1, 48, 200], [16, 500, 15, 17])):
        st = b.prefill(ids, new, device=device)
        t = sum(new)
        key, val = randn_bf16(t, KH, D, seed=10 + chunk).to(device), randn_bf16(t, KH, D, seed=20 + chunk).to(device)
        store_kvcache(key, val, k1, v1, st["slot_mapping"])
        for cache in (k1, v1):
            mean_pooling_prefill(cache, st["y_cu_seqlens"], st["y_maxlen"], st["block_tables"],
                                 st["cmp_slot_mapping"])
        store_kvcache_and_pool_prefill(key, val, k2, v2, st["x_cu_seqlens"], st["x_maxlen"], st["context_lens"],
                                       st["slot_mapping"], st["y_cu_seqlens"], st["y_maxlen"],
                                       st["cmp_slot_mapping"], st["block_tables"])
        assert torch.equal(k1, k2) and torch.equal(v1, v2), f"chunk {chunk}"
    assert float(k1.abs().sum()) > 0


@pytest.mark.parametrize("QH,KH,D,caps", [(64, 4, 128, (512, 64)), (16, 2, 128, (8192, 2048))])
def test_generation_loop_equals_training_forward(device, QH, KH, D, caps):
    """Two prefill chunks and 40 decode steps for three sequences, the K/V of every step handed to nsa_prefill /
    nsa_decode as new rows (cache write fused into the step) with tables from the PageTableBuilder: every output row
    equals the row of the training forward on the whole sequence.  caps = (fixed_y_maxlen, fixed_num_slc_blocks):
    the first setting takes the one-launch decode kernel, the second the two-launch path with a separate writer."""
    from flash_nsa import NSAConfig, NSACore, nsa_prefill, nsa_decode
    from flash_nsa.inference import PageTableBuilder, allocate_kv_pools
    page, n_dec = 128, 40
    prompts = [(300, 213), (64, 31), (1, 700)]          # two chunks per sequence
    total = [a + c + n_dec for a, c in prompts]
    (kc, vc), = allocate_kv_pools(40, page, KH, D, device=device)
    kc.zero_(); vc.zero_()
    b = PageTableBuilder(40, page)
    ids = [10, 20, 30]
    q = [randn_bf16(L, QH, D, seed=100 + i).to(device) for i, L in enumerate(total)]
    k = [randn_bf16(L, KH, D, seed=200 + i).to(device) for i, L in enumerate(total)]
    v = [randn_bf16(L, KH, D, seed=300 + i).to(device) for i, L in enumerate(total)]
    w = [randn_bf16(L, QH, 3, seed=400 + i).to(device) for i, L in enumerate(total)]
    kw = dict(fixed_y_maxlen=caps[0], fixed_num_slc_blocks=caps[1])
    outs = [[] for _ in ids]
    pos = [0, 0, 0]
    for chunk in range(2):
        new = [p[chunk] for p in prompts]
        st = b.prefill(ids, new, device=device)
        cat = lambda xs: torch.cat([x[pos[i]:pos[i] + new[i]] for i, x in enumerate(xs)])
        slot_mapping = st.pop("slot_mapping")
        o = nsa_prefill(cat(q), kc, vc, cat(w), new_k=cat(k), new_v=cat(v), slot_mapping=slot_mapping, **st, **kw)
        off = 0
        for i in range(3):
            outs[i].append(o[off:off + new[i]])
            off += new[i]
            pos[i] += new[i]
    for step in range(n_dec):
        st = b.decode(ids, device=device)
        row = lambda xs: torch.stack([x[pos[i]] for i, x in enumerate(xs)])
        slot_mapping = st.pop("slot_mapping")
        o = nsa_decode(row(q), kc, vc, row(w), st["context_lens"], st["block_tables"], st["cmp_slot_mapping"],
                       st["cmp_block_tables"], new_k=row(k), new_v=row(v), slot_mapping=slot_mapping, **kw)
        for i in range(3):
            outs[i].append(o[i:i + 1])
            pos[i] += 1
    core = NSACore(NSAConfig(head_dim=D, num_heads=QH, num_kv_heads=KH))
    for i, L in enumerate(total):
        with torch.no_grad():
            full = core(q[i], k[i], v[i], w[i], torch.tensor([0, L], dtype=torch.int32, device=device))
        got = torch.cat(outs[i])
        assert got.shape == full.shape
        assert_close(got, full, f"sequence {i}: paged generation vs training forward", atol=1e-2, rtol=1e-2)
        # the pool holds the sequence's rows and compressed rows
        rows = torch.tensor([b.slot(ids[i], p) for p in range(L)], device=device)
        assert torch.equal(kc.view(-1, KH, D)[rows], k[i]) and torch.equal(vc.view(-1, KH, D)[rows], v[i])


@pytest.mark.parametrize("window", [64, 128, 512])
def test_fused_cache_write_is_ordered_before_the_window_reads(device, window):
    """The one-launch decode kernel writes the newest token's K/V row itself when the caller passes it.  On steps that
    pool nothing the row is stored after the kernel's first barrier, and with a short context or a narrow window the
    wave that attends the window's last unit (which holds that row) is ready for it early: its fetch must come after
    the store.  The pool rows of the newest tokens hold large finite garbage before the step, so a read that overtakes
    the store changes the output; the reference is the separate writer followed by the same kernel without new rows."""
    from flash_nsa.inference import decode_one_launch, store_kvcache, decode_one_launch_fits
    from paged_util import build_pool, prepool, decode_slot_mapping
    QH, KH, D, page = 64, 4, 128, 128
    ctx = [1, 2, 17, 31, 33, 47, 63, 65, 97, 130, 200, 223, 225, 300, 513, 1000]   # none completes a compressed row
    B = len(ctx)
    case = build_pool(ctx, KH, D, D, page=page, seed=41)
    prepool(case, ctx)
    slots = decode_slot_mapping(case)
    assert int((slots >= 0).sum()) == 0, "this test is about steps that pool nothing"
    raw_slot = torch.tensor([int(case["bt"][b, (L - 1) // page]) * page + (L - 1) % page for b, L in enumerate(ctx)],
                            dtype=torch.int32)
    new_k, new_v = randn_bf16(B, KH, D, seed=42), randn_bf16(B, KH, D, seed=43)
    q, w = randn_bf16(B, QH, D, seed=44).to(device), randn_bf16(B, QH, 3, seed=45).to(device)
    ctx_t = torch.tensor(ctx, dtype=torch.int32, device=device)
    # garbage where the newest rows go
    for name in ("k", "v"):
        case[name].view(-1, KH, D)[raw_slot.long()] = 3.0e4
    kw = dict(fixed_y_maxlen=256, fixed_num_slc_blocks=32, window_size=window, return_parts=True)
    d1 = {k: (v.to(device) if torch.is_tensor(v) else v) for k, v in case.items()}
    d2 = {k: (v.to(device) if torch.is_tensor(v) else v) for k, v in case.items()}
    assert decode_one_launch_fits(q, d1["k"], d1["v"], d1["bt"], 256, 32)
    store_kvcache(new_k.to(device), new_v.to(device), d1["k"], d1["v"], raw_slot.to(device))
    ref = decode_one_launch(q, d1["k"], d1["v"], w, d1["bt"], d1["cbt"], ctx_t, cmp_slot_mapping=slots.to(device), **kw)
    for rep in range(3):
        d2["k"].copy_(case["k"].to(device)); d2["v"].copy_(case["v"].to(device))
        got = decode_one_launch(q, d2["k"], d2["v"], w, d2["bt"], d2["cbt"], ctx_t, cmp_slot_mapping=slots.to(device),
                                new_k=new_k.to(device), new_v=new_v.to(device), slot_mapping=raw_slot.to(device), **kw)
        torch.cuda.synchronize()
        for name, a, r in zip(("out", "cmp_o", "slc_o", "swa_o", "topk", "lse"), got, ref):
            assert torch.equal(a, r), f"{name}: fused cache write differs from store + decode (repeat {rep})"
        assert torch.equal(d1["k"], d2["k"]) and torch.equal(d1["v"], d2["v"])
    assert torch.isfinite(ref[0].float()).all()
