"""Host-side page-table builder (no GPU): the tensors it hands to nsa_prefill / nsa_decode, checked against a
position-by-position restatement of the paging rules."""
import random

import pytest
import torch

from flash_nsa.inference.paging import PageTableBuilder, allocate_kv_pools
from oracle import nsa_oracle as O


def cmp_len(L, kernel=32, stride=16):
    return max((L - kernel) // stride + 1, 0)


def check_tables(b, ids, step, page):
    """every listed page is owned by exactly one sequence; tables are padded with -1"""
    owned = {}
    for row, sid in enumerate(ids):
        s = b.seqs[sid]
        assert len(s.pages) == -(-s.length // page) and len(s.cmp_pages) == -(-cmp_len(s.length) // page)
        for pg in s.pages + s.cmp_pages:
            assert pg not in owned, "a page is listed twice"
            owned[pg] = sid
        bt, cbt = step["block_tables"][row].tolist(), step["cmp_block_tables"][row].tolist()
        assert bt[:len(s.pages)] == s.pages and all(x == -1 for x in bt[len(s.pages):])
        assert cbt[:len(s.cmp_pages)] == s.cmp_pages and all(x == -1 for x in cbt[len(s.cmp_pages):])
    assert not (set(owned) & set(b.free))


def test_prefill_chunks_then_decode_steps_follow_the_paging_rules():
    page = 64
    b = PageTableBuilder(num_pages=400, page_size=page)
    rnd = random.Random(0)
    ids = [3, 7, 11]
    lens = {i: 0 for i in ids}
    pooled = {i: 0 for i in ids}
    for chunk in range(3):  # three prefill chunks per sequence
        new = [rnd.randint(1, 300) for _ in ids]
        st = b.prefill(ids, new, device="cpu")
        x_cu, y_cu = st["x_cu_seqlens"].tolist(), st["y_cu_seqlens"].tolist()
        assert st["x_maxlen"] == max(new)
        for r, sid in enumerate(ids):
            old = lens[sid]
            lens[sid] += new[r]
            assert x_cu[r + 1] - x_cu[r] == new[r] and st["context_lens"][r] == lens[sid]
            slots = st["slot_mapping"][x_cu[r]:x_cu[r + 1]].tolist()
            assert slots == [b.seqs[sid].pages[p // page] * page + p % page for p in range(old, lens[sid])]
            y = cmp_len(lens[sid])
            assert y_cu[r + 1] - y_cu[r] == y
            cs = st["cmp_slot_mapping"][y_cu[r]:y_cu[r + 1]].tolist()
            want = [-1 if i < pooled[sid] else b.seqs[sid].cmp_pages[i // page] * page + i % page for i in range(y)]
            assert cs == want
            pooled[sid] = y
        assert st["y_maxlen"] == max(cmp_len(lens[i]) for i in ids)
        check_tables(b, ids, st, page)
    for _ in range(70):  # decode steps
        st = b.decode(ids, device="cpu")
        for r, sid in enumerate(ids):
            lens[sid] += 1
            L = lens[sid]
            assert st["context_lens"][r] == L
            assert st["slot_mapping"][r] == b.seqs[sid].pages[(L - 1) // page] * page + (L - 1) % page
            y = cmp_len(L)
            if L >= 32 and (L - 32) % 16 == 0:
                assert y == pooled[sid] + 1
                assert st["cmp_slot_mapping"][r] == b.seqs[sid].cmp_pages[(y - 1) // page] * page + (y - 1) % page
                pooled[sid] = y
            else:
                assert st["cmp_slot_mapping"][r] == -1
        check_tables(b, ids, st, page)
    used = sum(len(s.pages) + len(s.cmp_pages) for s in b.seqs.values())
    assert used + len(b.free) == 400
    b.release(7)
    assert 7 not in b.seqs and used - len(b.free) + 400 - used >= 0
    assert sum(len(s.pages) + len(s.cmp_pages) for s in b.seqs.values()) + len(b.free) == 400


def test_decode_padding_for_a_captured_graph_and_exhaustion():
    b = PageTableBuilder(num_pages=6, page_size=64)
    b.prefill([0, 1], [64, 10], device="cpu")
    st = b.decode([0, 1], device="cpu", pad_to=4, raw_width=5, cmp_width=2)
    assert st["context_lens"].tolist() == [65, 11, 0, 0]
    assert st["slot_mapping"].tolist()[2:] == [-1, -1] and st["cmp_slot_mapping"].tolist()[2:] == [-1, -1]
    assert st["block_tables"].shape == (4, 5) and st["cmp_block_tables"].shape == (4, 2)
    assert (st["block_tables"][2:] == -1).all()
    assert b.pages_needed(2, 200) == 4 + 1 and not b.can_extend(2, 200)   # 6 pages, 4 taken: 2 free
    with pytest.raises(RuntimeError, match="exhausted"):
        b.prefill([2], [200], device="cpu")


def test_pools_of_a_layer_share_one_allocation_with_the_v_pool_staggered():
    """K pool then V pool of every layer inside one allocation, none overlapping; every K pool starts on a 1 KB
    boundary and its V pool 256 bytes past one, so that the K rows and the V rows of one kv head fall on different
    quarters of a 1 KB window (the decode kernels stream both at once)."""
    pools = allocate_kv_pools(5, 64, 2, 32, 16, num_layers=3, device="cpu", dtype=torch.float32)
    spans = []
    for k, v in pools:
        assert k.shape == (5, 64, 2, 32) and v.shape == (5, 64, 2, 16)
        assert k.is_contiguous() and v.is_contiguous()
        assert k.data_ptr() % 1024 == 0 and v.data_ptr() % 1024 == 256
        assert 0 <= v.data_ptr() - (k.data_ptr() + k.numel() * k.element_size()) < 2048
        spans += [(t.data_ptr(), t.data_ptr() + t.numel() * t.element_size()) for t in (k, v)]
    spans.sort()
    assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:])), "pools overlap"
    assert k.untyped_storage().data_ptr() == pools[0][0].untyped_storage().data_ptr()


def test_oracle_store_kvcache_is_an_indexed_row_copy():
    g = torch.Generator().manual_seed(0)
    kc, vc = torch.zeros(3, 4, 2, 8), torch.zeros(3, 4, 2, 4)
    key, val = torch.randn(5, 2, 8, generator=g), torch.randn(5, 2, 4, generator=g)
    slots = torch.tensor([7, -1, 0, 11, 3])
    O.store_kvcache(key, val, kc, vc, slots)
    want_k = torch.zeros(12, 2, 8).index_copy_(0, torch.tensor([7, 0, 11, 3]), key[[0, 2, 3, 4]])
    want_v = torch.zeros(12, 2, 4).index_copy_(0, torch.tensor([7, 0, 11, 3]), val[[0, 2, 3, 4]])
    assert torch.equal(kc.view(12, 2, 8), want_k) and torch.equal(vc.view(12, 2, 4), want_v)


def test_decode_picks_parts_only_for_small_batches_of_long_contexts():
    """auto_cmp_splits: one workgroup per (request, kv head) while those pairs fill the GPU or the capacity is below
    16K tokens; a capacity the one-launch kernel holds is cut (into 8) only for up to 16 pairs; larger capacities into
    the power of two of parts, at most 8, that brings the workgroup count back to about the CU count."""
    from flash_nsa.inference import auto_cmp_splits
    assert auto_cmp_splits(64, 4, 4096) == 1          # 256 pairs: the GPU is full
    assert auto_cmp_splits(33, 4, 4096) == 1          # more than half full
    assert auto_cmp_splits(32, 4, 4096) == 2
    assert auto_cmp_splits(16, 4, 8192) == 4
    assert auto_cmp_splits(8, 4, 8192) == 8
    assert auto_cmp_splits(1, 1, 8192) == 16          # 16 only for a handful of pairs at a large capacity
    assert auto_cmp_splits(2, 4, 8192) == 16 and auto_cmp_splits(3, 4, 8192) == 8
    assert auto_cmp_splits(1, 4, 4096) == 8
    assert auto_cmp_splits(1, 1, 2048) == 8           # 32K tokens of capacity: worth the second launch
    assert auto_cmp_splits(4, 4, 2048) == 8 and auto_cmp_splits(5, 4, 2048) == 1   # ... for up to 16 pairs
    assert auto_cmp_splits(8, 4, 2048) == 1 and auto_cmp_splits(8, 4, 2048, one_launch_fits=False) == 8
    assert auto_cmp_splits(1, 1, 1000) == 1           # below 16K tokens of capacity: one launch
    for b in range(1, 80):
        n = auto_cmp_splits(b, 4, 4096)
        assert n in (1, 2, 4, 8) and (n == 1 or b * 4 * n <= 256)
