"""Paged-KV inference entry points (mirrors upstream flash_nsa/inference/__init__.py:21-257).

Both functions expect the new tokens' K/V to be already written into the pool and `context_lens` to include
them; they write the newly completed compressed rows into the same pool (mean pooling only, as upstream) and
never synchronise with the host, so the decode step can be captured in a HIP graph."""
from .stages import (mean_pooling_prefill, kv_mean_pooling_decode, cmp_attn_prefill, cmp_attn_decode, topk_prefill,
                     topk_decode, slc_attn_prefill, fused_slc_swa_attn_decode, swa_prefill, combine_prefill,
                     combine_decode, mean_pooling_decode, slc_attn_decode, fused_decode_supported, decode_cmp_topk,
                     decode_slc_swa_combine, decode_cmp_split, decode_one_launch, decode_one_launch_fits,
                     store_kvcache, store_kvcache_and_pool_prefill, decode_split, decode_split_fits)
from .paging import PageTableBuilder, allocate_kv_pools


def nsa_prefill(q, k, v, w, x_cu_seqlens, y_cu_seqlens, x_maxlen, y_maxlen, context_lens, block_tables,
                cmp_slot_mapping, cmp_block_tables, fixed_y_maxlen=8192, fixed_num_slc_blocks=2048, kernel_size=32,
                stride=16, block_size=64, top_n=16, num_init_blocks=1, num_local_blocks=2, window_size=512,
                sm_scale=None, new_k=None, new_v=None, slot_mapping=None):
    """Chunked / prefix-cached prefill.
    q [t,QH,D] new tokens only; k, v [pages, page_size, KH, D|VD] pools; w [t,QH,3];
    x_cu_seqlens [B+1] offsets of the new tokens; y_cu_seqlens [B+1] offsets of ALL compressed rows per request;
    context_lens [B] total lengths; block_tables [B,N1]; cmp_slot_mapping [y_cu[-1]] flat destination row of each
    compressed row or -1 if it was pooled by an earlier chunk; cmp_block_tables [B,N2].  Returns o [t,QH,VD].
    As upstream, the new tokens' K/V are expected in the pools already; alternatively pass them as new_k / new_v
    [t,KH,*] with their flat pool rows slot_mapping [t] and the cache write is fused with the pooling (one launch)."""
    assert k.size(1) % 64 == 0, "page size must be a multiple of 64"
    if sm_scale is None:
        sm_scale = q.size(-1) ** -0.5
    if new_k is not None:
        store_kvcache_and_pool_prefill(new_k, new_v, k, v, x_cu_seqlens, x_maxlen, context_lens, slot_mapping,
                                       y_cu_seqlens, y_maxlen, cmp_slot_mapping, block_tables,
                                       kernel_size=kernel_size, stride=stride)
    else:
        mean_pooling_prefill(k, y_cu_seqlens, y_maxlen, block_table=block_tables, slot_mapping=cmp_slot_mapping,
                             kernel_size=kernel_size, stride=stride)
        mean_pooling_prefill(v, y_cu_seqlens, y_maxlen, block_table=block_tables, slot_mapping=cmp_slot_mapping,
                             kernel_size=kernel_size, stride=stride)
    cmp_o, lse = cmp_attn_prefill(q, k, v, x_cu_seqlens, x_maxlen, block_tables=cmp_block_tables,
                                  context_lens=context_lens, kernel_size=kernel_size, stride=stride,
                                  sm_scale=sm_scale)
    topk = topk_prefill(q, k, lse, x_cu_seqlens, x_maxlen, y_maxlen, block_tables=cmp_block_tables,
                        context_lens=context_lens, fixed_y_maxlen=fixed_y_maxlen,
                        fixed_num_slc_blocks=fixed_num_slc_blocks, sm_scale=sm_scale, kernel_size=kernel_size,
                        stride=stride, block_size=block_size, top_n=top_n, num_inital=num_init_blocks,
                        num_local=num_local_blocks)
    slc_o, _ = slc_attn_prefill(q, k, v, topk, x_cu_seqlens, x_maxlen, block_tables=block_tables,
                                context_lens=context_lens, block_size=block_size, top_n=top_n, sm_scale=sm_scale)
    swa_o = swa_prefill(q, k, v, x_cu_seqlens, x_maxlen, block_tables=block_tables, context_lens=context_lens,
                        window_size=window_size, sm_scale=sm_scale)
    return combine_prefill(cmp_o, slc_o, swa_o, w)


def auto_cmp_splits(batch, num_kv_heads, fixed_y_maxlen, num_cus=256, one_launch_fits=None):
    """Parts the compressed branch of a decode step is cut into per (request, kv head); 1 = not cut.
    one_launch_fits: whether the one-launch kernel holds this capacity (None: assumed up to 2048 compressed rows).
    Measured on MI355X (4 kv heads, d = 128, graph replay, microseconds for 1 / 2 / 4 / 8 parts):
      capacity 2048 rows (one launch possible): 1 x 32K 50 / 49 / 46 / 42, 4 x 32K 52 / 54 / 51 / 47, 4 x 4K
      38 / 39 / 40 / 39, 8 x 32K 54 / 59 / 58 / 55, 16 x 32K 61 / 62 / 62 / 65 -- parts pay for up to 16 (request,
      kv head) pairs and then only with 8 of them; short contexts in a large capacity lose 1-2 us to them;
      capacity 8192 rows (two launches without parts): 8 x 64K 105 / 72 / 68 / 64, 16 x 64K 114 / 80 / 77 / 80,
      16 x 128K 192 / 127 / 114 / 114, 32 x 64K 140 / 111 / 119 / 126, 32 x 128K 240 / 185 / 188 / 191;
      8 / 16 / 32 / 64 parts: 1 x 128K 61.3 / 58.8 / 61.1 / 69.1, 2 x 128K 64.8 / 62.7 / 65.9 / 76.8, 4 x 128K
      67.9 / 68.3 / 76.7 / 89.6 -- 16 parts pay for up to 8 pairs."""
    pairs = batch * num_kv_heads
    if fixed_y_maxlen < 1024:
        return 1
    if one_launch_fits is None:
        one_launch_fits = fixed_y_maxlen <= 2048
    scale = num_cus / 256.0
    if one_launch_fits:
        return 8 if pairs <= 16 * scale else 1
    if pairs <= 8 * scale and fixed_y_maxlen >= 8192:
        return 16
    if pairs <= 32 * scale:
        return 8
    if pairs <= 64 * scale:
        return 4
    if pairs <= 128 * scale:
        return 2
    return 1


def nsa_decode(q, k, v, w, context_lens, block_tables, cmp_slot_mapping, cmp_block_tables, cmp_num_splits=0,
               slc_num_splits=0, fixed_y_maxlen=8192, fixed_num_slc_blocks=2048, kernel_size=32, stride=16,
               block_size=64, top_n=16, num_init_blocks=1, num_local_blocks=2, window_size=512, sm_scale=None,
               new_k=None, new_v=None, slot_mapping=None):
    """One query token per request.  q [B,QH,D]; w [B,QH,3]; cmp_slot_mapping [B] (-1: no compressed row completes
    at this step).  Rows with context_lens == 0 (graph padding) produce zeros.  Returns o [B,QH,VD].
    cmp_num_splits: 0 = chosen from the batch size and fixed_y_maxlen (auto_cmp_splits), 1 = never split.
    slc_num_splits (upstream flash_nsa/inference/__init__.py:195-196): > 1 cuts the window and selected blocks of a
    request over that many workgroups; honoured where the compressed branch is cut as well (the two-launch path for
    small batches of long contexts, plus a merging launch), ignored by the one-launch kernel, whose batches fill the
    GPU without it.  Measured, it does not pay on MI355X (one request of 128K tokens: 61.5 us with or without).
    As upstream, the newest token's K/V are expected in the pools already; alternatively pass them as new_k / new_v
    [B,KH,*] with their flat pool rows slot_mapping [B] (-1: padding) and the cache write happens here (inside the
    single decode launch when that path is taken)."""
    assert k.size(1) % 64 == 0, "page size must be a multiple of 64"
    if sm_scale is None:
        sm_scale = q.size(-1) ** -0.5
    if cmp_num_splits == 0:
        # the split kernels exist for the shapes of the fused decode kernels (head dims 128/128 or 64/64, at most 16
        # q-heads per kv head)
        if fused_decode_supported(q, k, v):
            fits = decode_one_launch_fits(q, k, v, block_tables, fixed_y_maxlen, fixed_num_slc_blocks)
            cmp_num_splits = auto_cmp_splits(q.size(0), k.size(2), fixed_y_maxlen, one_launch_fits=fits)
        else:
            cmp_num_splits = 1
    one_launch = (fused_decode_supported(q, k, v) and cmp_num_splits <= 1 and
                  decode_one_launch_fits(q, k, v, block_tables, fixed_y_maxlen, fixed_num_slc_blocks))
    if one_launch:
        # pooling of the newest compressed row included
        return decode_one_launch(q, k, v, w, block_tables, cmp_block_tables, context_lens,
                                 fixed_y_maxlen=fixed_y_maxlen, fixed_num_slc_blocks=fixed_num_slc_blocks,
                                 kernel_size=kernel_size, stride=stride, block_size=block_size, top_n=top_n,
                                 num_inital=num_init_blocks, num_local=num_local_blocks, window_size=window_size,
                                 sm_scale=sm_scale, cmp_slot_mapping=cmp_slot_mapping, new_k=new_k, new_v=new_v,
                                 slot_mapping=slot_mapping)
    if new_k is not None:
        store_kvcache(new_k, new_v, k, v, slot_mapping)
    if (fused_decode_supported(q, k, v) and cmp_num_splits > 1 and
            decode_split_fits(q, k, v, block_tables, fixed_y_maxlen, fixed_num_slc_blocks)):
        # small batches of long contexts: the compressed branch is cut in that many key-interleaved parts per
        # (request, kv head); two launches.  From 8 requests on the first of them also pools the newest compressed
        # row (2 us less than the pooling launch at 16-32 requests); below that the pooling, which sits in front of
        # the one workgroup that owns the last unit, costs more than its launch (46 -> 49 us for one request).
        fuse_pool = q.size(0) >= 8
        if not fuse_pool:
            kv_mean_pooling_decode(k, v, block_table=block_tables, slot_mapping=cmp_slot_mapping,
                                   context_lens=context_lens, kernel_size=kernel_size, stride=stride)
        return decode_split(q, k, v, w, block_tables, cmp_block_tables, context_lens, nsplit=cmp_num_splits,
                            fixed_y_maxlen=fixed_y_maxlen, fixed_num_slc_blocks=fixed_num_slc_blocks,
                            kernel_size=kernel_size, stride=stride, block_size=block_size, top_n=top_n,
                            num_inital=num_init_blocks, num_local=num_local_blocks, window_size=window_size,
                            sm_scale=sm_scale, cmp_slot_mapping=cmp_slot_mapping if fuse_pool else None,
                            slc_nsplit=max(1, min(int(slc_num_splits), 16)))
    kv_mean_pooling_decode(k, v, block_table=block_tables, slot_mapping=cmp_slot_mapping, context_lens=context_lens,
                           kernel_size=kernel_size, stride=stride)
    if fused_decode_supported(q, k, v):
        if cmp_num_splits <= 1:
            # two fused launches: (compressed attention + importance + selection), (selected + window + combine)
            cmp_o, topk = decode_cmp_topk(q, k, v, cmp_block_tables, context_lens, fixed_y_maxlen=fixed_y_maxlen,
                                          fixed_num_slc_blocks=fixed_num_slc_blocks, kernel_size=kernel_size,
                                          stride=stride, block_size=block_size, top_n=top_n,
                                          num_inital=num_init_blocks, num_local=num_local_blocks, sm_scale=sm_scale)
            return decode_slc_swa_combine(q, k, v, w, topk, cmp_o, block_tables, context_lens, block_size=block_size,
                                          top_n=top_n, window_size=window_size, sm_scale=sm_scale)
        # parts with capacities beyond the LDS of the two-launch path: three launches after the pooling, the
        # probabilities recomputed from the keys
        cmp_o, pg = decode_cmp_split(q, k, v, cmp_block_tables, context_lens, nsplit=cmp_num_splits,
                                     fixed_y_maxlen=fixed_y_maxlen, kernel_size=kernel_size, stride=stride,
                                     sm_scale=sm_scale)
        out, _topk = decode_slc_swa_combine(q, k, v, w, None, cmp_o, block_tables, context_lens,
                                            block_size=block_size, top_n=top_n, window_size=window_size,
                                            sm_scale=sm_scale, pg=pg, fixed_num_slc_blocks=fixed_num_slc_blocks,
                                            kernel_size=kernel_size, stride=stride, num_inital=num_init_blocks,
                                            num_local=num_local_blocks)
        return out
    return nsa_decode_staged(q, k, v, w, context_lens, block_tables, cmp_block_tables, cmp_num_splits, slc_num_splits,
                             fixed_y_maxlen, fixed_num_slc_blocks, kernel_size, stride, block_size, top_n,
                             num_init_blocks, num_local_blocks, window_size, sm_scale)


def nsa_decode_staged(q, k, v, w, context_lens, block_tables, cmp_block_tables, cmp_num_splits=0, slc_num_splits=0,
                      fixed_y_maxlen=8192, fixed_num_slc_blocks=2048, kernel_size=32, stride=16, block_size=64,
                      top_n=16, num_init_blocks=1, num_local_blocks=2, window_size=512, sm_scale=None):
    """The decode step stage by stage (after pooling), through the stage functions that mirror upstream's; used when
    a kv head has more than 16 q-heads, and by the tests as a second implementation of the fused path."""
    if sm_scale is None:
        sm_scale = q.size(-1) ** -0.5
    cmp_o, lse = cmp_attn_decode(q, k, v, block_tables=cmp_block_tables, context_lens=context_lens,
                                 num_splits=cmp_num_splits, kernel_size=kernel_size, stride=stride,
                                 sm_scale=sm_scale)
    topk = topk_decode(q, k, lse, fixed_y_maxlen=fixed_y_maxlen, fixed_num_slc_blocks=fixed_num_slc_blocks,
                       block_tables=cmp_block_tables, context_lens=context_lens, kernel_size=kernel_size,
                       stride=stride, block_size=block_size, top_n=top_n, num_inital=num_init_blocks,
                       num_local=num_local_blocks, sm_scale=sm_scale)
    slc_o, swa_o = fused_slc_swa_attn_decode(q, k, v, topk, num_splits=slc_num_splits, block_tables=block_tables,
                                             context_lens=context_lens, block_size=block_size, top_n=top_n,
                                             window_size=window_size, sm_scale=sm_scale)
    return combine_decode(cmp_o, slc_o, swa_o, w)
