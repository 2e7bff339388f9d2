"""Stages of the paged-KV inference path (mirrors the stage functions of upstream flash_nsa/inference/*.py).
Prefill stages take the new tokens of every request packed as [t, heads, dim] with x_cu_seqlens; decode stages
take one token per request [B, heads, dim]."""
import torch

from .. import _lib
from ..ops._common import check_bf16
from ..ops.combine import combine_fwd
from ..ops.topk import topk_workspace

_ARANGE = {}


def _decode_cu(B, device):
    """[0,1,...,B] int32 on the device, cached so that a captured decode step allocates nothing for it."""
    key = (B, str(device))
    t = _ARANGE.get(key)
    if t is None:
        t = torch.arange(B + 1, dtype=torch.int32, device=device)
        _ARANGE[key] = t
    return t


def _pool_args(cache):
    assert cache.dim() == 4 and cache.is_contiguous(), "cache must be a contiguous [pages, page_size, KH, D] tensor"
    check_bf16(cache)
    P, page, KH, D = cache.shape
    return page, KH, D, cache.stride(1), cache.stride(2)


def _i32(t):
    assert t.dtype == torch.int32 and t.is_contiguous(), "index tensors must be contiguous int32"
    return t


# ------------------------------------------------------------------------------------------------ cache writer
def store_kvcache(key, value, k_cache, v_cache, slot_mapping):
    """Scatter of new K/V rows into the paged pools (upstream nano-vllm/nanovllm/layers/attention.py:123-153):
    key [N,KH,D], value [N,KH,VD] -> flat pool rows slot_mapping[n] of k_cache / v_cache [pages,page,KH,*]
    (-1: skip the token)."""
    check_bf16(key)
    N, KH, D = key.shape
    VD = value.size(-1)
    assert value.shape[:2] == (N, KH) and key.stride(-1) == 1 and value.stride(-1) == 1
    assert key.stride(1) == D and value.stride(1) == VD, "the heads of a token must be contiguous"
    assert k_cache.dim() == 4 and k_cache.is_contiguous() and v_cache.is_contiguous()
    assert k_cache.shape[2:] == (KH, D) and v_cache.shape[2:] == (KH, VD)
    assert slot_mapping.numel() == N
    _lib.call("nsa_store_kvcache", key.data_ptr(), key.stride(0), value.data_ptr(), value.stride(0),
              k_cache.data_ptr(), KH * D, v_cache.data_ptr(), KH * VD, _i32(slot_mapping).data_ptr(), N, KH * D,
              KH * VD, _lib.stream_ptr())


def store_kvcache_and_pool_prefill(key, value, k_cache, v_cache, x_cu_seqlens, x_maxlen, context_lens, slot_mapping,
                                   y_cu_seqlens, y_maxlen, cmp_slot_mapping, block_tables, kernel_size=32, stride=16):
    """One launch for a prefill chunk: store_kvcache of the new tokens (key/value [t,KH,*] packed by x_cu_seqlens)
    and mean pooling of the compressed rows named by cmp_slot_mapping (what two mean_pooling_prefill calls do after a
    separate store)."""
    check_bf16(key)
    t, KH, D = key.shape
    VD = value.size(-1)
    page = k_cache.size(1)
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and key.stride(-1) == 1 and value.stride(-1) == 1
    assert k_cache.shape[2:] == (KH, D) and v_cache.shape[2:] == (KH, VD) and slot_mapping.numel() == t
    B = x_cu_seqlens.numel() - 1
    _lib.call("nsa_paged_store_pool_prefill", key.data_ptr(), key.stride(0), key.stride(1), D, value.data_ptr(),
              value.stride(0), value.stride(1), VD, k_cache.data_ptr(), k_cache.stride(1), k_cache.stride(2),
              v_cache.data_ptr(), v_cache.stride(1), v_cache.stride(2), _i32(x_cu_seqlens).data_ptr(),
              _i32(context_lens).data_ptr(), _i32(slot_mapping).data_ptr(), _i32(y_cu_seqlens).data_ptr(),
              _i32(cmp_slot_mapping).data_ptr(), _i32(block_tables).data_ptr(), block_tables.stride(0), B,
              int(x_maxlen), int(y_maxlen), page, KH, kernel_size, stride, _lib.stream_ptr())


# ------------------------------------------------------------------------------------------------ pooling
def mean_pooling_prefill(x, y_cu_seqlens, y_maxlen, block_table, slot_mapping, kernel_size=32, stride=16):
    """In place: every compressed row whose slot != -1 is pooled from the raw rows (read through block_table)
    and written to flat pool row `slot` of the same tensor x [pages, page_size, H, D]."""
    page, H, D, sr, sh = _pool_args(x)
    B = y_cu_seqlens.numel() - 1
    _lib.call("nsa_paged_pool_prefill", x.data_ptr(), sr, sh, _i32(y_cu_seqlens).data_ptr(),
              _i32(block_table).data_ptr(), block_table.stride(0), _i32(slot_mapping).data_ptr(), B, int(y_maxlen),
              page, H, D, kernel_size, stride, _lib.stream_ptr())
    return x


def kv_mean_pooling_decode(k, v, block_table, slot_mapping, context_lens, kernel_size=32, stride=16):
    """In place: requests with slot != -1 and len >= kernel pool their last complete window of K and V."""
    page, H, Dk, ksr, ksh = _pool_args(k)
    _, _, Dv, vsr, vsh = _pool_args(v)
    B = context_lens.numel()
    _lib.call("nsa_paged_pool_decode", k.data_ptr(), ksr, ksh, Dk, v.data_ptr(), vsr, vsh, Dv,
              _i32(context_lens).data_ptr(), _i32(block_table).data_ptr(), block_table.stride(0),
              _i32(slot_mapping).data_ptr(), B, page, H, kernel_size, stride, _lib.stream_ptr())


def mean_pooling_decode(x, block_table, slot_mapping, context_lens, kernel_size=32, stride=16):
    kv_mean_pooling_decode(x, x, block_table, slot_mapping, context_lens, kernel_size, stride)


# ------------------------------------------------------------------------------------------------ compressed attn
def cmp_attn_prefill(q, k, v, x_cu_seqlens, x_maxlen, block_tables, context_lens, kernel_size=32, stride=16,
                     sm_scale=None):
    """-> (o [t,QH,VD], lse [QH,t] fp32 log2).  block_tables: the COMPRESSED-row tables."""
    check_bf16(q)
    page, KH, D, ksr, ksh = _pool_args(k)
    _, _, VD, vsr, vsh = _pool_args(v)
    t, QH, _ = q.shape
    B = x_cu_seqlens.numel() - 1
    sm_scale = q.size(-1) ** -0.5 if sm_scale is None else sm_scale
    o = torch.empty(t, QH, VD, device=q.device, dtype=q.dtype)
    lse = torch.empty(QH, t, device=q.device, dtype=torch.float32)
    _lib.call("nsa_paged_cmp_attn_fwd", q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), ksr, ksh, v.data_ptr(),
              vsr, vsh, o.data_ptr(), o.stride(0), o.stride(1), lse.data_ptr(), lse.stride(1), lse.stride(0),
              _i32(x_cu_seqlens).data_ptr(), _i32(context_lens).data_ptr(), _i32(block_tables).data_ptr(),
              block_tables.stride(0), page, B, int(x_maxlen), QH, KH, D, VD, kernel_size, stride, sm_scale,
              _lib.stream_ptr())
    return o, lse


def cmp_attn_decode(q, k, v, block_tables, context_lens, num_splits=0, kernel_size=32, stride=16, sm_scale=None,
                    bench=False):
    """q [B,QH,D] -> (o [B,QH,VD], lse [B,QH]).  num_splits is accepted for call compatibility."""
    B = q.size(0)
    o, lse = cmp_attn_prefill(q, k, v, _decode_cu(B, q.device), 1, block_tables, context_lens, kernel_size, stride,
                              sm_scale)
    return o, lse.t()


# ------------------------------------------------------------------------------------------------ top-k
def topk_prefill(q, k, lse, x_cu_seqlens, x_maxlen, y_maxlen, block_tables, context_lens, fixed_y_maxlen=8192,
                 fixed_num_slc_blocks=2048, sm_scale=None, kernel_size=32, stride=16, block_size=64, top_n=16,
                 num_inital=1, num_local=2):
    """-> topk [KH,t,top_n] int32, unused slots = -1.  lse [QH,t] from cmp_attn_prefill."""
    check_bf16(q)
    page, KH, D, ksr, ksh = _pool_args(k)
    t, QH, _ = q.shape
    B = x_cu_seqlens.numel() - 1
    sm_scale = q.size(-1) ** -0.5 if sm_scale is None else sm_scale
    assert lse.dtype == torch.float32 and lse.shape == (QH, t)
    topk = torch.empty(KH, t, top_n, device=q.device, dtype=torch.int32)
    ws = topk_workspace(t, int(fixed_num_slc_blocks), KH, q.device)
    _lib.call("nsa_paged_topk_select_ws", q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), ksr, ksh,
              lse.data_ptr(), lse.stride(1), lse.stride(0), topk.data_ptr(), topk.stride(0), topk.stride(1),
              _i32(x_cu_seqlens).data_ptr(), _i32(context_lens).data_ptr(), _i32(block_tables).data_ptr(),
              block_tables.stride(0), page, B, int(x_maxlen), int(fixed_num_slc_blocks), QH, KH, D, kernel_size,
              stride, block_size, top_n, num_inital, num_local, -1, sm_scale, t, _lib.ptr(ws),
              ws.numel() if ws is not None else 0, _lib.stream_ptr())
    return topk


def topk_decode(q, k, lse, block_tables, context_lens, fixed_y_maxlen=8192, fixed_num_slc_blocks=2048,
                kernel_size=32, stride=16, block_size=64, top_n=16, num_inital=1, num_local=2, sm_scale=None):
    """q [B,QH,D], lse [B,QH] -> topk [KH,B,top_n] int32"""
    B = q.size(0)
    return topk_prefill(q, k, lse.t(), _decode_cu(B, q.device), 1, fixed_y_maxlen, block_tables, context_lens,
                        fixed_y_maxlen, fixed_num_slc_blocks, sm_scale, kernel_size, stride, block_size, top_n,
                        num_inital, num_local)


# ------------------------------------------------------------------------------------------------ selected / window
def slc_attn_prefill(q, k, v, topk, x_cu_seqlens, x_maxlen, block_tables, context_lens, block_size=64, top_n=16,
                     sm_scale=None):
    """-> (o [t,QH,VD], lse [t,QH])"""
    check_bf16(q)
    page, KH, D, ksr, ksh = _pool_args(k)
    _, _, VD, vsr, vsh = _pool_args(v)
    t, QH, _ = q.shape
    B = x_cu_seqlens.numel() - 1
    sm_scale = q.size(-1) ** -0.5 if sm_scale is None else sm_scale
    assert topk.dtype == torch.int32 and topk.shape == (KH, t, top_n) and topk.stride(-1) == 1
    o = torch.empty(t, QH, VD, device=q.device, dtype=q.dtype)
    lse = torch.empty(t, QH, device=q.device, dtype=torch.float32)
    _lib.call("nsa_paged_slc_attn_fwd", q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), ksr, ksh, v.data_ptr(),
              vsr, vsh, topk.data_ptr(), topk.stride(0), topk.stride(1), o.data_ptr(), o.stride(0), o.stride(1),
              lse.data_ptr(), lse.stride(0), lse.stride(1), _i32(x_cu_seqlens).data_ptr(),
              _i32(context_lens).data_ptr(), _i32(block_tables).data_ptr(), block_tables.stride(0), page, B,
              int(x_maxlen), QH, KH, D, VD, block_size, top_n, sm_scale, _lib.stream_ptr())
    return o, lse


def swa_prefill(q, k, v, x_cu_seqlens, x_maxlen, block_tables, context_lens, window_size=512, sm_scale=None):
    """Paged causal sliding-window attention (upstream calls FlashAttention with a page table here)."""
    check_bf16(q)
    page, KH, D, ksr, ksh = _pool_args(k)
    _, _, VD, vsr, vsh = _pool_args(v)
    t, QH, _ = q.shape
    B = x_cu_seqlens.numel() - 1
    sm_scale = q.size(-1) ** -0.5 if sm_scale is None else sm_scale
    o = torch.empty(t, QH, VD, device=q.device, dtype=q.dtype)
    _lib.call("nsa_paged_swa_fwd", q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), ksr, ksh, v.data_ptr(), vsr,
              vsh, o.data_ptr(), o.stride(0), o.stride(1), None, 0, 0, _i32(x_cu_seqlens).data_ptr(),
              _i32(context_lens).data_ptr(), _i32(block_tables).data_ptr(), block_tables.stride(0), page, B,
              int(x_maxlen), QH, KH, D, VD, window_size, sm_scale, _lib.stream_ptr())
    return o


def slc_attn_decode(q, k, v, topk, block_tables, context_lens, num_splits=0, block_size=64, top_n=16,
                    sm_scale=None):
    B = q.size(0)
    return slc_attn_prefill(q, k, v, topk, _decode_cu(B, q.device), 1, block_tables, context_lens, block_size,
                            top_n, sm_scale)


def fused_slc_swa_attn_decode(q, k, v, topk, block_tables, context_lens, num_splits=0, block_size=64, top_n=16,
                              window_size=512, sm_scale=None, bench=False):
    """-> (slc_o, swa_o), each [B,QH,VD]"""
    B = q.size(0)
    cu = _decode_cu(B, q.device)
    slc_o, _ = slc_attn_prefill(q, k, v, topk, cu, 1, block_tables, context_lens, block_size, top_n, sm_scale)
    swa_o = swa_prefill(q, k, v, cu, 1, block_tables, context_lens, window_size, sm_scale)
    return slc_o, swa_o


# ------------------------------------------------------------------------------------------------ combine
def combine_prefill(a, b, c, w):
    return combine_fwd(a, b, c, w)


def combine_decode(a, b, c, w):
    return combine_fwd(a, b, c, w)


# ------------------------------------------------------------------------------------------------ fused decode
def fused_decode_supported(q, k, v):
    QH, KH = q.size(1), k.size(2)
    return QH // KH <= 16 and (q.size(-1), v.size(-1)) in ((128, 128), (64, 64))


def decode_one_launch_fits(q, k, v, block_tables, fixed_y_maxlen, fixed_num_slc_blocks):
    """True when the whole decode step fits the one-launch kernel (its LDS holds per-request tables and the
    probabilities of fixed_y_maxlen compressed keys)."""
    return bool(_lib.value("nsa_decode_fused_fits", q.size(-1), v.size(-1), int(fixed_y_maxlen),
                           int(fixed_num_slc_blocks), int(block_tables.stride(0)), int(k.size(1))))


def decode_one_launch(q, k, v, w, block_tables, cmp_block_tables, context_lens, fixed_y_maxlen=8192,
                      fixed_num_slc_blocks=2048, kernel_size=32, stride=16, block_size=64, top_n=16, num_inital=1,
                      num_local=2, window_size=512, sm_scale=None, return_parts=False, cmp_slot_mapping=None,
                      new_k=None, new_v=None, slot_mapping=None):
    """The decode step in one launch (one workgroup per request and kv head): compressed attention,
    block scores, selection, window and selected-block attention, gated combine -> o [B,QH,VD]
    (return_parts: also cmp_o, slc_o, swa_o, topk [KH,B,top_n], lse [B,QH]).  With cmp_slot_mapping [B] the kernel
    first pools the compressed K/V row completed by the newest token (what kv_mean_pooling_decode does); without it
    the caller has pooled already.  With new_k / new_v [B,KH,*] and slot_mapping [B] it also writes the newest token's
    K/V rows into the pools first (what store_kvcache does)."""
    check_bf16(q)
    page, KH, D, ksr, ksh = _pool_args(k)
    _, _, VD, vsr, vsh = _pool_args(v)
    B, QH, _ = q.shape
    sm_scale = q.size(-1) ** -0.5 if sm_scale is None else sm_scale
    dev = q.device
    out = torch.empty(B, QH, VD, device=dev, dtype=q.dtype)
    parts = [torch.empty_like(out) for _ in range(3)] if return_parts else [None] * 3
    store = new_k is not None
    if store:
        assert new_v is not None and slot_mapping is not None and new_k.shape == (B, KH, D)
        assert new_v.shape == (B, KH, VD) and new_k.stride(-1) == 1 and new_v.stride(-1) == 1
    topk = torch.empty(KH, B, top_n, device=dev, dtype=torch.int32) if return_parts else None
    lse = torch.empty(B, QH, device=dev, dtype=torch.float32) if return_parts else None
    _lib.call("nsa_decode_fused", q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), ksr, ksh, v.data_ptr(), vsr,
              vsh, w.data_ptr(), w.stride(0), w.stride(1), out.data_ptr(), out.stride(0), out.stride(1),
              _lib.ptr(parts[0]), _lib.ptr(parts[1]), _lib.ptr(parts[2]), out.stride(0), out.stride(1),
              _lib.ptr(lse), lse.stride(0) if return_parts else 0, lse.stride(1) if return_parts else 0,
              _lib.ptr(topk), topk.stride(0) if return_parts else 0, topk.stride(1) if return_parts else 0,
              _i32(context_lens).data_ptr(), _i32(block_tables).data_ptr(), block_tables.stride(0),
              _i32(cmp_block_tables).data_ptr(), cmp_block_tables.stride(0),
              None if cmp_slot_mapping is None else _i32(cmp_slot_mapping).data_ptr(), _lib.ptr(new_k),
              new_k.stride(0) if store else 0, new_k.stride(1) if store else 0, _lib.ptr(new_v),
              new_v.stride(0) if store else 0, new_v.stride(1) if store else 0,
              _i32(slot_mapping).data_ptr() if store else None, page, B, QH, KH, D, VD,
              int(fixed_y_maxlen), int(fixed_num_slc_blocks), kernel_size, stride, block_size, top_n, num_inital,
              num_local, -1, window_size, sm_scale, _lib.stream_ptr())
    if return_parts:
        return out, parts[0], parts[1], parts[2], topk, lse
    return out


def decode_cmp_topk(q, k, v, cmp_block_tables, context_lens, fixed_y_maxlen=8192, fixed_num_slc_blocks=2048,
                    kernel_size=32, stride=16, block_size=64, top_n=16, num_inital=1, num_local=2, sm_scale=None,
                    return_lse=False):
    """One launch: compressed attention + block importance + top-n selection for one token per request.
    -> (cmp_o [B,QH,VD], topk [KH,B,top_n] int32[, lse [B,QH]])"""
    check_bf16(q)
    page, KH, D, ksr, ksh = _pool_args(k)
    _, _, VD, vsr, vsh = _pool_args(v)
    B, QH, _ = q.shape
    sm_scale = q.size(-1) ** -0.5 if sm_scale is None else sm_scale
    cmp_o = torch.empty(B, QH, VD, device=q.device, dtype=q.dtype)
    topk = torch.empty(KH, B, top_n, device=q.device, dtype=torch.int32)
    lse = torch.empty(B, QH, device=q.device, dtype=torch.float32) if return_lse else None
    _lib.call("nsa_decode_cmp_topk", q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), ksr, ksh, v.data_ptr(),
              vsr, vsh, cmp_o.data_ptr(), cmp_o.stride(0), cmp_o.stride(1), _lib.ptr(lse),
              lse.stride(0) if return_lse else 0, lse.stride(1) if return_lse else 0, topk.data_ptr(),
              topk.stride(0), topk.stride(1), _i32(context_lens).data_ptr(), _i32(cmp_block_tables).data_ptr(),
              cmp_block_tables.stride(0), page, B, QH, KH, D, VD, int(fixed_y_maxlen), int(fixed_num_slc_blocks),
              kernel_size, stride, block_size, top_n, num_inital, num_local, -1, sm_scale, _lib.stream_ptr())
    if return_lse:
        return cmp_o, topk, lse
    return cmp_o, topk


def decode_cmp_split(q, k, v, cmp_block_tables, context_lens, nsplit=4, fixed_y_maxlen=8192, kernel_size=32,
                     stride=16, sm_scale=None, return_lse=False):
    """Compressed branch of the decode step, split over `nsplit` workgroups per (request, kv head) so that a batch
    with very different context lengths still fills the chip.
    -> (cmp_o [B,QH,VD], pg [B,KH,fixed_y_maxlen] fp32 head-summed probabilities[, lse [B,QH]])"""
    check_bf16(q)
    page, KH, D, ksr, ksh = _pool_args(k)
    _, _, VD, vsr, vsh = _pool_args(v)
    B, QH, _ = q.shape
    sm_scale = q.size(-1) ** -0.5 if sm_scale is None else sm_scale
    dev = q.device
    cmp_o = torch.empty(B, QH, VD, device=dev, dtype=q.dtype)
    pg = torch.empty(B, KH, int(fixed_y_maxlen), device=dev, dtype=torch.float32)
    sp_ml = torch.empty(2, B, KH, nsplit, 16, device=dev, dtype=torch.float32)
    sp_o = torch.empty(B, KH, nsplit, 16, VD, device=dev, dtype=torch.float32)
    lse = torch.empty(B, QH, device=dev, dtype=torch.float32) if return_lse else None
    _lib.call("nsa_decode_cmp_split", q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), ksr, ksh, v.data_ptr(),
              vsr, vsh, cmp_o.data_ptr(), cmp_o.stride(0), cmp_o.stride(1), _lib.ptr(lse),
              lse.stride(0) if return_lse else 0, lse.stride(1) if return_lse else 0, pg.data_ptr(),
              sp_ml[0].data_ptr(), sp_ml[1].data_ptr(), sp_o.data_ptr(), nsplit, _i32(context_lens).data_ptr(),
              _i32(cmp_block_tables).data_ptr(), cmp_block_tables.stride(0), page, B, QH, KH, D, VD,
              int(fixed_y_maxlen), kernel_size, stride, sm_scale, _lib.stream_ptr())
    if return_lse:
        return cmp_o, pg, lse
    return cmp_o, pg


def decode_split_fits(q, k, v, block_tables, fixed_y_maxlen, fixed_num_slc_blocks):
    """True when decode_split's second kernel holds its tables and scores in LDS for these capacities."""
    return bool(_lib.value("nsa_decode_split_fits", q.size(-1), v.size(-1), int(fixed_y_maxlen),
                           int(fixed_num_slc_blocks), block_tables.size(1)))


def decode_split(q, k, v, w, block_tables, cmp_block_tables, context_lens, nsplit=4, fixed_y_maxlen=8192,
                 fixed_num_slc_blocks=2048, kernel_size=32, stride=16, block_size=64, top_n=16, num_inital=1,
                 num_local=2, window_size=512, sm_scale=None, return_parts=False, cmp_slot_mapping=None,
                 static_scratch=False, slc_nsplit=1):
    """The decode step in two launches, for small batches of long contexts: the compressed branch cut into `nsplit`
    parts per (request, kv head) so that it fills the GPU, then one workgroup per pair for the merge, the block
    selection, selected + window attention and the gated combine.  -> o [B,QH,VD]
    (return_parts: also cmp_o, slc_o, swa_o, topk [KH,B,top_n], lse [B,QH]).
    cmp_slot_mapping [B] (-1: none): the first launch also pools the compressed row that the newest token completes;
    None: that row is in the pool already.
    static_scratch: the library's own static device buffer holds the parts' partial results (entry point
    nsa_decode_split_static, which allocates nothing); sizes beyond that buffer raise.
    slc_nsplit > 1: the second launch runs with that many workgroups per (request, kv head), which share the window
    and the selected blocks, and a third launch merges them (upstream's slc_num_splits,
    flash_nsa/inference/__init__.py:195-196)."""
    check_bf16(q)
    page, KH, D, ksr, ksh = _pool_args(k)
    _, _, VD, vsr, vsh = _pool_args(v)
    B, QH, _ = q.shape
    sm_scale = q.size(-1) ** -0.5 if sm_scale is None else sm_scale
    dev = q.device
    out = torch.empty(B, QH, VD, device=dev, dtype=q.dtype)
    parts = [torch.empty_like(out) for _ in range(3)] if return_parts else [None] * 3
    topk = torch.empty(KH, B, top_n, device=dev, dtype=torch.int32) if return_parts else None
    lse = torch.empty(B, QH, device=dev, dtype=torch.float32) if return_parts else None
    if static_scratch:
        if slc_nsplit > 1:
            raise ValueError("decode_split: the static-scratch entry point has no parts of the window / selected "
                             "branches (slc_nsplit must be 1)")
        _lib.call("nsa_decode_split_static", q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), ksr, ksh,
                  v.data_ptr(), vsr, vsh, w.data_ptr(), w.stride(0), w.stride(1), out.data_ptr(), out.stride(0),
                  out.stride(1), _lib.ptr(parts[0]), _lib.ptr(parts[1]), _lib.ptr(parts[2]), out.stride(0),
                  out.stride(1), _lib.ptr(lse), lse.stride(0) if return_parts else 0,
                  lse.stride(1) if return_parts else 0, _lib.ptr(topk), topk.stride(0) if return_parts else 0,
                  topk.stride(1) if return_parts else 0, nsplit,
                  _lib.ptr(None if cmp_slot_mapping is None else _i32(cmp_slot_mapping)),
                  _i32(context_lens).data_ptr(), _i32(block_tables).data_ptr(), block_tables.stride(0),
                  _i32(cmp_block_tables).data_ptr(), cmp_block_tables.stride(0), page, B, QH, KH, D, VD,
                  int(fixed_y_maxlen), int(fixed_num_slc_blocks), kernel_size, stride, block_size, top_n, num_inital,
                  num_local, -1, window_size, sm_scale, _lib.stream_ptr())
        if return_parts:
            return out, parts[0], parts[1], parts[2], topk, lse
        return out
    ycap32 = (int(fixed_y_maxlen) + 31) // 32 * 32
    sp_ml = torch.empty(2, B, KH, nsplit, 16, device=dev, dtype=torch.float32)
    sp_o = torch.empty(B, KH, nsplit, 16, VD, device=dev, dtype=torch.float32)
    keep_p = torch.empty(B, KH, 16, ycap32, device=dev, dtype=torch.float16)
    keep_m = torch.empty(B, KH, ycap32 // 32, 16, device=dev, dtype=torch.float32)
    args = (q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), ksr, ksh, v.data_ptr(), vsr,
            vsh, w.data_ptr(), w.stride(0), w.stride(1), out.data_ptr(), out.stride(0), out.stride(1),
            _lib.ptr(parts[0]), _lib.ptr(parts[1]), _lib.ptr(parts[2]), out.stride(0), out.stride(1),
            _lib.ptr(lse), lse.stride(0) if return_parts else 0, lse.stride(1) if return_parts else 0,
            _lib.ptr(topk), topk.stride(0) if return_parts else 0, topk.stride(1) if return_parts else 0,
            sp_ml[0].data_ptr(), sp_ml[1].data_ptr(), sp_o.data_ptr(), keep_p.data_ptr(), keep_m.data_ptr(), nsplit,
            _lib.ptr(None if cmp_slot_mapping is None else _i32(cmp_slot_mapping)), _i32(context_lens).data_ptr(),
            _i32(block_tables).data_ptr(), block_tables.stride(0),
            _i32(cmp_block_tables).data_ptr(), cmp_block_tables.stride(0), page, B, QH, KH, D, VD,
            int(fixed_y_maxlen), int(fixed_num_slc_blocks), kernel_size, stride, block_size, top_n, num_inital,
            num_local, -1, window_size, sm_scale)
    if slc_nsplit > 1:
        sp2_ml = torch.empty(B, KH, slc_nsplit, 2, 2, 16, device=dev, dtype=torch.float32)
        sp2_o = torch.empty(B, KH, slc_nsplit, 2, 16, VD, device=dev, dtype=torch.float32)
        cmp_tmp = torch.empty_like(out)
        _lib.call("nsa_decode_split_parts", *args, int(slc_nsplit), sp2_ml.data_ptr(), sp2_o.data_ptr(),
                  cmp_tmp.data_ptr(), _lib.stream_ptr())
    else:
        _lib.call("nsa_decode_split", *args, _lib.stream_ptr())
    if return_parts:
        return out, parts[0], parts[1], parts[2], topk, lse
    return out


def decode_slc_swa_combine(q, k, v, w, topk, cmp_o, block_tables, context_lens, block_size=64, top_n=16,
                           window_size=512, sm_scale=None, return_branches=False, pg=None, fixed_num_slc_blocks=2048,
                           kernel_size=32, stride=16, num_inital=1, num_local=2):
    """One launch: selected-block + window attention and the gated combine -> o [B,QH,VD]
    (with return_branches also slc_o, swa_o).  With `pg` (from decode_cmp_split) the block selection runs in the
    kernel's prologue and `topk` may be None; the selection is then returned as a third/fifth value."""
    check_bf16(q)
    page, KH, D, ksr, ksh = _pool_args(k)
    _, _, VD, vsr, vsh = _pool_args(v)
    B, QH, _ = q.shape
    sm_scale = q.size(-1) ** -0.5 if sm_scale is None else sm_scale
    out = torch.empty(B, QH, VD, device=q.device, dtype=q.dtype)
    slc_o = torch.empty_like(out) if return_branches else None
    swa_o = torch.empty_like(out) if return_branches else None
    assert cmp_o.stride() == out.stride()
    select_here = pg is not None
    if select_here:
        topk = torch.empty(KH, B, top_n, device=q.device, dtype=torch.int32)
    _lib.call("nsa_decode_slc_swa_combine", q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), ksr, ksh,
              v.data_ptr(), vsr, vsh, w.data_ptr(), w.stride(0), w.stride(1), topk.data_ptr(), topk.stride(0),
              topk.stride(1), _lib.ptr(pg), pg.size(-1) if select_here else 0, int(fixed_num_slc_blocks), kernel_size,
              stride, num_inital, num_local, -1, cmp_o.data_ptr(), _lib.ptr(slc_o), _lib.ptr(swa_o), cmp_o.stride(0),
              cmp_o.stride(1), out.data_ptr(), out.stride(0), out.stride(1), _i32(context_lens).data_ptr(),
              _i32(block_tables).data_ptr(), block_tables.stride(0), page, B, QH, KH, D, VD, block_size, top_n,
              window_size, sm_scale, _lib.stream_ptr())
    res = (out, slc_o, swa_o) if return_branches else (out,)
    if select_here:
        res = res + (topk,)
    return res if len(res) > 1 else res[0]
