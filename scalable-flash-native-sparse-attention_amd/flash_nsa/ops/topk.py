"""Block-importance scoring and top-n block selection (upstream flash_nsa/ops/topk.py:630-775)."""
import torch

from .. import _lib
from ..utils import NSAHelper, cdiv
from ._common import check_thd, default_scale


@torch.no_grad()
def slc_topk_indices(q, k, lse, sm_scale=None, return_slc_prob=False, align=True, ignore_index=None, fp32=True,
                     maybe_efficient_version=True, scale_slc_p=True):
    """q [T,QH,D], k [y_len,KH,D] compressed keys, lse [QH,T] (log2 units) from the compressed attention.
    Returns (topk [KH,T,top_n] int32, block scores or None).  Slot order: initial blocks, then local blocks
    (current, previous, ...), then the remaining blocks by descending score (lowest index on ties); unused slots
    hold ignore_index (default: number of selection blocks of the longest sequence).

    The scores never leave the chip unless return_slc_prob is set, in which case they are returned in fp32
    [KH,T,cols].  `fp32`, `maybe_efficient_version` and `scale_slc_p` are accepted for call compatibility: there
    is a single fp32 code path."""
    check_thd(q, "q"), check_thd(k, "k")
    helper = NSAHelper
    T, QH, D = q.shape
    Y, KH, _ = k.shape
    assert lse.shape == (QH, T) and lse.dtype == torch.float32
    sm_scale = default_scale(q, sm_scale)
    nblk = max(cdiv(helper.x_maxlen, helper.block_size), 1)
    assert ignore_index is None or ignore_index >= nblk or ignore_index < 0
    ignore_index = nblk if ignore_index is None else ignore_index
    topk = torch.empty(KH, T, helper.top_n, device=q.device, dtype=torch.int32)
    probs = None
    cols = 0
    if return_slc_prob:
        cols = nblk
        if align:
            cols = max(1 << (nblk - 1).bit_length(), 8)
        probs = torch.empty(KH, T, cols, device=q.device, dtype=torch.float32)
    ws = topk_workspace(T, nblk, KH, q.device)
    _lib.call("nsa_topk_select_ws", q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), k.stride(0), k.stride(1),
              lse.data_ptr(), lse.stride(1), lse.stride(0), topk.data_ptr(), topk.stride(0), topk.stride(1),
              _lib.ptr(probs), probs.stride(0) if probs is not None else 0,
              probs.stride(1) if probs is not None else 0, cols, helper.x_cu_seqlens.data_ptr(),
              helper.y_cu_seqlens.data_ptr(), helper.batch, helper.x_maxlen, QH, KH, D, helper.kernel_size,
              helper.stride, helper.block_size, helper.top_n, helper.num_init_blocks, helper.num_local_blocks,
              ignore_index, sm_scale, T, _lib.ptr(ws), ws.numel() if ws is not None else 0, _lib.stream_ptr())
    return topk, probs


# most bytes of block scores held between the two launches of the selector; batches that need more run in chunks
TOPK_WORKSPACE_LIMIT = 2 << 30
# below this many tokens the one-launch selector (scores in LDS, no workspace) is at least as fast
TOPK_TWO_PASS_MIN_TOKENS = 256


def topk_workspace(total_tokens, max_blocks, KH, device):
    """Scratch for the two-launch block selector (fp32 block scores of a chunk of tokens), from torch's caching
    allocator; None for batches too small to gain from it."""
    if total_tokens < TOPK_TWO_PASS_MIN_TOKENS:
        return None
    need = _lib.value("nsa_topk_workspace_bytes", int(total_tokens), int(max_blocks), int(KH))
    return torch.empty(min(need, TOPK_WORKSPACE_LIMIT), dtype=torch.uint8, device=device)


@torch.no_grad()
def get_bind_from_find(topk, helper=NSAHelper, chunk_tokens=None):
    """Inverse of the selection: for every (kv head, selection block) the ascending list of query tokens that
    selected it.  Returns a dict with the CSR (csr_off [KH,nblk+1], csr_tok [KH*T*top_n]), the work-item prefix
    (item_off [KH,nblk+1]) and the static bound on the number of work items per kv head."""
    KH, T, N = topk.shape
    dev = topk.device
    nblk = helper.k_len
    if chunk_tokens is None:
        chunk_tokens = _lib.value("nsa_slc_bwd_chunk_tokens", T, KH, N)
    csr_off = torch.empty(KH, nblk + 1, device=dev, dtype=torch.int32)
    item_off = torch.empty(KH, nblk + 1, device=dev, dtype=torch.int32)
    csr_tok = torch.empty(KH * T * N, device=dev, dtype=torch.int32)
    ws_elems = _lib.value("nsa_inverse_index_workspace_elems", T, KH, nblk)
    ws = torch.empty(ws_elems, device=dev, dtype=torch.int32)
    _lib.call("nsa_build_inverse_index", topk.data_ptr(), topk.stride(0), topk.stride(1), N,
              helper.x_cu_seqlens.data_ptr(), helper.k_cu_seqlens.data_ptr(), helper.batch, T, KH, nblk,
              helper.block_size, chunk_tokens, csr_off.data_ptr(), csr_tok.data_ptr(), item_off.data_ptr(),
              ws.data_ptr(), ws_elems, _lib.stream_ptr())
    n_items_bound = (T * N + chunk_tokens - 1) // chunk_tokens + nblk
    return dict(csr_off=csr_off, csr_tok=csr_tok, item_off=item_off, n_items_bound=n_items_bound,
                chunk_tokens=chunk_tokens, nblk=nblk)
