"""Selected-block attention (upstream flash_nsa/ops/select_attn.py:439-748)."""
import torch

from .. import _lib
from ..utils import NSAHelper
from ._common import check_thd, default_scale


def slc_attn_fwd(q, k, v, topk, sm_scale=None, helper=NSAHelper):
    """q [T,QH,D], k [T,KH,D], v [T,KH,VD], topk [KH,T,top_n] int32 -> o [T,QH,VD], lse [T,QH] fp32 (log2).
    Query t of a sequence attends the keys <= t of the blocks in its first min(top_n, t//block+1) slots."""
    check_thd(q, "q"), check_thd(k, "k"), check_thd(v, "v")
    T, QH, D = q.shape
    _, KH, VD = v.shape
    assert topk.dtype == torch.int32 and topk.shape[:2] == (KH, T) and topk.stride(-1) == 1
    sm_scale = default_scale(q, sm_scale)
    o = torch.empty(T, QH, VD, device=q.device, dtype=q.dtype)
    lse = torch.empty(T, QH, device=q.device, dtype=torch.float32)
    _lib.call("nsa_slc_attn_fwd", q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), k.stride(0), k.stride(1),
              v.data_ptr(), v.stride(0), v.stride(1), topk.data_ptr(), topk.stride(0), topk.stride(1), o.data_ptr(),
              o.stride(0), o.stride(1), lse.data_ptr(), lse.stride(0), lse.stride(1),
              helper.x_cu_seqlens.data_ptr(), helper.batch, helper.x_maxlen, QH, KH, D, VD, helper.block_size,
              topk.size(-1), sm_scale, _lib.stream_ptr())
    return o, lse
