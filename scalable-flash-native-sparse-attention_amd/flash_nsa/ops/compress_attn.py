"""Compressed attention (upstream flash_nsa/ops/compress_attn.py:531-776)."""
import torch

from .. import _lib
from ..utils import NSAHelper
from ._common import check_thd, default_scale


def cmp_attn_fwd(q, k, v, sm_scale=None, helper=NSAHelper):
    """q [T,QH,D], k [y_len,KH,D], v [y_len,KH,VD] (compressed rows) -> o [T,QH,VD], lse [QH,T] fp32 (log2 units).
    Query t sees compressed row i iff t >= stride*i + kernel-1; rows that see nothing give o = 0, lse = 0."""
    check_thd(q, "q"), check_thd(k, "k"), check_thd(v, "v")
    T, QH, D = q.shape
    Y, KH, VD = v.shape
    assert k.shape == (Y, KH, D) and QH % KH == 0 and Y == helper.y_len
    sm_scale = default_scale(q, sm_scale)
    o = torch.empty(T, QH, VD, device=q.device, dtype=q.dtype)
    lse = torch.empty(QH, T, device=q.device, dtype=torch.float32)
    _lib.call("nsa_cmp_attn_fwd", q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), k.stride(0), k.stride(1),
              v.data_ptr(), v.stride(0), v.stride(1), o.data_ptr(), o.stride(0), o.stride(1), lse.data_ptr(),
              lse.stride(1), lse.stride(0), helper.x_cu_seqlens.data_ptr(), helper.y_cu_seqlens.data_ptr(),
              helper.batch, helper.x_maxlen, QH, KH, D, VD, helper.kernel_size, helper.stride, sm_scale,
              _lib.stream_ptr())
    return o, lse
