"""Causal sliding-window attention over packed sequences (upstream
flash_nsa/ops/sliding_window_attention.py:26-157, which delegates to FlashAttention with window=(W,-1))."""
import torch

from .. import _lib
from ..utils import NSAHelper
from ._common import check_thd, default_scale


def swa_fwd(q, k, v, sm_scale=None, helper=NSAHelper):
    """-> o [T,QH,VD], lse [T,QH] fp32 in log2 units.  Query t attends keys max(0,t-W) .. t of its sequence."""
    check_thd(q, "q"), check_thd(k, "k"), check_thd(v, "v")
    T, QH, D = q.shape
    _, KH, VD = v.shape
    sm_scale = default_scale(q, sm_scale)
    o = torch.empty(T, QH, VD, device=q.device, dtype=q.dtype)
    lse = torch.empty(T, QH, device=q.device, dtype=torch.float32)
    _lib.call("nsa_swa_fwd", q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), k.stride(0), k.stride(1),
              v.data_ptr(), v.stride(0), v.stride(1), o.data_ptr(), o.stride(0), o.stride(1), lse.data_ptr(),
              lse.stride(0), lse.stride(1), helper.x_cu_seqlens.data_ptr(), helper.batch, helper.x_maxlen, QH, KH, D,
              VD, helper.window_size, sm_scale, _lib.stream_ptr())
    return o, lse
