"""Causal sliding-window attention over packed sequences (upstream
flash_nsa/ops/sliding_window_attention.py:26-157, which delegates to FlashAttention with window=(W,-1))."""
import torch

from .. import _lib
from ..utils import NSAHelper
from ._common import check_thd, default_scale, delta_of, dq_target


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


def swa_bwd(q, k, v, o, lse, do, sm_scale=None, helper=NSAHelper, delta=None, dq=None, dkv_fp32=False, parts="both"):
    """Backward of the window branch.  Returns (dq, dk, dv); dq is a fresh bf16 tensor or the caller's fp32
    buffer (added into); dk/dv are freshly written (bf16, or fp32 when dkv_fp32), one writer per element.
    parts = "dq" / "dkdv" launches only that kernel (the other results are None), so that a caller can put the
    two on different streams."""
    check_thd(do, "do")
    T, QH, D = q.shape
    _, KH, VD = v.shape
    sm_scale = default_scale(q, sm_scale)
    if delta is None:
        delta = delta_of(o, do)
    common = (q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), k.stride(0), k.stride(1), v.data_ptr(),
              v.stride(0), v.stride(1), do.data_ptr(), do.stride(0), do.stride(1), lse.data_ptr(), lse.stride(0),
              lse.stride(1), delta.data_ptr(), delta.stride(0), delta.stride(1))
    dq_buf = dk = dv = None
    if parts in ("both", "dq"):
        dq_buf, mode = dq_target(q, dq)
        _lib.call("nsa_swa_bwd_dq", *common, dq_buf.data_ptr(), dq_buf.stride(0), dq_buf.stride(1), mode,
                  helper.x_cu_seqlens.data_ptr(), helper.batch, helper.x_maxlen, QH, KH, D, VD, helper.window_size,
                  sm_scale, _lib.stream_ptr())
    if parts in ("both", "dkdv"):
        kv_dtype = torch.float32 if dkv_fp32 else k.dtype
        dk = torch.empty(T, KH, D, device=q.device, dtype=kv_dtype)
        dv = torch.empty(T, KH, VD, device=q.device, dtype=kv_dtype)
        _lib.call("nsa_swa_bwd_dkdv", *common, dk.data_ptr(), dk.stride(0), dk.stride(1), dv.data_ptr(),
                  dv.stride(0), dv.stride(1), int(dkv_fp32), helper.x_cu_seqlens.data_ptr(), helper.batch,
                  helper.x_maxlen, QH, KH, D, VD, helper.window_size, sm_scale, _lib.stream_ptr())
    return dq_buf, dk, dv


class _SWA(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, sm_scale):
        o, lse = swa_fwd(q, k, v, sm_scale)
        ctx.save_for_backward(q, k, v, o, lse)
        ctx.sm_scale = sm_scale
        ctx.helper = NSAHelper.get_bwd_helper()
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, lse = ctx.saved_tensors
        do = do if do.stride(-1) == 1 else do.contiguous()
        dq, dk, dv = swa_bwd(q, k, v, o, lse, do, sm_scale=ctx.sm_scale, helper=ctx.helper)
        return dq, dk, dv, None


def swa_varlen_func(q, k, v, sm_scale=None):
    """Differentiable causal sliding-window attention over the registered packed batch."""
    return _SWA.apply(q, k, v, sm_scale)
