"""Compressed attention (upstream flash_nsa/ops/compress_attn.py:531-776)."""
import torch

from .. import _lib
from ..utils import NSAHelper
from ._common import check_thd, default_scale, delta_of, dq_target


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


def cmp_attn_bwd(q, k, v, o, lse, do, dq=None, dkdv_repeat=False, sm_scale=None, helper=NSAHelper, delta=None,
                 q_chunk_tokens=0, finalize_dq=False, parts="both"):
    """Backward of compressed attention.  Returns (dq, dk, dv).
    dq: fresh bf16 tensor, or the caller's fp32 buffer, which is added into; with finalize_dq the fp32 buffer is
    only read and the returned dq is a fresh tensor in q's dtype holding buffer + this branch.
    parts = "dq" / "dkdv" launches only that kernel (the other results are None).
    dk, dv: fp32 [y_len,KH,*].  dkdv_repeat=False (default, as upstream): the work items (query chunks) add their
    partial results with fp32 atomics, so the summation order changes from run to run; dkdv_repeat=True (or
    NSAHelper.set_deterministic(True)): every work item stores into its own slot of a scratch buffer and a second
    launch sums the slots in a fixed order -- bit-identical results across runs.
    delta may be passed when already known (delta[T,QH] fp32 = rowsum(o*do)).
    q_chunk_tokens: queries per work item of the dk/dv kernel (0: chosen by the library from the sizes)."""
    check_thd(do, "do")
    T, QH, D = q.shape
    Y, KH, VD = v.shape
    sm_scale = default_scale(q, sm_scale)
    if delta is None:
        delta = delta_of(o, do)
    common = (q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), k.stride(0), k.stride(1), v.data_ptr(),
              v.stride(0), v.stride(1), do.data_ptr(), do.stride(0), do.stride(1), lse.data_ptr(), lse.stride(1),
              lse.stride(0), delta.data_ptr(), delta.stride(0), delta.stride(1))
    tail = (helper.x_cu_seqlens.data_ptr(), helper.y_cu_seqlens.data_ptr(), helper.batch, helper.x_maxlen, QH, KH,
            D, VD, helper.kernel_size, helper.stride, sm_scale, _lib.stream_ptr())
    dq_buf = dk = dv = None
    if parts in ("both", "dq"):
        if finalize_dq:
            # last branch of a fused backward: dq (fp32 sum of the other branches) + this branch -> fresh tensor in
            # q's dtype
            assert dq is not None and dq.dtype == torch.float32 and dq.shape == q.shape and dq.stride(-1) == 1
            dq_buf = torch.empty_like(q)
            _lib.call("nsa_cmp_attn_bwd_dq_final", *common, dq.data_ptr(), dq.stride(0), dq.stride(1),
                      dq_buf.data_ptr(), dq_buf.stride(0), dq_buf.stride(1), *tail)
        else:
            dq_buf, mode = dq_target(q, dq)
            _lib.call("nsa_cmp_attn_bwd_dq", *common, dq_buf.data_ptr(), dq_buf.stride(0), dq_buf.stride(1), mode,
                      *tail)
    if parts in ("both", "dkdv"):
        dk = torch.zeros(Y, KH, D, device=q.device, dtype=torch.float32)
        dv = torch.zeros(Y, KH, VD, device=q.device, dtype=torch.float32)
        sizes = (helper.batch, helper.x_maxlen, helper.y_maxlen, QH, KH, D, VD, helper.kernel_size, helper.stride,
                 q_chunk_tokens)
        args = (*common, dk.data_ptr(), dk.stride(0), dk.stride(1), dv.data_ptr(), dv.stride(0), dv.stride(1),
                helper.x_cu_seqlens.data_ptr(), helper.y_cu_seqlens.data_ptr(), *sizes, sm_scale)
        if dkdv_repeat or getattr(helper, "deterministic", False):
            ws = torch.empty(max(_lib.value("nsa_cmp_attn_bwd_dkdv_det_bytes", *sizes), 1), dtype=torch.uint8,
                             device=q.device)
            _lib.call("nsa_cmp_attn_bwd_dkdv_det", *args, ws.data_ptr(), ws.numel(), _lib.stream_ptr())
        else:
            _lib.call("nsa_cmp_attn_bwd_dkdv", *args, _lib.stream_ptr())
    return dq_buf, dk, dv


class _CompressAttn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, sm_scale):
        o, lse = cmp_attn_fwd(q, k, v, sm_scale)
        ctx.save_for_backward(q, k, v, o, lse)
        ctx.sm_scale = sm_scale
        ctx.helper = NSAHelper.get_bwd_helper()
        ctx.mark_non_differentiable(lse)
        return o, lse

    @staticmethod
    def backward(ctx, do, _dlse):
        q, k, v, o, lse = ctx.saved_tensors
        do = do if do.stride(-1) == 1 else do.contiguous()
        dq, dk, dv = cmp_attn_bwd(q, k, v, o, lse, do, sm_scale=ctx.sm_scale, helper=ctx.helper)
        return dq, dk.to(k.dtype), dv.to(v.dtype), None


def compress_attn(q, k, v, sm_scale=None):
    """Differentiable compressed attention -> (o, lse)."""
    return _CompressAttn.apply(q, k, v, sm_scale)
