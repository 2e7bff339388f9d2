"""Fused rotary embedding of q and k (mirrors upstream flash_nsa/ops/rope.py:126-232)."""
import torch

from .. import _lib
from ._common import check_bf16


def _strides3(t):
    assert t.stride(-1) == 1, "the head dimension must be contiguous"
    return t.stride(0), t.stride(1), t.stride(2)


def _launch(q, k, qe, ke, cos, sin, backward):
    B, N, QH, D = q.shape
    KH = k.size(2)
    assert k.shape == (B, N, KH, D) and cos.shape == (B, N, D) and sin.shape == cos.shape
    assert cos.dtype == sin.dtype and cos.dtype in (torch.bfloat16, torch.float32)
    assert cos.stride(-1) == 1 and sin.stride() == cos.stride()
    _lib.call("nsa_rope", q.data_ptr(), *_strides3(q), k.data_ptr(), *_strides3(k), qe.data_ptr(), *_strides3(qe),
              ke.data_ptr(), *_strides3(ke), cos.data_ptr(), sin.data_ptr(), cos.stride(0), cos.stride(1),
              int(cos.dtype == torch.float32), B, N, QH, KH, D, int(backward), _lib.stream_ptr())


class _FusedApplyRope(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, cos, sin, inplace):
        check_bf16(q), check_bf16(k)
        if inplace:
            qe, ke = q, k
            # Autograd cannot track one function that rewrites two views (the slices of a fused projection are
            # such views), so those are rotated behind its back, as upstream does (flash_nsa/ops/rope.py:139-168):
            # correct as long as no earlier node saved the un-rotated rows, which holds for a projection's output.
            if not (q._is_view() or k._is_view()):
                ctx.mark_dirty(q, k)
        else:
            qe, ke = torch.empty_like(q), torch.empty_like(k)
        _launch(q, k, qe, ke, cos, sin, False)
        ctx.save_for_backward(cos, sin)
        return qe, ke

    @staticmethod
    def backward(ctx, dqe, dke):
        cos, sin = ctx.saved_tensors
        dqe = dqe if dqe.stride(-1) == 1 else dqe.contiguous()
        dke = dke if dke.stride(-1) == 1 else dke.contiguous()
        dq, dk = torch.empty_like(dqe), torch.empty_like(dke)
        _launch(dqe, dke, dq, dk, cos, sin, True)
        return dq, dk, None, None, None


def fused_apply_rope(q, k, cos, sin, inplace=False):
    """Rotate-half RoPE.  q [b,s,qh,d], k [b,s,kh,d] bf16; cos, sin [b,s,d] (or [1,s,d], or with a singleton head
    axis), bf16 or fp32.  Returns (qe, ke); with inplace they are q and k themselves."""
    if cos.dim() == 4:
        cos = cos.squeeze(-2)
    if sin.dim() == 4:
        sin = sin.squeeze(-2)
    if cos.size(0) != q.size(0):
        b = q.size(0)
        _, s, d = cos.shape
        cos, sin = cos.expand(b, s, d), sin.expand(b, s, d)
    return _FusedApplyRope.apply(q, k, cos, sin, inplace)
