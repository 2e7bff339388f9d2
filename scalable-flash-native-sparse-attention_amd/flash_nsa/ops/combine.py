"""Sigmoid-gated sum of the three branch outputs (upstream flash_nsa/ops/combine.py:114-216)."""
import torch

from .. import _lib
from ._common import check_thd, check_bf16


def combine_fwd(a, b, c, w):
    """o = a*sigmoid(w[...,0]) + b*sigmoid(w[...,1]) + c*sigmoid(w[...,2]);  a,b,c [T,H,D], w [T,H,3]."""
    for t, n in ((a, "a"), (b, "b"), (c, "c")):
        check_thd(t, n)
    assert a.shape == b.shape == c.shape and a.stride() == b.stride() == c.stride()
    check_bf16(w)
    assert w.shape == (a.size(0), a.size(1), 3)
    T, H, D = a.shape
    o = torch.empty(T, H, D, device=a.device, dtype=a.dtype)
    _lib.call("nsa_combine_fwd", a.data_ptr(), b.data_ptr(), c.data_ptr(), a.stride(0), a.stride(1), w.data_ptr(),
              w.stride(0), w.stride(1), o.data_ptr(), o.stride(0), o.stride(1), T, H, D, _lib.stream_ptr())
    return o


def combine_bwd(a, b, c, w, do, return_delta=False):
    """Returns da, db, dc (contiguous [T,H,D]), dw [T,H,3] and optionally delta [3,T,H] fp32 with
    delta[k] = rowsum(branch_k * d branch_k), which the attention backward kernels consume."""
    T, H, D = a.shape
    assert a.stride() == b.stride() == c.stride()
    do = do if do.stride(-1) == 1 else do.contiguous()
    da = torch.empty(T, H, D, device=a.device, dtype=a.dtype)
    db = torch.empty_like(da)
    dc = torch.empty_like(da)
    dw = torch.empty(T, H, 3, device=a.device, dtype=w.dtype)
    delta = torch.empty(3, T, H, device=a.device, dtype=torch.float32) if return_delta else None
    _lib.call("nsa_combine_bwd", a.data_ptr(), b.data_ptr(), c.data_ptr(), a.stride(0), a.stride(1), w.data_ptr(),
              w.stride(0), w.stride(1), do.data_ptr(), do.stride(0), do.stride(1), da.data_ptr(), db.data_ptr(),
              dc.data_ptr(), dw.data_ptr(), _lib.ptr(delta), T, H, D, _lib.stream_ptr())
    if return_delta:
        return da, db, dc, dw, delta
    return da, db, dc, dw


class _Combine(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a, b, c, w):
        ctx.save_for_backward(a, b, c, w)
        return combine_fwd(a, b, c, w)

    @staticmethod
    def backward(ctx, do):
        a, b, c, w = ctx.saved_tensors
        return combine_bwd(a, b, c, w, do)


def fused_sigmoid_combine(a, b, c, w):
    return _Combine.apply(a, b, c, w)
