"""Gated activations of the learned compression: sigmoid(gate)*up and silu(gate)*up
(upstream flash_nsa/ops/act.py:13-247).  Input [..., 2d] = gate | up, output [..., d]."""
import torch

from .. import _lib
from ._common import check_bf16

_ACT = {"sigmoid-mul": 0, "swiglu": 1}


def _glu_fwd(x, act):
    check_bf16(x)
    x = x.contiguous()
    d = x.size(-1) // 2
    y = torch.empty(*x.shape[:-1], d, device=x.device, dtype=x.dtype)
    _lib.call("nsa_glu_fwd", x.data_ptr(), y.data_ptr(), x.numel() // (2 * d), d, _ACT[act], _lib.stream_ptr())
    return y


def _glu_bwd(x, dy, act, inplace=True):
    """Returns [dgate | dup]; like upstream, the saved pre-activation is overwritten when inplace."""
    x = x if x.is_contiguous() else x.contiguous()
    dy = dy.contiguous()
    d = x.size(-1) // 2
    dx = x if inplace else torch.empty_like(x)
    _lib.call("nsa_glu_bwd", x.data_ptr(), dy.data_ptr(), dx.data_ptr(), x.numel() // (2 * d), d, _ACT[act],
              _lib.stream_ptr())
    return dx


def sigmoid_mul_fwd(x):
    return _glu_fwd(x, "sigmoid-mul")


def sigmoid_mul_bwd(x, dy, inplace=True):
    return _glu_bwd(x, dy, "sigmoid-mul", inplace)


def swiglu_fwd(x):
    return _glu_fwd(x, "swiglu")


def swiglu_bwd(x, dy, inplace=True):
    return _glu_bwd(x, dy, "swiglu", inplace)


class _Glu(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, act):
        ctx.act = act
        ctx.save_for_backward(x)
        return _glu_fwd(x, act)

    @staticmethod
    def backward(ctx, dy):
        (x,) = ctx.saved_tensors
        return _glu_bwd(x, dy, ctx.act, inplace=False), None


def sigmoid_mul_impl(x):
    return _Glu.apply(x, "sigmoid-mul")


def swiglu_impl(x):
    return _Glu.apply(x, "swiglu")
