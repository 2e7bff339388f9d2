"""KV compression operators: mean pooling and im2col of the compression windows
(upstream flash_nsa/ops/compress_kv.py:126-426)."""
import torch

from .. import _lib
from ..utils import NSAHelper
from ._common import check_thd


def mean_pooling_fwd(x, helper=NSAHelper):
    """x [T,H,D] -> y [y_len,H,D]: mean over windows [stride*i, stride*i+kernel) of every sequence."""
    check_thd(x, "x")
    T, H, D = x.shape
    y = torch.empty(helper.y_len, H, D, device=x.device, dtype=x.dtype)
    _lib.call("nsa_mean_pool_fwd", x.data_ptr(), x.stride(0), x.stride(1), y.data_ptr(), y.stride(0), y.stride(1),
              helper.x_cu_seqlens.data_ptr(), helper.y_cu_seqlens.data_ptr(), helper.batch, helper.y_maxlen, H, D,
              helper.kernel_size, helper.stride, _lib.stream_ptr())
    return y


def mean_pooling_bwd(x, dy, dx=None, helper=NSAHelper):
    """Gradient of mean pooling.  With dx=None a new tensor of x's dtype is returned; an fp32 dx is
    accumulated into (each element has a single writer, so the result is deterministic)."""
    check_thd(dy, "dy")
    T, H, D = x.shape
    accumulate = dx is not None
    if dx is None:
        dx = torch.empty(T, H, D, device=x.device, dtype=x.dtype)
    else:
        assert dx.dtype == torch.float32 and dx.shape == x.shape and dx.stride(-1) == 1
    _lib.call("nsa_mean_pool_bwd", dy.data_ptr(), dy.stride(0), dy.stride(1), dx.data_ptr(), dx.stride(0),
              dx.stride(1), int(dx.dtype == torch.float32), int(accumulate), helper.x_cu_seqlens.data_ptr(),
              helper.y_cu_seqlens.data_ptr(), helper.batch, helper.x_maxlen, H, D, helper.kernel_size, helper.stride,
              _lib.stream_ptr())
    return dx


def construct_block_fwd(x, helper=NSAHelper):
    """x [T,H,D] -> [y_len,H,kernel,D] (im2col of the compression windows)."""
    check_thd(x, "x")
    T, H, D = x.shape
    y = torch.empty(helper.y_len, H, helper.kernel_size, D, device=x.device, dtype=x.dtype)
    _lib.call("nsa_construct_block_fwd", x.data_ptr(), x.stride(0), x.stride(1), y.data_ptr(),
              helper.x_cu_seqlens.data_ptr(), helper.y_cu_seqlens.data_ptr(), helper.batch, helper.y_maxlen, H, D,
              helper.kernel_size, helper.stride, _lib.stream_ptr())
    return y


def construct_block_bwd(x, dy, dx=None, helper=NSAHelper):
    T, H, D = x.shape
    dy = dy.contiguous()
    accumulate = dx is not None
    if dx is None:
        dx = torch.empty(T, H, D, device=x.device, dtype=x.dtype)
    else:
        assert dx.dtype == torch.float32 and dx.shape == x.shape and dx.stride(-1) == 1
    _lib.call("nsa_construct_block_bwd", dy.data_ptr(), dx.data_ptr(), dx.stride(0), dx.stride(1),
              int(dx.dtype == torch.float32), int(accumulate), helper.x_cu_seqlens.data_ptr(),
              helper.y_cu_seqlens.data_ptr(), helper.batch, helper.x_maxlen, H, D, helper.kernel_size, helper.stride,
              _lib.stream_ptr())
    return dx


class _MeanPooling(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        ctx.helper = NSAHelper.get_bwd_helper()
        ctx.x_meta = x
        return mean_pooling_fwd(x)

    @staticmethod
    def backward(ctx, dy):
        return mean_pooling_bwd(ctx.x_meta, dy.contiguous(), helper=ctx.helper)


class _ConstructBlock(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        ctx.helper = NSAHelper.get_bwd_helper()
        ctx.x_meta = x
        return construct_block_fwd(x)

    @staticmethod
    def backward(ctx, dy):
        return construct_block_bwd(ctx.x_meta, dy, helper=ctx.helper)


def mean_pooling(x):
    return _MeanPooling.apply(x)


def construct_block(x):
    return _ConstructBlock.apply(x)
