"""Argument checks shared by the operator wrappers."""
import torch


def check_bf16(*tensors):
    for t in tensors:
        assert t.is_cuda, "tensor must live on the GPU"
        assert t.dtype == torch.bfloat16, f"this build computes in bf16 only (got {t.dtype})"
        assert t.stride(-1) == 1, "last dimension must be contiguous"


def check_thd(t, name):
    assert t.dim() == 3, f"{name} must be [tokens, heads, dim]"
    check_bf16(t)
    assert t.stride(0) % 8 == 0 and t.stride(1) % 8 == 0, f"{name}: token/head strides must be 16-byte aligned"
    assert t.data_ptr() % 16 == 0, f"{name}: base address must be 16-byte aligned"


def default_scale(q, sm_scale):
    return q.size(-1) ** -0.5 if sm_scale is None else float(sm_scale)


def delta_of(o, do):
    """delta[T,H] fp32 = rowsum(o * do): the softmax-backward correction term."""
    from .. import _lib
    T, H, D = o.shape
    delta = torch.empty(T, H, device=o.device, dtype=torch.float32)
    _lib.call("nsa_delta", o.data_ptr(), o.stride(0), o.stride(1), do.data_ptr(), do.stride(0), do.stride(1),
              delta.data_ptr(), T, H, D, _lib.stream_ptr())
    return delta


def dq_target(q, dq):
    """(buffer, mode) for a dq output: fresh bf16 store, or accumulation into a caller-provided fp32 buffer."""
    if dq is None:
        return torch.empty_like(q), 0
    if hasattr(dq, "buf"):  # fp32 buffer to be overwritten (first branch of a fused backward)
        return dq.buf, 1
    assert dq.dtype == torch.float32 and dq.shape == q.shape and dq.stride(-1) == 1, \
        "an accumulation target for dq must be fp32 with q's shape"
    return dq, 2
