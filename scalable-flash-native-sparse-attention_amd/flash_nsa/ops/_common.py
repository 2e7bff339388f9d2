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
