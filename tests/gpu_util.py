"""Helpers shared by the GPU parity tests: seeded inputs generated on the CPU (so that oracle and device see the
same bf16 values) and the tolerance of the parity bar."""
import numpy as np
import torch

# parity bar for bf16 outputs and gradients against the fp32 oracle
ATOL = 2e-2
RTOL = 1e-2


def make_cu(lens):
    return torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32)


def randn_bf16(*shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float32).to(torch.bfloat16)


def make_qkvw(T, QH, KH, D, VD=None, seed=0):
    VD = D if VD is None else VD
    q = randn_bf16(T, QH, D, seed=seed)
    k = randn_bf16(T, KH, D, seed=seed + 1)
    v = randn_bf16(T, KH, VD, seed=seed + 2)
    w = randn_bf16(T, QH, 3, seed=seed + 3)
    return q, k, v, w


def assert_close(dev, ref, name, atol=ATOL, rtol=RTOL, row_scale=False):
    """|dev - ref| <= atol + rtol * |ref| elementwise.  With row_scale=True the relative term uses
    max(|ref|, rms of ref over the last dim): for gradients that sum bf16-rounded products over thousands of
    query rows (dK, dV) the rounding error of an element scales with the magnitude of its row, not with the
    element's own value, which may be near zero by cancellation."""
    dev = dev.detach().float().cpu()
    ref = ref.detach().float().cpu()
    assert dev.shape == ref.shape, (name, dev.shape, ref.shape)
    assert torch.isfinite(dev).all(), f"{name}: non-finite values on device"
    err = (dev - ref).abs()
    mag = ref.abs()
    if row_scale and ref.numel():
        mag = torch.maximum(mag, ref.pow(2).mean(-1, keepdim=True).sqrt())
    bound = atol + rtol * mag
    bad = err > bound
    assert not bad.any(), (f"{name}: {int(bad.sum())}/{bad.numel()} outside atol={atol} rtol={rtol}; "
                           f"max abs err {float(err.max()):.4g} at {np.unravel_index(int(err.argmax()), err.shape)}")
    return float(err.max())


def bar_violations(dev, ref, atol=ATOL, rtol=RTOL, row_scale=False):
    """(number of elements outside atol + rtol * base, number of elements, largest |dev - ref|), base as in
    assert_close.  For assertions that state how many elements miss the plain bar instead of hiding them behind the
    row-scaled one."""
    dev = dev.detach().float().cpu()
    ref = ref.detach().float().cpu()
    assert dev.shape == ref.shape and torch.isfinite(dev).all()
    err = (dev - ref).abs()
    mag = ref.abs()
    if row_scale and ref.numel():
        mag = torch.maximum(mag, ref.pow(2).mean(-1, keepdim=True).sqrt())
    return int((err > atol + rtol * mag).sum()), ref.numel(), float(err.max()) if ref.numel() else 0.0
