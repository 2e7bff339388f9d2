"""Selected-block attention (upstream flash_nsa/ops/select_attn.py:439-748)."""
import torch

from .. import _lib
from ..utils import NSAHelper
from ._common import check_thd, default_scale, delta_of, dq_target


def slc_attn_fwd(q, k, v, topk, sm_scale=None, helper=NSAHelper):
    """q [T,QH,D], k [T,KH,D], v [T,KH,VD], topk [KH,T,top_n] int32 -> o [T,QH,VD], lse [T,QH] fp32 (log2).
    Query t of a sequence attends the keys <= t of the blocks in its first min(top_n, t//block+1) slots."""
    check_thd(q, "q"), check_thd(k, "k"), check_thd(v, "v")
    T, QH, D = q.shape
    _, KH, VD = v.shape
    assert topk.dtype == torch.int32 and topk.shape[:2] == (KH, T) and topk.stride(-1) == 1
    sm_scale = default_scale(q, sm_scale)
    o = torch.empty(T, QH, VD, device=q.device, dtype=q.dtype)
    lse = torch.empty(T, QH, device=q.device, dtype=torch.float32)
    _lib.call("nsa_slc_attn_fwd", q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), k.stride(0), k.stride(1),
              v.data_ptr(), v.stride(0), v.stride(1), topk.data_ptr(), topk.stride(0), topk.stride(1), o.data_ptr(),
              o.stride(0), o.stride(1), lse.data_ptr(), lse.stride(0), lse.stride(1),
              helper.x_cu_seqlens.data_ptr(), helper.batch, helper.x_maxlen, QH, KH, D, VD, helper.block_size,
              topk.size(-1), sm_scale, _lib.stream_ptr())
    return o, lse


def slc_attn_bwd(q, k, v, topk, o, lse, do, dq=None, dk=None, dv=None, sm_scale=None, helper=NSAHelper, delta=None,
                 bind=None, parts="both", dkdv_repeat=False):
    """Backward of selected attention.  Returns (dq, dk, dv).
    dq: fresh bf16 tensor, or the caller's fp32 buffer (added into).  dk/dv: fp32 [T,KH,*]; the caller's buffers
    are added into, otherwise zero-filled ones are created.  dkdv_repeat=False (default): with fp32 atomics, so the
    summation order changes from run to run (as upstream's dkdv_repeat=False); dkdv_repeat=True (or
    NSAHelper.set_deterministic(True)): the work items store into slots of a scratch buffer that a second launch adds
    in a fixed order -- bit-identical results across runs.  `bind` is the inverse index from get_bind_from_find (built here when absent).
    parts = "dq" / "dkdv" launches only that kernel (the other results are None)."""
    from .topk import get_bind_from_find
    check_thd(do, "do")
    T, QH, D = q.shape
    _, KH, VD = v.shape
    sm_scale = default_scale(q, sm_scale)
    if delta is None:
        delta = delta_of(o, do)
    common = (q.data_ptr(), q.stride(0), q.stride(1), k.data_ptr(), k.stride(0), k.stride(1), v.data_ptr(),
              v.stride(0), v.stride(1), do.data_ptr(), do.stride(0), do.stride(1), lse.data_ptr(), lse.stride(0),
              lse.stride(1), delta.data_ptr(), delta.stride(0), delta.stride(1))
    dq_buf = None
    if parts in ("both", "dq"):
        dq_buf, mode = dq_target(q, dq)
        _lib.call("nsa_slc_attn_bwd_dq", *common, topk.data_ptr(), topk.stride(0), topk.stride(1), dq_buf.data_ptr(),
                  dq_buf.stride(0), dq_buf.stride(1), mode, helper.x_cu_seqlens.data_ptr(), helper.batch,
                  helper.x_maxlen, QH, KH, D, VD, helper.block_size, topk.size(-1), sm_scale, _lib.stream_ptr())
    if parts == "dq":
        return dq_buf, None, None
    if dk is None:
        dk = torch.zeros(T, KH, D, device=q.device, dtype=torch.float32)
    if dv is None:
        dv = torch.zeros(T, KH, VD, device=q.device, dtype=torch.float32)
    assert dk.dtype == torch.float32 and dv.dtype == torch.float32
    if bind is None:
        bind = get_bind_from_find(topk, helper)
    args = (*common, dk.data_ptr(), dk.stride(0), dk.stride(1), dv.data_ptr(), dv.stride(0), dv.stride(1),
            helper.x_cu_seqlens.data_ptr(), helper.k_cu_seqlens.data_ptr(), helper.blk_seq.data_ptr(),
            bind["csr_off"].data_ptr(), bind["csr_tok"].data_ptr(), bind["item_off"].data_ptr(), bind["nblk"],
            bind["chunk_tokens"], bind["n_items_bound"], helper.batch, QH, KH, D, VD, helper.block_size, sm_scale)
    if dkdv_repeat or getattr(helper, "deterministic", False):
        nbytes = _lib.value("nsa_slc_attn_bwd_dkdv_det_bytes", bind["n_items_bound"], KH, D, VD, helper.block_size)
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=q.device)
        _lib.call("nsa_slc_attn_bwd_dkdv_det", *args, ws.data_ptr(), ws.numel(), _lib.stream_ptr())
    else:
        _lib.call("nsa_slc_attn_bwd_dkdv", *args, _lib.stream_ptr())
    return dq_buf, dk, dv


class _SelectAttn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, topk, sm_scale):
        o, lse = slc_attn_fwd(q, k, v, topk, sm_scale)
        ctx.save_for_backward(q, k, v, topk, o, lse)
        ctx.sm_scale = sm_scale
        ctx.helper = NSAHelper.get_bwd_helper()
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, topk, o, lse = ctx.saved_tensors
        do = do if do.stride(-1) == 1 else do.contiguous()
        dq, dk, dv = slc_attn_bwd(q, k, v, topk, o, lse, do, sm_scale=ctx.sm_scale, helper=ctx.helper)
        return dq, dk.to(k.dtype), dv.to(v.dtype), None, None


def select_attn(q, k, v, topk, sm_scale=None):
    """Differentiable selected-block attention (no gradient flows into topk)."""
    return _SelectAttn.apply(q, k, v, topk, sm_scale)
