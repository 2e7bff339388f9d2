"""Megatron-level NSA core: the whole sparse attention as ONE autograd node with fp32 dq/dk/dv accumulation
across the three branches and optional recomputation of saved activations
(mirrors the interface of upstream flash_nsa/modules/megatron_level_nsa.py:46-159, 386-545; the
context-parallel function of that file is outside this single-GPU build)."""
import math

import torch

from ..config import NSAConfig, check_supported
from ..utils import NSAHelper
from ..ops.compress_kv import construct_block_fwd, construct_block_bwd, mean_pooling_fwd, mean_pooling_bwd
from ..ops.compress_attn import cmp_attn_fwd, cmp_attn_bwd
from ..ops.select_attn import slc_attn_fwd, slc_attn_bwd
from ..ops.topk import slc_topk_indices
from ..ops.act import swiglu_fwd, swiglu_bwd, sigmoid_mul_fwd, sigmoid_mul_bwd
from ..ops.combine import combine_fwd, combine_bwd
from ..ops.sliding_window_attention import swa_fwd, swa_bwd


# The backward runs on two streams: the memory-bound selected-block dq kernel leaves the matrix cores idle and the
# dense dk/dv kernels leave the memory side idle, so the dq chain (window -> selected -> compressed) runs next to the
# dk/dv kernels (measured: about 1 ms of a 75 ms step; the same split of the forward gained nothing).
# Setting this module attribute to False puts everything back on the caller's stream.
OVERLAP_STREAMS = True
_side_streams = {}


def _side_stream(device):
    key = device.index if device.index is not None else torch.cuda.current_device()
    s = _side_streams.get(key)
    if s is None:
        s = _side_streams[key] = torch.cuda.Stream(device=device)
    return s


def weight_grad(inp, grad_out, weight):
    """dW = grad_out^T @ inp; accumulated into weight.main_grad (fp32) when the optimizer keeps one."""
    inp = inp.reshape(-1, inp.size(-1))
    grad_out = grad_out.reshape(-1, grad_out.size(-1))
    main_grad = getattr(weight, "main_grad", None)
    if main_grad is None:
        return torch.matmul(grad_out.t(), inp)
    # bf16 operands, fp32 accumulator added to the fp32 buffer in the GEMM's epilogue: no rounding of dW to bf16
    # (upstream's wgrad GEMM adds its fp32 accumulator tiles the same way, flash_nsa/ops/gemm.py:131-133)
    torch.addmm(main_grad, grad_out.t(), inp, out_dtype=torch.float32, out=main_grad)
    if hasattr(weight, "grad_added_to_main_grad"):
        weight.grad_added_to_main_grad = True
        return torch.empty(main_grad.shape, dtype=inp.dtype, device=inp.device)
    return None


def compress_kv_fwd(x, weight, version, helper=NSAHelper):
    """-> (windows or None, pre-activation or None, compressed rows)"""
    if version == "mean":
        return None, None, mean_pooling_fwd(x, helper=helper)
    windows = construct_block_fwd(x, helper=helper)
    hidden = torch.matmul(windows.flatten(-2, -1), weight.t())
    if version == "linear":
        out = hidden
    elif version == "sigmoid-mul":
        out = sigmoid_mul_fwd(hidden)
    elif version == "swiglu":
        out = swiglu_fwd(hidden)
    else:
        raise ValueError(version)
    return windows, hidden, out


def compress_kv_bwd(x, weight, windows, hidden, dout, dx, version, helper=NSAHelper, async_dw=False):
    """Adds the compression gradient into the fp32 buffer dx and returns (dx, dW or a thunk computing it)."""
    dout = dout.to(x.dtype)
    if version == "mean":
        mean_pooling_bwd(x, dout, dx, helper=helper)
        return dx, None
    if version == "linear":
        dhidden = dout
    elif version == "sigmoid-mul":
        dhidden = sigmoid_mul_bwd(hidden, dout, inplace=False)
    else:
        dhidden = swiglu_bwd(hidden, dout, inplace=False)
    dwindows = torch.matmul(dhidden, weight).view(*windows.shape)
    construct_block_bwd(x, dwindows, dx, helper=helper)

    def dw_fn():
        return weight_grad(windows.flatten(-2, -1), dhidden, weight)

    return dx, (dw_fn if async_dw else dw_fn())


class NSAFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, combine_weight, cmp_k_weight, cmp_v_weight, sm_scale=None):
        if sm_scale is None:
            sm_scale = q.size(-1) ** -0.5
        H = NSAHelper
        win_k, hid_k, cmp_k = compress_kv_fwd(k, cmp_k_weight, H.cmp_k_method)
        win_v, hid_v, cmp_v = compress_kv_fwd(v, cmp_v_weight, H.cmp_v_method)
        cmp_o, cmp_lse = cmp_attn_fwd(q, cmp_k, cmp_v, sm_scale=sm_scale)
        topk, _ = slc_topk_indices(q, cmp_k, cmp_lse, sm_scale=sm_scale)
        slc_o, slc_lse = slc_attn_fwd(q, k, v, topk, sm_scale=sm_scale)
        swa_o, swa_lse = swa_fwd(q, k, v, sm_scale=sm_scale)
        out = combine_fwd(cmp_o, slc_o, swa_o, combine_weight)

        keep = lambda flag, *ts: [None if flag else t for t in ts]
        saved = [q, k, v, combine_weight, cmp_k_weight, cmp_v_weight, topk]
        saved += keep(H.recompute_cmp_kv, win_k, hid_k, cmp_k, win_v, hid_v, cmp_v)
        saved += keep(H.recompute_cmp_o, cmp_o, cmp_lse)
        saved += keep(H.recompute_slc_o, slc_o, slc_lse)
        saved += keep(H.recompute_swa_o, swa_o, swa_lse)
        ctx.save_for_backward(*saved)
        ctx.sm_scale = sm_scale
        ctx.helper = H.get_bwd_helper()
        ctx.methods = (H.cmp_k_method, H.cmp_v_method)
        return out

    @staticmethod
    def backward(ctx, do):
        (q, k, v, combine_weight, cmp_k_weight, cmp_v_weight, topk, win_k, hid_k, cmp_k, win_v, hid_v, cmp_v, cmp_o,
         cmp_lse, slc_o, slc_lse, swa_o, swa_lse) = ctx.saved_tensors
        sm_scale, helper = ctx.sm_scale, ctx.helper
        k_method, v_method = ctx.methods
        do = do if do.stride(-1) == 1 else do.contiguous()

        if cmp_k is None:
            win_k, hid_k, cmp_k = compress_kv_fwd(k, cmp_k_weight, k_method, helper)
            win_v, hid_v, cmp_v = compress_kv_fwd(v, cmp_v_weight, v_method, helper)
        if cmp_o is None:
            cmp_o, cmp_lse = cmp_attn_fwd(q, cmp_k, cmp_v, sm_scale=sm_scale, helper=helper)
        if slc_o is None:
            slc_o, slc_lse = slc_attn_fwd(q, k, v, topk, sm_scale=sm_scale, helper=helper)
        if swa_o is None:
            swa_o, swa_lse = swa_fwd(q, k, v, sm_scale=sm_scale, helper=helper)

        # the combine backward also yields rowsum(branch * dbranch) of the three branches
        dcmp_o, dslc_o, dswa_o, dw, delta = combine_bwd(cmp_o, slc_o, swa_o, combine_weight, do, return_delta=True)
        dq32 = torch.empty(q.shape, device=q.device, dtype=torch.float32)
        kw = dict(sm_scale=sm_scale, helper=helper)
        if OVERLAP_STREAMS:
            main, side = torch.cuda.current_stream(), _side_stream(q.device)
            side.wait_stream(main)
            with torch.cuda.stream(side):
                # dq chain: the selected branch (memory bound) stores, the window branch (matrix bound, with
                # bandwidth to spare for the read-modify-write) adds, the compressed branch adds and writes q's dtype
                slc_attn_bwd(q, k, v, topk, slc_o, slc_lse, dslc_o, _store_into(dq32), delta=delta[1], parts="dq", **kw)
                swa_bwd(q, k, v, swa_o, swa_lse, dswa_o, delta=delta[2], dq=dq32, parts="dq", **kw)
                dq, _, _ = cmp_attn_bwd(q, cmp_k, cmp_v, cmp_o, cmp_lse, dcmp_o, dq32, delta=delta[0],
                                        finalize_dq=True, parts="dq", **kw)
                dq.record_stream(main)
            # dk/dv kernels on the caller's stream.  The compressed branch (matrix bound) goes first, next to the
            # selected dq kernel (bound by the gather path) on the other stream: 0.7-1.7 ms per step less at T = 64K
            # (67.7 -> 67.0 and 67.2 -> 65.5 ms on two GPUs) than the order window, selected, compressed, which ran the
            # two selected kernels side by side.  The
            # window branch writes every element of dk / dv, the selected branch then adds to them.
            _, dcmp_k, dcmp_v = cmp_attn_bwd(q, cmp_k, cmp_v, cmp_o, cmp_lse, dcmp_o, delta=delta[0], parts="dkdv",
                                             **kw)
            _, dk, dv = swa_bwd(q, k, v, swa_o, swa_lse, dswa_o, delta=delta[2], dkv_fp32=True, parts="dkdv", **kw)
            slc_attn_bwd(q, k, v, topk, slc_o, slc_lse, dslc_o, None, dk, dv, delta=delta[1], parts="dkdv", **kw)
        else:
            # the selected branch stores dq, the window branch adds to it and writes every element of dk / dv, to
            # which the selected branch then adds
            slc_attn_bwd(q, k, v, topk, slc_o, slc_lse, dslc_o, _store_into(dq32), delta=delta[1], parts="dq", **kw)
            _, dk, dv = swa_bwd(q, k, v, swa_o, swa_lse, dswa_o, delta=delta[2], dq=dq32, dkv_fp32=True, **kw)
            slc_attn_bwd(q, k, v, topk, slc_o, slc_lse, dslc_o, None, dk, dv, delta=delta[1], parts="dkdv", **kw)
            dq, dcmp_k, dcmp_v = cmp_attn_bwd(q, cmp_k, cmp_v, cmp_o, cmp_lse, dcmp_o, dq32, delta=delta[0],
                                              finalize_dq=True, **kw)
        _, dwk = compress_kv_bwd(k, cmp_k_weight, win_k, hid_k, dcmp_k, dk, k_method, helper)
        _, dwv = compress_kv_bwd(v, cmp_v_weight, win_v, hid_v, dcmp_v, dv, v_method, helper)
        if OVERLAP_STREAMS:
            main.wait_stream(side)
        return dq, dk, dv, dw, dwk, dwv, None


class _StoreTarget:
    """Marks an fp32 dq buffer that the first branch overwrites instead of adding into."""

    def __init__(self, buf):
        self.buf = buf


def _store_into(buf):
    return _StoreTarget(buf)


def flash_nsa_varlen_func(q, k, v, combine_weight, cmp_k_weight=None, cmp_v_weight=None, sm_scale=None):
    return NSAFunction.apply(q, k, v, combine_weight, cmp_k_weight, cmp_v_weight, sm_scale)


def cp_flash_nsa_varlen_func(*args, **kwargs):
    raise NotImplementedError("context parallelism is outside this single-GPU build")


class NSACore(torch.nn.Module):
    def __init__(self, config: NSAConfig, process_group=None, pp_size=1):
        super().__init__()
        assert process_group is None, "context parallelism is outside this single-GPU build"
        self.config = config
        self.qk_head_dim = config.qk_head_dim if config.qk_head_dim is not None else config.head_dim
        self.v_head_dim = config.v_head_dim if config.v_head_dim is not None else config.head_dim
        g = lambda name, default: getattr(config, name, default)
        self.kernel_size, self.stride, self.block_size = g("kernel_size", 32), g("stride", 16), g("block_size", 64)
        self.top_n, self.window_size = g("top_n", 16), g("window_size", 512)
        self.num_init_blocks, self.num_local_blocks = g("num_init_blocks", 1), g("num_local_blocks", 2)
        self.cmp_k_method, self.cmp_v_method = g("cmp_k_method", "mean"), g("cmp_v_method", "mean")
        self.recompute = dict(recompute_cmp_kv=g("recompute_cmp_kv", False), recompute_cmp_o=g("recompute_cmp_o", False),
                              recompute_slc_o=g("recompute_slc_o", False), recompute_swa_o=g("recompute_swa_o", False))
        self.pp_size = pp_size
        self.sm_scale = self.qk_head_dim ** -0.5
        # the core also accepts config objects other than NSAConfig (any object with these attributes): validate here too
        check_supported(self.qk_head_dim, self.v_head_dim, self.kernel_size, self.stride, self.block_size)
        self._set_helper()

        def make_weight(method, dim):
            if method == "mean":
                return None
            out_features = dim if method == "linear" else 2 * dim
            w = torch.empty(out_features, self.kernel_size * dim)
            torch.nn.init.kaiming_uniform_(w, a=math.sqrt(5))
            return torch.nn.Parameter(w)

        self.cmp_k_weight = make_weight(self.cmp_k_method, self.qk_head_dim)
        self.cmp_v_weight = make_weight(self.cmp_v_method, self.v_head_dim)

    def _set_helper(self):
        NSAHelper.set_hyperparameters(kernel_size=self.kernel_size, stride=self.stride, block_size=self.block_size,
                                      window_size=self.window_size, top_n=self.top_n,
                                      num_init_blocks=self.num_init_blocks, num_local_blocks=self.num_local_blocks)
        NSAHelper.set_recompute(**self.recompute)
        NSAHelper.set_cmp_kv_method(cmp_k_method=self.cmp_k_method, cmp_v_method=self.cmp_v_method)
        NSAHelper.set_pipeline_parallel_world_size(pp_size=self.pp_size)

    def forward(self, q, k, v, combine_weight, cu_seqlens, cu_seqlens_np=None, cp_mode=None):
        """q [T,QH,Dqk], k [T,KH,Dqk], v [T,KH,Dv], combine_weight [T,QH,3], cu_seqlens int32 [B+1] -> [T,QH,Dv]"""
        assert cu_seqlens is not None
        self._set_helper()
        NSAHelper.init_cu_seqlens(cu_seqlens)
        return flash_nsa_varlen_func(q, k, v, combine_weight, self.cmp_k_weight, self.cmp_v_weight, self.sm_scale)
