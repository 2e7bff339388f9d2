"""HuggingFace-level NSA core: one autograd node per stage, learned or mean KV compression
(mirrors the interface of upstream flash_nsa/modules/hf_level_nsa.py:17-158)."""

import torch

from ..config import NSAConfig, check_supported
from ..utils import NSAHelper
from ..ops.compress_kv import construct_block, mean_pooling
from ..ops.compress_attn import compress_attn
from ..ops.select_attn import select_attn
from ..ops.topk import slc_topk_indices
from ..ops.act import swiglu_impl, sigmoid_mul_impl
from ..ops.combine import fused_sigmoid_combine
from ..ops.sliding_window_attention import swa_varlen_func

_METHODS = ("mean", "sigmoid-mul", "swiglu", "linear")


class CompressKV(torch.nn.Module):
    """Compresses [T,H,D] into one row per window of kernel_size tokens every stride tokens.
    mean: average; linear: fc over the flattened window; sigmoid-mul / swiglu: gated fc (2*D outputs)."""

    def __init__(self, config: NSAConfig, head_dim=128, version=None):
        super().__init__()
        assert version in _METHODS, f"compression method must be one of {_METHODS}"
        self.head_dim = head_dim
        self.kernel_size = getattr(config, "kernel_size", 32)
        self.stride = getattr(config, "stride", 16)
        self.version = version
        if version != "mean":
            out_features = head_dim if version == "linear" else 2 * head_dim
            self.fc = torch.nn.Linear(self.kernel_size * head_dim, out_features, bias=False)

    def forward(self, x):
        if self.version == "mean":
            return mean_pooling(x)
        windows = construct_block(x)                    # [y_len, H, kernel, D]
        hidden = self.fc(windows.flatten(-2, -1))        # flatten order: (position in window, channel)
        if self.version == "linear":
            return hidden
        if self.version == "sigmoid-mul":
            return sigmoid_mul_impl(hidden)
        return swiglu_impl(hidden)


class HFNSACore(torch.nn.Module):
    def __init__(self, config: NSAConfig):
        super().__init__()
        self.config = config
        self.qk_head_dim = config.qk_head_dim if config.qk_head_dim is not None else config.head_dim
        self.v_head_dim = config.v_head_dim if config.v_head_dim is not None else config.head_dim
        self.kernel_size = getattr(config, "kernel_size", 32)
        self.stride = getattr(config, "stride", 16)
        self.block_size = getattr(config, "block_size", 64)
        self.top_n = getattr(config, "top_n", 16)
        self.num_init_blocks = getattr(config, "num_init_blocks", 1)
        self.num_local_blocks = getattr(config, "num_local_blocks", 2)
        self.window_size = getattr(config, "window_size", 512)
        self.sm_scale = self.qk_head_dim ** -0.5
        # the core also accepts config objects other than NSAConfig (any object with these attributes): validate here too
        check_supported(self.qk_head_dim, self.v_head_dim, self.kernel_size, self.stride, self.block_size)
        self._set_helper()
        self.compress_k = CompressKV(config, head_dim=self.qk_head_dim, version=config.cmp_k_method)
        self.compress_v = CompressKV(config, head_dim=self.v_head_dim, version=config.cmp_v_method)

    def _set_helper(self):
        NSAHelper.set_hyperparameters(kernel_size=self.kernel_size, stride=self.stride, block_size=self.block_size,
                                      window_size=self.window_size, top_n=self.top_n,
                                      num_init_blocks=self.num_init_blocks, num_local_blocks=self.num_local_blocks)

    def forward(self, q, k, v, combine_weight, cu_seqlens, bench: bool = False, print_result: bool = True):
        """q [T,QH,Dqk], k [T,KH,Dqk], v [T,KH,Dv], combine_weight [T,QH,3], cu_seqlens int32 [B+1] -> o [T,QH,Dv].
        With bench=True also returns a pandas Series of per-stage forward milliseconds."""
        assert cu_seqlens is not None
        self._set_helper()
        NSAHelper.init_cu_seqlens(cu_seqlens)
        stages = {}

        def run(name, fn):
            out = fn()
            if bench:
                stages[name] = fn
            return out

        cmp_k = run("cmp_k", lambda: self.compress_k(k))
        cmp_v = run("cmp_v", lambda: self.compress_v(v))
        cmp_o, cmp_lse = run("cmp_o", lambda: compress_attn(q, cmp_k, cmp_v, sm_scale=self.sm_scale))
        topk, _ = run("top_k", lambda: slc_topk_indices(q, cmp_k, cmp_lse, sm_scale=self.sm_scale))
        slc_o = run("slc_o", lambda: select_attn(q, k, v, topk, sm_scale=self.sm_scale))
        swa_o = run("swa_o", lambda: swa_varlen_func(q, k, v, self.sm_scale))
        out = run("combine", lambda: fused_sigmoid_combine(cmp_o, slc_o, swa_o, combine_weight))
        if not bench:
            return out
        import pandas as pd
        times = {}
        with torch.no_grad():
            for name, fn in stages.items():
                times[name] = _time_ms(fn)
        series = pd.Series(times)
        if print_result:
            print("forward time (ms):")
            print(series)
        return out, series


def _time_ms(fn, warmup=2, reps=5):
    for _ in range(warmup):
        fn()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(reps):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / reps
