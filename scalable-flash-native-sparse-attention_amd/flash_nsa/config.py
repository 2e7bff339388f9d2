"""NSAConfig: hyper-parameters of the sparse attention (mirrors upstream flash_nsa/config.py:16-86)."""
import json
from dataclasses import dataclass, fields
from typing import Optional


def _is_pow2(n: int) -> bool:
    return n > 0 and (n & (n - 1)) == 0


# (qk head dim, v head dim) pairs the kernels are built for
SUPPORTED_HEAD_DIMS = ((128, 128), (64, 64), (192, 128), (32, 32), (256, 256))


def check_supported(qk_head_dim, v_head_dim, kernel_size, stride, block_size):
    """The constraints of upstream (flash_nsa/config.py:48-52) plus the ones of this build's kernels, checked where a
    model is configured so that an unsupported shape fails there and not at its first launch."""
    assert _is_pow2(stride), "stride must be a power of 2"
    assert kernel_size % stride == 0, "kernel_size must be a multiple of stride"
    assert block_size >= kernel_size, "block_size must be >= kernel_size"
    assert block_size % stride == 0, "block_size must be a multiple of stride"
    assert block_size % 32 == 0, (
        f"block_size {block_size}: the selected-attention kernels work in units of 32 keys; block sizes that are "
        "multiples of 32 are supported (32, 64, 96, 128, 256, ...)")
    assert (qk_head_dim, v_head_dim) in SUPPORTED_HEAD_DIMS, (
        f"head dims qk={qk_head_dim} / v={v_head_dim} are not built; supported (qk, v) pairs: {SUPPORTED_HEAD_DIMS}")


@dataclass
class NSAConfig:
    hidden_size: int = 4096
    head_dim: int = 128
    qk_head_dim: Optional[int] = None
    v_head_dim: Optional[int] = None
    num_heads: int = 64
    num_kv_heads: int = 4

    kernel_size: int = 32
    stride: int = 16
    cmp_k_method: str = "mean"
    cmp_v_method: str = "mean"
    block_size: int = 64
    top_n: int = 16
    num_init_blocks: int = 1
    num_local_blocks: int = 2
    window_size: int = 512

    recompute_swa_o: bool = False
    recompute_slc_o: bool = False
    recompute_cmp_kv: bool = False
    recompute_cmp_o: bool = False

    # context-parallel knobs are accepted for config-file compatibility; this build runs on one GPU
    cp_mode: int = 1
    kv_head_stride: int = 1
    use_overlap_swa: bool = False

    def __post_init__(self):
        assert _is_pow2(self.stride), "stride must be a power of 2"
        assert self.kernel_size % self.stride == 0
        assert self.block_size >= self.kernel_size
        assert self.block_size % self.stride == 0
        if self.qk_head_dim is None:
            assert self.head_dim is not None
            self.qk_head_dim = self.head_dim
        if self.v_head_dim is None:
            assert self.head_dim is not None
            self.v_head_dim = self.head_dim
        assert self.num_heads % self.num_kv_heads == 0
        check_supported(self.qk_head_dim, self.v_head_dim, self.kernel_size, self.stride, self.block_size)

    @classmethod
    def from_json(cls, json_file: str):
        with open(json_file, "r", encoding="utf-8") as f:
            data = json.load(f)
        known = {f.name for f in fields(cls)}
        inst = cls(**{k: v for k, v in data.items() if k in known})
        for k, v in data.items():  # unknown keys ride along as plain attributes, as upstream does
            if k not in known:
                setattr(inst, k, v)
        return inst
