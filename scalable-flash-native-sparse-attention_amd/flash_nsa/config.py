"""NSAConfig: hyper-parameters of the sparse attention (mirrors upstream flash_nsa/config.py:16-86)."""
import json
from dataclasses import dataclass, fields
from typing import Optional


def _is_pow2(n: int) -> bool:
    return n > 0 and (n & (n - 1)) == 0


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
