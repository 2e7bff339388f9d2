"""Attention layer around NSACore with ONE fused projection producing q, k, v and the three gates per head
(the demo layer of upstream flash_nsa/layers/megatron_level_nsa.py:9-113, without the Megatron tensor-/context-
parallel wrappers: one GPU).  Sequence-first activations [s, b, hidden], as Megatron passes them."""
import torch
import torch.nn as nn

from ..config import NSAConfig
from ..modules.megatron_level_nsa import NSACore
from ..ops.rope import fused_apply_rope


def _batch_first_tables(t, b, s):
    """cos / sin as [b|1, s, d]: accepts that layout, the sequence-first one [s, b|1, d] and either with an extra
    singleton head axis (Megatron's [s, 1, 1, d])."""
    if t.dim() == 4:
        t = t.squeeze(-2)
    if t.size(0) in (b, 1) and t.size(1) == s:
        return t
    assert t.size(0) == s and t.size(1) in (b, 1), f"rotary table of shape {tuple(t.shape)} for b={b}, s={s}"
    return t.transpose(0, 1)


class NSA(nn.Module):
    def __init__(self, config: NSAConfig):
        super().__init__()
        self.config = config
        self.hidden_size = config.hidden_size
        self.num_heads, self.num_kv_heads = config.num_heads, config.num_kv_heads
        self.qk_head_dim, self.v_head_dim = config.qk_head_dim, config.v_head_dim
        self.nsa = NSACore(config)
        # columns: q | k | v | gates | padding to a multiple of 8 (every slice then starts 16-byte aligned for bf16
        # whenever the head dims are multiples of 8)
        self.split_size = [self.num_heads * self.qk_head_dim, self.num_kv_heads * self.qk_head_dim,
                           self.num_kv_heads * self.v_head_dim, self.num_heads * 3]
        out = sum(self.split_size)
        pad = -out % 8
        self.split_size.append(pad)
        self.qkv_proj = nn.Linear(self.hidden_size, out + pad, bias=False)
        self.o_proj = nn.Linear(self.num_heads * self.v_head_dim, self.hidden_size, bias=False)

    def forward(self, hidden_states, rotary_pos_emb, extra_kwargs=None):
        """hidden_states [s,b,hidden]; rotary_pos_emb = (cos, sin) [b|1,s,d] or [s,b|1,d];
        extra_kwargs["cu_seqlens"] over the b*s tokens in batch-major order.  Returns [s,b,hidden]."""
        s, b, _ = hidden_states.shape
        q, k, v, w, _ = self.qkv_proj(hidden_states).split(self.split_size, -1)
        q = q.view(s, b, self.num_heads, self.qk_head_dim)
        k = k.view(s, b, self.num_kv_heads, self.qk_head_dim)
        v = v.view(s, b, self.num_kv_heads, self.v_head_dim)
        w = w.view(s, b, self.num_heads, 3)
        cos, sin = (_batch_first_tables(t, b, s) for t in rotary_pos_emb)
        # with one sequence per batch the batch-first views are the projection's own memory and are rotated in
        # place; otherwise the rotation writes the packed batch-major copy that the core needs anyway
        q, k = fused_apply_rope(q.transpose(0, 1), k.transpose(0, 1), cos, sin, inplace=(b == 1))
        cu_seqlens = (extra_kwargs or {}).get("cu_seqlens")
        assert cu_seqlens is not None, "extra_kwargs['cu_seqlens'] is required"
        o = self.nsa(q.flatten(0, 1), k.flatten(0, 1), v.transpose(0, 1).flatten(0, 1),
                     w.transpose(0, 1).flatten(0, 1), cu_seqlens)
        o = o.view(b, s, self.num_heads * self.v_head_dim).transpose(0, 1)
        return self.o_proj(o)
