"""Attention layer around HFNSACore: separate q / k / v / gate projections, rotary embedding, output projection
(the demo layer of upstream flash_nsa/layers/hf_level_nsa.py:8-58).  The projections are plain library GEMMs
(torch.nn.Linear -> hipBLASLt); everything between them is this package's HIP path."""
import torch
import torch.nn as nn

from ..config import NSAConfig
from ..modules.hf_level_nsa import HFNSACore
from ..ops.rope import fused_apply_rope


class HFNSA(nn.Module):
    def __init__(self, config: NSAConfig) -> None:
        super().__init__()
        self.hidden_size = config.hidden_size
        self.num_heads, self.num_kv_heads = config.num_heads, config.num_kv_heads
        self.qk_head_dim, self.v_head_dim = config.qk_head_dim, config.v_head_dim
        self.q_proj = nn.Linear(self.hidden_size, self.num_heads * self.qk_head_dim, bias=False)
        self.k_proj = nn.Linear(self.hidden_size, self.num_kv_heads * self.qk_head_dim, bias=False)
        self.v_proj = nn.Linear(self.hidden_size, self.num_kv_heads * self.v_head_dim, bias=False)
        self.o_proj = nn.Linear(self.num_heads * self.v_head_dim, self.hidden_size, bias=False)
        self.combine_proj = nn.Linear(self.hidden_size, self.num_heads * 3, bias=False)
        self.nsa = HFNSACore(config)

    def forward(self, hidden_states, position_embeddings, cu_seqlens=None):
        """hidden_states [b,s,hidden]; position_embeddings = (cos, sin) [b|1,s,d]; cu_seqlens over the b*s packed
        tokens (default: b sequences of s tokens)."""
        b, s, _ = hidden_states.shape
        q = self.q_proj(hidden_states).view(b, s, self.num_heads, self.qk_head_dim)
        k = self.k_proj(hidden_states).view(b, s, self.num_kv_heads, self.qk_head_dim)
        v = self.v_proj(hidden_states).view(b, s, self.num_kv_heads, self.v_head_dim)
        w = self.combine_proj(hidden_states).view(b, s, self.num_heads, 3)
        cos, sin = position_embeddings
        q, k = fused_apply_rope(q, k, cos, sin, inplace=True)
        if cu_seqlens is None:
            cu_seqlens = torch.arange(b + 1, device=q.device, dtype=torch.int32) * s
        o = self.nsa(q.flatten(0, 1), k.flatten(0, 1), v.flatten(0, 1), w.flatten(0, 1), cu_seqlens)
        return self.o_proj(o.view(b, s, -1))
