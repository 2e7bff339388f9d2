from .hf_level_nsa import HFNSA
from .megatron_level_nsa import NSA
