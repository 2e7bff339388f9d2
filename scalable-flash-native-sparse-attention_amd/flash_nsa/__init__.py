"""flash_nsa for MI355X: drop-in Python surface of Native Sparse Attention backed by hand-written gfx950 HIP
kernels (libnsa_hip.so).  Import surface mirrors upstream flash_nsa/__init__.py:1-23."""
from .utils import NSAHelper
from .config import NSAConfig
