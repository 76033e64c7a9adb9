"""MI355X-native FP8 training hot path with the Python API of chinoll/viola:
`nn.Linear`, `nn.MLP`, `nn.grouped_linear`, `optim.FP8Muon`, the FP8 gradient wire codec.
Every operator is a hand-written HIP kernel for gfx950 behind a C ABI (include/viola_hip.h)."""

__version__ = "0.1.0"

from . import distributed, nn, optim, precision
from .precision import set_gradient_dtype, set_master_weight_dtype

__all__ = ["distributed", "nn", "optim", "precision", "set_master_weight_dtype", "set_gradient_dtype"]
