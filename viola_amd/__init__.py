"""MI355X-native FP8 training hot path with the Python API of chinoll/viola.

What is here, by sub-package:

  nn           `Linear` (grouped FP32 scales, per-tensor `current` / `delayed` scaling, MXFP8), `MLP` (gated, the
               activation fused into the GEMM epilogues), `grouped_linear` for variable-sized expert groups
  optim        `FP8Muon` (FP8 momentum state, Newton-Schulz orthogonalisation in bf16 or fp16), `bind_optimizer`
               (master weights behind FP8 / 16-bit parameters)
  distributed  `FP8Communication`, the FP8 wire codec for gradient buckets, and `packet_bytes`
  precision    process-wide dtype policy (`set_master_weight_dtype`, `set_gradient_dtype`)

Every operator is a hand-written HIP kernel for gfx950 behind a C ABI (include/viola_hip.h, loaded by `_lib`);
nothing falls back to PyTorch arithmetic, and an operator raises if the library is missing.
"""

from . import precision
from . import nn, optim, distributed
from .precision import set_master_weight_dtype, set_gradient_dtype

__version__ = "0.1.0"
__all__ = ["nn", "optim", "distributed", "precision", "set_master_weight_dtype", "set_gradient_dtype"]
