"""Stand-alone PyTorch optimizers on HIP kernels and the master-weight binding for FP8-stored modules.

    FP8Muon          Muon with FP8 momentum (Newton-Schulz on matrices, AdamW on vectors)
    MatrixOptimizer  its base: per-matrix stepping, state layout, checkpoint hooks
    bind_optimizer   FP32/BF16 masters for modules whose weights live as FP8 codes
"""

from .master_weights import bind_optimizer
from .matrix import MatrixOptimizer
from .muon import FP8Muon

__all__ = ("FP8Muon", "MatrixOptimizer", "bind_optimizer")
