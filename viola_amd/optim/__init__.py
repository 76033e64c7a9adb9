"""Stand-alone PyTorch optimizers on HIP kernels: FP8Muon, its MatrixOptimizer base and the master-weight binding."""

from .matrix import MatrixOptimizer
from .muon import FP8Muon
from .master_weights import bind_optimizer

__all__ = ["MatrixOptimizer", "FP8Muon", "bind_optimizer"]
