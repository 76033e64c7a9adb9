"""Stand-alone PyTorch optimizers on HIP kernels: FP8Muon and its MatrixOptimizer base."""

from .matrix import MatrixOptimizer
from .muon import FP8Muon

__all__ = ["MatrixOptimizer", "FP8Muon"]
