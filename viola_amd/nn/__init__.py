"""FP8 modules: Linear, gated MLP, and the variable-group (expert) linear."""

from .linear import Linear
from .mlp import MLP
from ._varlen import grouped_linear, GroupedExperts

__all__ = ["Linear", "MLP", "grouped_linear", "GroupedExperts"]
