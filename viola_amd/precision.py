"""Process-wide training precision policy, read by Linear, the variable-group experts, FP8Muon and bind_optimizer
when they are constructed (the role of viola/precision.py:5-35).

Three knobs: the dtype master weights are kept in (None = update the model's own weights, no separate copy), how a
master is rounded when it is narrower than FP32, and the dtype parameter gradients (dW, db) are produced in. Layers
and optimizers that already exist keep what they were built with.
"""

import torch

_NAMES = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}
_ROUNDINGS = ("nearest", "stochastic")

# the live policy; settings() hands out copies
_settings = {
    "master_weight_dtype": torch.float32,
    "gradient_dtype": None,
    "master_rounding": "nearest",
    "master_rounding_seed": 0,
}


def _resolve(dtype):
    """'fp32' / 'bf16' / 'fp16' or the torch dtype itself -> torch dtype."""
    resolved = _NAMES.get(dtype, dtype) if isinstance(dtype, str) else dtype
    assert resolved in _NAMES.values(), f"unsupported floating dtype {dtype!r}"
    return resolved


def set_master_weight_dtype(dtype, *, rounding="nearest", seed=0):
    assert rounding in _ROUNDINGS, rounding
    assert 0 <= seed < 2 ** 63, "the seed is a 63-bit Philox key"
    _settings["master_weight_dtype"] = _resolve(dtype) if dtype is not None else None
    _settings["master_rounding"] = rounding
    _settings["master_rounding_seed"] = seed


def set_gradient_dtype(dtype):
    _settings["gradient_dtype"] = _resolve(dtype)


def settings():
    """A snapshot of the policy: later set_* calls do not reach into it."""
    return {key: value for key, value in _settings.items()}
