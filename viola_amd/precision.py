"""Training precision policy (mirrors viola/precision.py:5-35): master-weight dtype,
parameter-gradient dtype and master rounding, read by Linear and FP8Muon at construction."""

import torch

_DTYPES = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}
_settings = dict(master_weight_dtype=torch.float32, gradient_dtype=None,
                 master_rounding="nearest", master_rounding_seed=0)


def _dtype(value):
    value = _DTYPES[value] if isinstance(value, str) else value
    assert value in _DTYPES.values()
    return value


def set_master_weight_dtype(dtype, *, rounding="nearest", seed=0):
    """Master storage dtype; None updates model weights in place without a separate copy."""
    assert rounding in ("nearest", "stochastic") and 0 <= seed < (1 << 63)
    _settings.update(master_weight_dtype=None if dtype is None else _dtype(dtype),
                     master_rounding=rounding, master_rounding_seed=seed)


def set_gradient_dtype(dtype):
    """dtype in which parameter gradients are produced (dW, db) for layers and optimizers built afterwards."""
    _settings["gradient_dtype"] = _dtype(dtype)


def settings():
    return dict(_settings)
