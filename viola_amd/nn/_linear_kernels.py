"""Byte-matrix kernels shared with the grouped path (operator seam of
viola/nn/_linear_kernels.py; only `transpose` :253-257 is on the grouped hot path)."""

import torch

from .. import _lib


def transpose(x, out=None):
    """FP8 code matrix [rows, cols] -> [cols, rows] (or a stack [batch, rows, cols] -> [batch, cols, rows]), one HIP launch."""
    assert x.is_cuda and x.dim() in (2, 3) and x.element_size() == 1
    x = x.contiguous()
    if out is None:
        out = torch.empty((*x.shape[:-2], x.shape[-1], x.shape[-2]), device=x.device, dtype=x.dtype)
    _lib.call("viola_fp8_transpose", _lib.ptr(x), _lib.ptr(out), x.shape[0] if x.dim() == 3 else 1, x.shape[-2], x.shape[-1])
    return out
