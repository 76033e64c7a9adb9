"""Hadamard-64 rotation ahead of per-tensor FP8 quantization (operator seam of viola/nn/_rotation_kernels.py:100-123):
`tensor_scale` and `quantize` of the rotated tensor without a full-sized floating temporary, and the in-place
rotation `inverse_` (H64 is its own inverse). Rotation runs along the last dimension in runs of 64 columns."""

import torch

from .. import _lib


def tensor_scale(x, *, history=None, index=0, delayed=False, fp8_dtype=torch.float8_e4m3fn, quantization_limit=None):
    """The per-tensor scale of rotate(x): max |rotate(x)| (or the history's maximum) / limit, one float per 64 x 64
    tile as scratch."""
    assert x.is_cuda and x.dim() == 2 and x.numel() > 0
    x = x.contiguous()
    rows, cols = x.shape
    parts = -(-rows // 64) * -(-cols // 64)
    maxima = torch.empty(parts, device=x.device, dtype=torch.float32)
    if history is None:
        history = torch.zeros(1, device=x.device, dtype=torch.float32)
    scale = torch.empty(1, device=x.device, dtype=torch.float32)
    limit = torch.finfo(fp8_dtype).max if quantization_limit is None else quantization_limit
    _lib.call("viola_rotation_amax", _lib.ptr(x), _lib.code(x.dtype), rows, cols, _lib.ptr(maxima), parts)
    _lib.call("viola_tensor_scale", _lib.ptr(maxima), parts, _lib.ptr(history), history.numel(), int(index), int(bool(delayed)),
              float(limit), _lib.ptr(scale))
    return scale


def quantize(x, scale, *, rowwise=True, transpose=False, fp8_dtype=torch.float8_e4m3fn, out=None, out_t=None,
             quantization_limit=None):
    """(q, qt): the codes of rotate(x) / scale in x's layout and / or transposed; absent ones are (0, 0)-shaped."""
    assert x.is_cuda and x.dim() == 2
    x = x.contiguous()
    q = out if out is not None else torch.empty(x.shape if rowwise else (0, 0), device=x.device, dtype=fp8_dtype)
    qt = out_t if out_t is not None else torch.empty(x.shape[::-1] if transpose else (0, 0), device=x.device, dtype=fp8_dtype)
    assert q.is_contiguous() and qt.is_contiguous() and q.dtype == qt.dtype
    limit = torch.finfo(q.dtype).max if quantization_limit is None else quantization_limit
    _lib.call("viola_rotation_quantize", _lib.ptr(x), _lib.code(x.dtype), x.shape[0], x.shape[1], _lib.ptr(scale),
              _lib.ptr(q), _lib.ptr(qt), _lib.code(q.dtype), float(limit))
    return q, qt


def inverse_(x):
    """x <- rotate(x) in place (rounded to x's dtype); returns x."""
    assert x.is_cuda and x.dim() == 2 and x.is_contiguous()
    _lib.call("viola_rotation_inverse", _lib.ptr(x), _lib.code(x.dtype), x.shape[0], x.shape[1])
    return x
