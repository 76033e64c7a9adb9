"""Per-tensor FP8 scaling operators (operator seam of viola/nn/_linear_kernels.py:231-293): `tensor_scale`,
`quantize`, `transpose`, `gemm`. `transpose` also serves the grouped path."""

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


def tensor_scale_and_column_sum(x, sum_dtype, *, history=None, index=0, delayed=False, fp8_dtype=torch.float8_e4m3fn,
                                quantization_limit=None):
    """(tensor_scale(x), x.sum(0, dtype=sum_dtype)) of a matrix from one read of x; fp32 sums in a fixed order. Falls
    back to two passes when the columns are not whole 16-byte pieces."""
    assert x.is_cuda and x.dim() == 2
    x = x.contiguous()
    rows, cols = x.shape
    piece = 16 // x.element_size()
    if rows == 0 or cols % piece or x.data_ptr() % 16:
        scale = tensor_scale(x, history=history, index=index, delayed=delayed, fp8_dtype=fp8_dtype, quantization_limit=quantization_limit)
        return scale, x.sum(dim=0, dtype=sum_dtype)
    blocks_x = -(-(cols // piece) // 256)
    slices = max(1, min(-(-rows // 8), 512 // blocks_x, 65535))
    parts = blocks_x * slices
    maxima = torch.empty(parts, device=x.device, dtype=torch.float32)
    partial = torch.empty((slices, cols), device=x.device, dtype=torch.float32)
    if history is None:
        history = torch.zeros(1, device=x.device, dtype=torch.float32)
    scale = torch.empty(1, device=x.device, dtype=torch.float32)
    total = torch.empty(cols, device=x.device, dtype=sum_dtype)
    limit = torch.finfo(fp8_dtype).max if quantization_limit is None else quantization_limit
    _lib.call("viola_tensor_amax_columns_scale", _lib.ptr(x), _lib.code(x.dtype), rows, cols, slices, _lib.ptr(maxima),
              _lib.ptr(partial), _lib.ptr(history), history.numel(), int(index), int(bool(delayed)), float(limit), _lib.ptr(scale),
              _lib.ptr(total), _lib.code(sum_dtype))
    return scale, total


def tensor_scale(x, *, history=None, index=0, delayed=False, fp8_dtype=torch.float8_e4m3fn, quantization_limit=None):
    """scale [1] = max(amax(x) or, delayed after the first call, the history's maximum, 1e-30) / limit; the new amax
    goes into history[index % len]. Scratch is one float per 64 Ki elements, never a full-sized temporary."""
    assert x.is_cuda
    x = x.contiguous()
    parts = max(1, min(-(-x.numel() // 65536), 1024))
    maxima = torch.empty(parts, device=x.device, dtype=torch.float32)
    if history is None:
        history = torch.zeros(1, device=x.device, dtype=torch.float32)
    scale = torch.empty(1, device=x.device, dtype=torch.float32)
    limit = torch.finfo(fp8_dtype).max if quantization_limit is None else quantization_limit
    _lib.call("viola_tensor_amax_scale", _lib.ptr(x), _lib.code(x.dtype), x.numel(), _lib.ptr(maxima), parts, _lib.ptr(history),
              history.numel(), int(index), int(bool(delayed)), float(limit), _lib.ptr(scale))
    return scale


def quantize(x, scale, *, rowwise=True, transpose=False, fp8_dtype=torch.float8_e4m3fn, out=None, out_t=None,
             quantization_limit=None):
    """(q, qt): the codes of x / scale in x's layout and / or transposed, from one read; absent ones are (0, 0)-shaped."""
    assert x.is_cuda and x.dim() == 2
    x = x.contiguous()
    q = out if out is not None else torch.empty(x.shape if rowwise else (0, 0), device=x.device, dtype=fp8_dtype)
    qt = out_t if out_t is not None else torch.empty(x.shape[::-1] if transpose else (0, 0), device=x.device, dtype=fp8_dtype)
    assert q.is_contiguous() and qt.is_contiguous() and q.dtype == qt.dtype
    limit = torch.finfo(q.dtype).max if quantization_limit is None else quantization_limit
    _lib.call("viola_tensor_quantize", _lib.ptr(x), _lib.code(x.dtype), x.shape[0], x.shape[1], _lib.ptr(scale),
              _lib.ptr(q), _lib.ptr(qt), _lib.code(q.dtype), float(limit))
    return q, qt


def gemm(a, b, sa, sb, *, out_dtype, bias=None, autotune=False, accum_dtype="fp32", accum_block_size=0,
         accum_reduce_dtype="fp32"):
    """(a * sa) @ (b * sb).T + bias with the scaling in the epilogue; a [m, k] and b [n, k] are FP8 codes.
    accum_dtype="fp16" takes the FP16-accumulator model of the reference's kernel (FP16 partial sums over
    accum_block_size k, totals in accum_reduce_dtype); with FP32 accumulation the other two options change nothing."""
    assert accum_dtype in ("fp32", "fp16") and accum_reduce_dtype in ("fp32", "bf16") and accum_block_size % 32 == 0
    assert a.is_cuda and a.is_contiguous() and b.is_contiguous() and a.shape[1] == b.shape[1]
    out = torch.empty((a.shape[0], b.shape[0]), device=a.device, dtype=out_dtype)
    has_bias = bias is not None and bias.numel() > 0
    if accum_dtype == "fp16":
        _lib.call("viola_tensor_gemm_half", _lib.ptr(a), _lib.code(a.dtype), _lib.ptr(b), _lib.code(b.dtype), _lib.ptr(sa), _lib.ptr(sb),
                  a.shape[0], b.shape[0], a.shape[1], _lib.ptr(bias) if has_bias else None, _lib.code(bias.dtype) if has_bias else 0,
                  _lib.ptr(out), _lib.code(out_dtype), accum_block_size, _lib.BF16 if accum_reduce_dtype == "bf16" else _lib.F32)
        return out
    _lib.call("viola_tensor_gemm", _lib.ptr(a), _lib.code(a.dtype), _lib.ptr(b), _lib.code(b.dtype), _lib.ptr(sa), _lib.ptr(sb),
              a.shape[0], b.shape[0], a.shape[1], _lib.ptr(bias) if has_bias else None, _lib.code(bias.dtype) if has_bias else 0,
              _lib.ptr(out), _lib.code(out_dtype))
    return out
