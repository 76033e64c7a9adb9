"""Group-scaled FP8 quantization and GEMM operators (operator seam of
viola/nn/_grouped_kernels.py: scale_shape :16, dequantize :44, quantize :127,
transpose_group :161, transpose :166, gemm :310), each one call into libviola_hip.

`native=True` is the MXFP8 recipe: scales are E8M0 bytes (uint8, value 2^(byte - 127)) of 32-wide K groups, and the
GEMM scales inside the block-scaled MFMA.
"""

import torch

from .. import _lib
from ._linear_kernels import transpose as transpose_payload


def scale_shape(shape, group):
    return tuple(-(-n // g) for n, g in zip(shape, group))


def _scale_dtype(native):
    return torch.uint8 if native else torch.float32


def decode_scale(scale):
    """E8M0 bytes -> the FP32 scales they stand for (exact); FP32 scales pass through."""
    return torch.exp2(scale.float() - 127.) if scale.dtype == torch.uint8 else scale


def dequantize(q, scale, group):
    """fp32 [rows, cols] = float(q) * scale[r // gr, c // gc]."""
    assert q.is_cuda, "viola_amd kernels run on the GPU only"
    q = q.contiguous()
    scale = decode_scale(scale)
    out = torch.empty(q.shape, device=q.device, dtype=torch.float32)
    _lib.call("viola_group_dequantize", _lib.ptr(q), _lib.code(q.dtype), _lib.ptr(scale.contiguous()),
              q.shape[0], q.shape[1], group[0], group[1], _lib.ptr(out))
    return out


def quantize(x, dtype, group, *, native=False, limit=None, transposed=False,
             source_scale=None, source_group=(1, 32), out=None, scale_out=None):
    """Group amax quantization of a 2-D tensor; returns (codes, fp32 scales), or (codes, E8M0 bytes) with native=True.

    transposed=True yields the quantized transpose (codes [cols, rows]) with the groups laid
    along the new last dimension, read straight from the floating input. source_scale re-encodes
    existing codes. out/scale_out let the caller own the outputs (nothing is allocated then).
    """
    assert x.is_cuda and x.dim() == 2, "viola_amd kernels run on the GPU only"
    x = x.contiguous()
    shape = tuple(x.shape[::-1]) if transposed else tuple(x.shape)
    limit = torch.finfo(dtype).max if limit is None else limit
    q = out if out is not None else torch.empty(shape, device=x.device, dtype=dtype)
    s = scale_out if scale_out is not None else torch.empty(scale_shape(shape, group), device=x.device, dtype=_scale_dtype(native))
    assert q.is_contiguous() and s.is_contiguous() and tuple(q.shape) == shape and tuple(s.shape) == scale_shape(shape, group)
    assert s.dtype == _scale_dtype(native) and (source_scale is None or source_scale.dtype == s.dtype)
    source = source_scale.contiguous() if source_scale is not None else None
    _lib.call("viola_group_quantize", _lib.ptr(x), _lib.code(x.dtype), x.shape[0], x.shape[1],
              _lib.ptr(q), _lib.code(q.dtype), _lib.ptr(s), group[0], group[1], float(limit), int(transposed),
              _lib.ptr(source), source_group[0], source_group[1], int(bool(native)))
    return q, s


def quantize_dual(x, dtype, group, *, limit=None, column_sum_dtype=None, native=False):
    """Row-wise codes/scales and the quantized transpose of x from ONE read of x.

    Same values as quantize(x, ...) and quantize(x, ..., transposed=True); 1-D groups of 32 only.
    Returns (q, s, qt, st), plus x.sum(0) in column_sum_dtype (fp32 accumulation, from the same read)
    when that is given.
    """
    assert x.is_cuda and x.dim() == 2 and tuple(group) == (1, 32)
    x = x.contiguous()
    rows, cols = x.shape
    limit = torch.finfo(dtype).max if limit is None else limit
    q = torch.empty((rows, cols), device=x.device, dtype=dtype)
    s = torch.empty(scale_shape((rows, cols), group), device=x.device, dtype=_scale_dtype(native))
    qt = torch.empty((cols, rows), device=x.device, dtype=dtype)
    st = torch.empty(scale_shape((cols, rows), group), device=x.device, dtype=_scale_dtype(native))
    parts = -(-rows // 32)
    partial = torch.empty((parts, cols), device=x.device, dtype=torch.float32) if column_sum_dtype is not None else None
    _lib.call("viola_group_quantize_dual", _lib.ptr(x), _lib.code(x.dtype), rows, cols, _lib.ptr(q), _lib.ptr(s),
              _lib.ptr(qt), _lib.ptr(st), _lib.code(dtype), group[1], float(limit), _lib.ptr(partial), int(bool(native)))
    if column_sum_dtype is None:
        return q, s, qt, st
    total = torch.empty(cols, device=x.device, dtype=column_sum_dtype)
    _lib.call("viola_column_reduce", _lib.ptr(partial), parts, cols, _lib.ptr(total), _lib.code(column_sum_dtype))
    return q, s, qt, st, total


def gated_quantize_dual(z, activation, dtype, *, limit=None, native=False):
    """quantize_dual of h = act(g) * u (rounded to z's dtype) straight from z = [g | u] [rows, 2 h], bf16 / fp16:
    the codes an MLP's down projection reads (viola/nn/_mlp_kernels.py:195-230) without h ever being stored.
    Returns (q, s, qt, st), or None for shapes the kernel does not take."""
    assert z.is_cuda and z.dim() == 2 and z.shape[1] % 2 == 0
    z = z.contiguous()
    rows, h = z.shape[0], z.shape[1] // 2
    limit = torch.finfo(dtype).max if limit is None else limit
    q = torch.empty((rows, h), device=z.device, dtype=dtype)
    s = torch.empty(scale_shape((rows, h), (1, 32)), device=z.device, dtype=_scale_dtype(native))
    qt = torch.empty((h, rows), device=z.device, dtype=dtype)
    st = torch.empty(scale_shape((h, rows), (1, 32)), device=z.device, dtype=_scale_dtype(native))
    status = _lib.call("viola_gated_quantize_dual", _lib.ptr(z), _lib.code(z.dtype), rows, h, _lib.ACTIVATION[activation], _lib.ptr(q),
                       _lib.ptr(s), _lib.ptr(qt), _lib.ptr(st), _lib.code(dtype), 32, float(limit), int(bool(native)), unsupported_ok=True)
    return (q, s, qt, st) if status == 0 else None


def transpose_group(group):
    """A 2-D block (>= 32 rows) transposes exactly; a 1-D row group keeps its shape and needs new K groups."""
    return tuple(group[::-1]) if group[0] >= 32 else tuple(group)


def transpose(q, scale, group, *, native=False, limit=None):
    if group[0] >= 32:
        # a 2-D block transposes exactly: codes and scale grid move in one launch
        assert q.is_cuda and q.dim() == 2 and scale.dim() == 2
        q, scale = q.contiguous(), scale.contiguous()
        out = torch.empty((q.shape[1], q.shape[0]), device=q.device, dtype=q.dtype)
        scale_out = torch.empty((scale.shape[1], scale.shape[0]), device=q.device, dtype=scale.dtype)
        if q.numel():
            _lib.call("viola_block_transpose", _lib.ptr(q), _lib.ptr(out), q.shape[0], q.shape[1], _lib.ptr(scale), _lib.ptr(scale_out),
                      group[0], group[1], int(scale.dtype == torch.uint8))
        return out, scale_out
    return quantize(q, q.dtype, group, native=native, limit=limit, transposed=True, source_scale=scale, source_group=group)


def gemm(a, b, sa, sb, group_a, group_b, *, out_dtype, native=False, bias=None, autotune=False,
         accum_dtype="fp32", accum_block_size=0, accum_reduce_dtype="fp32"):
    """out[m, n] = sum over 32-wide K groups of (a_codes . b_codes^T) * sa * sb (+ bias); a [m, k], b [n, k].

    accum_dtype="fp16" (FP32 scales only) takes the FP16-accumulator model of the reference's kernel: FP16 partial sums
    per scale group, totals in accum_reduce_dtype. With FP32 accumulation the other two options change nothing (the
    MFMA's sums are FP32 throughout)."""
    assert accum_dtype in ("fp32", "fp16") and accum_reduce_dtype in ("fp32", "bf16") and accum_block_size % 32 == 0
    assert a.is_cuda and b.is_cuda and a.shape[1] == b.shape[1]
    a, b, sa, sb = a.contiguous(), b.contiguous(), sa.contiguous(), sb.contiguous()
    m, k = a.shape
    n = b.shape[0]
    assert tuple(sa.shape) == scale_shape((m, k), group_a) and tuple(sb.shape) == scale_shape((n, k), group_b)
    out = torch.empty((m, n), device=a.device, dtype=out_dtype)
    bias_c = bias.contiguous() if bias is not None else None
    if accum_dtype == "fp16":
        assert not native, "MXFP8 MMA uses FP32 accumulation."
        _lib.call("viola_group_gemm_half", _lib.ptr(a), _lib.code(a.dtype), _lib.ptr(b), _lib.code(b.dtype), _lib.ptr(sa), _lib.ptr(sb),
                  m, n, k, group_a[0], group_a[1], group_b[0], group_b[1], _lib.ptr(bias_c),
                  _lib.code(bias_c.dtype) if bias_c is not None else 0, _lib.ptr(out), _lib.code(out_dtype), accum_block_size,
                  _lib.BF16 if accum_reduce_dtype == "bf16" else _lib.F32)
        return out
    if native:
        assert sa.dtype == torch.uint8 and sb.dtype == torch.uint8 and group_a[1] == 32 and group_b[1] == 32
        status = _lib.call("viola_mx_gemm", _lib.ptr(a), _lib.code(a.dtype), _lib.ptr(b), _lib.code(b.dtype), _lib.ptr(sa),
                           _lib.ptr(sb), m, n, k, group_a[0], group_b[0], _lib.ptr(bias_c),
                           _lib.code(bias_c.dtype) if bias_c is not None else 0, _lib.ptr(out), _lib.code(out_dtype),
                           unsupported_ok=True)
        if status == 0:
            return out
        # shapes the block-scaled MFMA kernel declines: the same products with the scales spelled out in FP32
        sa, sb = decode_scale(sa), decode_scale(sb)
    _lib.call("viola_group_gemm", _lib.ptr(a), _lib.code(a.dtype), _lib.ptr(b), _lib.code(b.dtype), _lib.ptr(sa), _lib.ptr(sb),
              m, n, k, group_a[0], group_a[1], group_b[0], group_b[1],
              _lib.ptr(bias_c), _lib.code(bias_c.dtype) if bias_c is not None else 0, _lib.ptr(out), _lib.code(out_dtype))
    return out
