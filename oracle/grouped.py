"""Group-scaled FP8 quantization and GEMM on CPU tensors. TEST INFRASTRUCTURE ONLY.

Restates the reference's group quantizer and the "dequantize then FP32 matmul"
recipe its checks use as the expected value.
"""

import torch
import torch.nn.functional as F

FP8 = {"e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2}


def scale_shape(shape, group):
    """ceil(n / g) per dimension (viola/nn/_grouped_kernels.py:16-17)."""
    return tuple((n + g - 1) // g for n, g in zip(shape, group))


def decode_scale(scale):
    """E8M0 bytes (uint8, the `native` recipe) -> 2^(byte - 127) (viola/nn/_grouped_kernels.py:35,72); FP32 passes."""
    return torch.exp2(scale.float() - 127.) if scale.dtype == torch.uint8 else scale.float()


def pow2_ceil(scales):
    """The smallest power of two that is not below each (positive, finite) scale: the mathematical value of the
    reference's exp2(ceil(log2(s))) (viola/nn/_grouped_kernels.py:81-83 on the GPU, :143-146 on the CPU), found from
    the binary exponent instead of a rounded fp32 logarithm. PARITY UNPINNED where the reference's own log2 rounds:
    for s within a few ulp above a power of two with |log2 s| >= 4 its fp32 log2 comes out an integer and the
    reference keeps the smaller power; nothing in the reference pins that case (its CPU and CUDA log2 differ too)."""
    mantissa, exponent = torch.frexp(scales.float())                       # s = mantissa * 2^exponent, mantissa in [0.5, 1)
    exponent = torch.where(mantissa == 0.5, exponent - 1, exponent)
    return torch.ldexp(torch.ones_like(scales, dtype=torch.float32), exponent), (exponent + 127).to(torch.uint8)


def dequantize(q, scale, group):
    """float(q) * scale[r // gr, c // gc]  (viola/nn/_grouped_kernels.py:37-40,49-50)."""
    expanded = decode_scale(scale).repeat_interleave(group[0], 0).repeat_interleave(group[1], 1)
    return q.float() * expanded[:q.shape[0], :q.shape[1]]


def quantize(x, dtype, group, *, limit=None, transposed=False, source_scale=None, source_group=(1, 32), native=False):
    """Group amax quantization (viola/nn/_grouped_kernels.py:127-158).

    Follows the CPU branch at :135-151 (pad -> reshape (nr, gr, nc, gc) -> amax ->
    clamp_min(1e-30) / limit -> divide -> clamp -> cast), except for NaN inside a
    group, where the device kernel's behaviour is restated instead
    (encode_kernel :69-91): the abs-max reduction ignores NaN, so only the NaN
    element itself becomes a NaN code. Every step is an IEEE fp32 operation.
    """
    limit = torch.finfo(dtype).max if limit is None else limit
    value = dequantize(x, source_scale, source_group) if source_scale is not None else x.float()
    value = value.T if transposed else value
    shape = tuple(value.shape)
    gr, gc = group
    nr, nc = scale_shape(shape, group)
    blocks = F.pad(value, (0, nc * gc - shape[1], 0, nr * gr - shape[0])).reshape(nr, gr, nc, gc)
    magnitude = torch.where(blocks.isnan(), torch.zeros_like(blocks), blocks.abs())
    scales = magnitude.amax((1, 3)).clamp_min(1e-30) / limit
    stored = scales
    if native:                                                             # E8M0: power-of-two scale, stored as its exponent byte
        scales, stored = pow2_ceil(scales)
    codes = (blocks / scales[:, None, :, None]).clamp(-limit, limit)      # clamp keeps NaN
    q = codes.reshape(nr * gr, nc * gc)[:shape[0], :shape[1]].to(dtype)
    return q.contiguous(), stored.contiguous()


def transpose_group(group):
    """2-D blocks transpose exactly; 1-D row groups keep their shape (:161-163)."""
    return group[::-1] if group[0] >= 32 else group


def transpose(q, scale, group, *, limit=None, native=False):
    """Byte transpose + scale.T for 2-D blocks, otherwise re-encode (:166-171)."""
    if group[0] >= 32:
        return q.T.contiguous(), scale.T.contiguous()
    return quantize(q, q.dtype, group, limit=limit, transposed=True, source_scale=scale, source_group=group, native=native)


def gemm(a, b, sa, sb, group_a, group_b, *, out_dtype=torch.float32, bias=None, witness=False):
    """(deq(a) @ deq(b).T + bias) -> out dtype (checks/check_grouped_linear.py:32,39).

    witness=True evaluates the same sum in fp64 (the reference's FP64 witness,
    viola/nn/_grouped_tuning.py:40-46).
    """
    da, db = dequantize(a, sa, group_a), dequantize(b, sb, group_b)
    if witness:
        da, db = da.double(), db.double()
    out = da @ db.T
    if bias is not None:
        out = out + bias.to(out.dtype)
    return out.to(out_dtype)


def gemm_kgroup_order(a, b, sa, sb, group_a, group_b, *, bias=None):
    """The device kernel's own summation order: per 32-wide K group, the raw code
    product is formed first and then scaled, total += (acc*sa)*sb, K groups in
    ascending order (viola/nn/_grouped_kernels.py:268-292). Used to show that the
    order does not matter beyond fp32 rounding."""
    m, k = a.shape
    n = b.shape[0]
    total = torch.zeros(m, n)
    af, bf = a.float(), b.float()
    rows = torch.arange(m) // group_a[0]
    cols = torch.arange(n) // group_b[0]
    for k0 in range(0, k, 32):
        acc = af[:, k0:k0 + 32] @ bf[:, k0:k0 + 32].T
        total = total + (acc * sa[rows, k0 // group_a[1]][:, None]) * sb[cols, k0 // group_b[1]][None, :]
    if bias is not None:
        total = total + bias.float()
    return total


def gemm_half(a, b, sa, sb, group_a, group_b, *, accum_block_size=0, reduce_dtype=torch.float32, bias=None,
              out_dtype=torch.float32):
    """gemm_kernel with accum_dtype='float16' (viola/nn/_grouped_kernels.py:268-292, :310-318).

    `acc` is an FP16 fragment advanced by the 32-k tensor-core step `mma.mma(al, bl, acc)`: modelled as
    acc = fp16(acc + the 32 products summed exactly), the best a unit with an FP16 accumulator can return (what the
    reference's GPU does inside that step is not written in its source: parity with it is held to the bound of
    checks/check_grouped_linear.py:41, not to the bit). Every partial_k = gcd(group K sizes, accum_block_size) k:
    total = reduce_dtype(float(total) + float(acc) * sa * sb), acc = 0.
    """
    import math
    m, k = a.shape
    n = b.shape[0]
    partial_k = math.gcd(group_a[1], group_b[1])
    if accum_block_size:
        partial_k = math.gcd(partial_k, accum_block_size)
    total = torch.zeros(m, n, dtype=reduce_dtype)
    acc = torch.zeros(m, n, dtype=torch.float16)
    af, bf = a.double(), b.double()
    rows = torch.arange(m) // group_a[0]
    cols = torch.arange(n) // group_b[0]
    for k0 in range(0, k, 32):
        step = af[:, k0:k0 + 32] @ bf[:, k0:k0 + 32].T                    # exact in float64
        acc = (acc.double() + step).to(torch.float16)
        if (k0 + 32) % partial_k == 0 or k0 + 32 >= k:
            scaled = (acc.float() * sa[rows, k0 // group_a[1]][:, None]) * sb[cols, k0 // group_b[1]][None, :]
            total = (total.float() + scaled).to(reduce_dtype)
            acc = torch.zeros_like(acc)
    value = total.float()
    if bias is not None:
        value = value + bias.float()
    return value.to(out_dtype)

