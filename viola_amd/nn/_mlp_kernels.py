"""FP8 GEMMs with the gated-activation forward/backward epilogues fused (operator seam of
viola/nn/_mlp_kernels.py `gemm` :243-277) for every scaling recipe: FP32 group scales, E8M0 block scales on the
block-scaled MFMA, and one FP32 scale per tensor."""

import torch

from .. import _lib
from . import _gated_kernels, _grouped_kernels


def gemm(a, b, sa, sb, *, layer, out_dtype, activation, backward=False, aux=None, bias=None, save=True,
         group_a=None, group_b=None, encode_output=False, save_output_transpose=False):
    """forward: out = act(a.Wg^T) * (a.Wu^T), aux = [g, u] if save; backward: out = [d*u*act'(g), d*act(g)].

    Returns (out, aux, (out_scale, out_t, out_t_scale)). With encode_output (MXFP8 forward only,
    _mlp_kernels.py:195-230) out holds the FP8 codes of h with E8M0 scales per 32 columns in out_scale, and with
    save_output_transpose out_t / out_t_scale hold the quantized transpose: written by the GEMM's epilogue where
    the block-scaled MFMA path takes the shape, by the dual-layout quantizer from a BF16 h otherwise (the same
    codes and scales either way). Without encode_output the triple is empty.
    """
    assert a.is_cuda and not (save_output_transpose and not encode_output)
    if encode_output:
        return _encoded_forward(a, b, sa, sb, layer=layer, out_dtype=out_dtype, activation=activation, bias=bias, save=save,
                                group_a=group_a, group_b=group_b, transpose=save_output_transpose)
    a, b, sa, sb = a.contiguous(), b.contiguous(), sa.contiguous(), sb.contiguous()
    m, k = a.shape
    h = b.shape[0] if backward else b.shape[0] // 2
    if getattr(layer, "accum_dtype", "fp32") == "fp16":
        # the FP16-accumulator model exists for the plain product: the same values as a fused epilogue from the plain
        # GEMM (which rounds g, u and d to out_dtype as the epilogue does) and the elementwise kernels
        if not layer._grouped_scaling:
            # Per-tensor scales: the reference's MLP kernel clears its FP16 partial every accum_block_size k counted in
            # 32-k steps (viola/nn/_mlp_kernels.py:19-20,129-130), its Linear kernel, which the plain product here
            # models, after whole 64-k chunks (viola/nn/_linear_kernels.py:150-153). The two agree for 32 and for
            # multiples of 64; other periods are refused rather than computed with the wrong clearing points.
            block = getattr(layer, "accum_block_size", 0)
            assert block in (0, 32) or block % 64 == 0, \
                "MLP with per-tensor scaling and accum_dtype='fp16' takes accum_block_size 0, 32 or a multiple of 64"
        plain = (lambda bias_: layer._group_gemm(a, b, sa, sb, tuple(group_a or layer.input_group_shape),
                                                 tuple(group_b or layer.weight_group_shape), out_dtype=out_dtype, bias=bias_)) \
            if layer._grouped_scaling else (lambda bias_: layer._tensor_gemm(a, b, sa, sb, out_dtype=out_dtype, bias=bias_))
        empty = torch.empty((0, 0), device=a.device, dtype=torch.uint8)
        extra = (empty, a.new_empty((0, 0)), empty)
        if backward:
            return _gated_kernels.gated_backward(aux, plain(None), activation), aux, extra
        z, out = _gated_kernels.gated_forward(plain(bias), activation)
        return out, (z if save else z.new_empty((0, 0))), extra
    out = torch.empty((m, 2 * h if backward else h), device=a.device, dtype=out_dtype)
    if aux is None:
        aux = torch.empty((m, 2 * h) if save else (0, 0), device=a.device, dtype=out_dtype)
    else:
        assert aux.dtype == out_dtype and aux.is_contiguous() and tuple(aux.shape) == (m, 2 * h)
    bias_c = bias.contiguous() if bias is not None else None
    bias_code = _lib.code(bias_c.dtype) if bias_c is not None else 0
    empty = torch.empty((0, 0), device=a.device, dtype=torch.uint8)
    extra = (empty, out.new_empty((0, 0), dtype=a.dtype), empty)
    operands = (_lib.ptr(a), _lib.code(a.dtype), _lib.ptr(b), _lib.code(b.dtype), _lib.ptr(sa), _lib.ptr(sb), m, h, k)
    tail = (_lib.ptr(bias_c), bias_code, _lib.ptr(aux), _lib.ptr(out), _lib.code(out_dtype), _lib.ACTIVATION[activation], int(backward))
    if not layer._grouped_scaling:
        _lib.call("viola_tensor_gated_gemm", *operands, *tail)
        return out, aux, extra
    ga = tuple(group_a or layer.input_group_shape)
    gb = tuple(group_b or layer.weight_group_shape)
    if not layer._native_scaling:
        _lib.call("viola_gated_gemm", *operands, ga[0], ga[1], gb[0], gb[1], *tail)
        return out, aux, extra
    status = -2
    if ga[1] == 32 and gb[1] == 32:
        status = _lib.call("viola_mx_gated_gemm", *operands, ga[0], gb[0], *tail, unsupported_ok=True)
    if status != 0:
        # shapes the block-scaled MFMA path does not take: the same values from the plain GEMM and the elementwise kernels
        if backward:
            d = _grouped_kernels.gemm(a, b, sa, sb, ga, gb, out_dtype=out_dtype, native=True)
            out = _gated_kernels.gated_backward(aux, d, activation)
        else:
            z = _grouped_kernels.gemm(a, b, sa, sb, ga, gb, out_dtype=out_dtype, native=True, bias=bias)
            z, out = _gated_kernels.gated_forward(z, activation)
            aux = z if save else aux
    return out, aux, extra


def _encoded_forward(a, b, sa, sb, *, layer, out_dtype, activation, bias, save, group_a, group_b, transpose):
    assert layer._native_scaling, "only the MXFP8 recipe re-encodes H in the GEMM"
    a, b, sa, sb = a.contiguous(), b.contiguous(), sa.contiguous(), sb.contiguous()
    m, k = a.shape
    h = b.shape[0] // 2
    ga = tuple(group_a or layer.input_group_shape)
    gb = tuple(group_b or layer.weight_group_shape)
    fp8 = layer.fp8_dtype
    limit = layer._group_limit(layer.input_group_shape, fp8) or torch.finfo(fp8).max
    if ga[1] == 32 and gb[1] == 32 and m % 32 == 0 and h % 32 == 0:
        aux = torch.empty((m, 2 * h) if save else (0, 0), device=a.device, dtype=out_dtype)
        codes = torch.empty((m, h), device=a.device, dtype=fp8)
        scale = torch.empty((m, h // 32), device=a.device, dtype=torch.uint8)
        codes_t = torch.empty((h, m) if transpose else (0, 0), device=a.device, dtype=fp8)
        scale_t = torch.empty((h, m // 32) if transpose else (0, 0), device=a.device, dtype=torch.uint8)
        bias_c = bias.contiguous() if bias is not None else None
        status = _lib.call("viola_mx_gated_gemm_encode", _lib.ptr(a), _lib.code(a.dtype), _lib.ptr(b), _lib.code(b.dtype),
                           _lib.ptr(sa), _lib.ptr(sb), m, h, k, ga[0], gb[0], _lib.ptr(bias_c),
                           _lib.code(bias_c.dtype) if bias_c is not None else 0, _lib.ptr(aux) if save else None,
                           _lib.code(out_dtype), _lib.ptr(codes), _lib.ptr(scale), _lib.ptr(codes_t) if transpose else None,
                           _lib.ptr(scale_t) if transpose else None, _lib.code(fp8), float(limit), _lib.ACTIVATION[activation],
                           unsupported_ok=True)
        if status == 0:
            return codes, aux, (scale, codes_t, scale_t)
    hidden, aux, _ = gemm(a, b, sa, sb, layer=layer, out_dtype=out_dtype, activation=activation, bias=bias, save=save,
                          group_a=group_a, group_b=group_b)
    if transpose:
        codes, scale, codes_t, scale_t = _grouped_kernels.quantize_dual(hidden, fp8, (1, 32), limit=limit, native=True)
    else:
        codes, scale = _grouped_kernels.quantize(hidden, fp8, (1, 32), limit=limit, native=True)
        codes_t, scale_t = hidden.new_empty((0, 0), dtype=fp8), scale.new_empty((0, 0))
    return codes, aux, (scale, codes_t, scale_t)
