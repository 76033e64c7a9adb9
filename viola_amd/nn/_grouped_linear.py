"""Forward / dgrad / wgrad orchestration of Linear(scaling="grouped") (the role of
viola/nn/_grouped_linear.py:10-102), shared by Linear and by the two projections of MLP.

Differences from the reference's schedule, none of which change a value:
  * when the FP8 transpose of X is saved for wgrad, X is read ONCE: one kernel emits both the
    row-wise codes for the forward GEMM and the quantized transpose (the reference launches two
    quantize kernels, _grouped_linear.py:21 and :46-47);
  * likewise dY is read once for dgrad + wgrad when both are needed (:73 and :92).
"""

from types import SimpleNamespace

import torch

from . import _grouped_kernels as kernels
from . import _mlp_kernels

_FLOAT = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


def _one_d32(group):
    return tuple(group) == (1, 32)


def forward_core(x, weight, bias, layer, need_backward, needs, *, gated=None, encode=(False, False), encoded=None,
                 input_dtype=None):
    """Returns (y, aux, record). `needs` = (needs dX, needs dW, needs db); aux is the gated
    projection's [g, u] (None otherwise); record carries what backward_core needs.

    encode = (codes, transposed codes too): the gated projection hands h over as MXFP8 codes, and y becomes the tuple
    (codes, scale, codes_t, scale_t) (_grouped_linear.py:28-32). encoded = (scale, codes_t, scale_t) marks x as such
    codes, of an activation of dtype input_dtype (_grouped_linear.py:11-18, 44-46)."""
    shape = x.shape
    x_dtype = x.dtype if encoded is None else input_dtype
    x2 = x.reshape(-1, layer.in_features).contiguous()
    gx, gw = layer.input_group_shape, layer.weight_group_shape
    native = layer._native_scaling
    limit = layer._group_limit(gx, layer.fp8_dtype)
    save_fp8 = need_backward and needs[1] and layer.saved_input_dtype == "fp8"
    xt = sxt = None
    if encoded is not None:
        qx, sx = x2, encoded[0]
        if save_fp8:
            xt, sxt = encoded[1:]
    elif save_fp8 and _one_d32(gx):
        qx, sx, xt, sxt = kernels.quantize_dual(x2, layer.fp8_dtype, gx, limit=limit, native=native)
    else:
        qx, sx = kernels.quantize(x2, layer.fp8_dtype, gx, limit=limit, native=native)
        if save_fp8:
            xt, sxt = kernels.quantize(x2, layer.fp8_dtype, gx, limit=limit, transposed=True, native=native)
    weight_limit = layer._group_limit(gw, layer.fp8_dtype, weight=True)
    if layer.weight_dtype != "fp8":
        qw, sw = kernels.quantize(weight, layer.fp8_dtype, gw, limit=weight_limit, native=native)
    else:
        qw, sw = weight, layer.weight_scale
    aux = None
    extra = None
    if gated:
        y, aux, extra = _mlp_kernels.gemm(qx, qw, sx, sw, layer=layer, out_dtype=x_dtype, bias=bias,
                                          activation=gated, save=need_backward, encode_output=encode[0],
                                          save_output_transpose=encode[1])
    else:
        y = layer._group_gemm(qx, qw, sx, sw, gx, gw, out_dtype=x_dtype, bias=bias)
    record = None
    if need_backward:
        wt, st = layer.weight_transpose, layer.weight_transpose_scale
        if layer.weight_dtype != "fp8" and needs[0] and layer.cache_weight_transpose:
            wt, st = kernels.quantize(weight, layer.fp8_dtype, kernels.transpose_group(gw), limit=weight_limit, transposed=True, native=native)
        if save_fp8:
            saved_x, saved_scale = xt, sxt
        elif needs[1]:
            saved_x, saved_scale = x2.to(_FLOAT[layer.saved_input_dtype]), x2.new_empty(0)
        else:
            saved_x, saved_scale = x2.new_empty(0), x2.new_empty(0)
        record = SimpleNamespace(tensors=(saved_x, saved_scale, weight, sw, wt, st), layer=layer, shape=shape,
                                 x_dtype=x_dtype, save_fp8=save_fp8, input_limit=limit,
                                 weight_grad_dtype=weight.grad_dtype or weight.dtype,
                                 bias_grad_dtype=(bias.grad_dtype or bias.dtype) if bias is not None else None)
    if encode[0]:
        return (y, *extra), aux, record
    return y.reshape(*shape[:-1], y.shape[-1]), aux, record


def backward_core(record, tensors, dy, needs, *, gated=None, aux=None):
    """Returns (dx, dw, db). With `gated`, dx is dz = [d*u*act'(g), d*act(g)] of width 2h and the
    weight gradient is produced first, as in the reference (_grouped_linear.py:69-70)."""
    saved_x, saved_scale, w, sw, cached_wt, cached_st = tensors
    layer = record.layer
    dy = dy.reshape(-1, layer.out_features).contiguous()
    gg, gx, gw = layer.grad_group_shape, layer.input_group_shape, layer.weight_group_shape
    fp8, bwd = layer.fp8_dtype, layer.backward_fp8_dtype
    native = layer._native_scaling
    limit = layer._group_limit(gg, bwd)
    weight_limit = layer._group_limit(gw, fp8, weight=True)
    qg = sg = gt = sgt = None
    dx = dw = db = None
    if needs[0] and needs[1] and _one_d32(gg):
        if needs[2] and dy.shape[0] > 0:
            # the bias gradient rides on the quantizer's read of dy
            qg, sg, gt, sgt, db = kernels.quantize_dual(dy, bwd, gg, limit=limit, column_sum_dtype=record.bias_grad_dtype, native=native)
        else:
            qg, sg, gt, sgt = kernels.quantize_dual(dy, bwd, gg, limit=limit, native=native)
    for op in ((1, 0) if gated else (0, 1)):
        if op == 0 and needs[0]:
            if qg is None:
                qg, sg = kernels.quantize(dy, bwd, gg, limit=limit, native=native)
            if cached_wt.numel():
                wt, st = cached_wt, cached_st
            elif layer.weight_dtype != "fp8":
                wt, st = kernels.quantize(w, fp8, kernels.transpose_group(gw), limit=weight_limit, transposed=True, native=native)
            else:
                wt, st = kernels.transpose(w, sw, gw, native=native, limit=weight_limit)
            gwt = kernels.transpose_group(gw)
            if gated:
                dx, _, _ = _mlp_kernels.gemm(qg, wt, sg, st, layer=layer, out_dtype=record.x_dtype, backward=True,
                                             activation=gated, aux=aux, group_a=gg, group_b=gwt)
            else:
                dx = layer._group_gemm(qg, wt, sg, st, gg, gwt, out_dtype=record.x_dtype)
            dx = dx.reshape(*record.shape[:-1], dx.shape[-1])
            qg = sg = wt = st = None
        if op == 1 and needs[1]:
            if gt is None:
                gt, sgt = kernels.quantize(dy, bwd, gg, limit=limit, transposed=True, native=native)
            if record.save_fp8:
                xt, sxt = saved_x, saved_scale
            else:
                xt, sxt = kernels.quantize(saved_x, fp8, gx, limit=record.input_limit, transposed=True, native=native)
            dw = layer._group_gemm(gt, xt, sgt, sxt, gg, gx, out_dtype=record.weight_grad_dtype)
            gt = sgt = xt = sxt = None
    if needs[2] and db is None:
        db = dy.sum(0, dtype=record.bias_grad_dtype)
    return dx, dw, db


class GroupedLinear(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, layer, need_backward):
        y, _, record = forward_core(x, weight, bias, layer, need_backward, ctx.needs_input_grad[:3])
        if record is not None:
            ctx.save_for_backward(*record.tensors)
            record.tensors = None
            ctx.record = record
        return y

    @staticmethod
    def backward(ctx, dy):
        dx, dw, db = backward_core(ctx.record, ctx.saved_tensors, dy, ctx.needs_input_grad[:3])
        return dx, dw, db, None, None
