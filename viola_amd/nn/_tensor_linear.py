"""Forward / dgrad / wgrad of Linear(scaling="current" | "delayed"): one FP32 scale per tensor, applied in the
GEMM epilogue (the role of `_Linear`, viola/nn/linear.py:36-147), shared by Linear and by the two projections of MLP.
Each operand is read twice at most: once for its amax, once by the quantizer, which writes the row-wise and the
transposed codes together when both are needed.

With `rotation_size=64`, X and W are Hadamard-rotated along in_features inside their amax and quantize kernels
((X H)(W H)^T = X W^T), dY is not, and the two gradients that come out in rotated coordinates, dX = dY (W H) and
dW = dY^T (X H), are rotated back in place (linear.py:42-52, :113-115, :142-143)."""

from types import SimpleNamespace

import torch

from . import _gated_kernels
from . import _linear_kernels as kernels
from . import _mlp_kernels
from . import _rotation_kernels as rotation

_FLOAT = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


def forward_core(x, weight, bias, layer, need_backward, needs, *, gated=None):
    """Returns (y, aux, record). `needs` = (needs dX, needs dW, needs db); with `gated`, y = act(g) * u and aux is
    the projection's [g, u] (linear.py:54-57); record carries what backward_core needs."""
    shape = x.shape
    x2 = x.reshape(-1, layer.in_features).contiguous()
    fp8 = layer.fp8_dtype
    input_limit = layer._quantization_limit(max(x2.shape), fp8)
    sx = layer.input_quantizer.scale(x2, fp8, input_limit, layer.rotation_size)
    quantize = rotation.quantize if layer.rotation_size else kernels.quantize
    needs_x, needs_w = needs[0], needs[1]
    save_fp8 = need_backward and needs_w and layer.saved_input_dtype == "fp8"
    qx, qxt = quantize(x2, sx, transpose=save_fp8, fp8_dtype=fp8, quantization_limit=input_limit)
    if layer.weight_dtype != "fp8":
        weight_limit = layer._quantization_limit(max(weight.shape), fp8)
        sw = layer.weight_quantizer.scale(weight, fp8, weight_limit, layer.rotation_size)
        qw, wt = quantize(weight, sw, fp8_dtype=fp8, quantization_limit=weight_limit,
                          transpose=need_backward and needs_x and layer.cache_weight_transpose)
    else:
        qw, sw, wt = weight, layer.weight_scale, layer.weight_transpose
    aux = None
    if gated:
        y, aux, _ = _mlp_kernels.gemm(qx, qw, sx, sw, layer=layer, out_dtype=x2.dtype, bias=bias, activation=gated, save=need_backward)
    else:
        y = layer._tensor_gemm(qx, qw, sx, sw, out_dtype=x2.dtype, bias=bias)
    record = None
    if need_backward:
        if save_fp8:
            saved_x = qxt
        elif needs_w:
            saved_x = x2.to(_FLOAT[layer.saved_input_dtype])
        else:
            saved_x = x2.new_empty(0)
        # the scales this very forward used, not the quantizers' mutable state
        record = SimpleNamespace(tensors=(saved_x, sx, weight, sw, wt), layer=layer, shape=shape, x_dtype=x2.dtype,
                                 save_fp8=save_fp8, input_limit=input_limit,
                                 weight_grad_dtype=weight.grad_dtype or weight.dtype,
                                 bias_grad_dtype=(bias.grad_dtype or bias.dtype) if bias is not None else None)
    return y.reshape(*shape[:-1], y.shape[-1]), aux, record


def backward_core(record, tensors, dy, needs, *, gated=None, aux=None):
    """Returns (dx, dw, db). With `gated`, dx is dz = [d*u*act'(g), d*act(g)] of width 2h, from the dgrad GEMM's
    epilogue, or, under rotation, from the elementwise kernel after dX is rotated back (linear.py:106-122)."""
    saved_x, sx, weight, sw, cached_wt = tensors
    layer = record.layer
    fp8, bwd = layer.fp8_dtype, layer.backward_fp8_dtype
    dy = dy.reshape(-1, layer.out_features).contiguous()
    needs_x, needs_w, needs_b = needs
    grad_limit = layer._quantization_limit(max(dy.shape), bwd)
    dx = dw = db = None
    quantize = rotation.quantize if layer.rotation_size else kernels.quantize
    if needs_b:
        # the bias gradient rides on the amax pass over dy
        sg, db = layer.grad_quantizer.scale_and_column_sum(dy, record.bias_grad_dtype, bwd, grad_limit)
    else:
        sg = layer.grad_quantizer.scale(dy, bwd, grad_limit)
    # one read of dy serves dgrad (row-wise codes) and wgrad (transposed codes) when both are wanted
    qg, qgt = kernels.quantize(dy, sg, rowwise=needs_x, transpose=needs_w, fp8_dtype=bwd, quantization_limit=grad_limit)
    if needs_x:
        if cached_wt.numel():
            wt = cached_wt
        elif layer.weight_dtype != "fp8":
            # this forward's scale again: the delayed history does not advance in backward
            _, wt = quantize(weight, sw, rowwise=False, transpose=True, fp8_dtype=fp8,
                             quantization_limit=layer._quantization_limit(max(weight.shape), fp8))
        else:
            wt = kernels.transpose(weight)
        if gated and not layer.rotation_size:
            dx, _, _ = _mlp_kernels.gemm(qg, wt, sg, sw, layer=layer, out_dtype=record.x_dtype, activation=gated, backward=True, aux=aux)
        else:
            dx = layer._tensor_gemm(qg, wt, sg, sw, out_dtype=record.x_dtype)
            if layer.rotation_size:
                rotation.inverse_(dx)
            if gated:
                dx = _gated_kernels.gated_backward(aux, dx, gated)               # the inverse rotation comes before the derivative
        dx = dx.reshape(*record.shape[:-1], dx.shape[-1])
        del wt, qg
    if needs_w:
        if record.save_fp8:
            xt = saved_x
        else:
            _, xt = quantize(saved_x, sx, rowwise=False, transpose=True, fp8_dtype=fp8, quantization_limit=record.input_limit)
        dw = layer._tensor_gemm(qgt, xt, sg, sx, out_dtype=record.weight_grad_dtype)
        if layer.rotation_size:
            rotation.inverse_(dw)
    return dx, dw, db


class TensorLinear(torch.autograd.Function):
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
