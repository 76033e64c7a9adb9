"""Variable-group (MoE-expert style) FP8 linear: `groups` independent Linear(scaling="grouped")
problems that share in/out features and differ in how many rows each owns.

The reference has no such operator (its "grouped" means group-scaled quantization); the semantics
here are "a Python loop of per-group viola.nn.Linear(scaling='grouped')": rows are quantized with
(1, 32) tiles, weights with (32, 32) blocks per group, and the weight gradient of a group uses the
transposed (1, 32) quantization of that group's own rows (32-token tiles counted from the group's
first row). One launch covers all groups; empty groups yield no rows and a zero dW.
"""

import math

import torch
from torch import nn

from .. import _lib
from . import _grouped_kernels as kernels
from ._linear_kernels import transpose as transpose_payload
from ..precision import settings

_FORMATS = {"e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2}
GX, GW = (1, 32), (32, 32)


def _offsets(counts, device):
    counts = [int(c) for c in (counts.tolist() if isinstance(counts, torch.Tensor) else counts)]
    assert all(c >= 0 for c in counts)
    offsets, padded = [0], [0]
    for c in counts:
        offsets.append(offsets[-1] + c)
        padded.append(padded[-1] + (c + 31) // 32 * 32)
    # The padded token axis is the row length of the transposed codes: rounded up to 128 (empty slots at the end of the
    # last group, zero codes) so that every row starts on a cache line and the quantizer's 64-byte pieces never straddle one.
    padded[-1] = (padded[-1] + 127) // 128 * 128
    both = torch.tensor([offsets, padded], dtype=torch.int64).to(device, non_blocking=True)
    return offsets, padded, both[0], both[1]


def varlen_gemm(a, b, sa, sb, offsets_dev, *, out_dtype):
    """a [M, K] codes with (1, 32) scales; b [G, N, K] codes with (32, 32) scales [G, N/32, K/32]."""
    m, k = a.shape
    groups, n, _ = b.shape
    out = torch.empty((m, n), device=a.device, dtype=out_dtype)
    _lib.call("viola_varlen_group_gemm", _lib.ptr(a), _lib.code(a.dtype), _lib.ptr(b), _lib.code(b.dtype),
              _lib.ptr(sa), _lib.ptr(sb), _lib.ptr(offsets_dev), groups, m, n, k, GX[0], GX[1], GW[0], GW[1],
              n * k, sb.shape[1] * sb.shape[2], _lib.ptr(out), _lib.code(out_dtype))
    return out


def quantize_transposed_segmented(x, dtype, offsets_dev, padded_dev, groups, t_total, *, rowwise=False):
    """Per-group quantized transpose of x [M, C]: codes [C, t_total], scales [C, t_total/32]. With rowwise, also the
    plain (1, 32) row-wise codes and scales of x from the same read: returns (qt, st, q, s)."""
    rows, cols = x.shape
    qt = torch.empty((cols, t_total), device=x.device, dtype=dtype)
    st = torch.empty((cols, t_total // 32), device=x.device, dtype=torch.float32)
    fused = rowwise and x.element_size() == 2 and cols % 8 == 0 and x.data_ptr() % 16 == 0
    q = torch.empty((rows, cols), device=x.device, dtype=dtype) if fused else None
    s = torch.empty((rows, -(-cols // 32)), device=x.device, dtype=torch.float32) if fused else None
    _lib.call("viola_varlen_quantize_transposed", _lib.ptr(x), _lib.code(x.dtype), rows, cols, _lib.ptr(offsets_dev),
              _lib.ptr(padded_dev), groups, t_total, _lib.ptr(qt), _lib.ptr(st), _lib.code(dtype),
              float(torch.finfo(dtype).max), _lib.ptr(q), _lib.ptr(s))
    if not rowwise:
        return qt, st
    if not fused:
        q, s = kernels.quantize(x, dtype, GX)
    return qt, st, q, s


def varlen_wgrad(gt, xt, sgt, sxt, padded_dev, groups, *, out_dtype):
    n, t_total = gt.shape
    kout = xt.shape[0]
    out = torch.empty((groups, n, kout), device=gt.device, dtype=out_dtype)
    _lib.call("viola_varlen_wgrad_gemm", _lib.ptr(gt), _lib.code(gt.dtype), _lib.ptr(xt), _lib.code(xt.dtype),
              _lib.ptr(sgt), _lib.ptr(sxt), _lib.ptr(padded_dev), groups, t_total, n, kout, _lib.ptr(out), _lib.code(out_dtype))
    return out


class _VarlenLinear(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, weight_scale, counts, fp8, bwd_fp8, grad_dtype):
        assert x.is_cuda and x.dim() == 2
        x = x.contiguous()
        groups = weight.shape[0]
        offsets, padded, offsets_dev, padded_dev = _offsets(counts, x.device)
        assert offsets[-1] == x.shape[0] and len(offsets) == groups + 1
        need_w = ctx.needs_input_grad[1]
        if need_w and x.shape[0]:
            xt, sxt, qx, sx = quantize_transposed_segmented(x, fp8, offsets_dev, padded_dev, groups, padded[-1], rowwise=True)
        else:
            qx, sx = kernels.quantize(x, fp8, GX)
            xt = sxt = x.new_empty(0)
        y = varlen_gemm(qx, weight, sx, weight_scale, offsets_dev, out_dtype=x.dtype)
        ctx.save_for_backward(xt, sxt, weight, weight_scale, offsets_dev, padded_dev)
        ctx.meta = (groups, padded[-1], bwd_fp8, grad_dtype, x.dtype)
        return y

    @staticmethod
    def backward(ctx, dy):
        xt, sxt, weight, weight_scale, offsets_dev, padded_dev = ctx.saved_tensors
        groups, t_total, bwd_fp8, grad_dtype, x_dtype = ctx.meta
        dy = dy.contiguous()
        dx = dw = None
        gt = None
        if ctx.needs_input_grad[0]:
            if ctx.needs_input_grad[1] and dy.shape[0]:
                gt, sgt, qg, sg = quantize_transposed_segmented(dy, bwd_fp8, offsets_dev, padded_dev, groups, t_total, rowwise=True)
            else:
                qg, sg = kernels.quantize(dy, bwd_fp8, GX)
            wt = transpose_payload(weight)
            st = weight_scale.transpose(1, 2).contiguous()
            dx = varlen_gemm(qg, wt, sg, st, offsets_dev, out_dtype=x_dtype)
        if ctx.needs_input_grad[1]:
            if gt is None:
                gt, sgt = quantize_transposed_segmented(dy, bwd_fp8, offsets_dev, padded_dev, groups, t_total)
            dw = varlen_wgrad(gt, xt, sgt, sxt, padded_dev, groups, out_dtype=grad_dtype)
        return dx, dw, None, None, None, None, None


def grouped_linear(x, weight, weight_scale, counts, *, forward_dtype="e4m3", backward_dtype="e4m3", grad_dtype=None):
    """y[rows of group g] = x[rows of group g] @ dequant(weight[g]).T for every group, one launch.

    weight [G, N, K] FP8 codes, weight_scale [G, ceil(N/32), ceil(K/32)] fp32, counts: rows per group
    (host list or CPU tensor, sum == x.shape[0])."""
    grad_dtype = grad_dtype or weight.grad_dtype or torch.float32
    return _VarlenLinear.apply(x, weight, weight_scale, counts, _FORMATS[forward_dtype], _FORMATS[backward_dtype], grad_dtype)


class GroupedExperts(nn.Module):
    """`groups` expert weight matrices [out, in] stored as FP8 codes with (32, 32) block scales."""

    def __init__(self, groups, in_features, out_features, *, forward_dtype="e4m3", backward_dtype="e4m3",
                 device=None, dtype=None):
        super().__init__()
        self.groups, self.in_features, self.out_features = groups, in_features, out_features
        self.forward_dtype, self.backward_dtype = forward_dtype, backward_dtype
        policy = settings()
        shape = (groups, out_features, in_features)
        self._initial_weight = torch.empty(shape, device=device, dtype=policy["master_weight_dtype"] or torch.float32)
        self.weight = nn.Parameter(torch.empty(shape, device=device, dtype=_FORMATS[forward_dtype]))
        self.weight.grad_dtype = policy["gradient_dtype"] or torch.float32
        self.register_buffer("weight_scale", torch.ones((groups, *kernels.scale_shape(shape[1:], GW)), device=device,
                                                        dtype=torch.float32))
        self.reset_parameters()

    @torch.no_grad()
    def reset_parameters(self):
        for g in range(self.groups):
            nn.init.kaiming_uniform_(self._initial_weight[g], a=math.sqrt(5))
        self.refresh_weight(self._initial_weight)

    @torch.no_grad()
    def refresh_weight(self, master):
        assert master.is_cuda, "viola_amd kernels run on the GPU only: construct GroupedExperts on the GPU"
        for g in range(self.groups):
            kernels.quantize(master[g], self.weight.dtype, GW, out=self.weight[g], scale_out=self.weight_scale[g])

    def dequantize_weight(self):
        return torch.stack([kernels.dequantize(self.weight[g], self.weight_scale[g], GW) for g in range(self.groups)])

    def forward(self, x, counts):
        assert x.is_cuda, "viola_amd kernels run on the GPU only"
        return grouped_linear(x, self.weight, self.weight_scale, counts, forward_dtype=self.forward_dtype,
                              backward_dtype=self.backward_dtype, grad_dtype=self.weight.grad_dtype)
