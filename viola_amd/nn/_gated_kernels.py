"""Stand-alone elementwise gated activations (operator seam of viola/nn/_gated_kernels.py
`GatedActivation` :121-141): out = act(z[:, :h]) * z[:, h:], and its derivative."""

import torch

from .. import _lib


def gated_forward(z, activation):
    hidden = z.shape[-1] // 2
    flat = z.reshape(-1, 2 * hidden).contiguous()
    out = torch.empty((flat.shape[0], hidden), device=z.device, dtype=z.dtype)
    _lib.call("viola_gated_forward", _lib.ptr(flat), _lib.ptr(out), flat.shape[0], hidden, _lib.code(z.dtype),
              _lib.ACTIVATION[activation])
    return flat, out


def gated_backward(flat, dy, activation):
    hidden = flat.shape[-1] // 2
    dy = dy.reshape(-1, hidden).contiguous()
    dz = torch.empty_like(flat)
    _lib.call("viola_gated_backward", _lib.ptr(flat), _lib.ptr(dy), _lib.ptr(dz), flat.shape[0], hidden,
              _lib.code(flat.dtype), _lib.ACTIVATION[activation])
    return dz


class GatedActivation(torch.autograd.Function):
    @staticmethod
    def forward(ctx, z, activation, autotune=False):
        assert z.is_cuda
        flat, out = gated_forward(z, activation)
        ctx.save_for_backward(flat)
        ctx.shape, ctx.activation = z.shape, activation
        return out.reshape(*z.shape[:-1], out.shape[-1])

    @staticmethod
    def backward(ctx, dy):
        flat, = ctx.saved_tensors
        return gated_backward(flat, dy, ctx.activation).reshape(ctx.shape), None, None
