"""Gated MLP: down(act(gate(x)) * up(x)) with the gating fused into the FP8 GEMMs' epilogues under every scaling
recipe (module surface of viola/nn/mlp.py:76-113; autograd wiring :22-73)."""

import torch
from torch import nn

from .linear import Linear
from . import _grouped_linear, _tensor_linear


def forward_core(x, weight, bias, layer, *args, **kwargs):
    cores = _grouped_linear if layer._grouped_scaling else _tensor_linear
    return cores.forward_core(x, weight, bias, layer, *args, **kwargs)


def backward_core(record, *args, **kwargs):
    cores = _grouped_linear if record.layer._grouped_scaling else _tensor_linear
    return cores.backward_core(record, *args, **kwargs)


class _GateUp(torch.autograd.Function):
    """x -> (h, z): h = act(g) * u is produced by the GEMM epilogue and is not differentiable;
    z = [g, u] carries the gradient between the two projections."""

    @staticmethod
    def forward(ctx, x, weight, bias, layer, activation, need_backward):
        ctx.set_materialize_grads(False)
        h, z, record = forward_core(x, weight, bias, layer, need_backward, ctx.needs_input_grad[:3], gated=activation)
        if record is not None:
            ctx.save_for_backward(*record.tensors)
            record.tensors = None
            ctx.record = record
        if z is None:
            z = h.new_empty((0, 0))
        ctx.mark_non_differentiable(h)
        return h, z

    @staticmethod
    def backward(ctx, unused_dh, dz):
        dx, dw, db = backward_core(ctx.record, ctx.saved_tensors, dz, ctx.needs_input_grad[:3])
        return dx, dw, db, None, None, None


class _Down(torch.autograd.Function):
    """(h, z) -> y. Its backward runs the down projection's dgrad with the activation derivative
    fused, so the gradient it returns is already dz; h never needs a dH buffer."""

    @staticmethod
    def forward(ctx, h, z, weight, bias, layer, activation, need_backward, need_up):
        needs = (need_up, ctx.needs_input_grad[2], ctx.needs_input_grad[3])
        y, _, record = forward_core(h, weight, bias, layer, need_backward, needs)
        if record is not None:
            ctx.save_for_backward(*record.tensors, z)
            record.tensors = None
            ctx.record, ctx.needs, ctx.activation = record, needs, activation
        return y

    @staticmethod
    def backward(ctx, dy):
        *tensors, z = ctx.saved_tensors
        dz, dw, db = backward_core(ctx.record, tensors, dy, ctx.needs, gated=ctx.activation, aux=z)
        if dz is not None:
            dz = dz.reshape(z.shape)
        return None, dz, dw, db, None, None, None, None


class MLP(nn.Module):
    """hidden_features is the width of each branch; gate_up holds [gate; up] stacked on the output
    axis. Linear's storage, FP8 format, scaling and caching options pass through unchanged."""

    def __init__(self, in_features, hidden_features, out_features=None, *, activation="silu",
                 autotune=False, **linear_options):
        super().__init__()
        assert activation in ("silu", "gelu", "relu")
        self.in_features = in_features
        self.hidden_features = hidden_features
        self.out_features = in_features if out_features is None else out_features
        self.activation, self.autotune = activation, autotune
        self.gate_up = Linear(in_features, 2 * hidden_features, autotune=autotune, **linear_options)
        self.down = Linear(hidden_features, self.out_features, autotune=autotune, **linear_options)

    def forward(self, x):
        assert x.is_cuda, "viola.nn.MLP executes on CUDA."
        if torch.is_autocast_enabled("cuda"):
            x = x.to(torch.get_autocast_dtype("cuda"))
        need_backward = torch.is_grad_enabled() and (x.requires_grad or any(p.requires_grad for p in self.parameters()))
        need_up = need_backward and (x.requires_grad or any(p.requires_grad for p in self.gate_up.parameters()))
        shape = x.shape
        h, z = _GateUp.apply(x.reshape(-1, shape[-1]), self.gate_up.weight, self.gate_up.bias, self.gate_up,
                             self.activation, need_up)
        y = _Down.apply(h, z, self.down.weight, self.down.bias, self.down, self.activation, need_backward, need_up)
        return y.reshape(*shape[:-1], y.shape[-1])

    def extra_repr(self):
        return (f"in_features={self.in_features}, hidden_features={self.hidden_features}, "
                f"out_features={self.out_features}, activation={self.activation!r}, autotune={self.autotune}")
