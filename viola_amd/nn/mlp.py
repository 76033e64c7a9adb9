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
    def forward(ctx, x, weight, bias, layer, activation, need_backward, encode_output, encode_transpose):
        ctx.set_materialize_grads(False)
        options = dict(encode=(True, encode_transpose)) if encode_output else {}
        h, z, record = forward_core(x, weight, bias, layer, need_backward, ctx.needs_input_grad[:3], gated=activation, **options)
        if record is not None:
            ctx.save_for_backward(*record.tensors)
            record.tensors = None
            ctx.record = record
        if encode_output:
            h, scale, ht, st = h                                              # MXFP8 codes of h in both layouts (mlp.py:29-33)
        else:
            scale, ht, st = (h.new_empty((0, 0), dtype=torch.uint8) for _ in range(3))
        if z is None:
            z = x.new_empty((0, 0))
        ctx.mark_non_differentiable(h, scale, ht, st)
        return h, scale, ht, st, z

    @staticmethod
    def backward(ctx, unused_dh, unused_ds, unused_dht, unused_dst, dz):
        dx, dw, db = backward_core(ctx.record, ctx.saved_tensors, dz, ctx.needs_input_grad[:3])
        return dx, dw, db, None, None, None, None, None


class _Down(torch.autograd.Function):
    """(h, z) -> y. Its backward runs the down projection's dgrad with the activation derivative
    fused, so the gradient it returns is already dz; h never needs a dH buffer."""

    @staticmethod
    def forward(ctx, h, scale, ht, st, z, weight, bias, layer, activation, need_backward, need_up, input_dtype):
        needs = (need_up, ctx.needs_input_grad[5], ctx.needs_input_grad[6])
        options = dict(encoded=(scale, ht, st), input_dtype=input_dtype) if scale.numel() else {}
        y, _, record = forward_core(h, weight, bias, layer, need_backward, needs, **options)
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
        return None, None, None, None, dz, dw, db, None, None, None, None, None


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
        # MXFP8 with (1, 32) input groups and FP8-saved inputs: h goes from the gate/up GEMM to the down projection as
        # codes and scales, never as a BF16 tensor (mlp.py:103-107)
        encode = self.down._native_scaling and self.down.input_group_shape == (1, 32) and self.down.saved_input_dtype == "fp8"
        h, scale, ht, st, z = _GateUp.apply(x.reshape(-1, shape[-1]), self.gate_up.weight, self.gate_up.bias, self.gate_up,
                                            self.activation, need_up, encode,
                                            encode and need_backward and self.down.weight.requires_grad)
        y = _Down.apply(h, scale, ht, st, z, self.down.weight, self.down.bias, self.down, self.activation, need_backward,
                        need_up, x.dtype)
        return y.reshape(*shape[:-1], y.shape[-1])

    def extra_repr(self):
        return (f"in_features={self.in_features}, hidden_features={self.hidden_features}, "
                f"out_features={self.out_features}, activation={self.activation!r}, autotune={self.autotune}")
