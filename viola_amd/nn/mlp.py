"""Gated MLP: down(act(gate(x)) * up(x)) with the gating fused into the FP8 GEMMs' epilogues under every scaling
recipe (module surface of viola/nn/mlp.py:76-113; autograd wiring :22-73).

Two autograd nodes make up one MLP call. The first runs the stacked [gate; up] projection and returns the hidden
activation h together with z = [g | u]; h comes out of the GEMM's epilogue and carries no gradient, z does. The second
runs the down projection; its backward is the down projection's data-gradient GEMM with the activation's derivative
in the epilogue, so what flows back along z is already dz and no dH buffer ever exists.
"""

from collections import namedtuple

import torch
from torch import nn

from .linear import Linear
from . import _grouped_linear, _tensor_linear

ACTIVATIONS = ("silu", "gelu", "relu")

# How the hidden activation travels between the two nodes: as a tensor of the input's dtype, or (MXFP8, mlp.py:29-33)
# as FP8 codes with their E8M0 scales in both layouts. The three extra slots are empty tensors in the first case.
_Hidden = namedtuple("_Hidden", "value scale transposed transposed_scale")


def _cores(layer):
    return _grouped_linear if layer._grouped_scaling else _tensor_linear


def forward_core(x, weight, bias, layer, *args, **kwargs):
    return _cores(layer).forward_core(x, weight, bias, layer, *args, **kwargs)


def backward_core(record, *args, **kwargs):
    return _cores(record.layer).backward_core(record, *args, **kwargs)


def _keep(ctx, record, *more):
    """Parks a projection's saved tensors in the autograd context and the rest of its record beside them."""
    if record is None:
        return False
    ctx.save_for_backward(*record.tensors, *more)
    record.tensors = None
    ctx.record = record
    return True


class _GateUp(torch.autograd.Function):
    """(layer, activation, plan, x, weight, bias) -> (*hidden, z); plan = (save for backward, hand h over as codes,
    with the transposed codes too)."""

    @staticmethod
    def forward(ctx, layer, activation, plan, x, weight, bias):
        save, as_codes, with_transpose = plan
        ctx.set_materialize_grads(False)
        ctx.wanted = ctx.needs_input_grad[3:6]
        extra = {"encode": (True, with_transpose)} if as_codes else {}
        h, z, record = forward_core(x, weight, bias, layer, save, ctx.wanted, gated=activation, **extra)
        _keep(ctx, record)
        if as_codes:
            hidden = _Hidden(*h)
        else:
            hidden = _Hidden(h, *(h.new_empty((0, 0), dtype=torch.uint8) for _ in range(3)))
        ctx.mark_non_differentiable(*hidden)
        return (*hidden, x.new_empty((0, 0)) if z is None else z)

    @staticmethod
    def backward(ctx, *gradients):
        dz = gradients[-1]                                                    # the four hidden slots carry none
        dx, dw, db = backward_core(ctx.record, ctx.saved_tensors, dz, ctx.wanted)
        return None, None, None, dx, dw, db


class _Down(torch.autograd.Function):
    """(layer, activation, plan, input dtype, z, weight, bias, *hidden) -> y; plan = (save for backward, the gate/up
    side wants dz)."""

    @staticmethod
    def forward(ctx, layer, activation, plan, input_dtype, z, weight, bias, *hidden):
        save, wants_dz = plan
        hidden = _Hidden(*hidden)
        ctx.wanted = (wants_dz, ctx.needs_input_grad[5], ctx.needs_input_grad[6])
        extra = {}
        if hidden.scale.numel():
            extra = {"encoded": (hidden.scale, hidden.transposed, hidden.transposed_scale), "input_dtype": input_dtype}
        y, _, record = forward_core(hidden.value, weight, bias, layer, save, ctx.wanted, **extra)
        if _keep(ctx, record, z):
            ctx.activation = activation
        return y

    @staticmethod
    def backward(ctx, dy):
        *saved, z = ctx.saved_tensors
        dz, dw, db = backward_core(ctx.record, saved, dy, ctx.wanted, gated=ctx.activation, aux=z)
        return (None, None, None, None, None if dz is None else dz.reshape(z.shape), dw, db, None, None, None, None)


def _trains(module):
    return any(p.requires_grad for p in module.parameters())


class MLP(nn.Module):
    """hidden_features is the width of each branch; gate_up holds [gate; up] stacked on the output
    axis. Linear's storage, FP8 format, scaling and caching options pass through unchanged."""

    def __init__(self, in_features, hidden_features, out_features=None, *, activation="silu",
                 autotune=False, **linear_options):
        super().__init__()
        if activation not in ACTIVATIONS:
            raise AssertionError(f"activation must be one of {ACTIVATIONS}")
        widths = dict(in_features=in_features, hidden_features=hidden_features,
                      out_features=in_features if out_features is None else out_features)
        for name, width in widths.items():
            setattr(self, name, width)
        self.activation = activation
        self.autotune = autotune
        shared = dict(linear_options, autotune=autotune)
        self.gate_up = Linear(widths["in_features"], 2 * widths["hidden_features"], **shared)
        self.down = Linear(widths["hidden_features"], widths["out_features"], **shared)

    def _hands_over_codes(self):
        """MXFP8 with (1, 32) input groups and FP8-saved inputs: h goes from the gate/up GEMM to the down projection as
        codes and scales, never as a 16-bit tensor (mlp.py:103-107)."""
        down = self.down
        return bool(down._native_scaling) and down.input_group_shape == (1, 32) and down.saved_input_dtype == "fp8"

    def forward(self, x):
        assert x.is_cuda, "viola.nn.MLP executes on CUDA."
        if torch.is_autocast_enabled("cuda"):
            x = x.to(torch.get_autocast_dtype("cuda"))
        recording = torch.is_grad_enabled()
        first_half = recording and (x.requires_grad or _trains(self.gate_up))      # anything upstream of z wants a gradient
        whole = recording and (first_half or _trains(self.down))
        as_codes = self._hands_over_codes()
        leading = x.shape[:-1]
        *hidden, z = _GateUp.apply(self.gate_up, self.activation,
                                   (first_half, as_codes, as_codes and whole and self.down.weight.requires_grad),
                                   x.reshape(-1, x.shape[-1]), self.gate_up.weight, self.gate_up.bias)
        y = _Down.apply(self.down, self.activation, (whole, first_half), x.dtype, z, self.down.weight, self.down.bias, *hidden)
        return y.reshape(*leading, y.shape[-1])

    def extra_repr(self):
        shown = {name: getattr(self, name) for name in ("in_features", "hidden_features", "out_features")}
        shown["activation"] = repr(self.activation)
        shown["autotune"] = self.autotune
        return ", ".join(f"{name}={value}" for name, value in shown.items())
