"""FP8 Linear with FP8 / BF16 / FP16 weight storage (module surface of viola/nn/linear.py:150-412).

Built here: `scaling="grouped"` (FP32 scales per 2-D weight block and per 1-D activation /
gradient tile), `scaling="mxfp8"` (the same groups with E8M0 power-of-two scales, GEMMs on the block-scaled
MFMA) and the per-tensor recipes `scaling="current"` / `"delayed"` (one FP32 scale per tensor,
delayed = the maximum of an amax history), e4m3 / e5m2 operand formats.

Accumulation: `accum_dtype="fp16"` (with `accum_block_size`, `accum_reduce_dtype`) is the reference's ablation of
narrow accumulators. The quantization limits it implies (linear.py:232-253) are applied, so codes and scales are the
ones the reference stores, and the GEMMs follow the FP16-accumulator model of its kernels: FP16 partial sums advanced
every 32 k, cleared into an FP32 or BF16 total per scale group / accumulation block. The FP8 MFMA of gfx950 sums in
FP32, so the model runs on the generic kernel with explicit roundings; with `accum_dtype="fp32"` the other two options
change nothing. `rotation_size=64` (per-tensor recipes only) stores and multiplies Hadamard-rotated X and W.

How the module is put together: `_Numerics` checks the recipe options once and answers every question about clamp
limits and scale storage; `_WeightStore` turns a master weight into what the module stores (codes, scales, the cached
transpose) on the GPU; `Linear` itself owns the parameters and buffers under the names a checkpoint of the reference
carries, and keeps their dtypes through module-wide casts.
"""

import math

import torch
from torch import nn

from . import _grouped_kernels as grouped
from . import _linear_kernels as kernels
from . import _rotation_kernels as rotation
from ..precision import settings

_FORMATS = {"e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2}
_STORAGE = {"bf16": torch.bfloat16, "fp16": torch.float16}
_HOST_MASTER = ("The FP8 weight has not been quantized yet: its master is still on the host. Move the model to the GPU "
                "before binding an optimizer (the quantizer runs on the GPU only).")


class _Quantizer(nn.Module):
    """Amax history and call counter of one per-tensor-scaled operand (viola/nn/linear.py:14-33); the grouped
    recipe never advances it, but its state_dict carries the same keys."""

    def __init__(self, scaling, history_len, device):
        super().__init__()
        self.scaling, self.index = scaling, 0
        self.register_buffer("history", torch.zeros(history_len, device=device, dtype=torch.float32))

    def _options(self, fp8_dtype, quantization_limit):
        return dict(history=self.history, index=self.index, delayed=self.scaling == "delayed", fp8_dtype=fp8_dtype,
                    quantization_limit=quantization_limit)

    def scale(self, x, fp8_dtype=torch.float8_e4m3fn, quantization_limit=None, rotation_size=0):
        scale = (rotation if rotation_size else kernels).tensor_scale(x, **self._options(fp8_dtype, quantization_limit))
        self.index += 1
        return scale

    def scale_and_column_sum(self, x, sum_dtype, fp8_dtype=torch.float8_e4m3fn, quantization_limit=None):
        """scale(x) and x.sum(0) from one read of the matrix x."""
        result = kernels.tensor_scale_and_column_sum(x, sum_dtype, **self._options(fp8_dtype, quantization_limit))
        self.index += 1
        return result

    def get_extra_state(self):
        return {"index": self.index, "scaling": self.scaling}

    def set_extra_state(self, state):
        self.index, self.scaling = state["index"], state["scaling"]


def _half_sum_limit(reduction):
    """Largest power of two L with reduction * L * L <= 32768: `reduction` products of two codes of
    magnitude <= L then sum to at most half of FP16's range (linear.py:237-241, :250-253)."""
    return 2.0 ** math.floor(math.log2(math.sqrt(32768.0 / reduction)))


class _Numerics:
    """The arithmetic options of one Linear, validated together (the assertions of linear.py:169-200)."""

    FIELDS = ("forward_dtype", "backward_dtype", "fp8_dtype", "backward_fp8_dtype", "_grouped_scaling", "_native_scaling",
              "weight_group_shape", "input_group_shape", "grad_group_shape", "accum_dtype", "accum_block_size",
              "accum_reduce_dtype", "quantization_limit", "rotation_size")

    def __init__(self, in_features, scaling, forward_dtype, backward_dtype, accum_dtype, accum_block_size, accum_reduce_dtype,
                 quantization_limit, rotation_size, weight_group_shape, input_group_shape, grad_group_shape):
        assert scaling in ("current", "delayed", "grouped", "mxfp8")
        assert accum_dtype in ("fp32", "fp16") and accum_reduce_dtype in ("fp32", "bf16")
        assert accum_block_size >= 0 and accum_block_size % 32 == 0 and rotation_size in (0, 64)
        assert not rotation_size or in_features % rotation_size == 0
        self.forward_dtype, self.backward_dtype = forward_dtype, backward_dtype
        self.fp8_dtype, self.backward_fp8_dtype = _FORMATS[forward_dtype], _FORMATS[backward_dtype]
        self._native_scaling = scaling == "mxfp8"
        self._grouped_scaling = self._native_scaling or scaling == "grouped"
        groups = [tuple(weight_group_shape), tuple(input_group_shape), tuple(grad_group_shape)]
        self.weight_group_shape, self.input_group_shape, self.grad_group_shape = groups
        for rows, cols in groups:
            assert all(side > 0 and side & (side - 1) == 0 for side in (rows, cols)) and cols >= 32
        if self._grouped_scaling:
            assert rotation_size == 0, "Grouped scaling does not combine with rotation_size."
        if self._native_scaling:
            assert (accum_dtype, accum_block_size, accum_reduce_dtype) == ("fp32", 0, "fp32"), "MXFP8 MMA uses FP32 accumulation."
        self.accum_dtype, self.accum_block_size, self.accum_reduce_dtype = accum_dtype, accum_block_size, accum_reduce_dtype
        self.quantization_limit, self.rotation_size = quantization_limit, rotation_size

    def _clamp(self, reduction, dtype):
        """Clamp magnitude when `reduction` code products meet in one FP16 partial sum; None = the format's maximum."""
        largest = torch.finfo(dtype).max
        if self.quantization_limit is not None:
            return min(self.quantization_limit, largest)
        return None if self.accum_dtype == "fp32" else min(_half_sum_limit(reduction), largest)

    def group_limit(self, shape, dtype, weight=False):
        # a weight block is reduced along either of its sides (forward and dgrad); linear.py:244-253
        reduction = max(shape) if weight else shape[1]
        return self._clamp(math.gcd(reduction, self.accum_block_size) if self.accum_block_size else reduction, dtype)

    def tensor_limit(self, reduction, dtype):
        return self._clamp(self.accum_block_size or reduction, dtype)                      # linear.py:232-242

    def scale_storage(self, weight_shape, fp8_storage):
        """(shape, dtype, initial value) of `weight_scale`: FP32 scales start at 1, E8M0 bytes at 127 = 2^0
        (linear.py:218-226); without FP8 storage the buffer is empty."""
        if self._grouped_scaling:
            shape = grouped.scale_shape(weight_shape, self.weight_group_shape) if fp8_storage else (0, 0)
        else:
            shape = (1,) if fp8_storage else (0,)
        return (shape, torch.uint8, 127) if self._native_scaling else (shape, torch.float32, 1)


class _WeightStore:
    """Derives what a Linear stores from a master weight: FP8 codes + scales (+ the cached transpose), or a plain
    copy for BF16 / FP16 storage. The quantizers exist on the GPU only, so a master that is still on the host is
    remembered (`pending`) and encoded when the module arrives on the GPU."""

    def __init__(self, layer):
        self.pending = False
        self._layer = layer                                                    # plain attribute: not a submodule

    def encode(self, master):
        layer = self._layer
        if layer.weight_dtype != "fp8":
            if master is not layer.weight:
                layer.weight.copy_(master)
            return
        self.pending = not master.is_cuda
        if self.pending:
            return
        if layer._grouped_scaling:
            limit = layer._group_limit(layer.weight_group_shape, layer.fp8_dtype, weight=True)
            grouped.quantize(master, layer.fp8_dtype, layer.weight_group_shape, limit=limit, native=layer._native_scaling,
                             out=layer.weight, scale_out=layer.weight_scale)
            if layer.cache_weight_transpose:
                self.transpose(limit)
            return
        # one scale for the tensor; the transposed codes, when cached, come from the same read (linear.py:288-297)
        limit = layer._quantization_limit(max(layer.in_features, layer.out_features), layer.fp8_dtype)
        transposed = None
        if layer.cache_weight_transpose:
            if layer.weight_transpose.numel() == 0:
                layer.weight_transpose = layer.weight.new_empty((layer.in_features, layer.out_features))
            transposed = layer.weight_transpose
        scale = layer.weight_quantizer.scale(master, layer.fp8_dtype, limit, layer.rotation_size)
        layer.weight_scale.copy_(scale)
        (rotation if layer.rotation_size else kernels).quantize(master, scale, transpose=transposed is not None,
                                                                 fp8_dtype=layer.fp8_dtype, out=layer.weight, out_t=transposed,
                                                                 quantization_limit=limit)

    def transpose(self, limit=None):
        """W^T from the stored codes and scales, without requantizing W."""
        layer = self._layer
        if layer._grouped_scaling:
            layer.weight_transpose, layer.weight_transpose_scale = grouped.transpose(
                layer.weight, layer.weight_scale, layer.weight_group_shape, native=layer._native_scaling, limit=limit)
        else:
            layer.weight_transpose = kernels.transpose(layer.weight)

    def decode(self):
        layer = self._layer
        if layer.weight_dtype != "fp8":
            return layer.weight.float()
        assert layer.weight.is_cuda, "viola_amd kernels run on the GPU only"
        if layer._grouped_scaling:
            return grouped.dequantize(layer.weight, layer.weight_scale, layer.weight_group_shape)
        real = layer.weight.float() * layer.weight_scale
        return rotation.inverse_(real) if layer.rotation_size else real         # back to the original coordinates


def _destination(fn, tensor):
    """The device a module-wide `_apply` function sends `tensor` to, found by handing it an empty FP32 tensor from the
    same device (the function may also cast floating dtypes, which is exactly what must not reach FP8 codes and scales)."""
    return fn(torch.empty(0, device=tensor.device)).device


class Linear(nn.Module):
    """y = x W^T + b computed with FP8 GEMMs on the GPU; inputs/outputs are ordinary BF16/FP16/FP32.

    weight_dtype selects FP8 codes (+ FP32 block scales in `weight_scale`) or BF16/FP16 real
    weights as storage; dequantize_weight() returns real weights in the original coordinates.
    """

    _KEPT_BUFFERS = ("weight_scale", "weight_transpose", "weight_transpose_scale")

    def __init__(self, in_features, out_features, bias=True, *, mode="memory", weight_dtype="fp8",
                 forward_dtype="e4m3", backward_dtype="e5m2", cache_weight_transpose=None,
                 saved_input_dtype="fp8", scaling="current", history_len=16, autotune=False,
                 accum_dtype="fp32", accum_block_size=0, accum_reduce_dtype="fp32", quantization_limit=None,
                 rotation_size=0, weight_group_shape=(32, 32), input_group_shape=(1, 32),
                 grad_group_shape=(1, 32), device=None, dtype=None):
        super().__init__()
        assert mode in ("memory", "fast") and weight_dtype in ("fp8", "bf16", "fp16")
        assert saved_input_dtype in ("fp8", "bf16", "fp16", "fp32") and history_len > 0
        numerics = _Numerics(in_features, scaling, forward_dtype, backward_dtype, accum_dtype, accum_block_size,
                             accum_reduce_dtype, quantization_limit, rotation_size, weight_group_shape,
                             input_group_shape, grad_group_shape)
        self._numerics = numerics
        for field in _Numerics.FIELDS:                                         # the attributes the autograd functions read
            setattr(self, field, getattr(numerics, field))
        self.in_features, self.out_features = in_features, out_features
        self.mode, self.weight_dtype, self.saved_input_dtype, self.autotune = mode, weight_dtype, saved_input_dtype, autotune
        self.cache_weight_transpose = (mode == "fast") if cache_weight_transpose is None else cache_weight_transpose
        self._store = _WeightStore(self)
        self._master_ref = None
        self._allocate(bias, device, dtype or torch.get_default_dtype(), settings())
        for operand in ("weight", "input", "grad"):
            setattr(self, f"{operand}_quantizer", _Quantizer(scaling, history_len, device))
        self.reset_parameters()

    def _allocate(self, bias, device, dtype, policy):
        """Parameters and buffers under the reference's names (linear.py:203-226). With FP8 storage the initial
        values live in a master-precision tensor that the optimizer binding takes over; BF16 / FP16 storage
        initialises the parameter itself."""
        shape = (self.out_features, self.in_features)
        fp8_storage = self.weight_dtype == "fp8"
        on = dict(device=device)
        self._initial_weight = torch.empty(shape, dtype=policy["master_weight_dtype"] or torch.float32, **on) if fp8_storage else None
        self.weight = nn.Parameter(torch.empty(shape, dtype=self.fp8_dtype if fp8_storage else _STORAGE[self.weight_dtype], **on))
        self.bias = nn.Parameter(torch.empty(self.out_features, dtype=dtype, **on)) if bias else None
        self._set_grad_dtype(policy["gradient_dtype"] or torch.float32)
        scale_shape, scale_dtype, one = self._numerics.scale_storage(shape, fp8_storage)
        self.register_buffer("weight_scale", torch.full(scale_shape, one, dtype=scale_dtype, **on), persistent=fp8_storage)
        self.register_buffer("weight_transpose", torch.empty(0, 0, dtype=self.fp8_dtype, **on), persistent=False)
        self.register_buffer("weight_transpose_scale", torch.empty(0, 0, dtype=scale_dtype, **on), persistent=False)

    def _set_grad_dtype(self, grad_dtype):
        for parameter in (self.weight, self.bias):
            if parameter is not None:
                parameter.grad_dtype = grad_dtype

    @property
    def _pending_refresh(self):
        return self._store.pending

    # ------------------------------------------------------------------ quantization policy
    def _group_limit(self, shape, dtype, weight=False):
        """Clamp magnitude for a group; None means the format's own maximum (linear.py:244-253)."""
        return self._numerics.group_limit(shape, dtype, weight)

    def _quantization_limit(self, reduction, fp8_dtype):
        """Clamp magnitude of a per-tensor-scaled operand; None means the format's own maximum (linear.py:232-242)."""
        return self._numerics.tensor_limit(reduction, fp8_dtype)

    def _accumulation(self):
        return dict(accum_dtype=self.accum_dtype, accum_block_size=self.accum_block_size, accum_reduce_dtype=self.accum_reduce_dtype)

    def _group_gemm(self, a, b, sa, sb, ga, gb, *, out_dtype, bias=None):
        return grouped.gemm(a, b, sa, sb, ga, gb, out_dtype=out_dtype, bias=bias, native=self._native_scaling, **self._accumulation())

    def _tensor_gemm(self, a, b, sa, sb, *, out_dtype, bias=None):
        return kernels.gemm(a, b, sa, sb, out_dtype=out_dtype, bias=bias, **self._accumulation())

    # ------------------------------------------------------------------ weights
    def _master(self):
        """The tensor the stored weight is derived from: the bound optimizer's master, else the initial values (FP8
        storage) or the parameter itself."""
        if self._master_ref is not None:
            return self._master_ref()
        return self._initial_weight if self.weight_dtype == "fp8" else self.weight

    @torch.no_grad()
    def reset_parameters(self):
        master = self._master()
        nn.init.kaiming_uniform_(master, a=math.sqrt(5))
        if self.bias is not None:
            spread = 1 / math.sqrt(self.in_features)
            self.bias.uniform_(-spread, spread)
        self.refresh_weight(master)

    @torch.no_grad()
    def refresh_weight(self, master):
        """Re-derive the stored weight from an updated master (called after each optimizer step)."""
        self._store.encode(master)

    def dequantize_weight(self):
        return self._store.decode()

    @classmethod
    @torch.no_grad()
    def from_float(cls, linear, **kwargs):
        """An FP8 Linear holding the weights of a torch.nn.Linear (linear.py:324-340)."""
        source_bias = linear.bias
        layer = cls(linear.in_features, linear.out_features, source_bias is not None, device=linear.weight.device,
                    dtype=linear.weight.dtype, **kwargs)
        # the amax history must describe the loaded weight, not the initialiser that was quantized a moment ago
        layer.weight_quantizer.index = 0
        layer.weight_quantizer.history.zero_()
        layer.refresh_weight(layer._master().copy_(linear.weight))
        for ours, theirs in ((layer.weight, linear.weight), (layer.bias, source_bias)):
            if theirs is not None:
                ours.requires_grad_(theirs.requires_grad)
        if source_bias is not None:
            layer.bias.copy_(source_bias)
        return layer

    # ------------------------------------------------------------------ execution
    def forward(self, x):
        assert x.is_cuda, "viola.nn.Linear executes on CUDA."
        if torch.is_autocast_enabled("cuda"):
            x = x.to(torch.get_autocast_dtype("cuda"))
        if self._store.pending:
            self.refresh_weight(self._master())
            assert not self._store.pending, _HOST_MASTER
        trainable = [t for t in (x, self.weight, self.bias) if t is not None and t.requires_grad]
        need_backward = torch.is_grad_enabled() and bool(trainable)
        if self._grouped_scaling:
            from ._grouped_linear import GroupedLinear as function
        else:
            from ._tensor_linear import TensorLinear as function
        return function.apply(x, self.weight, self.bias, self, need_backward)

    # ------------------------------------------------------------------ module plumbing
    def _kept(self):
        """(owner dict, key) of every tensor that `.to()` / `.cuda()` / `.bfloat16()` may move but never cast: the
        weight (FP8 codes or its chosen storage dtype), the scales and cached transpose, the amax histories
        (linear.py:355-380)."""
        slots = [(self._parameters, "weight")] + [(self._buffers, name) for name in self._KEPT_BUFFERS]
        return slots + [(q._buffers, "history") for q in (self.weight_quantizer, self.input_quantizer, self.grad_quantizer)]

    def _apply(self, fn, recurse=True):
        slots = self._kept()
        held = [owner[key] for owner, key in slots]
        grad_dtype = held[0].grad_dtype
        for owner, key in slots:
            owner[key] = None                                                  # out of sight of the generic walk
        try:
            super()._apply(fn, recurse)                                        # the bias (and nothing else) follows casts
        finally:
            for (owner, key), tensor in zip(slots, held):
                owner[key] = tensor
        for (owner, key), tensor in zip(slots, held):
            device = _destination(fn, tensor)
            if isinstance(tensor, nn.Parameter):                               # the same Parameter object, relocated
                tensor.data = tensor.data.to(device)
                if tensor.grad is not None:
                    tensor.grad = tensor.grad.to(device)
            else:
                owner[key] = tensor.to(device)
        if self._initial_weight is not None:
            self._initial_weight = self._initial_weight.to(_destination(fn, self._initial_weight))
        self._set_grad_dtype(grad_dtype)
        master = self._master()
        if self._store.pending and master is not None and master.is_cuda and self.weight.is_cuda:
            self.refresh_weight(master)                                        # built on the host, now on the GPU
        return self

    def _save_to_state_dict(self, destination, prefix, keep_vars):
        assert not self._store.pending, \
            "This Linear was built on the host and its FP8 codes do not exist yet: move it to the GPU before saving."
        super()._save_to_state_dict(destination, prefix, keep_vars)

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        stored = state_dict[prefix + "weight"].dtype
        assert stored == self.weight.dtype, "Construct Linear with the checkpoint's weight storage and FP8 format."
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)
        # the checkpoint's codes are the weight now: neither the initial values nor a deferred encode apply any more
        self._initial_weight, self._store.pending = None, False
        self.rebuild_weight_cache()

    @torch.no_grad()
    def rebuild_weight_cache(self):
        """Rebuild W^T from the loaded codes and scales without requantizing W."""
        if self.cache_weight_transpose and self.weight_dtype == "fp8" and self.weight.is_cuda:
            grouped_limit = self._group_limit(self.weight_group_shape, self.fp8_dtype, weight=True) if self._grouped_scaling else None
            self._store.transpose(grouped_limit)

    def extra_repr(self):
        shown = dict(in_features=self.in_features, out_features=self.out_features, bias=self.bias is not None, mode=self.mode,
                     weight_dtype=self.weight_dtype, forward_dtype=self.forward_dtype, backward_dtype=self.backward_dtype,
                     cache_weight_transpose=self.cache_weight_transpose, saved_input_dtype=self.saved_input_dtype,
                     scaling=self.weight_quantizer.scaling, accum_dtype=self.accum_dtype, accum_block_size=self.accum_block_size,
                     accum_reduce_dtype=self.accum_reduce_dtype, rotation_size=self.rotation_size,
                     weight_group_shape=self.weight_group_shape, input_group_shape=self.input_group_shape,
                     grad_group_shape=self.grad_group_shape)
        return ", ".join(f"{name}={value!r}" for name, value in shown.items())
