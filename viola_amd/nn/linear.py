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


class _Quantizer(nn.Module):
    """Amax history and call counter of one per-tensor-scaled operand (viola/nn/linear.py:14-33); the grouped
    recipe never advances it, but its state_dict carries the same keys."""

    def __init__(self, scaling, history_len, device):
        super().__init__()
        self.scaling, self.index = scaling, 0
        self.register_buffer("history", torch.zeros(history_len, device=device, dtype=torch.float32))

    def scale(self, x, fp8_dtype=torch.float8_e4m3fn, quantization_limit=None, rotation_size=0):
        implementation = rotation if rotation_size else kernels
        scale = implementation.tensor_scale(x, history=self.history, index=self.index, delayed=self.scaling == "delayed",
                                            fp8_dtype=fp8_dtype, quantization_limit=quantization_limit)
        self.index += 1
        return scale

    def scale_and_column_sum(self, x, sum_dtype, fp8_dtype=torch.float8_e4m3fn, quantization_limit=None):
        """scale(x) and x.sum(0) from one read of the matrix x."""
        result = kernels.tensor_scale_and_column_sum(x, sum_dtype, history=self.history, index=self.index,
                                                     delayed=self.scaling == "delayed", fp8_dtype=fp8_dtype,
                                                     quantization_limit=quantization_limit)
        self.index += 1
        return result

    def get_extra_state(self):
        return {"index": self.index, "scaling": self.scaling}

    def set_extra_state(self, state):
        self.index, self.scaling = state["index"], state["scaling"]


def _pow2(v):
    return v > 0 and v & (v - 1) == 0


def _half_sum_limit(reduction):
    """Largest power of two L with reduction * L * L <= 32768: `reduction` products of two codes of
    magnitude <= L then sum to at most half of FP16's range (linear.py:237-241, :250-253)."""
    return 2.0 ** math.floor(math.log2(math.sqrt(32768.0 / reduction)))


class Linear(nn.Module):
    """y = x W^T + b computed with FP8 GEMMs on the GPU; inputs/outputs are ordinary BF16/FP16/FP32.

    weight_dtype selects FP8 codes (+ FP32 block scales in `weight_scale`) or BF16/FP16 real
    weights as storage; dequantize_weight() returns real weights in the original coordinates.
    """

    def __init__(self, in_features, out_features, bias=True, *, mode="memory", weight_dtype="fp8",
                 forward_dtype="e4m3", backward_dtype="e5m2", cache_weight_transpose=None,
                 saved_input_dtype="fp8", scaling="current", history_len=16, autotune=False,
                 accum_dtype="fp32", accum_block_size=0, accum_reduce_dtype="fp32", quantization_limit=None,
                 rotation_size=0, weight_group_shape=(32, 32), input_group_shape=(1, 32),
                 grad_group_shape=(1, 32), device=None, dtype=None):
        super().__init__()
        assert mode in ("memory", "fast") and weight_dtype in ("fp8", "bf16", "fp16")
        assert saved_input_dtype in ("fp8", "bf16", "fp16", "fp32")
        assert scaling in ("current", "delayed", "grouped", "mxfp8") and history_len > 0
        assert accum_dtype in ("fp32", "fp16") and accum_reduce_dtype in ("fp32", "bf16")
        assert accum_block_size >= 0 and accum_block_size % 32 == 0 and rotation_size in (0, 64)

        assert not rotation_size or in_features % rotation_size == 0
        if scaling in ("grouped", "mxfp8"):
            assert rotation_size == 0, "Grouped scaling does not combine with rotation_size."
        if scaling == "mxfp8":
            assert accum_dtype == "fp32" and accum_block_size == 0 and accum_reduce_dtype == "fp32", "MXFP8 MMA uses FP32 accumulation."
        self.in_features, self.out_features = in_features, out_features
        self.mode, self.weight_dtype, self.saved_input_dtype = mode, weight_dtype, saved_input_dtype
        self.forward_dtype, self.backward_dtype = forward_dtype, backward_dtype
        self.fp8_dtype, self.backward_fp8_dtype = _FORMATS[forward_dtype], _FORMATS[backward_dtype]
        self._grouped_scaling, self._native_scaling = scaling in ("grouped", "mxfp8"), scaling == "mxfp8"
        self.weight_group_shape = tuple(weight_group_shape)
        self.input_group_shape = tuple(input_group_shape)
        self.grad_group_shape = tuple(grad_group_shape)
        for gr, gc in (self.weight_group_shape, self.input_group_shape, self.grad_group_shape):
            assert _pow2(gr) and _pow2(gc) and gc >= 32
        self.autotune = autotune
        self.accum_dtype, self.accum_block_size, self.accum_reduce_dtype = accum_dtype, accum_block_size, accum_reduce_dtype
        self.quantization_limit, self.rotation_size = quantization_limit, rotation_size
        self.cache_weight_transpose = (mode == "fast") if cache_weight_transpose is None else cache_weight_transpose
        policy = settings()
        gradient_dtype = policy["gradient_dtype"] or torch.float32
        dtype = dtype or torch.get_default_dtype()
        shape = (out_features, in_features)
        fp8_storage = weight_dtype == "fp8"
        # FP8 storage: the initialiser lives in a master-precision tensor that the optimizer binding
        # takes over; BF16/FP16 storage initialises the parameter itself.
        self._initial_weight = (torch.empty(shape, device=device, dtype=policy["master_weight_dtype"] or torch.float32)
                                if fp8_storage else None)
        self._master_ref = None
        self._pending_refresh = False
        self.weight = nn.Parameter(torch.empty(shape, device=device, dtype=self.fp8_dtype if fp8_storage else _STORAGE[weight_dtype]))
        self.weight.grad_dtype = gradient_dtype
        self.bias = nn.Parameter(torch.empty(out_features, device=device, dtype=dtype)) if bias else None
        if self.bias is not None:
            self.bias.grad_dtype = gradient_dtype
        if self._grouped_scaling:
            scale_shape = grouped.scale_shape(shape, self.weight_group_shape) if fp8_storage else (0, 0)
        else:
            scale_shape = (1,) if fp8_storage else (0,)
        # FP32 scales start at 1, E8M0 bytes at 127 = 2^0 (linear.py:221-226)
        scale_dtype = torch.uint8 if self._native_scaling else torch.float32
        self.register_buffer("weight_scale", torch.full(scale_shape, 127 if self._native_scaling else 1, device=device, dtype=scale_dtype),
                             persistent=fp8_storage)
        self.register_buffer("weight_transpose", torch.empty(0, 0, device=device, dtype=self.fp8_dtype), persistent=False)
        self.register_buffer("weight_transpose_scale", torch.empty(0, 0, device=device, dtype=scale_dtype), persistent=False)
        self.weight_quantizer = _Quantizer(scaling, history_len, device)
        self.input_quantizer = _Quantizer(scaling, history_len, device)
        self.grad_quantizer = _Quantizer(scaling, history_len, device)
        self.reset_parameters()

    # ------------------------------------------------------------------ quantization policy
    def _group_limit(self, shape, dtype, weight=False):
        """Clamp magnitude for a group; None means the format's own maximum (linear.py:244-253)."""
        if self.quantization_limit is not None:
            return min(self.quantization_limit, torch.finfo(dtype).max)
        if self.accum_dtype == "fp32":
            return None
        # a weight block is reduced along either of its sides (forward and dgrad)
        reduction = max(shape) if weight else shape[1]
        if self.accum_block_size:
            reduction = math.gcd(reduction, self.accum_block_size)
        return min(_half_sum_limit(reduction), torch.finfo(dtype).max)

    def _quantization_limit(self, reduction, fp8_dtype):
        """Clamp magnitude of a per-tensor-scaled operand; None means the format's own maximum (linear.py:232-242)."""
        if self.quantization_limit is not None:
            return min(self.quantization_limit, torch.finfo(fp8_dtype).max)
        if self.accum_dtype == "fp32":
            return None
        return min(_half_sum_limit(self.accum_block_size or reduction), torch.finfo(fp8_dtype).max)

    def _group_gemm(self, a, b, sa, sb, ga, gb, *, out_dtype, bias=None):
        return grouped.gemm(a, b, sa, sb, ga, gb, out_dtype=out_dtype, bias=bias, native=self._native_scaling,
                            accum_dtype=self.accum_dtype, accum_block_size=self.accum_block_size,
                            accum_reduce_dtype=self.accum_reduce_dtype)

    def _tensor_gemm(self, a, b, sa, sb, *, out_dtype, bias=None):
        return kernels.gemm(a, b, sa, sb, out_dtype=out_dtype, bias=bias, accum_dtype=self.accum_dtype,
                            accum_block_size=self.accum_block_size, accum_reduce_dtype=self.accum_reduce_dtype)

    # ------------------------------------------------------------------ weights
    def _master(self):
        if self._master_ref is not None:
            return self._master_ref()
        return self.weight if self.weight_dtype != "fp8" else self._initial_weight

    @torch.no_grad()
    def reset_parameters(self):
        master = self._master()
        nn.init.kaiming_uniform_(master, a=math.sqrt(5))
        if self.bias is not None:
            bound = 1 / math.sqrt(self.in_features)
            nn.init.uniform_(self.bias, -bound, bound)
        self.refresh_weight(master)

    @torch.no_grad()
    def refresh_weight(self, master):
        """Re-derive the stored weight from an updated master (called after each optimizer step)."""
        if self.weight_dtype != "fp8":
            if master is not self.weight:
                self.weight.copy_(master)
            return
        if not master.is_cuda:
            # Built on the host: the codes and scales are produced by the GPU kernels as soon as the
            # module is moved to the GPU (there is no host implementation of the quantizer).
            self._pending_refresh = True
            return
        self._pending_refresh = False
        if not self._grouped_scaling:
            # one scale for the tensor; the transposed codes, when cached, come from the same read (linear.py:288-297)
            limit = self._quantization_limit(max(self.in_features, self.out_features), self.fp8_dtype)
            if self.cache_weight_transpose and self.weight_transpose.numel() == 0:
                self.weight_transpose = torch.empty((self.in_features, self.out_features), device=master.device, dtype=self.fp8_dtype)
            scale = self.weight_quantizer.scale(master, self.fp8_dtype, limit, self.rotation_size)
            self.weight_scale.copy_(scale)
            quantize = rotation.quantize if self.rotation_size else kernels.quantize
            quantize(master, scale, transpose=self.cache_weight_transpose, fp8_dtype=self.fp8_dtype, out=self.weight,
                     out_t=self.weight_transpose if self.cache_weight_transpose else None, quantization_limit=limit)
            return
        limit = self._group_limit(self.weight_group_shape, self.fp8_dtype, weight=True)
        grouped.quantize(master, self.fp8_dtype, self.weight_group_shape, limit=limit, native=self._native_scaling,
                         out=self.weight, scale_out=self.weight_scale)
        if self.cache_weight_transpose:
            self._build_transpose(limit)

    def _build_transpose(self, limit):
        if not self._grouped_scaling:
            self.weight_transpose = kernels.transpose(self.weight)
            return
        self.weight_transpose, self.weight_transpose_scale = grouped.transpose(
            self.weight, self.weight_scale, self.weight_group_shape, native=self._native_scaling, limit=limit)

    def dequantize_weight(self):
        if self.weight_dtype != "fp8":
            return self.weight.float()
        assert self.weight.is_cuda, "viola_amd kernels run on the GPU only"
        if not self._grouped_scaling:
            weight = self.weight.float() * self.weight_scale
            return rotation.inverse_(weight) if self.rotation_size else weight   # back to the original coordinates
        return grouped.dequantize(self.weight, self.weight_scale, self.weight_group_shape)

    @classmethod
    @torch.no_grad()
    def from_float(cls, linear, **kwargs):
        layer = cls(linear.in_features, linear.out_features, linear.bias is not None,
                    device=linear.weight.device, dtype=linear.weight.dtype, **kwargs)
        master = layer._master()
        master.copy_(linear.weight)
        layer.weight_quantizer.history.zero_()
        layer.weight_quantizer.index = 0
        layer.refresh_weight(master)
        if linear.bias is not None:
            layer.bias.copy_(linear.bias)
            layer.bias.requires_grad_(linear.bias.requires_grad)
        layer.weight.requires_grad_(linear.weight.requires_grad)
        return layer

    # ------------------------------------------------------------------ execution
    def forward(self, x):
        assert x.is_cuda, "viola.nn.Linear executes on CUDA."
        if torch.is_autocast_enabled("cuda"):
            x = x.to(torch.get_autocast_dtype("cuda"))
        if self._pending_refresh:
            self.refresh_weight(self._master())
            assert not self._pending_refresh, \
                "The FP8 weight has not been quantized yet: its master is still on the host. Move the model to the GPU " \
                "before binding an optimizer (the quantizer runs on the GPU only)."
        need_backward = torch.is_grad_enabled() and (
            x.requires_grad or self.weight.requires_grad or (self.bias is not None and self.bias.requires_grad))
        if self._grouped_scaling:
            from ._grouped_linear import GroupedLinear
            return GroupedLinear.apply(x, self.weight, self.bias, self, need_backward)
        from ._tensor_linear import TensorLinear
        return TensorLinear.apply(x, self.weight, self.bias, self, need_backward)

    # ------------------------------------------------------------------ module plumbing
    def _apply(self, fn, recurse=True):
        """`.to()` / `.cuda()` / `.bfloat16()` move devices but never change the FP8 codes, the FP32
        scales or the amax histories: only the bias follows a dtype cast (linear.py:355-380)."""
        weight = self._parameters["weight"]
        self._parameters["weight"] = None
        grad_dtype = weight.grad_dtype
        pinned = [(self, name, self._buffers.pop(name)) for name in ("weight_scale", "weight_transpose", "weight_transpose_scale")]
        for quantizer in (self.weight_quantizer, self.input_quantizer, self.grad_quantizer):
            pinned.append((quantizer, "history", quantizer._buffers.pop("history")))
        super()._apply(fn, recurse)

        def move(t):
            return t.to(device=fn(torch.empty(0, device=t.device, dtype=t.dtype)).device)

        weight.data = move(weight.data)
        if weight.grad is not None:
            weight.grad = move(weight.grad)
        weight.grad_dtype = grad_dtype
        self._parameters["weight"] = weight
        for module, name, tensor in pinned:
            module._buffers[name] = move(tensor)
        if self._initial_weight is not None:
            self._initial_weight = move(self._initial_weight)
        if self.bias is not None:
            self.bias.grad_dtype = grad_dtype
        if self._pending_refresh and weight.is_cuda and self._master() is not None and self._master().is_cuda:
            self.refresh_weight(self._master())
        return self

    def _save_to_state_dict(self, destination, prefix, keep_vars):
        assert not self._pending_refresh, \
            "This Linear was built on the host and its FP8 codes do not exist yet: move it to the GPU before saving."
        super()._save_to_state_dict(destination, prefix, keep_vars)

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        expected = self.fp8_dtype if self.weight_dtype == "fp8" else _STORAGE[self.weight_dtype]
        assert state_dict[prefix + "weight"].dtype == expected, \
            "Construct Linear with the checkpoint's weight storage and FP8 format."
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)
        self._initial_weight = None
        self._pending_refresh = False
        self.rebuild_weight_cache()

    @torch.no_grad()
    def rebuild_weight_cache(self):
        """Rebuild W^T from the loaded codes and scales without requantizing W."""
        if self.cache_weight_transpose and self.weight_dtype == "fp8" and self.weight.is_cuda:
            self._build_transpose(self._group_limit(self.weight_group_shape, self.fp8_dtype, weight=True) if self._grouped_scaling else None)

    def extra_repr(self):
        return (f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}, "
                f"mode={self.mode!r}, weight_dtype={self.weight_dtype!r}, forward_dtype={self.forward_dtype!r}, "
                f"backward_dtype={self.backward_dtype!r}, cache_weight_transpose={self.cache_weight_transpose}, "
                f"saved_input_dtype={self.saved_input_dtype!r}, scaling={self.weight_quantizer.scaling!r}, "
                f"accum_dtype={self.accum_dtype!r}, accum_block_size={self.accum_block_size}, "
                f"accum_reduce_dtype={self.accum_reduce_dtype!r}, rotation_size={self.rotation_size}, "
                f"weight_group_shape={self.weight_group_shape}, input_group_shape={self.input_group_shape}, "
                f"grad_group_shape={self.grad_group_shape}")
