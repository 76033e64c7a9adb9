"""ctypes binding of libviola_hip.so (include/viola_hip.h) and tensor marshalling.

PyTorch only supplies device memory and the current HIP stream here; every
operator is one C-ABI call. There is no CPU or PyTorch fallback: if the library
is missing, or a tensor is not on the GPU, the call raises.
"""

import ctypes
from pathlib import Path

import torch

F32, BF16, F16, E4M3, E5M2 = range(5)
DTYPE = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16,
         torch.float8_e4m3fn: E4M3, torch.float8_e5m2: E5M2}
ACTIVATION = {"silu": 0, "gelu": 1, "relu": 2}
ROUNDING = {"nearest": 0, "stochastic": 1}
LIBRARY = Path(__file__).resolve().parent / "csrc" / "libviola_hip.so"

_i, _l, _f, _p = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p
_SIGNATURES = {
    "viola_group_quantize": [_p, _i, _l, _l, _p, _i, _p, _i, _i, _f, _i, _p, _i, _i, _i, _p],
    "viola_group_quantize_dual": [_p, _i, _l, _l, _p, _p, _p, _p, _i, _i, _f, _p, _i, _p],
    "viola_gated_quantize_dual": [_p, _i, _l, _l, _i, _p, _p, _p, _p, _i, _i, _f, _i, _p],
    "viola_column_reduce": [_p, _l, _l, _p, _i, _p],
    "viola_group_dequantize": [_p, _i, _p, _l, _l, _i, _i, _p, _p],
    "viola_fp8_transpose": [_p, _p, _l, _l, _l, _p],
    "viola_block_transpose": [_p, _p, _l, _l, _p, _p, _i, _i, _i, _p],
    "viola_group_gemm": [_p, _i, _p, _i, _p, _p, _l, _l, _l, _i, _i, _i, _i, _p, _i, _p, _i, _p],
    "viola_group_gemm_half": [_p, _i, _p, _i, _p, _p, _l, _l, _l, _i, _i, _i, _i, _p, _i, _p, _i, _i, _i, _p],
    "viola_tensor_gemm_half": [_p, _i, _p, _i, _p, _p, _l, _l, _l, _p, _i, _p, _i, _i, _i, _p],
    "viola_gated_gemm": [_p, _i, _p, _i, _p, _p, _l, _l, _l, _i, _i, _i, _i, _p, _i, _p, _p, _i, _i, _i, _p],
    "viola_varlen_group_gemm": [_p, _i, _p, _i, _p, _p, _p, _i, _l, _l, _l, _i, _i, _i, _i, _l, _l, _p, _i, _p],
    "viola_varlen_wgrad_gemm": [_p, _i, _p, _i, _p, _p, _p, _i, _l, _l, _l, _p, _i, _p],
    "viola_varlen_quantize_transposed": [_p, _i, _l, _l, _p, _p, _i, _l, _p, _p, _i, _f, _p, _p, _p],
    "viola_gated_forward": [_p, _p, _l, _l, _i, _i, _p],
    "viola_gated_backward": [_p, _p, _p, _l, _l, _i, _i, _p],
    "viola_momentum_update": [_p, _i, _p, _p, _p, _p, _p, _l, _f, _f, _i, _i, _i, _l, _l, _l, _i, _i, _i, _l, _l, _p],
    "viola_weight_update": [_p, _i, _p, _i, _l, _f, _f, _f, _i, _l, _l, _l, _p],
    "viola_adam_update": [_p, _i, _p, _i, _p, _p, _i, _l, _f, _f, _f, _f, _f, _f, _f, _i, _l, _l, _l, _i, _i, _p],
    "viola_tensor_amax": [_p, _i, _l, _p, _l, _p],
    "viola_tensor_scale": [_p, _l, _p, _i, _l, _i, _f, _p, _p],
    "viola_tensor_amax_columns": [_p, _i, _l, _l, _l, _p, _p, _p],
    "viola_tensor_amax_columns_scale": [_p, _i, _l, _l, _l, _p, _p, _p, _i, _l, _i, _f, _p, _p, _i, _p],
    "viola_tensor_amax_scale": [_p, _i, _l, _p, _l, _p, _i, _l, _i, _f, _p, _p],
    "viola_tensor_quantize": [_p, _i, _l, _l, _p, _p, _p, _i, _f, _p],
    "viola_rotation_amax": [_p, _i, _l, _l, _p, _l, _p],
    "viola_rotation_quantize": [_p, _i, _l, _l, _p, _p, _p, _i, _f, _p],
    "viola_rotation_inverse": [_p, _i, _l, _l, _p],
    "viola_tensor_gemm": [_p, _i, _p, _i, _p, _p, _l, _l, _l, _p, _i, _p, _i, _p],
    "viola_mx_gemm": [_p, _i, _p, _i, _p, _p, _l, _l, _l, _i, _i, _p, _i, _p, _i, _p],
    "viola_tensor_gated_gemm": [_p, _i, _p, _i, _p, _p, _l, _l, _l, _p, _i, _p, _p, _i, _i, _i, _p],
    "viola_mx_gated_gemm": [_p, _i, _p, _i, _p, _p, _l, _l, _l, _i, _i, _p, _i, _p, _p, _i, _i, _i, _p],
    "viola_mx_gated_gemm_encode": [_p, _i, _p, _i, _p, _p, _l, _l, _l, _i, _i, _p, _i, _p, _i, _p, _p, _p, _p, _i, _f, _i, _p],
    "viola_momentum_update_table": [_p, _l, _l, _i, _i, _f, _f, _i, _i, _l, _p],
    "viola_weight_update_table": [_p, _l, _l, _i, _f, _f, _f, _p],
    "viola_adam_update_table": [_p, _l, _l, _i, _i, _i, _f, _f, _f, _f, _f, _f, _f, _i, _l, _i, _i, _p],
    "viola_copy_scaled": [_p, _i, _p, _i, _l, _l, _l, _f, _p],
    "viola_momentum_dequantize": [_p, _p, _p, _l, _i, _i, _l, _l, _l, _i, _i, _p],
    "viola_ns_gemm": [_p, _p, _p, _p, _i, _i, _i, _l, _l, _l, _l, _f, _p, _i, _p],
    "viola_ns_prepare": [_p, _i, _p, _i, _l, _l, _l, _p, _p],
    "viola_ns_prepare_static": [_p, _i, _p, _i, _l, _l, _l, _p],
    "viola_comm_pack": [_p, _l, _p, _l, _l, _i, _i, _p],
    "viola_comm_unpack": [_p, _p, _l, _l, _l, _i, _i, _i, _p],
    "viola_comm_pack_table": [_p, _l, _l, _i, _i, _p],
    "viola_comm_unpack_table": [_p, _l, _l, _i, _i, _i, _p],
    "viola_selftest_fp8": [_p, _p],
    "viola_selftest_philox": [_p, _p, _l, _p],
}
EXPORTS = tuple(_SIGNATURES) + ("viola_abi_version", "viola_error_string", "viola_ns_plan")

_lib = None


def library():
    """Load the HIP library once; raise loudly if it has not been built."""
    global _lib
    if _lib is None:
        if not LIBRARY.exists():
            raise RuntimeError(f"{LIBRARY} is missing: build it with `python -m viola_amd.csrc.build` "
                               "(viola_amd has no CPU or PyTorch fallback)")
        lib = ctypes.CDLL(str(LIBRARY))
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = argtypes, ctypes.c_int
        lib.viola_abi_version.restype = ctypes.c_int
        lib.viola_error_string.argtypes, lib.viola_error_string.restype = [ctypes.c_int], ctypes.c_char_p
        lib.viola_ns_plan.argtypes, lib.viola_ns_plan.restype = [_l, _l, _l, _l, _i, _i, _i, ctypes.POINTER(ctypes.c_int)], ctypes.c_int
        assert lib.viola_abi_version() == 1
        _lib = lib
    return _lib


def ptr(tensor):
    """Device pointer of a tensor, or NULL for None / empty (the "absent" convention)."""
    if tensor is None or tensor.numel() == 0:
        return None
    assert tensor.is_cuda, "viola_amd kernels run on the GPU only"
    return tensor.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def stream():
    """Handle of the current stream of the current device (the raw accessors cost a tenth of building a Stream object,
    which matters with a dozen launches in a 0.2 ms step)."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


timeline = None   # when a list, every call appends (name, start_event, end_event) recorded on the current stream


def call(name, *args, unsupported_ok=False):
    """Invoke one entry point on the current stream; non-zero status raises (VIOLA_EUNSUPPORTED is returned instead
    when the caller has another route)."""
    lib = library()
    if timeline is not None:
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        status = getattr(lib, name)(*args, stream())
        end.record()
        timeline.append((name, start, end))
    else:
        status = getattr(lib, name)(*args, stream())
    if status == -2 and unsupported_ok:
        return status
    if status:
        raise RuntimeError(f"{name} failed: {lib.viola_error_string(status).decode()} (status {status})")
    return status


def code(dtype):
    return DTYPE[dtype]
