"""The C-ABI library loads and exports every symbol include/viola_hip.h declares (no compute calls)."""

import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]


def declared_symbols():
    text = (ROOT / "include" / "viola_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(viola_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_operator_set():
    names = declared_symbols()
    for required in ("viola_group_quantize", "viola_group_quantize_dual", "viola_group_gemm", "viola_gated_gemm",
                     "viola_varlen_group_gemm", "viola_momentum_update", "viola_weight_update", "viola_adam_update",
                     "viola_ns_gemm", "viola_comm_pack", "viola_comm_unpack", "viola_fp8_transpose"):
        assert required in names


def test_library_exports_every_declared_symbol():
    from viola_amd import _lib
    assert _lib.LIBRARY.exists(), "build first: python -m viola_amd.csrc.build"
    lib = ctypes.CDLL(str(_lib.LIBRARY))
    for name in declared_symbols():
        assert hasattr(lib, name), name
    assert set(_lib.EXPORTS) == set(declared_symbols())
    assert _lib.library().viola_abi_version() == 1
    assert b"invalid" in _lib.library().viola_error_string(-1)


def test_host_side_geometry():
    from viola_amd.nn import _grouped_kernels as g
    from viola_amd.optim._kernels import state_sizes
    from viola_amd.distributed import packet_bytes
    assert g.scale_shape((8192, 1024), (1, 32)) == (8192, 32) and g.scale_shape((4096, 1024), (32, 32)) == (128, 32)
    assert g.scale_shape((65, 96), (32, 64)) == (3, 2)
    assert g.transpose_group((32, 64)) == (64, 32) and g.transpose_group((1, 32)) == (1, 32)
    assert state_sizes((17, 31), tile_size=64) == (576, 9)
    assert state_sizes((2, 33, 67), granularity="block", block_shape=(16, 32)) == (4422, 2 * 3 * 3)
    assert packet_bytes(25600, 256) == 6656000


def test_product_never_imports_the_oracle():
    for path in (ROOT / "viola_amd").rglob("*.py"):
        text = path.read_text()
        assert "import oracle" not in text and "from oracle" not in text, path


def test_cpu_tensors_are_rejected():
    import torch
    from viola_amd.nn import _grouped_kernels as g
    with pytest.raises(AssertionError):
        g.quantize(torch.randn(4, 32), torch.float8_e4m3fn, (1, 32))


def test_rejected_calls_return_codes_and_launch_nothing():
    """Argument checks come before any launch, so they can be exercised without a GPU: VIOLA_EINVAL (-1) for bad
    dtypes / sizes / missing operands, VIOLA_EUNSUPPORTED (-2) for shapes an entry point does not take, 0 for empty
    problems. The pointers are never dereferenced on these paths."""
    from viola_amd import _lib
    lib = _lib.library()
    P = 0x10000                                                                # a non-null address that is never touched
    F32, BF16, E4M3, E5M2 = 0, 1, 3, 4
    # grouped GEMM: an FP8 code matrix cannot be an output, a float one cannot be an operand; group k must be >= 32
    assert lib.viola_group_gemm(P, E4M3, P, E4M3, P, P, 64, 64, 64, 1, 32, 32, 32, None, 0, P, E4M3, None) == -1
    assert lib.viola_group_gemm(P, BF16, P, E4M3, P, P, 64, 64, 64, 1, 32, 32, 32, None, 0, P, BF16, None) == -1
    assert lib.viola_group_gemm(P, E4M3, P, E4M3, P, P, 64, 64, 64, 1, 16, 32, 32, None, 0, P, BF16, None) == -1
    assert lib.viola_group_gemm(P, E4M3, P, E4M3, P, P, -1, 64, 64, 1, 32, 32, 32, None, 0, P, BF16, None) == -1
    assert lib.viola_group_gemm(P, E4M3, P, E4M3, P, P, 0, 64, 64, 1, 32, 32, 32, None, 0, P, BF16, None) == 0      # empty: done
    assert lib.viola_group_gemm(P, E4M3, P, E4M3, P, P, 64, 64, 64, 1, 32, 32, 32, None, 0, None, BF16, None) == -1  # no output
    # per-tensor GEMM and quantizer
    assert lib.viola_tensor_gemm(P, E4M3, P, E5M2, None, P, 64, 64, 64, None, 0, P, BF16, None) == -1               # no a scale
    assert lib.viola_tensor_quantize(P, E4M3, 64, 64, P, P, None, E4M3, 448.0, None) == -1                           # FP8 input
    assert lib.viola_tensor_quantize(P, BF16, 64, 64, P, P, None, E4M3, 0.0, None) == -1                             # limit <= 0
    assert lib.viola_tensor_quantize(P, BF16, 0, 64, P, P, None, E4M3, 448.0, None) == 0
    assert lib.viola_tensor_quantize(P, BF16, 64, 64, P, None, None, E4M3, 448.0, None) == 0                         # nothing asked for
    # block-scaled MFMA entries: unsupported shapes are reported, not guessed at
    assert lib.viola_mx_gemm(P, E4M3, P, E4M3, P, P, 64, 64, 96, 1, 32, None, 0, P, BF16, None) == -2                # k % 128
    assert lib.viola_mx_gemm(P + 8, E4M3, P, E4M3, P, P, 64, 64, 128, 1, 32, None, 0, P, BF16, None) == -2           # a not 16-byte aligned
    assert lib.viola_mx_gemm(P, E4M3, P, E4M3, P, P, 64, 64, 128, 1, 8, None, 0, P, BF16, None) == -2                # 8-row weight groups
    assert lib.viola_mx_gated_gemm(P, E4M3, P, E4M3, P, P, 64, 48, 128, 1, 32, None, 0, P, P, BF16, 0, 0, None) == -2  # up rows off the scale grid
    assert lib.viola_mx_gated_gemm(P, E4M3, P, E4M3, P, P, 64, 64, 128, 1, 32, None, 0, P, P, BF16, 7, 0, None) == -1  # no such activation
    assert lib.viola_mx_gated_gemm(P, E4M3, P, E4M3, P, P, 64, 64, 128, 1, 32, None, 0, None, P, BF16, 0, 1, None) == -1  # backward without [g, u]
    assert lib.viola_mx_gated_gemm_encode(P, E4M3, P, E4M3, P, P, 66, 64, 128, 1, 32, None, 0, P, BF16, P, P, P, P, E4M3, 448.0, 0, None) == -2
    assert lib.viola_mx_gated_gemm_encode(P, E4M3, P, E4M3, P, P, 64, 64, 128, 1, 32, None, 0, P, BF16, P, None, P, P, E4M3, 448.0, 0, None) == -1
    # rotation: the scratch size is part of the contract
    assert lib.viola_rotation_amax(P, BF16, 100, 200, P, 7, None) == -1                                              # needs 2 * 4 = 8 parts
    assert lib.viola_rotation_inverse(P, E4M3, 64, 64, None) == -1
    assert lib.viola_rotation_inverse(P, BF16, 0, 64, None) == 0
    # gated elementwise kernels
    assert lib.viola_gated_forward(P, P, 8, 8, E4M3, 0, None) == -1
    assert lib.viola_gated_forward(None, P, 8, 8, BF16, 0, None) == -1
    assert lib.viola_gated_forward(P, P, 0, 8, BF16, 0, None) == 0
    # the dual quantizer fed from [g | u]
    assert lib.viola_gated_quantize_dual(None, BF16, 64, 64, 0, P, P, P, P, E4M3, 32, 448.0, 0, None) == -1          # no input
    assert lib.viola_gated_quantize_dual(P, BF16, 64, 64, 9, P, P, P, P, E4M3, 32, 448.0, 0, None) == -1             # no such activation
    assert lib.viola_gated_quantize_dual(P, BF16, 64, 64, 0, P, P, P, P, BF16, 32, 448.0, 0, None) == -1             # codes must be FP8
    assert lib.viola_gated_quantize_dual(P, F32, 64, 64, 0, P, P, P, P, E4M3, 32, 448.0, 0, None) == -2              # 16-bit [g | u] only
    assert lib.viola_gated_quantize_dual(P, BF16, 64, 60, 0, P, P, P, P, E4M3, 32, 448.0, 0, None) == -2             # rows of h not 16-byte pieces
    assert lib.viola_gated_quantize_dual(P, BF16, 64, 64, 0, P, P, P, P, E4M3, 64, 448.0, 0, None) == -2             # groups of 32 only
    assert lib.viola_gated_quantize_dual(P, BF16, 0, 64, 0, P, P, P, P, E4M3, 32, 448.0, 0, None) == 0               # empty: done
    for status in (-1, -2):
        assert lib.viola_error_string(status)
