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
