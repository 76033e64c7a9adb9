"""viola_ns_prepare_static: the Newton-Schulz normalisation for callers that cannot allocate device memory. Same
kernels as viola_ns_prepare with the partial sums in an array built into the library, so its output must equal
viola_ns_prepare's bit for bit: on two calls in a row, the second on a smaller input (the array keeps the first
call's contents), for both working dtypes and the tall (transposed) case; sizes beyond the array are rejected."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(matrix, dtype):
    from viola_amd import _lib
    from viola_amd.optim import _orthogonalize_kernels as nk
    batch, rows, cols = matrix.shape
    expect = nk.prepare(matrix, dtype)                                          # viola_ns_prepare, caller's workspace
    out = torch.full_like(expect, float("nan"))
    _lib.call("viola_ns_prepare_static", _lib.ptr(matrix), _lib.code(matrix.dtype), _lib.ptr(out), _lib.code(dtype),
              batch, rows, cols)
    return out, expect


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("in_dtype", [torch.float32, torch.bfloat16])
def test_static_scratch_prepare_equals_the_workspace_entry_point(dtype, in_dtype):
    from viola_amd import _lib
    _lib.call("viola_ns_prepare_static", None, _lib.code(in_dtype), None, _lib.code(dtype), 0, 0, 0)   # set-up call
    torch.manual_seed(77)
    first = (torch.randn(28, 192, 576, device="cuda") * 3).to(in_dtype)
    second = (torch.randn(3, 96, 40, device="cuda") * 1e-3).to(in_dtype)         # smaller, tall, other magnitude
    third = torch.randn(1, 33, 70, device="cuda").to(in_dtype)                   # ragged: the scalar kernels
    for matrix in (first, second, third, first):
        out, expect = _both(matrix, dtype)
        torch.cuda.synchronize()
        assert out.shape == expect.shape and torch.equal(out, expect)
        assert torch.isfinite(out).all()


def test_static_scratch_prepare_rejects_what_does_not_fit():
    from viola_amd import _lib
    x = torch.zeros(8, device="cuda")
    with pytest.raises(RuntimeError, match="built-in scratch"):
        _lib.call("viola_ns_prepare_static", _lib.ptr(x), _lib.F32, _lib.ptr(x), _lib.BF16, 1025, 1, 1)
    # the largest batch that fits runs
    big = torch.randn(1024, 8, 16, device="cuda")
    out, expect = _both(big, torch.bfloat16)
    assert torch.equal(out, expect)
