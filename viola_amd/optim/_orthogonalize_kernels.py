"""Newton-Schulz orthogonalization as a chain of HIP bf16/fp16 MFMA GEMMs with fused epilogues
(operator seam of viola/optim/_orthogonalize_kernels.py: _matmul :53, run :77, orthogonalize :200).

`standard` is the bf16 quintic iteration, `gram` the fp16 Gram recurrence with one restart; both
follow the rounding points of the reference's device chain: fp32 accumulate -> round -> fp32
epilogue -> round."""

import torch

from .. import _lib

A_COEFF = 3.4445


def _matmul(a, b, *, transpose_b=False, residual=None, epilogue=0, add_diag=None, transpose_out=False):
    """One chain GEMM. With add_diag, also returns a copy of the result with add_diag on its diagonal;
    transpose_out stores the result as [batch, n, m]."""
    batch, m, k = a.shape
    n = b.shape[-2] if transpose_b else b.shape[-1]
    out = a.new_empty((batch, n, m) if transpose_out else (batch, m, n))
    second = a.new_empty(out.shape) if add_diag is not None else None
    _lib.call("viola_ns_gemm", _lib.ptr(a), _lib.ptr(b), _lib.ptr(residual), _lib.ptr(out), _lib.code(a.dtype),
              int(transpose_b), epilogue, batch, m, n, k, float(add_diag or 0.0), _lib.ptr(second), int(transpose_out))
    return out if add_diag is None else (out, second)


def plan(batch, m, n, k, *, transpose_b=False, same_operand=False, transpose_out=False):
    """The tile shape one chain GEMM of this size runs on (the counterpart of the reference's timed `plan`,
    viola/optim/_orthogonalize_kernels.py:114): host arithmetic of the library, usable without a GPU."""
    import ctypes
    out = (ctypes.c_int * 4)()
    status = _lib.library().viola_ns_plan(batch, m, n, k, int(transpose_b), int(same_operand), int(transpose_out), out)
    assert status == 0, status
    return dict(bm=out[0], bn=out[1], mirrored=bool(out[2]), kernel=("generic", "64x64", "128x64", "128x128", "192x192", "384x192")[out[3]])


def prepare(matrix, dtype):
    """[B, rows, cols] (any float dtype) -> dtype, transposed if tall, divided by (||.||_F + 1e-7)."""
    batch, rows, cols = matrix.shape
    x = torch.empty((batch, min(rows, cols), max(rows, cols)), device=matrix.device, dtype=dtype)
    workspace = torch.empty(batch * 256, device=matrix.device, dtype=torch.float32)
    _lib.call("viola_ns_prepare", _lib.ptr(matrix), _lib.code(matrix.dtype), _lib.ptr(x), _lib.code(dtype),
              batch, rows, cols, _lib.ptr(workspace))
    return x


def run(matrix, steps, method):
    assert matrix.is_cuda, "viola_amd kernels run on the GPU only"
    shape = matrix.shape
    tall = shape[-2] > shape[-1]
    dtype = torch.bfloat16 if method == "standard" else torch.float16
    x = prepare(matrix.contiguous().reshape(-1, shape[-2], shape[-1]), dtype)
    if method == "standard" or x.shape[-2] == x.shape[-1]:
        for step in range(steps):
            r = _matmul(x, x, transpose_b=True)
            z = _matmul(r, r, transpose_b=True, residual=r, epilogue=1)      # r = x x^T is symmetric bit for bit: r r = r r^T
            x = _matmul(z, x, residual=x, epilogue=2, transpose_out=tall and step == steps - 1)
    else:
        segments = [length for length in (min(steps, 2), max(steps - 2, 0)) if length]
        for index, length in enumerate(segments):
            r = _matmul(x, x, transpose_b=True)
            q = None
            for i in range(length):
                if i == 0:
                    # Z and Q = Z + 3.4445 I from the one product
                    z, q = _matmul(r, r, transpose_b=True, residual=r, epilogue=1, add_diag=A_COEFF)
                else:
                    # past the first iteration r = 3.4445 rz + z rz is symmetric only up to rounding: r @ r as written
                    z = _matmul(r, r, residual=r, epilogue=1)
                    q = _matmul(z, q, residual=q, epilogue=2)
                if i + 1 < length:
                    rz = _matmul(z, r, residual=r, epilogue=2)
                    r = _matmul(z, rz, residual=rz, epilogue=2)
            x = _matmul(q, x, transpose_out=tall and index == len(segments) - 1)
    return x.reshape(shape)


def orthogonalize(matrix, steps=5, method="standard", autotune=True):
    return run(matrix, steps, method)
