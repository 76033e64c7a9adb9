"""Newton-Schulz orthogonalization on CPU. TEST INFRASTRUCTURE ONLY.

Two restatements of the same recurrences:
  * `standard` / `gram`: the eager recipe, every tensor op rounds to the working
    dtype (viola/optim/_orthogonalize.py:10-54);
  * `chain`: the GEMM-chain contract of the device kernels: fp32 accumulate ->
    round to dtype -> fp32 epilogue -> round once
    (viola/optim/_orthogonalize_kernels.py:38-49,77-108). The HIP chain follows this.
"""

import torch

A, B, C = 3.4445, -4.7750, 2.0315


def _prepare(matrix, dtype):
    tall = matrix.shape[-2] > matrix.shape[-1]
    x = matrix.to(dtype)
    if tall:
        x = x.mT
    return x / (x.norm(dim=(-2, -1), keepdim=True) + 1e-7), tall


def standard(matrix, steps=5):
    """bf16 quintic iteration (viola/optim/_orthogonalize.py:10-21)."""
    x, tall = _prepare(matrix, torch.bfloat16)
    for _ in range(steps):
        gram_ = x @ x.mT
        polynomial = B * gram_ + C * (gram_ @ gram_)
        x = A * x + polynomial @ x
    return x.mT if tall else x


def gram(matrix, steps=5):
    """fp16 Gram recurrence with one restart after two iterations (_orthogonalize.py:24-54)."""
    x, tall = _prepare(matrix, torch.float16)
    if x.shape[-2] == x.shape[-1]:
        for _ in range(steps):
            r = x @ x.mT
            x = A * x + (B * r + C * (r @ r)) @ x
    else:
        for length in (min(steps, 2), max(steps - 2, 0)):
            if length:
                r = x @ x.mT
                q = None
                for i in range(length):
                    z = B * r + C * (r @ r)
                    if i == 0:
                        q = z.clone()
                        q.diagonal(dim1=-2, dim2=-1).add_(A)
                    else:
                        q = A * q + z @ q
                    if i + 1 < length:
                        rz = A * r + z @ r
                        r = A * rz + z @ rz
                x = q @ x
    return x.mT if tall else x


def matmul(a, b, *, transpose_b=False, residual=None, epilogue=0):
    """One chain GEMM: acc fp32 -> dtype -> fp32 epilogue -> dtype (_orthogonalize_kernels.py:38-49)."""
    value = (a.float() @ (b.float().mT if transpose_b else b.float())).to(a.dtype).float()
    if epilogue == 1:
        value = torch.tensor(B) * residual.float() + torch.tensor(C) * value
    elif epilogue == 2:
        value = value + torch.tensor(A) * residual.float()
    return value.to(a.dtype)


def chain(matrix, steps=5, method="standard"):
    """The driver of the device GEMM chain (_orthogonalize_kernels.py:77-108)."""
    shape = matrix.shape
    x, tall = _prepare(matrix, torch.bfloat16 if method == "standard" else torch.float16)
    x = x.contiguous().reshape(-1, x.shape[-2], x.shape[-1])
    if method == "standard" or x.shape[-2] == x.shape[-1]:
        for _ in range(steps):
            r = matmul(x, x, transpose_b=True)
            z = matmul(r, r, residual=r, epilogue=1)
            x = matmul(z, x, residual=x, epilogue=2)
    else:
        for length in (min(steps, 2), max(steps - 2, 0)):
            if length:
                r = matmul(x, x, transpose_b=True)
                for i in range(length):
                    z = matmul(r, r, residual=r, epilogue=1)
                    if i == 0:
                        q = z.clone()
                        q.diagonal(dim1=-2, dim2=-1).add_(A)
                    else:
                        q = matmul(z, q, residual=q, epilogue=2)
                    if i + 1 < length:
                        rz = matmul(z, r, residual=r, epilogue=2)
                        r = matmul(z, rz, residual=rz, epilogue=2)
                x = matmul(q, x)
    if tall:
        x = x.mT
    return x.reshape(shape)


METHODS = {"standard": standard, "gram": gram}
