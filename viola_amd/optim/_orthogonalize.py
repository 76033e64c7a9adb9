"""Quintic Newton-Schulz orthogonalization entry points (viola/optim/_orthogonalize.py:10-57).
Both methods run the HIP GEMM chain; the reference's default instead traces the same recurrences
with torch.compile."""

from functools import partial

from ._orthogonalize_kernels import run


def standard(matrix, steps=5):
    return run(matrix, steps, "standard")


def gram(matrix, steps=5):
    return run(matrix, steps, "gram")


METHODS = {"standard": standard, "gram": gram}
