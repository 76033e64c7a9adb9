"""Which tile shape the Newton-Schulz GEMM picks is host arithmetic of the library (viola_ns_plan, the counterpart of
viola/optim/_orthogonalize_kernels.py:114 `plan`), so it can be replayed here without a GPU: over every shape the GPU
parity tests use, and over every product of the optimizer benchmark's DiT-XL step. A tile shape of the kernel, or a
product of that step, that no GPU test reaches fails this file."""

import itertools

import pytest

import test_gpu_ns_comm as cases
from viola_amd.optim._orthogonalize_kernels import plan

KERNELS = ("64x64", "128x64", "128x128", "192x192", "384x192")
MIRRORED = ("64x64", "128x128", "192x192")                                   # a Gram product keeps square tiles


def variant(batch, m, n, k, transpose_b=False, same_operand=False, transpose_out=False):
    p = plan(batch, m, n, k, transpose_b=transpose_b, same_operand=same_operand, transpose_out=transpose_out)
    return p["kernel"], p["mirrored"], bool(transpose_out)


def covered_by_the_gpu_tests():
    """(kernel, mirrored, transposed output) of every launch the parametrized GPU tests of the chain GEMM make."""
    seen = set()
    for (batch, m, n, k), (transpose_b, _) in itertools.product(cases.CONTRACT_SHAPES, cases.CONTRACT_MODES):
        seen.add(variant(batch, m, n, k, transpose_b))
    for batch, m, k in cases.GRAM_SHAPES + cases.GRAM_ASYMMETRIC_SHAPES + cases.DIAGONAL_SHAPES:
        seen.add(variant(batch, m, m, k, True, same_operand=True))
        seen.add(variant(batch, m, m, k, True))
    for batch, m, k in cases.DIAGONAL_SHAPES:
        seen.add(variant(batch, m, m, k, True, transpose_out=True))
        seen.add(variant(batch, m, m, k, True, same_operand=True, transpose_out=True))
    for (batch, m, n, k), (transpose_b, _) in itertools.product(cases.TRANSPOSED_SHAPES, cases.TRANSPOSED_MODES):
        seen.add(variant(batch, m, n, k, transpose_b))
        seen.add(variant(batch, m, n, k, transpose_b, transpose_out=True))
    for m, n, k in cases.DITXL_PRODUCTS:
        for transpose_out in (False, True):
            seen.add(variant(cases.DITXL_BATCH, m, n, k, transpose_out=transpose_out))
            seen.add(variant(1, m, n, k, transpose_out=transpose_out))
    for k in cases.DITXL_GRAM_K:
        seen.add(variant(cases.DITXL_BATCH, 1152, 1152, k, True, same_operand=True))
        seen.add(variant(cases.DITXL_BATCH, 1152, 1152, k, True))
        seen.add(variant(1, 1152, 1152, k, True, same_operand=True))
    return seen


def products_of_a_chain(batch, rows, cols, method):
    """The GEMMs of one orthogonalization (viola/optim/_orthogonalize.py:10-54 as the device chain runs it): tuples
    (batch, m, n, k, transpose_b, same_operand, transpose_out)."""
    tall = rows > cols
    m, n = min(rows, cols), max(rows, cols)
    if method == "standard" or m == n:
        return [(batch, m, m, n, True, True, False),                        # r = x x^T
                (batch, m, m, m, True, True, False),                        # z from r r^T
                (batch, m, n, m, False, False, False),                      # x = z x + 3.4445 x
                (batch, m, n, m, False, False, tall)]                       # ... stored transposed at the end of a tall matrix
    return [(batch, m, m, n, True, True, False),                            # r = x x^T
            (batch, m, m, m, True, True, False),                            # first z of a segment
            (batch, m, m, m, False, True, False),                           # later z: r r, r symmetric only up to rounding
            (batch, m, m, m, False, False, False),                          # z q, z r, z rz
            (batch, m, n, m, False, False, False),                          # x = q x
            (batch, m, n, m, False, False, tall)]


def test_every_tile_shape_has_a_covering_gpu_case():
    seen = covered_by_the_gpu_tests()
    for kernel in KERNELS:
        assert any(v[0] == kernel and not v[1] for v in seen), f"no GPU parity case runs the {kernel} tile"
        assert any(v[0] == kernel and not v[1] and v[2] for v in seen), f"no GPU parity case stores the {kernel} tile transposed"
    for kernel in MIRRORED:
        assert any(v[0] == kernel and v[1] for v in seen), f"no GPU parity case runs the mirrored {kernel} tile"
    assert any(v[0] == "generic" for v in seen)


@pytest.mark.parametrize("method", ["standard", "gram"])
def test_every_product_of_the_ditxl_step_has_a_covering_gpu_case(method):
    seen = covered_by_the_gpu_tests()
    d = 1152
    for batch, rows, cols in ((28, 3 * d, d), (28, d, d), (56, 4 * d, d), (28, 4 * d, d), (28, d, 4 * d)):
        for product in products_of_a_chain(batch, rows, cols, method):
            assert variant(*product) in seen, (method, product, variant(*product))


def test_plan_of_known_shapes():
    assert plan(28, 1152, 3456, 1152) == dict(bm=384, bn=192, mirrored=False, kernel="384x192")
    assert plan(28, 1152, 1152, 3456, transpose_b=True, same_operand=True)["mirrored"]
    assert not plan(28, 1152, 1152, 3456, transpose_b=True, same_operand=True, transpose_out=True)["mirrored"]
    assert plan(2, 33, 47, 65)["kernel"] == "generic"                        # k, n not multiples of 8
    assert plan(0, 64, 64, 64)["kernel"] == "generic"
