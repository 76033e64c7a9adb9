"""Writes tests/golden/ns_golden.pt: input/output vectors of the reference's eager Newton-Schulz
recipes, the one part of the hot path whose exact bf16/fp16 trajectory no closed form pins.

Run in the build container only (the reference tree is not available elsewhere):
    TORCH_COMPILE_DISABLE=1 python tests/golden/make_ns_golden.py
It loads viola/optim/_orthogonalize.py by file path (that file imports nothing but torch), with
torch.compile disabled so the functions run eagerly on the CPU. Only tensors are stored.
"""

import importlib.util
import os
import sys
from pathlib import Path

os.environ.setdefault("TORCH_COMPILE_DISABLE", "1")
import torch

REFERENCE = Path("/root/reference/viola/optim/_orthogonalize.py")
CASES = [("standard", (64, 256), 5), ("standard", (192, 64), 5), ("standard", (96, 96), 3),
         ("gram", (64, 256), 5), ("gram", (192, 64), 5), ("gram", (96, 96), 5), ("gram", (64, 160), 2),
         ("standard", (2, 48, 80), 5), ("gram", (2, 48, 80), 5)]
# The benchmark's single-matrix configuration: one 1024 x 4096 fp32 Gaussian matrix, seed 1, 5 steps. The 4 M-element
# input is regenerated from its seed by the tests (its sum and a strided sample are stored to make sure of that);
# of the output a strided sample and all singular values are stored.
LARGE = (1024, 4096)
LARGE_STRIDE = 16


def main():
    spec = importlib.util.spec_from_file_location("_reference_orthogonalize", REFERENCE)
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    torch.manual_seed(20261125)
    rows = []
    for method, shape, steps in CASES:
        matrix = torch.randn(*shape)
        out = module.METHODS[method](matrix, steps=steps)
        rows.append(dict(method=method, steps=steps, input=matrix, output=out.contiguous()))
    path = Path(__file__).with_name("ns_golden.pt")
    torch.save(rows, path)
    print(path, sum(r["input"].numel() for r in rows), "input elements")
    torch.manual_seed(1)
    matrix = torch.randn(*LARGE)
    large = dict(shape=LARGE, seed=1, steps=5, stride=LARGE_STRIDE, input_sum=matrix.double().sum(),
                 input_sample=matrix[::LARGE_STRIDE, ::LARGE_STRIDE].contiguous())
    for method in ("standard", "gram"):
        out = module.METHODS[method](matrix, steps=5)
        large[method] = dict(sample=out[::LARGE_STRIDE, ::LARGE_STRIDE].contiguous(),
                             singular_values=torch.linalg.svdvals(out.float()))
    path = Path(__file__).with_name("ns_golden_1024x4096.pt")
    torch.save(large, path)
    print(path)


if __name__ == "__main__":
    sys.exit(main())
