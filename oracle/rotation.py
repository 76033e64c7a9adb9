"""Hadamard-64 rotation on CPU. TEST INFRASTRUCTURE ONLY.

`rotate` restates the staged butterflies of the reference's kernels (viola/nn/_rotation_kernels.py:11-25, _regular64)
in their operation order, in float32, so the GPU result can be compared bit for bit; `hadamard64` is the matrix the
reference itself uses as the definition (rotate_cpu, _rotation_kernels.py:126-130). Pinned by: rotate == x @ H64
(exact on small integers, 1e-6 otherwise), H64 symmetric and orthogonal, rotate(rotate(x)) == x on integers.
"""

import numpy as np
import torch


def hadamard64():
    """kron(H4, H4, H4), H4 = (ones(4, 4) - 2 flip(eye(4))) / 2 (_rotation_kernels.py:128-129)."""
    h = (torch.ones(4, 4) - 2 * torch.eye(4).flip(1)) / 2
    return torch.kron(torch.kron(h, h), h)


def rotate(x):
    """Rotated copy of a [rows, cols] tensor in float32: each run of 64 columns (the last one completed with zeros)
    goes through three stages, stride 1, 4, 16:
    out[j] = ((v[b] + v[b + s]) + (v[b + 2 s] + v[b + 3 s])) * 0.5 - v[b + (3 - digit) s]."""
    rows, cols = x.shape
    padded = -(-cols // 64) * 64
    v = np.zeros((rows, padded), dtype=np.float32)
    v[:, :cols] = x.detach().float().cpu().numpy()
    j = np.arange(padded)
    half = np.float32(0.5)
    for stage in range(3):
        stride = 1 << (2 * stage)
        base = j // (4 * stride) * (4 * stride) + j % stride
        digit = j // stride % 4
        total = (v[:, base] + v[:, base + stride]) + (v[:, base + 2 * stride] + v[:, base + 3 * stride])
        v = (total * half - v[:, base + (3 - digit) * stride]).astype(np.float32)
    return torch.from_numpy(v[:, :cols].copy())


def amax(x):
    """max |rotate(x)| with NaN dropped, as the reference's reduction does (_rotation_kernels.py:44-46)."""
    r = rotate(x).abs()
    r = torch.where(torch.isnan(r), torch.zeros_like(r), r)
    return r.max() if r.numel() else torch.zeros(())
