"""Bit-level FP8 (OCP e4m3fn / e5m2) codecs in numpy. TEST INFRASTRUCTURE ONLY.

Independent of torch's casts, so tests can pin `tensor.to(torch.float8_*)`
(the cast the reference's CPU oracles rely on, nn/_grouped_kernels.py:149-150,
checks/fp8_communication.py:32-38) against a second implementation.

e4m3fn: 1-4-3, bias 7, max 448, min subnormal 2^-9, no Inf, NaN = 0x7f/0xff.
e5m2  : 1-5-2, bias 15, max 57344, Inf = 0x7c, NaN = 0x7d..0x7f.
"""

import numpy as np


def decode_table(fmt):
    """All 256 codes -> float32 values."""
    codes = np.arange(256, dtype=np.uint32)
    sign = np.where(codes & 0x80, -1.0, 1.0)
    if fmt == "e4m3":
        e, m = (codes >> 3) & 15, codes & 7
        value = np.where(e == 0, m * 2.0 ** -9, (1 + m / 8.0) * 2.0 ** (e.astype(np.float64) - 7))
        value = np.where((e == 15) & (m == 7), np.nan, value)
    else:
        e, m = (codes >> 2) & 31, codes & 3
        value = np.where(e == 0, m * 2.0 ** -16, (1 + m / 4.0) * 2.0 ** (e.astype(np.float64) - 15))
        value = np.where(e == 31, np.where(m == 0, np.inf, np.nan), value)
    return (sign * value).astype(np.float32)


def encode(x, fmt):
    """float32 array -> uint8 codes, round-to-nearest-even on the FP8 grid.

    Out-of-range policy is the one of PyTorch's casts: e4m3fn has no Inf, so a
    value that rounds above 448 becomes NaN (0x7f); e5m2 overflows to Inf.
    Found by exact search on the grid, not by bit tricks.
    """
    x = np.asarray(x, dtype=np.float32)
    table = decode_table(fmt)
    finite = table[:0x7f] if fmt == "e4m3" else table[:0x7c]          # non-negative finite codes, ascending
    grid = finite.astype(np.float64)
    a = np.abs(x.astype(np.float64)).ravel()
    hi = np.searchsorted(grid, a, side="left").clip(1, len(grid) - 1)
    lo = hi - 1
    dlo, dhi = a - grid[lo], grid[hi] - a
    pick_hi = (dhi < dlo) | ((dhi == dlo) & (hi % 2 == 0))            # ties to the even code
    code = np.where(pick_hi, hi, lo).astype(np.uint32)
    code = np.where(a <= 0, 0, code)
    top = grid[-1]
    step = grid[-1] - grid[-2]
    over = a >= top + step / 2                                         # rounds past the largest finite value
    # the tie exactly at top + step/2 goes to the (even-mantissa) neighbour: for e4m3fn the
    # largest finite code 0x7e is even, so the tie stays finite; for e5m2 0x7b is odd -> Inf.
    if fmt == "e4m3":
        over = a > top + step / 2
        code = np.where(over, 0x7f, code)
    else:
        code = np.where(over, 0x7c, code)
        code = np.where(np.isinf(a), 0x7c, code)
    code = np.where(np.isnan(a), 0x7f, code)
    sign = (x.view(np.uint32).ravel() >> 24) & 0x80
    return (code | sign).astype(np.uint8).reshape(x.shape)
