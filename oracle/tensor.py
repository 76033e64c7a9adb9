"""Per-tensor FP8 scaling (`current` / `delayed`) on CPU tensors. TEST INFRASTRUCTURE ONLY.

Restates viola/nn/_linear_kernels.py:33-104,124-163,231-293 and the Linear recipe around them
(viola/nn/linear.py:36-147). Pinned by the reference's own CPU definitions: `quantized()` in
checks/linear.py:17-20 and the CPU branch of `refresh_weight`, viola/nn/linear.py:298-312.
Unpinned corner: a tensor holding Inf has an infinite scale; the kernel text then sends Inf / Inf = NaN through
min(max(., -limit), limit), which yields -limit with IEEE-754 minNum / maxNum, while NaN inputs stay NaN.
"""

import torch


def amax(x):
    """max |x| with NaN dropped, 0 for an empty tensor (_amax_kernel, _linear_kernels.py:33-46)."""
    magnitude = x.float().abs().reshape(-1)
    magnitude = torch.where(magnitude.isnan(), torch.zeros_like(magnitude), magnitude)
    return magnitude.max() if magnitude.numel() else torch.zeros((), dtype=torch.float32)


def tensor_scale(x, history, index, *, delayed=False, limit=448.0):
    """(scale [1], history after the call) (_scale_kernel, _linear_kernels.py:49-71): the scale uses the history's
    maximum as it was before this call when delayed and index > 0, else this tensor's amax; the amax then goes into
    slot index % len."""
    current = amax(x)
    basis = history.max() if delayed and index != 0 else current
    scale = torch.maximum(basis, torch.tensor(1e-30, dtype=torch.float32)) / torch.tensor(limit, dtype=torch.float32)
    after = history.clone()
    after[index % history.numel()] = current
    return scale.reshape(1), after


def quantize(x, scale, dtype, *, limit=None, transpose=False):
    """fp8(isnan(x) ? x : clamp(x / scale, +-limit)) (_quantize_kernel, _linear_kernels.py:74-104), optionally transposed."""
    limit = torch.finfo(dtype).max if limit is None else limit
    value = x.float()
    quotient = value / scale.float().reshape(())
    low = torch.full_like(quotient, -limit)
    clamped = torch.where(quotient.isnan(), low, quotient.clamp(-limit, limit))     # maxNum(NaN, -limit) = -limit
    codes = torch.where(value.isnan(), value, clamped).to(dtype)
    return codes.T.contiguous() if transpose else codes


def gemm(a, b, sa, sb, *, bias=None, out_dtype=torch.float32):
    """(sum_k a b) * sa * sb + bias (_gemm_kernel epilogue, _linear_kernels.py:153-161), sums in float64."""
    acc = (a.double() @ b.double().T).float()
    value = acc * sa.float().reshape(()) * sb.float().reshape(())
    if bias is not None:
        value = value + bias.float()
    return value.to(out_dtype)


def gemm_half(a, b, sa, sb, *, accum_block_size=0, reduce_dtype=torch.float32, bias=None, out_dtype=torch.float32):
    """_gemm_kernel / _mixed_gemm_kernel with accum_dtype='float16' (viola/nn/_linear_kernels.py:139-161, :198-224).

    The FP16 fragment advances by 32-k tensor-core steps, acc = fp16(acc + the 32 products summed exactly) (the
    model of oracle.grouped.gemm_half). After whole chunks of bk k (bk = 64, or accum_block_size below that) that
    complete accum_block_size // bk chunks, and after the last chunk, total = reduce_dtype(float(total) + float(acc))
    and acc = 0; with accum_block_size = 0 the fragment runs over all of k. out = float(total) * sa * sb + bias."""
    m, k = a.shape
    n = b.shape[0]
    bk = accum_block_size if 0 < accum_block_size < 64 else 64
    acc = torch.zeros(m, n, dtype=torch.float16)
    total = torch.zeros(m, n, dtype=reduce_dtype)
    af, bf = a.double(), b.double()
    chunks = -(-k // bk)
    for chunk in range(chunks):
        for k0 in range(chunk * bk, min((chunk + 1) * bk, k), 32):
            acc = (acc.double() + af[:, k0:k0 + 32] @ bf[:, k0:k0 + 32].T).to(torch.float16)
        if accum_block_size and ((chunk + 1) % (accum_block_size // bk) == 0 or chunk == chunks - 1):
            total = (total.float() + acc.float()).to(reduce_dtype)
            acc = torch.zeros_like(acc)
    value = (total.float() if accum_block_size else acc.float()) * sa.float().reshape(()) * sb.float().reshape(())
    if bias is not None:
        value = value + bias.float()
    return value.to(out_dtype)


def linear(x, qw, sw, bias, dy, *, fp8=torch.float8_e4m3fn, bwd_fp8=torch.float8_e5m2, sx=None, sg=None,
           out_dtype=torch.bfloat16, grad_dtype=torch.bfloat16):
    """Expected y, dx, dw, db of Linear(scaling="current") from the stored weight codes (checks/linear.py:34-36):
    every operand quantized with its own tensor scale, products in fp32, db = dy.sum(0)."""
    limit_f, limit_b = torch.finfo(fp8).max, torch.finfo(bwd_fp8).max
    zero = torch.zeros(1)
    sx = tensor_scale(x, zero, 0, limit=limit_f)[0] if sx is None else sx
    sg = tensor_scale(dy, zero, 0, limit=limit_b)[0] if sg is None else sg
    qx, qg = quantize(x, sx, fp8), quantize(dy, sg, bwd_fp8)
    y = gemm(qx, qw, sx, sw, bias=bias, out_dtype=out_dtype)
    dx = gemm(qg, qw.T.contiguous(), sg, sw, out_dtype=out_dtype)
    dw = gemm(qg.T.contiguous(), qx.T.contiguous(), sg, sx, out_dtype=grad_dtype)
    return y, dx, dw, dy.float().sum(0).to(grad_dtype)
