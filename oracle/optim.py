"""FP8Muon state codec, Philox stochastic rounding, weight/AdamW updates on CPU.
TEST INFRASTRUCTURE ONLY.

Every sequence is the un-fused IEEE fp32 order of operations of the reference
kernels (no FMA contraction), which is what the HIP kernels are built to follow
bit for bit. The reference's own checks only hold the device kernels to
rtol 2e-6 (checks/quantization.py:105), because its CUDA build may contract.
"""

import math

import numpy as np
import torch
import torch.nn.functional as F

E4M3 = torch.float8_e4m3fn
MASK63 = (1 << 63) - 1


# ----------------------------------------------------------------------------- Philox / SR
def philox(element, step, key):
    """Philox4x32-10, word 0 (viola/optim/_kernels.py:13-26).

    counter = (element_lo, element_hi, step_lo, step_hi), key = (key_lo, key_hi).
    `element` may be a numpy uint64 array; step and key are Python ints.
    """
    element = np.asarray(element, dtype=np.uint64)
    m32 = np.uint64(0xFFFFFFFF)
    a, b = element & m32, element >> np.uint64(32)
    c = np.full_like(a, step & 0xFFFFFFFF)
    d = np.full_like(a, (step >> 32) & 0xFFFFFFFF)
    k0, k1 = key & 0xFFFFFFFF, (key >> 32) & 0xFFFFFFFF
    for _ in range(10):
        p0 = a * np.uint64(0xD2511F53)
        p1 = c * np.uint64(0xCD9E8D57)
        a, b, c, d = ((p1 >> np.uint64(32)) ^ b ^ np.uint64(k0), p1 & m32,
                      (p0 >> np.uint64(32)) ^ d ^ np.uint64(k1), p0 & m32)
        k0, k1 = (k0 + 0x9E3779B9) & 0xFFFFFFFF, (k1 + 0xBB67AE85) & 0xFFFFFFFF
    return a.astype(np.uint32)


def _spacing(a, mantissa_bits, min_exponent):
    exponent = ((a.view(np.uint32) >> 23) & 255).astype(np.int32) - 127
    return (((np.maximum(exponent - mantissa_bits, min_exponent) + 127).astype(np.uint32)) << 23).view(np.float32)


def _uniform(element, step, key):
    return (philox(element, step, key) >> 8).astype(np.float32) * np.float32(2.0 ** -24)


def stochastic_round_e4m3(x, element, step, key):
    """Round onto the e4m3 grid stochastically (viola/optim/_kernels.py:28-39).

    spacing = 2^max(e-3, -9); lower = floor(|x|/spacing)*spacing; round up iff
    uniform < (|x|-lower)/spacing; non-finite values pass through.
    """
    x = np.asarray(x, dtype=np.float32)
    a = np.abs(x)
    with np.errstate(all="ignore"):
        spacing = _spacing(a, 3, -9)
        lower = np.floor(a / spacing) * spacing
        probability = (a - lower) / spacing
        up = _uniform(element, step, key) < probability
        out = np.copysign(lower + np.where(up, spacing, np.float32(0)), x)
    return np.where(np.isfinite(x), out, x).astype(np.float32)


def stochastic_bf16(x, element, step, key):
    """bits += philox >> 16; bits &= 0xffff0000 (viola/optim/_kernels.py:41-47)."""
    x = np.asarray(x, dtype=np.float32)
    bits = (x.view(np.uint32) + (philox(element, step, key) >> 16)) & np.uint32(0xFFFF0000)
    return np.where(np.isfinite(x), bits.view(np.float32), x).astype(np.float32)


def stochastic_fp16(x, element, step, key):
    """fp16-grid stochastic rounding (viola/optim/_kernels.py:49-58)."""
    x = np.asarray(x, dtype=np.float32)
    a = np.abs(x)
    with np.errstate(all="ignore"):
        spacing = _spacing(a, 10, -24)
        lower = np.floor(a / spacing) * spacing
        up = _uniform(element, step, key) < (a - lower) / spacing
        out = np.copysign(lower + np.where(up, spacing, np.float32(0)), x)
    passthrough = ~np.isfinite(x) | (a > np.float32(65504.0))
    return np.where(passthrough, x, out).astype(np.float32)


# ----------------------------------------------------------------------------- state geometry
def state_sizes(shape, *, granularity="tile", tile_size=256, block_shape=(16, 16)):
    """(fp8 element count, scale count)  (viola/optim/_kernels.py:61-70)."""
    n = math.prod(shape)
    if granularity == "tile":
        blocks = (n + tile_size - 1) // tile_size
        return blocks * tile_size, blocks
    rows, cols = shape[-2:]
    tr, tc = block_shape
    tiles = (rows + tr - 1) // tr * ((cols + tc - 1) // tc)
    return n, math.prod(shape[:-2]) * tiles


def _expand(scales, shape, granularity, tile_size, block_shape):
    """Per-element scale, flat, in the payload's own order."""
    if granularity == "tile":
        return scales.repeat_interleave(tile_size)
    rows, cols = shape[-2:]
    tr, tc = block_shape
    e = scales.view(-1, (rows + tr - 1) // tr, (cols + tc - 1) // tc)
    return e.repeat_interleave(tr, 1).repeat_interleave(tc, 2)[:, :rows, :cols].flatten()


def dequantize(q, scales, shape, *, granularity="tile", tile_size=256, block_shape=(16, 16)):
    """viola/optim/_kernels.py:73-83."""
    n = math.prod(shape)
    values = q.view(E4M3).float() * _expand(scales, shape, granularity, tile_size, block_shape)
    return values[:n]


def _tile_amax(m, shape, granularity, tile_size, block_shape):
    """Per-tile abs-max (checks/quantization.py:27-38)."""
    if granularity == "tile":
        grouped = F.pad(m.flatten(), (0, (-m.numel()) % tile_size)).view(-1, tile_size)
    else:
        rows, cols = shape[-2:]
        tr, tc = block_shape
        padded = F.pad(m.view(-1, rows, cols), (0, (-cols) % tc, 0, (-rows) % tr))
        grouped = padded.view(-1, padded.shape[1] // tr, tr, padded.shape[2] // tc, tc)
        grouped = grouped.permute(0, 1, 3, 2, 4).reshape(-1, tr * tc)
    magnitude = torch.where(grouped.isnan(), torch.zeros_like(grouped), grouped.abs())
    return magnitude.amax(1)


def momentum_update(grad, q, scales, *, beta, shape, tile_size=256, nesterov=True, loss_scale=1.0,
                    granularity="tile", block_shape=(16, 16), rounding="nearest",
                    rounding_step=0, rounding_key=0):
    """One fused momentum step; returns (new_q uint8, new_scales fp32, update bf16).

    viola/optim/_kernels.py:114-142 (1-D tiles) and :166-198 (2-D blocks):
      g = f32(grad) * (1/loss_scale); m = beta*(f32(q)*scale) + (1-beta)*g
      scale' = max(amax_tile(m), 1e-30) / 448
      q' = e4m3(clamp(m/scale', +-448))   nearest, or stochastic with element = flat index
      update = bf16((1-beta)*g + beta*m) (nesterov) or bf16(m)
    The 1-D payload is padded with zeros to whole tiles and the stochastic element
    index is the padded flat index; the 2-D payload is unpadded.
    """
    n = math.prod(shape)
    beta32 = torch.tensor(beta, dtype=torch.float32)
    inv = torch.tensor(1.0 / float(loss_scale), dtype=torch.float32)
    g = grad.reshape(-1).float() * inv
    old = dequantize(q, scales, shape, granularity=granularity, tile_size=tile_size, block_shape=block_shape)
    one_minus = torch.tensor(1.0, dtype=torch.float32) - beta32
    m = beta32 * old + one_minus * g
    new_scales = _tile_amax(m, shape, granularity, tile_size, block_shape).clamp_min(1e-30) / 448.0
    qn, _ = state_sizes(shape, granularity=granularity, tile_size=tile_size, block_shape=block_shape)
    padded = F.pad(m, (0, qn - n))
    values = (padded / _expand(new_scales, shape, granularity, tile_size, block_shape)[:qn]).clamp(-448.0, 448.0)
    if rounding == "stochastic":
        element = np.arange(qn, dtype=np.uint64)
        values = torch.from_numpy(stochastic_round_e4m3(values.numpy(), element, rounding_step, rounding_key))
    new_q = values.to(E4M3).view(torch.uint8)
    update = (one_minus * g + beta32 * m if nesterov else m).bfloat16()
    return new_q, new_scales, update


def _store(value, dtype, rounding, element, step, key):
    if rounding == "stochastic" and dtype != torch.float32:
        fn = stochastic_bf16 if dtype == torch.bfloat16 else stochastic_fp16
        value = torch.from_numpy(fn(value.numpy(), element, step, key))
    return value.to(dtype)


def weight_update(weight, grad, lr, weight_decay, *, update_scale=1.0, rounding="nearest", step=0, key=0, offset=0):
    """w*(1 - lr*wd) - (lr*update_scale)*g in fp32 -> storage dtype (viola/optim/_kernels.py:247-253)."""
    f = lambda v: torch.tensor(float(v), dtype=torch.float32)
    lr, wd, us = f(lr), f(weight_decay), f(update_scale)
    value = weight.reshape(-1).float() * (f(1.0) - lr * wd) - (lr * us) * grad.reshape(-1).float()
    element = np.arange(value.numel(), dtype=np.uint64) + np.uint64(offset)
    return _store(value, weight.dtype, rounding, element, step, key).view(weight.shape)


def adam_update(weight, grad, first, second, *, lr, weight_decay, betas, eps, step, rounding="nearest",
                key=0, offset=0, adamw=True, maximize=False, bias_correction=True):
    """AdamW/Adam in fp32 (viola/optim/_kernels.py:273-291,331-337); returns (w, m, v)."""
    f = lambda v: torch.tensor(float(v), dtype=torch.float32)
    b1, b2 = betas
    inv_c1 = f(1. / (1. - b1 ** step) if bias_correction else 1.)
    inv_c2 = f(1. / (1. - b2 ** step) if bias_correction else 1.)
    lr, wd, b1, b2, eps = f(lr), f(weight_decay), f(b1), f(b2), f(eps)
    one = f(1.0)
    w = weight.reshape(-1).float()
    g = grad.reshape(-1).float()
    if maximize:
        g = -g
    if not adamw:
        g = g + wd * w
    m = b1 * first.reshape(-1).float() + (one - b1) * g
    v = b2 * second.reshape(-1).float() + ((one - b2) * g) * g
    if adamw:
        w = w * (one - lr * wd)
    # numpy's sqrt is correctly rounded; torch's vectorised CPU sqrt is not on every host
    root = torch.from_numpy(np.sqrt((v * inv_c2).numpy()))
    value = w - (lr * (m * inv_c1)) / (root + eps)
    element = np.arange(value.numel(), dtype=np.uint64) + np.uint64(offset)
    out = _store(value, weight.dtype, rounding, element, step - 1, key)
    return out.view(weight.shape), m.to(first.dtype).view(first.shape), v.to(second.dtype).view(second.shape)


def copy_scaled(update, partition, src, dst, count, scale):
    """out[dst+j] = f32(update[src+j]) * scale (viola/optim/_kernels.py:203-222,318-322)."""
    flat = update.contiguous().view(-1)
    out = partition.clone()
    out[dst:dst + count] = (flat[src:src + count].float() * torch.tensor(float(scale), dtype=torch.float32)).to(out.dtype)
    return out
