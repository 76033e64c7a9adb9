"""FP8Muon kernel operators (operator seam of viola/optim/_kernels.py: state_sizes :61, dequantize
:73, momentum_update :300, copy_scaled :318, weight_update :325, adam_update :331)."""

import math

import torch

from .. import _lib


def state_sizes(shape, *, granularity="tile", tile_size=256, block_shape=(16, 16)):
    """(FP8 payload elements, scale count). 1-D tiles pad the payload; 2-D blocks do not."""
    n = math.prod(shape)
    if granularity == "tile":
        blocks = -(-n // tile_size)
        return blocks * tile_size, blocks
    rows, cols = shape[-2:]
    tr, tc = block_shape
    return n, math.prod(shape[:-2]) * (-(-rows // tr)) * (-(-cols // tc))


def _geometry(n, granularity, tile_size, block_shape, matrix_shape):
    if granularity == "tile":
        return 0, int(tile_size), 1, 1, 1, 1, 1
    rows, cols = matrix_shape[-2:]
    planes = math.prod(matrix_shape[:-2])
    assert planes * rows * cols == n
    return 1, 0, planes, rows, cols, int(block_shape[0]), int(block_shape[1])


def dequantize(q, scales, shape, *, granularity="tile", tile_size=256, block_shape=(16, 16)):
    """Diagnostic: fp32 momentum of `shape` from the FP8 payload and its scales (flat)."""
    n = math.prod(shape)
    out = torch.empty(n, device=q.device, dtype=torch.float32)
    geometry = _geometry(n, granularity, tile_size, block_shape, shape)
    _lib.call("viola_momentum_dequantize", _lib.ptr(q), _lib.ptr(scales), _lib.ptr(out), n, *geometry)
    return out


def momentum_update(grad, q, scales, next_q, next_scales, out, *, beta, tile_size=256, nesterov=True,
                    loss_scale=1.0, granularity="tile", block_shape=(16, 16), matrix_shape=None,
                    rounding="nearest", rounding_step=0, rounding_key=0):
    """m = beta*deq(q) + (1-beta)*grad/loss_scale; (next_q, next_scales) = e4m3 tiles of m;
    out = bf16 update (Nesterov or plain). q/next_q and scales/next_scales may alias."""
    assert grad.is_cuda and out.dtype == torch.bfloat16
    flat = grad.reshape(-1)
    n = flat.numel()
    geometry = _geometry(n, granularity, tile_size, block_shape, matrix_shape)
    _lib.call("viola_momentum_update", _lib.ptr(flat), _lib.code(flat.dtype), _lib.ptr(q), _lib.ptr(scales),
              _lib.ptr(next_q), _lib.ptr(next_scales), _lib.ptr(out), n, float(beta), 1.0 / float(loss_scale),
              int(bool(nesterov)), *geometry, _lib.ROUNDING[rounding], int(rounding_step), int(rounding_key))


def copy_scaled(update, partition, src, dst, count, scale):
    flat = update.contiguous().view(-1)
    _lib.call("viola_copy_scaled", _lib.ptr(flat), _lib.code(flat.dtype), _lib.ptr(partition), _lib.code(partition.dtype),
              int(src), int(dst), int(count), float(scale))


def weight_update(weight, grad, lr, weight_decay, *, update_scale=1.0, rounding="nearest", step=0, key=0, offset=0):
    """weight = weight*(1 - lr*wd) - lr*update_scale*grad in fp32, stored in weight's dtype."""
    assert weight.is_cuda and weight.is_contiguous()
    flat = grad.reshape(-1)
    _lib.call("viola_weight_update", _lib.ptr(weight), _lib.code(weight.dtype), _lib.ptr(flat), _lib.code(flat.dtype),
              weight.numel(), float(lr), float(weight_decay), float(update_scale), _lib.ROUNDING[rounding],
              int(step), int(key), int(offset))


def adam_update(weight, grad, first, second, *, lr, weight_decay, betas, eps, step, rounding="nearest", key=0,
                offset=0, adamw=True, maximize=False, bias_correction=True):
    assert weight.is_cuda and weight.is_contiguous() and first.dtype == second.dtype
    b1, b2 = betas
    flat = grad.reshape(-1)
    _lib.call("viola_adam_update", _lib.ptr(weight), _lib.code(weight.dtype), _lib.ptr(flat), _lib.code(flat.dtype),
              _lib.ptr(first), _lib.ptr(second), _lib.code(first.dtype), weight.numel(), float(lr), float(weight_decay),
              float(b1), float(b2), 1. / (1. - b1 ** step) if bias_correction else 1.,
              1. / (1. - b2 ** step) if bias_correction else 1., float(eps), _lib.ROUNDING[rounding],
              int(step - 1), int(key), int(offset), int(bool(adamw)), int(bool(maximize)))


def _device_table(rows, device, cache):
    """int64 rows as a device tensor; `cache` (a dict) keeps it between calls and it is rebuilt when any entry changes."""
    held = cache.get("rows") if cache is not None else None
    if held == rows:
        return cache["table"]
    staging = torch.tensor(rows, dtype=torch.int64).pin_memory()
    table = staging.to(device, non_blocking=True)
    if cache is not None:
        cache.update(rows=rows, table=table, staging=staging)
    return table


def momentum_update_many(items, *, beta, tile_size=256, nesterov=True, loss_scale=1.0, rounding="nearest", rounding_step=0,
                         cache=None):
    """momentum_update (granularity="tile", state advanced in place) for a list of (grad, q, scales, out, key) with
    equal element counts (whole tiles), in one launch. Returns False, having done nothing, when the tensors do not fit
    the kernel (ragged tiles, small tiles, odd alignment, mixed dtypes)."""
    grad = items[0][0]
    n = grad.numel()
    if tile_size < 256 or n % tile_size or len(items) > 65535:
        return False
    rows = []
    for g, q, s, out, key in items:
        if (g.dtype != grad.dtype or g.numel() != n or not g.is_contiguous() or g.data_ptr() % (4 * g.element_size())
                or q.data_ptr() % 4 or out.data_ptr() % 8 or out.dtype != torch.bfloat16):
            return False
        rows.append((g.data_ptr(), q.data_ptr(), s.data_ptr(), q.data_ptr(), s.data_ptr(), out.data_ptr(), int(key), 0))
    table = _device_table(rows, grad.device, cache)
    _lib.call("viola_momentum_update_table", _lib.ptr(table), len(rows), n // tile_size, _lib.code(grad.dtype), int(tile_size),
              float(beta), 1.0 / float(loss_scale), int(bool(nesterov)), _lib.ROUNDING[rounding], int(rounding_step))
    return True


def weight_update_many(items, lr, weight_decay, *, update_scale=1.0, cache=None):
    """weight_update with nearest rounding for a list of (fp32 weight, update) of equal element counts, one launch.
    Returns False, having done nothing, when the tensors do not fit the kernel."""
    weight, update = items[0]
    n = weight.numel()
    if n % 4 or len(items) > 65535:
        return False
    rows = []
    for w, u in items:
        if (w.dtype != torch.float32 or u.dtype != update.dtype or w.numel() != n or u.numel() != n or not w.is_contiguous()
                or not u.is_contiguous() or w.data_ptr() % 16 or u.data_ptr() % (4 * u.element_size())):
            return False
        rows.append((w.data_ptr(), u.data_ptr()))
    table = _device_table(rows, weight.device, cache)
    _lib.call("viola_weight_update_table", _lib.ptr(table), len(rows), n, _lib.code(update.dtype), float(lr),
              float(weight_decay), float(update_scale))
    return True


def adam_update_many(items, *, lr, weight_decay, betas, eps, step, rounding="nearest", adamw=True, maximize=False,
                     bias_correction=True, cache=None):
    """adam_update for a list of (weight, grad, first, second, key, offset) sharing dtypes and step, in one launch.
    cache: a dict that keeps the device-side pointer table between calls (it is rebuilt when any pointer moves)."""
    weight, grad, first, second, _, _ = items[0]
    b1, b2 = betas
    rows = []
    for w, g, m, v, key, offset in items:
        assert w.is_cuda and w.is_contiguous() and g.is_contiguous() and m.is_contiguous() and v.is_contiguous()
        assert (w.dtype, g.dtype, m.dtype, v.dtype) == (weight.dtype, grad.dtype, first.dtype, first.dtype)
        assert g.numel() == m.numel() == v.numel() == w.numel()
        rows.append((w.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(), w.numel(), int(key), int(offset)))
    table = _device_table(rows, weight.device, cache)
    _lib.call("viola_adam_update_table", _lib.ptr(table), len(rows), max(r[4] for r in rows), _lib.code(weight.dtype),
              _lib.code(grad.dtype), _lib.code(first.dtype), float(lr), float(weight_decay), float(b1), float(b2),
              1. / (1. - b1 ** step) if bias_correction else 1., 1. / (1. - b2 ** step) if bias_correction else 1.,
              float(eps), _lib.ROUNDING[rounding], int(step - 1), int(bool(adamw)), int(bool(maximize)))
