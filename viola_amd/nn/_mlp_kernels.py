"""FP8 GEMMs with the gated-activation forward/backward epilogues fused (operator seam of
viola/nn/_mlp_kernels.py `gemm` :243-277), FP32 group scales."""

import torch

from .. import _lib


def gemm(a, b, sa, sb, *, layer, out_dtype, activation, backward=False, aux=None, bias=None, save=True,
         group_a=None, group_b=None, encode_output=False, save_output_transpose=False):
    """forward: out = act(a.Wg^T) * (a.Wu^T), aux = [g, u] if save; backward: out = [d*u*act'(g), d*act(g)].

    Returns (out, aux, (out_scale, out_t, out_t_scale)); the last triple is the reference's
    in-kernel MXFP8 re-encode of H, which only its E8M0 path produces: always empty here.
    """
    if encode_output or save_output_transpose or layer._native_scaling:
        raise NotImplementedError("in-kernel MXFP8 re-encode of H is not built in viola_amd")
    assert layer._grouped_scaling and a.is_cuda
    a, b, sa, sb = a.contiguous(), b.contiguous(), sa.contiguous(), sb.contiguous()
    m, k = a.shape
    h = b.shape[0] if backward else b.shape[0] // 2
    ga = tuple(group_a or layer.input_group_shape)
    gb = tuple(group_b or layer.weight_group_shape)
    out = torch.empty((m, 2 * h if backward else h), device=a.device, dtype=out_dtype)
    if aux is None:
        aux = torch.empty((m, 2 * h) if save else (0, 0), device=a.device, dtype=out_dtype)
    else:
        assert aux.dtype == out_dtype and aux.is_contiguous() and tuple(aux.shape) == (m, 2 * h)
    bias_c = bias.contiguous() if bias is not None else None
    _lib.call("viola_gated_gemm", _lib.ptr(a), _lib.code(a.dtype), _lib.ptr(b), _lib.code(b.dtype), _lib.ptr(sa), _lib.ptr(sb),
              m, h, k, ga[0], ga[1], gb[0], gb[1], _lib.ptr(bias_c), _lib.code(bias_c.dtype) if bias_c is not None else 0,
              _lib.ptr(aux), _lib.ptr(out), _lib.code(out_dtype), _lib.ACTIVATION[activation], int(backward))
    empty = torch.empty((0, 0), device=a.device, dtype=torch.uint8)
    return out, aux, (empty, out.new_empty((0, 0), dtype=a.dtype), empty)
