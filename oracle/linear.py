"""Linear / gated MLP / variable-group linear forward+backward on CPU.
TEST INFRASTRUCTURE ONLY.

Composition of oracle.grouped: quantize each operand the way the layer does, then
"dequantize and matmul in fp32" (checks/check_grouped_linear.py:64-75,
checks/mlp.py:12-16).
"""

import torch
import torch.nn.functional as F

from . import grouped


def _deq(x, dtype, group, limit=None, transposed=False, native=False):
    q, s = grouped.quantize(x, dtype, group, limit=limit, transposed=transposed, native=native)
    return grouped.dequantize(q, s, group)


def linear(x, w_real, bias, dy, *, fp8=torch.float8_e4m3fn, bwd_fp8=torch.float8_e4m3fn,
           gx=(1, 32), gw=(32, 32), gg=(1, 32), out_dtype=torch.bfloat16, grad_dtype=torch.bfloat16, native=False,
           limits=(None, None, None)):
    """Expected y, dx, dw, db of Linear(scaling='grouped') (check_grouped_linear.py:64-75); native=True is the same
    recipe with E8M0 scales (scaling='mxfp8').

    w_real is the dequantized weight in its original coordinates ([out, in] fp32); limits = the clamp
    magnitudes of (input, weight, gradient) groups, None = the format's maximum (layer._group_limit there).
    """
    x2, dy2 = x.reshape(-1, x.shape[-1]), dy.reshape(-1, dy.shape[-1])
    lx, lw, lg = limits
    ref_x = _deq(x2, fp8, gx, lx, native=native)
    ref_g = _deq(dy2, bwd_fp8, gg, lg, native=native)
    wt = w_real.T if gw[0] >= 32 else _deq(w_real, fp8, gw, lw, transposed=True, native=native)
    xt = _deq(x2, fp8, gx, lx, transposed=True, native=native)
    gt = _deq(dy2, bwd_fp8, gg, lg, transposed=True, native=native)
    y = ref_x @ w_real.T
    if bias is not None:
        y = y + bias.float()
    return dict(y=y.to(out_dtype).reshape(*x.shape[:-1], -1),
                dx=(ref_g @ wt.T).to(out_dtype).reshape(x.shape),
                dw=(gt @ xt.T).to(grad_dtype),
                db=None if bias is None else dy2.sum(0, dtype=grad_dtype))


def activation(name):
    return {"silu": F.silu, "relu": F.relu, "gelu": lambda a: F.gelu(a, approximate="tanh")}[name]


def gated_forward(g, u, name):
    """act(g)*u in fp32 from rounded g, u (viola/nn/_mlp_kernels.py:163-175,190-194)."""
    g, u = g.float(), u.float()
    if name == "silu":
        act = g * (1.0 / (1.0 + torch.exp(-g)))
    elif name == "gelu":
        act = 0.5 * g * (1.0 + torch.tanh(0.7978845608028654 * (g + 0.044715 * g * g * g)))
    else:
        act = g.clamp_min(0.0)
    return act * u


def gated_backward(d, g, u, name):
    """[d*u*act'(g), d*act(g)] (viola/nn/_mlp_kernels.py:158-189, _gated_kernels.py:54-66)."""
    d, g, u = d.float(), g.float(), u.float()
    if name == "silu":
        s = 1.0 / (1.0 + torch.exp(-g))
        act, derivative = g * s, s * (1.0 + g * (1.0 - s))
    elif name == "gelu":
        t = torch.tanh(0.7978845608028654 * (g + 0.044715 * g * g * g))
        act = 0.5 * g * (1.0 + t)
        derivative = 0.5 * (1.0 + t) + 0.5 * g * (1.0 - t * t) * 0.7978845608028654 * (1.0 + 0.134145 * g * g)
    else:
        act, derivative = g.clamp_min(0.0), (g > 0).float()
    return d * u * derivative, d * act


def mlp(x, w_gate_up, b_gate_up, w_down, b_down, dy, *, name="silu", fp8=torch.float8_e4m3fn,
        bwd_fp8=torch.float8_e4m3fn, gx=(1, 32), gw=(32, 32), gg=(1, 32), dtype=torch.bfloat16,
        grad_dtype=torch.bfloat16):
    """Fused gated MLP expected values: the unfused recipe with the same Linear rule
    (checks/mlp.py:12-16), with the rounding points of the fused kernels: g, u and dH are
    rounded to the activation dtype before the fp32 activation math."""
    kw = dict(fp8=fp8, bwd_fp8=bwd_fp8, gx=gx, gw=gw, gg=gg, out_dtype=dtype, grad_dtype=grad_dtype)
    x2 = x.reshape(-1, x.shape[-1])
    dy2 = dy.reshape(-1, dy.shape[-1])
    hidden = w_gate_up.shape[0] // 2
    z = linear(x2, w_gate_up, b_gate_up, torch.zeros(x2.shape[0], 2 * hidden, dtype=dtype), **kw)["y"]
    g, u = z[:, :hidden], z[:, hidden:]
    h = gated_forward(g, u, name).to(dtype)
    down = linear(h, w_down, b_down, dy2, **kw)
    dg, du = gated_backward(down["dx"], g, u, name)
    dz = torch.cat([dg, du], 1).to(dtype)
    up = linear(x2, w_gate_up, b_gate_up, dz, **kw)
    return dict(y=down["y"].reshape(*x.shape[:-1], -1), dx=up["dx"].reshape(x.shape), z=z, h=h, dz=dz,
                dw_gate_up=up["dw"], db_gate_up=up["db"], dw_down=down["dw"], db_down=down["db"])


def varlen_linear(x, weights, counts, dy, **kw):
    """Variable-group (MoE-expert style) linear: an independent Linear per row range.

    NOT in the reference (parity unpinned by it): group g owns rows
    [offset_g, offset_g + counts[g]) of x and dy and weight weights[g] ([out, in] real
    values). Empty groups give zero-row outputs and an all-zero dW.
    """
    ys, dxs, dws = [], [], []
    offset = 0
    for w, count in zip(weights, counts):
        rows = slice(offset, offset + count)
        if count:
            r = linear(x[rows], w, None, dy[rows], **kw)
            ys.append(r["y"]); dxs.append(r["dx"]); dws.append(r["dw"])
        else:
            dws.append(torch.zeros(w.shape, dtype=kw.get("grad_dtype", torch.bfloat16)))
        offset += count
    return dict(y=torch.cat(ys), dx=torch.cat(dxs), dw=torch.stack(dws))
