"""GPU checks at the full sizes of the named configurations, where the CPU oracle would take minutes: the HIP path is
held to size-independent properties (exact ones where the arithmetic gives them) and to a plain fp32 GPU matmul of
the dequantized operands, a library routine whose only difference from the contract is fp32 summation order."""

import math

import pytest
import torch

from conftest import rel_l2

pytestmark = pytest.mark.gpu
E4 = torch.float8_e4m3fn


def _quantized(rows, cols, group, seed):
    from viola_amd.nn import _grouped_kernels as g
    torch.manual_seed(seed)
    x = (torch.randn(rows, cols, device="cuda") * torch.exp2(torch.randint(-3, 4, (rows, 1), device="cuda").float())).bfloat16()
    q, s = g.quantize(x, E4, group)
    return x, q, s


@pytest.mark.parametrize("name,m,k,n,gb", [("forward", 8192, 1024, 4096, (32, 32)), ("dgrad", 8192, 4096, 1024, (32, 32)),
                                          ("wgrad", 4096, 8192, 1024, (1, 32))])
def test_linear_gemms_at_8192x1024x4096(name, m, k, n, gb):
    from viola_amd.nn import _grouped_kernels as g
    _, qa, sa = _quantized(m, k, (1, 32), 1)
    _, qb, sb = _quantized(n, k, gb, 2)
    out = g.gemm(qa, qb, sa, sb, (1, 32), gb, out_dtype=torch.float32)
    reference = g.dequantize(qa, sa, (1, 32)) @ g.dequantize(qb, sb, gb).T
    assert rel_l2(out, reference) < 2e-5
    # exact: scaling every a scale by a power of two scales the result by it
    assert torch.equal(g.gemm(qa, qb, sa * 4, sb, (1, 32), gb, out_dtype=torch.float32), out * 4)
    # exact: rows of a are independent, so permuting them permutes the output rows
    perm = torch.randperm(m, device="cuda")
    assert torch.equal(g.gemm(qa[perm].contiguous(), qb, sa[perm].contiguous(), sb, (1, 32), gb, out_dtype=torch.float32), out[perm])
    # bf16 output is the rounded fp32 output, bias added before the rounding
    bias = torch.randn(n, device="cuda")
    assert torch.equal(g.gemm(qa, qb, sa, sb, (1, 32), gb, out_dtype=torch.bfloat16, bias=bias), (out + bias).bfloat16())


@pytest.mark.parametrize("name,m,k,n,gb", [("forward", 8192, 1024, 4096, (32, 32)), ("dgrad", 8192, 4096, 1024, (32, 32)),
                                          ("wgrad", 4096, 8192, 1024, (1, 32))])
def test_linear_gemms_at_8192x1024x4096_against_the_cpu_oracle(name, m, k, n, gb):
    """The same three products held to the CPU oracle itself, on a sample the oracle finishes in seconds: 96 rows of the
    output spread over the whole matrix (first, last, one per 128-row tile boundary region, random ones) with every
    column, from the device's own codes and scales (which other tests pin to the oracle's bit for bit); the sum is
    taken in float64 on the CPU (the reference's witness, viola/nn/_grouped_tuning.py:40-46)."""
    from oracle import grouped as og
    from viola_amd.nn import _grouped_kernels as g
    _, qa, sa = _quantized(m, k, (1, 32), 1)
    _, qb, sb = _quantized(n, k, gb, 2)
    bias = torch.randn(n, device="cuda")
    out = g.gemm(qa, qb, sa, sb, (1, 32), gb, out_dtype=torch.float32, bias=bias)
    half = g.gemm(qa, qb, sa, sb, (1, 32), gb, out_dtype=torch.bfloat16, bias=bias)
    generator = torch.Generator().manual_seed(5)
    rows = torch.cat([torch.tensor([0, 1, 127, 128, m // 2 - 1, m // 2, m - 129, m - 128, m - 1]),
                      torch.randint(0, m, (87,), generator=generator)]).unique()
    witness = og.gemm(qa[rows.cuda()].cpu(), qb.cpu(), sa[rows.cuda()].cpu(), sb.cpu(), (1, 32), gb, bias=bias.cpu(), witness=True,
                      out_dtype=torch.float64)
    assert rel_l2(out[rows.cuda()], witness) < 2e-5                              # checks/check_grouped_linear.py:36-41
    assert rel_l2(half[rows.cuda()], witness) < 3e-3
    assert (out[rows.cuda()].cpu().double() - witness).abs().max() <= 1e-4 * witness.abs().max()


@pytest.mark.parametrize("rows,cols", [(8192, 1024), (8192, 4096)])
def test_dual_quantizer_at_full_size_against_the_cpu_oracle(rows, cols):
    """X and dY of the benchmark's Linear through the one-read dual-layout quantizer, against the CPU oracle on samples
    that cover both layouts: whole rows for the row-wise codes and scales (a row's groups depend on that row only) and
    whole columns for the transposed ones (a column's groups run along the tokens), bit for bit; the column sums the
    same pass produces against a float64 sum."""
    from oracle import grouped as og
    from viola_amd.nn import _grouped_kernels as g
    torch.manual_seed(6)
    x = (torch.randn(rows, cols, device="cuda") * torch.exp2(torch.randint(-6, 7, (rows, 1), device="cuda").float())).bfloat16()
    q, s, qt, st, column_sum = g.quantize_dual(x, E4, (1, 32), column_sum_dtype=torch.float32)
    generator = torch.Generator().manual_seed(7)
    some_rows = torch.cat([torch.tensor([0, 31, 32, rows - 1]), torch.randint(0, rows, (60,), generator=generator)]).unique()
    some_cols = torch.cat([torch.tensor([0, 63, 64, cols - 1]), torch.randint(0, cols, (60,), generator=generator)]).unique()
    host = x.cpu()
    want_q, want_s = og.quantize(host[some_rows], E4, (1, 32))
    assert torch.equal(q[some_rows.cuda()].cpu().view(torch.uint8), want_q.view(torch.uint8))
    assert torch.equal(s[some_rows.cuda()].cpu(), want_s)
    want_qt, want_st = og.quantize(host[:, some_cols].contiguous(), E4, (1, 32), transposed=True)
    assert torch.equal(qt[some_cols.cuda()].cpu().view(torch.uint8), want_qt.view(torch.uint8))
    assert torch.equal(st[some_cols.cuda()].cpu(), want_st)
    exact = host.double().sum(0)
    assert (column_sum.cpu().double() - exact).abs().max() <= 1e-5 * host.double().abs().sum(0).max()


def test_linear_module_at_8192x1024x4096():
    import viola_amd
    viola_amd.set_gradient_dtype("bf16")
    try:
        torch.manual_seed(3)
        layer = viola_amd.nn.Linear(1024, 4096, device="cuda", dtype=torch.bfloat16, scaling="grouped", forward_dtype="e4m3",
                                    backward_dtype="e4m3", mode="memory", weight_dtype="fp8")
    finally:
        viola_amd.precision._settings["gradient_dtype"] = None
    from viola_amd.nn import _grouped_kernels as g
    x = torch.randn(8192, 1024, device="cuda").bfloat16().requires_grad_()
    dy = (torch.randn(8192, 4096, device="cuda") * 1e-2).bfloat16()
    y = layer(x)
    y.backward(dy)
    w = g.dequantize(layer.weight.detach(), layer.weight_scale, (32, 32))
    xq = g.dequantize(*g.quantize(x.detach(), E4, (1, 32)), (1, 32))
    gq = g.dequantize(*g.quantize(dy, E4, (1, 32)), (1, 32))
    assert rel_l2(y, (xq @ w.T + layer.bias.float()).bfloat16()) < 3e-3
    assert rel_l2(x.grad, (gq @ w).bfloat16()) < 3e-3
    xt = g.dequantize(*g.quantize(x.detach(), E4, (1, 32), transposed=True), (1, 32))
    gt = g.dequantize(*g.quantize(dy, E4, (1, 32), transposed=True), (1, 32))
    assert rel_l2(layer.weight.grad, (gt @ xt.T).bfloat16()) < 3e-3
    assert rel_l2(layer.bias.grad, dy.float().sum(0).bfloat16()) < 3e-3


def test_gated_mlp_gemms_at_16384x4096x11008():
    from viola_amd.nn import _grouped_kernels as g, _mlp_kernels as mk
    m, d, h = 16384, 4096, 11008
    _, qx, sx = _quantized(m, d, (1, 32), 4)
    torch.manual_seed(5)
    w = torch.empty(2 * h, d, device="cuda").uniform_(-1 / 64, 1 / 64)
    qw, sw = g.quantize(w, E4, (32, 32))
    del w
    import types
    recipe = types.SimpleNamespace(_native_scaling=False, _grouped_scaling=True, input_group_shape=(1, 32), weight_group_shape=(32, 32))
    out, aux, _ = mk.gemm(qx, qw, sx, sw, layer=recipe, out_dtype=torch.bfloat16, activation="silu", save=True)
    assert out.shape == (m, h) and aux.shape == (m, 2 * h)
    rows = torch.arange(0, m, 61, device="cuda")                              # a 269-row sample keeps the fp32 reference small
    z = g.dequantize(qx[rows].contiguous(), sx[rows].contiguous(), (1, 32)) @ g.dequantize(qw, sw, (32, 32)).T
    assert rel_l2(aux[rows], z.bfloat16()) < 3e-3
    gate, up = aux[rows, :h].float(), aux[rows, h:].float()
    assert rel_l2(out[rows], (torch.nn.functional.silu(gate) * up).bfloat16()) < 3e-3
    # the fused forward equals the plain GEMM followed by the elementwise kernel
    plain = g.gemm(qx, qw, sx, sw, (1, 32), (32, 32), out_dtype=torch.bfloat16)
    assert torch.equal(plain, aux)
    del plain, z, qx, sx, qw, sw
    # the gated backward at the same size: dz = [d u act'(g) | d act(g)] with d = dY . W_down (a = dY codes, b = the down
    # projection's W^T [hidden, out]); bit-equal to the plain dgrad GEMM followed by the elementwise backward kernel, and
    # on the row sample within bf16 rounding of fp32 math on the dequantized operands
    from viola_amd.nn import _gated_kernels as gk
    _, qg, sg = _quantized(m, d, (1, 32), 6)
    torch.manual_seed(7)
    w2 = torch.empty(h, d, device="cuda").uniform_(-1 / 64, 1 / 64)
    qw2, sw2 = g.quantize(w2, E4, (32, 32))
    del w2
    dz, _, _ = mk.gemm(qg, qw2, sg, sw2, layer=recipe, out_dtype=torch.bfloat16, activation="silu", backward=True, aux=aux,
                       group_a=(1, 32), group_b=(32, 32))
    assert dz.shape == (m, 2 * h)
    dh = g.gemm(qg, qw2, sg, sw2, (1, 32), (32, 32), out_dtype=torch.bfloat16)
    assert torch.equal(dz, gk.gated_backward(aux, dh, "silu"))
    d_ref = (g.dequantize(qg[rows].contiguous(), sg[rows].contiguous(), (1, 32)) @ g.dequantize(qw2, sw2, (32, 32)).T).bfloat16().float()
    sig = torch.sigmoid(gate)
    expect = torch.cat([d_ref * up * (sig * (1 + gate * (1 - sig))), d_ref * gate * sig], 1).bfloat16()
    assert rel_l2(dz[rows], expect) < 6e-3


def test_gated_mlp_gemms_at_16384x4096x11008_against_the_cpu_oracle():
    """The gated forward and backward GEMMs of the MLP at full size, held to the CPU oracle itself on a row sample the
    oracle finishes in seconds (a row of either product depends on that row of the activations only): [g | u] against
    the float64 witness of oracle.grouped.gemm, h and dz against oracle.linear.gated_forward / gated_backward applied to
    the rounded values, as the fused kernels do (viola/nn/_mlp_kernels.py:158-194)."""
    import types
    from oracle import grouped as og, linear as ol
    from viola_amd.nn import _grouped_kernels as g, _mlp_kernels as mk
    m, d, h = 16384, 4096, 11008
    _, qx, sx = _quantized(m, d, (1, 32), 4)
    torch.manual_seed(5)
    w = torch.empty(2 * h, d, device="cuda").uniform_(-1 / 64, 1 / 64)
    qw, sw = g.quantize(w, E4, (32, 32))
    del w
    recipe = types.SimpleNamespace(_native_scaling=False, _grouped_scaling=True, input_group_shape=(1, 32), weight_group_shape=(32, 32))
    out, aux, _ = mk.gemm(qx, qw, sx, sw, layer=recipe, out_dtype=torch.bfloat16, activation="silu", save=True)
    generator = torch.Generator().manual_seed(9)
    rows = torch.cat([torch.tensor([0, 1, 127, 128, m // 2, m - 129, m - 1]), torch.randint(0, m, (25,), generator=generator)]).unique()
    on_gpu = rows.cuda()
    z = og.gemm(qx[on_gpu].cpu(), qw.cpu(), sx[on_gpu].cpu(), sw.cpu(), (1, 32), (32, 32), witness=True, out_dtype=torch.float64)
    assert rel_l2(aux[on_gpu], z) < 3e-3                                      # one bf16 rounding of [g | u]
    z16 = z.to(torch.bfloat16)
    assert (aux[on_gpu].cpu() == z16).float().mean() > 0.99                  # and the same rounded values but for summation order
    gate, up = aux[on_gpu, :h].cpu(), aux[on_gpu, h:].cpu()
    assert rel_l2(out[on_gpu], ol.gated_forward(gate, up, "silu")) < 4e-3
    del qx, sx, qw, sw, z, z16
    _, qg, sg = _quantized(m, d, (1, 32), 6)
    torch.manual_seed(7)
    w2 = torch.empty(h, d, device="cuda").uniform_(-1 / 64, 1 / 64)
    qw2, sw2 = g.quantize(w2, E4, (32, 32))
    del w2
    dz, _, _ = mk.gemm(qg, qw2, sg, sw2, layer=recipe, out_dtype=torch.bfloat16, activation="silu", backward=True, aux=aux,
                       group_a=(1, 32), group_b=(32, 32))
    dh = og.gemm(qg[on_gpu].cpu(), qw2.cpu(), sg[on_gpu].cpu(), sw2.cpu(), (1, 32), (32, 32), witness=True, out_dtype=torch.float64)
    dgate, dup = ol.gated_backward(dh.to(torch.bfloat16), gate, up, "silu")
    assert rel_l2(dz[on_gpu], torch.cat([dgate, dup], 1)) < 6e-3


def test_mlp_module_at_16384x4096x11008():
    """The whole viola_amd.nn.MLP forward + backward at the benchmark's size (grouped recipe, FP8 weight storage, memory
    mode) against fp32 GPU math on dequantized operands: y and dx on a row sample (row-wise quantization is per row, so
    a sample of rows stands alone), the two weight gradients on a sample of their rows with the full token contraction,
    the bias gradients as fp32 column sums."""
    import viola_amd
    from viola_amd.nn import _grouped_kernels as g
    m, d, h = 16384, 4096, 11008
    viola_amd.set_gradient_dtype("bf16")
    try:
        torch.manual_seed(11)
        mlp = viola_amd.nn.MLP(d, h, activation="silu", weight_dtype="fp8", scaling="grouped", mode="memory", backward_dtype="e4m3",
                               device="cuda", dtype=torch.bfloat16)
    finally:
        viola_amd.precision._settings["gradient_dtype"] = None
    x = torch.randn(m, d, device="cuda").bfloat16().requires_grad_()
    dy = torch.randn(m, d, device="cuda").bfloat16()
    y = mlp(x)
    y.backward(dy)
    fake = lambda t, transposed=False: g.dequantize(*g.quantize(t.contiguous(), E4, (1, 32), transposed=transposed), (1, 32))
    w_gu = g.dequantize(mlp.gate_up.weight.detach(), mlp.gate_up.weight_scale, (32, 32))
    w_dn = g.dequantize(mlp.down.weight.detach(), mlp.down.weight_scale, (32, 32))
    b_gu, b_dn = mlp.gate_up.bias.detach().float(), mlp.down.bias.detach().float()

    def hidden(x_rows):
        z = (fake(x_rows) @ w_gu.T + b_gu).bfloat16().float()
        gate, up = z[:, :h], z[:, h:]
        sig = 1 / (1 + torch.exp(-gate))
        return gate, up, sig, (gate * sig * up).bfloat16()

    def hidden_grad(dy_rows, gate, up, sig):
        dh = (fake(dy_rows) @ w_dn).bfloat16().float()
        return torch.cat([dh * up * (sig * (1 + gate * (1 - sig))), dh * gate * sig], 1).bfloat16()

    rows = torch.arange(0, m, 61, device="cuda")
    gate, up, sig, h_rows = hidden(x.detach()[rows])
    assert rel_l2(y[rows], (fake(h_rows) @ w_dn.T + b_dn).bfloat16()) < 4e-3
    dz_rows = hidden_grad(dy[rows], gate, up, sig)
    assert rel_l2(x.grad[rows], (fake(dz_rows) @ w_gu).bfloat16()) < 6e-3
    del gate, up, sig, h_rows, dz_rows
    # weight gradients contract over all 16384 tokens: rebuild h and dz in full (in slices of 2048 tokens)
    h_full = torch.empty(m, h, device="cuda", dtype=torch.bfloat16)
    dz_full = torch.empty(m, 2 * h, device="cuda", dtype=torch.bfloat16)
    for start in range(0, m, 2048):
        part = slice(start, start + 2048)
        gate, up, sig, h_full[part] = hidden(x.detach()[part])
        dz_full[part] = hidden_grad(dy[part], gate, up, sig)
    del gate, up, sig
    assert rel_l2(mlp.down.bias.grad, dy.float().sum(0)) < 3e-3                    # fp32 column sums in another order, one bf16 rounding
    assert rel_l2(mlp.gate_up.bias.grad, dz_full.float().sum(0)) < 4e-3
    out_rows = torch.arange(0, d, 97, device="cuda")
    got = mlp.down.weight.grad[out_rows]
    want = fake(dy[:, out_rows], transposed=True) @ fake(h_full, transposed=True).T
    assert rel_l2(got, want.bfloat16()) < 5e-3, rel_l2(got, want)
    del want, h_full
    hidden_rows = torch.arange(0, 2 * h, 501, device="cuda")
    got = mlp.gate_up.weight.grad[hidden_rows]
    want = fake(dz_full[:, hidden_rows], transposed=True) @ fake(x.detach(), transposed=True).T
    assert rel_l2(got, want.bfloat16()) < 6e-3, rel_l2(got, want)


@pytest.mark.parametrize("recipe", ["tensor", "mxfp8"])
def test_gated_mlp_gemms_other_recipes_at_16384x4096x11008(recipe):
    """The gated epilogues under per-tensor and E8M0 scales at the full MLP shape: the fused forward's [g, u] is the
    plain GEMM's output bit for bit, h is the elementwise kernel's to rounding, and the gated backward equals the plain
    dgrad GEMM followed by the elementwise backward kernel bit for bit (same expressions, same rounding points)."""
    import types
    from viola_amd.nn import _gated_kernels as gk, _grouped_kernels as g, _linear_kernels as lk, _mlp_kernels as mk
    m, d, h = 16384, 4096, 11008
    torch.manual_seed(6)
    x = (torch.randn(m, d, device="cuda") * torch.exp2(torch.randint(-3, 4, (m, 1), device="cuda").float())).bfloat16()
    w = torch.empty(2 * h, d, device="cuda").uniform_(-1 / 64, 1 / 64)
    dy = torch.randn(m, d, device="cuda").bfloat16()
    w2 = torch.empty(h, d, device="cuda").uniform_(-1 / 64, 1 / 64)          # the down projection's W^T: [hidden, out]
    if recipe == "mxfp8":
        layer = types.SimpleNamespace(_native_scaling=True, _grouped_scaling=True, input_group_shape=(1, 32), weight_group_shape=(32, 32))
        (qx, sx), (qw, sw) = g.quantize(x, E4, (1, 32), native=True), g.quantize(w, E4, (32, 32), native=True)
        (qg, sg), (qw2, sw2) = g.quantize(dy, E4, (1, 32), native=True), g.quantize(w2, E4, (32, 32), native=True)
        plain = lambda a, b, sa, sb: g.gemm(a, b, sa, sb, (1, 32), (32, 32), out_dtype=torch.bfloat16, native=True)
        extra = dict(group_a=(1, 32), group_b=(32, 32))
    else:
        layer = types.SimpleNamespace(_native_scaling=False, _grouped_scaling=False)
        sx, sw, sg, sw2 = (lk.tensor_scale(t) for t in (x, w, dy, w2))
        qx, qw, qg, qw2 = (lk.quantize(t, s)[0] for t, s in ((x, sx), (w, sw), (dy, sg), (w2, sw2)))
        plain = lambda a, b, sa, sb: lk.gemm(a, b, sa, sb, out_dtype=torch.bfloat16)
        extra = {}
    del w, w2
    out, aux, _ = mk.gemm(qx, qw, sx, sw, layer=layer, out_dtype=torch.bfloat16, activation="silu", save=True)
    assert out.shape == (m, h) and aux.shape == (m, 2 * h)
    assert torch.equal(aux, plain(qx, qw, sx, sw))
    assert rel_l2(out, gk.gated_forward(aux, "silu")[1]) < 3e-3              # the operator divides, the epilogue multiplies by 1 / (1 + exp(-g))
    rows = torch.arange(0, m, 61, device="cuda")
    assert rel_l2(out[rows], (torch.nn.functional.silu(aux[rows, :h].float()) * aux[rows, h:].float()).bfloat16()) < 3e-3
    dz, _, _ = mk.gemm(qg, qw2, sg, sw2, layer=layer, out_dtype=torch.bfloat16, activation="silu", backward=True, aux=aux, **extra)
    assert torch.equal(dz, gk.gated_backward(aux, plain(qg, qw2, sg, sw2), "silu"))


@pytest.mark.parametrize("scaling,backward", [("current", "e5m2"), ("mxfp8", "e4m3")])
def test_linear_module_other_recipes_at_8192x1024x4096(scaling, backward):
    """The headline layer under the per-tensor and the MXFP8 recipe against fp32 GPU matmuls of the dequantized operands."""
    import viola_amd
    from viola_amd.nn import _grouped_kernels as g, _linear_kernels as lk
    viola_amd.set_gradient_dtype("bf16")
    try:
        torch.manual_seed(3)
        layer = viola_amd.nn.Linear(1024, 4096, device="cuda", dtype=torch.bfloat16, scaling=scaling, forward_dtype="e4m3",
                                    backward_dtype=backward, mode="memory", weight_dtype="fp8")
    finally:
        viola_amd.precision._settings["gradient_dtype"] = None
    bwd = torch.float8_e5m2 if backward == "e5m2" else E4
    x = torch.randn(8192, 1024, device="cuda").bfloat16().requires_grad_()
    dy = (torch.randn(8192, 4096, device="cuda") * 1e-2).bfloat16()
    y = layer(x)
    y.backward(dy)
    w = layer.dequantize_weight()
    if scaling == "mxfp8":
        deq = lambda t, fmt, transposed=False: g.dequantize(*g.quantize(t, fmt, (1, 32), native=True, transposed=transposed), (1, 32))
        xq, gq, xt, gt = deq(x.detach(), E4), deq(dy, bwd), deq(x.detach(), E4, True), deq(dy, bwd, True)
    else:
        fake = lambda t, fmt: lk.quantize(t, lk.tensor_scale(t, fp8_dtype=fmt), fp8_dtype=fmt)[0].float() * lk.tensor_scale(t, fp8_dtype=fmt)
        xq, gq = fake(x.detach(), E4), fake(dy, bwd)
        xt, gt = xq.T, gq.T
    assert rel_l2(y, (xq @ w.T + layer.bias.float()).bfloat16()) < 3e-3
    assert rel_l2(x.grad, (gq @ w).bfloat16()) < 3e-3
    assert rel_l2(layer.weight.grad, (gt @ xt.T).bfloat16()) < 3e-3
    assert rel_l2(layer.bias.grad, dy.float().sum(0).bfloat16()) < 3e-3


def test_variable_groups_at_16x32768x4096x1024():
    from viola_amd.nn import _varlen as v, _grouped_kernels as g
    groups, k, n, total = 16, 4096, 1024, 32768
    generator = torch.Generator().manual_seed(6)
    counts = torch.bincount(torch.multinomial(torch.ones(groups) / groups, total, replacement=True, generator=generator), minlength=groups)
    counts[3] += counts[5] - 3
    counts[5] = 3
    counts[7] += counts[9]
    counts[9] = 0
    counts = counts.tolist()
    assert sum(counts) == total
    torch.manual_seed(7)
    x = torch.randn(total, k, device="cuda").bfloat16().requires_grad_()
    dy = torch.randn(total, n, device="cuda").bfloat16()
    experts = v.GroupedExperts(groups, k, n, device="cuda")
    y = experts(x, counts)
    y.backward(dy)
    w = experts.dequantize_weight()
    xq = g.dequantize(*g.quantize(x.detach(), E4, (1, 32)), (1, 32))
    gq = g.dequantize(*g.quantize(dy, E4, (1, 32)), (1, 32))
    start = 0
    for group, count in enumerate(counts):
        rows = slice(start, start + count)
        if count:
            assert rel_l2(y[rows], (xq[rows] @ w[group].T).bfloat16()) < 3e-3, group
            assert rel_l2(x.grad[rows], (gq[rows] @ w[group]).bfloat16()) < 3e-3, group
        else:
            assert experts.weight.grad[group].count_nonzero() == 0
        start += count
    # weight gradient of one full and one tiny group against the quantized transposes
    for group in (0, 5):
        begin = sum(counts[:group])
        rows = slice(begin, begin + counts[group])
        xt = g.dequantize(*g.quantize(x.detach()[rows].contiguous(), E4, (1, 32), transposed=True), (1, 32))
        gt = g.dequantize(*g.quantize(dy[rows].contiguous(), E4, (1, 32), transposed=True), (1, 32))
        assert rel_l2(experts.weight.grad[group], gt @ xt.T) < 3e-3, group


def test_variable_groups_at_16x32768x4096x1024_against_the_cpu_oracle():
    """The variable-group step at full size against the CPU oracle's Linear (oracle.linear.linear, which
    oracle.linear.varlen_linear applies per group): y and dx on a few rows of a full group, of the 3-row group and of the
    largest one (row-wise quantization makes a row's result depend on that row and the group's weight only), and the
    whole weight gradient of the 3-row group and of one full group."""
    from oracle import linear as ol
    from viola_amd.nn import _varlen as v
    groups, k, n, total = 16, 4096, 1024, 32768
    generator = torch.Generator().manual_seed(6)
    counts = torch.bincount(torch.multinomial(torch.ones(groups) / groups, total, replacement=True, generator=generator), minlength=groups)
    counts[3] += counts[5] - 3
    counts[5] = 3
    counts[7] += counts[9]
    counts[9] = 0
    counts = counts.tolist()
    torch.manual_seed(7)
    x = torch.randn(total, k, device="cuda").bfloat16().requires_grad_()
    dy = torch.randn(total, n, device="cuda").bfloat16()
    experts = v.GroupedExperts(groups, k, n, device="cuda")
    y = experts(x, counts)
    y.backward(dy)
    weights = experts.dequantize_weight().float().cpu()
    starts = [sum(counts[:group]) for group in range(groups)]
    for group in (0, 5, 3):
        begin, count = starts[group], counts[group]
        picks = torch.tensor(sorted({0, 1, count // 2, count - 1} & set(range(count)))) + begin
        want = ol.linear(x.detach()[picks.cuda()].cpu(), weights[group], None, dy[picks.cuda()].cpu())
        assert rel_l2(y[picks.cuda()], want["y"]) < 3e-3, group
        assert rel_l2(x.grad[picks.cuda()], want["dx"]) < 3e-3, group
    for group in (5, 0):
        rows = slice(starts[group], starts[group] + counts[group])
        want = ol.linear(x.detach()[rows].cpu(), weights[group], None, dy[rows].cpu(), grad_dtype=torch.float32)
        assert rel_l2(experts.weight.grad[group], want["dw"]) < 3e-3, group
    assert experts.weight.grad[9].count_nonzero() == 0


@pytest.mark.parametrize("method", ["standard", "gram"])
def test_newton_schulz_batched_equals_single_at_ditxl_shapes(method):
    from viola_amd.optim._orthogonalize import METHODS
    torch.manual_seed(8)
    for shape in ((3456, 1152), (1152, 1152), (1152, 4608)):
        batch = torch.randn(3, *shape, device="cuda").bfloat16()
        together = METHODS[method](batch, steps=5)
        for i in range(3):
            assert torch.equal(METHODS[method](batch[i:i + 1].clone(), steps=5)[0], together[i]), (shape, i)
        sigma = torch.linalg.svdvals(together[0].float())
        # a square Gaussian matrix has singular values arbitrarily close to zero, which five steps do not lift
        assert sigma.max() < 1.3 and (shape[0] == shape[1] or sigma.min() > .3), (shape, float(sigma.min()), float(sigma.max()))


@pytest.mark.parametrize("method,rounding", [("standard", "nearest"), ("gram", "nearest"), ("standard", "stochastic"), ("gram", "stochastic")])
def test_fp8muon_step_at_ditxl_block(method, rounding):
    """One transformer block of the DiT-XL set, two steps: the batched step equals stepping each parameter in its own
    optimizer, bit for bit, for both Newton-Schulz methods and both roundings of the momentum state (the stochastic
    rounding key depends on the parameter's index only, which the stand-alone optimizers are given)."""
    import viola_amd
    d = 1152
    shapes = ((3 * d, d), (d, d), (4 * d, d), (d, 4 * d), (d,), (3 * d,))

    def build(seed):
        torch.manual_seed(seed)
        params = [torch.nn.Parameter(torch.randn(*s, device="cuda") * .02) for s in shapes for _ in range(2)]
        for p in params:
            p.grad = torch.randn_like(p) * 1e-3
        return params

    options = dict(lr=1e-3, weight_decay=.01, adjust_lr_fn="match_rms_adamw", mode="balanced", tile_size=256, ns_method=method,
                   rounding=rounding, rounding_seed=42)
    together = build(9)
    batched = viola_amd.optim.FP8Muon(together, **options)
    batched.step()
    batched.step()
    alone = build(9)
    singles = []
    for index, p in enumerate(alone):
        singles.append(viola_amd.optim.FP8Muon([{"params": [p], "viola_parameter_indices": [index]}], **options))
        singles[-1].step()
        singles[-1].step()
    for a, b, opt in zip(together, alone, singles):
        assert torch.equal(a, b) and torch.isfinite(a).all()
        if a.ndim == 2:
            assert torch.equal(batched.state[a]["momentum_q"], opt.state[b]["momentum_q"])
            assert torch.equal(batched.state[a]["momentum_scale"], opt.state[b]["momentum_scale"])
    if rounding == "stochastic":
        nearest = build(9)
        viola_amd.optim.FP8Muon(nearest, **{**options, "rounding": "nearest"}).step()
        again = build(9)
        first = viola_amd.optim.FP8Muon(again, **options)
        first.step()
        # one step: the update itself does not depend on the rounding of the state that is stored for the next one
        assert all(torch.equal(a, b) for a, b in zip(nearest, again))


@pytest.mark.parametrize("method", ["standard", "gram"])
def test_fp8muon_step_at_the_ditxl_set(method):
    """The optimizer benchmark's whole parameter set (28 transformer blocks of width 1152: 112 matrices in three shape
    buckets of 28 and 56, plus the bias vectors), two steps: the batched step, whose Newton-Schulz products run on the
    large tiles that only a batch of this size selects, equals stepping every parameter in an optimizer of its own,
    bit for bit, weights and momentum state."""
    import viola_amd
    from viola_amd.optim import _orthogonalize_kernels as nk
    d, blocks = 1152, 28
    shapes = ((3 * d, d), (d, d), (4 * d, d), (d, 4 * d), (3 * d,), (d,), (4 * d,), (d,))
    assert nk.plan(blocks, d, 3 * d, d)["kernel"] != nk.plan(1, d, 3 * d, d)["kernel"]

    def build(seed):
        torch.manual_seed(seed)
        params = [torch.nn.Parameter(torch.randn(*s, device="cuda") * .02) for _ in range(blocks) for s in shapes]
        for p in params:
            p.grad = torch.randn_like(p) * 1e-3
        return params

    options = dict(lr=1e-3, weight_decay=.01, adjust_lr_fn="match_rms_adamw", mode="balanced", tile_size=256, ns_method=method,
                   rounding="nearest", rounding_seed=42)
    together = build(10)
    batched = viola_amd.optim.FP8Muon(together, **options)
    batched.step()
    batched.step()
    alone = build(10)
    for index, (a, b) in enumerate(zip(together, alone)):
        single = viola_amd.optim.FP8Muon([{"params": [b], "viola_parameter_indices": [index]}], **options)
        single.step()
        single.step()
        assert torch.equal(a, b) and torch.isfinite(a).all(), (index, tuple(a.shape))
        if a.ndim == 2:
            assert torch.equal(batched.state[a]["momentum_q"], single.state[b]["momentum_q"]), index
            assert torch.equal(batched.state[a]["momentum_scale"], single.state[b]["momentum_scale"]), index
        b.grad = None
        del single


@pytest.mark.parametrize("recipe", ["tensor", "mxfp8"])
@pytest.mark.parametrize("m,n,k,formats", [(4096, 12288, 256, (E4, E4)), (4100, 12300, 384, (torch.float8_e5m2, E4)),
                                           (8192, 8192, 1024, (E4, torch.float8_e5m2))])
def test_large_tile_gemm_of_the_fold_free_recipes(recipe, m, n, k, formats):
    """Products with at least 512 tiles of 256 x 256 take the one-block-per-CU kernel of the per-tensor and MXFP8
    recipes: held to an fp32 GPU matmul of the dequantized operands (ragged edges in m and n included), to the bias
    and rounding identity, and to the 128 x 128 kernel's result on a row sample (same products, same K order)."""
    from viola_amd.nn import _grouped_kernels as g, _linear_kernels as lk
    torch.manual_seed(8)
    a = (torch.randn(m, k, device="cuda") * torch.exp2(torch.randint(-3, 4, (m, 1), device="cuda").float())).bfloat16()
    b = (torch.randn(n, k, device="cuda") * torch.exp2(torch.randint(-3, 4, (n, 1), device="cuda").float())).bfloat16()
    bias = torch.randn(n, device="cuda")
    if recipe == "mxfp8":
        (qa, sa), (qb, sb) = g.quantize(a, formats[0], (1, 32), native=True), g.quantize(b, formats[1], (32, 32), native=True)
        run = lambda qa_, sa_, **kw: g.gemm(qa_, qb, sa_, sb, (1, 32), (32, 32), native=True, **kw)
        reference = g.dequantize(qa, sa, (1, 32)) @ g.dequantize(qb, sb, (32, 32)).T
    else:
        sa, sb = lk.tensor_scale(a, fp8_dtype=formats[0]), lk.tensor_scale(b, fp8_dtype=formats[1])
        qa, qb = lk.quantize(a, sa, fp8_dtype=formats[0])[0], lk.quantize(b, sb, fp8_dtype=formats[1])[0]
        run = lambda qa_, sa_, **kw: lk.gemm(qa_, qb, sa_, sb, **kw)
        reference = (qa.float() * sa) @ (qb.float() * sb).T
    out = run(qa, sa, out_dtype=torch.float32)
    assert rel_l2(out, reference) < 2e-5
    assert torch.equal(run(qa, sa, out_dtype=torch.bfloat16, bias=bias), (out + bias).bfloat16())
    rows = torch.arange(0, m, 37, device="cuda")[:96]                         # 96 rows: far below the large-tile threshold
    sample = run(qa[rows].contiguous(), sa[rows].contiguous() if recipe == "mxfp8" else sa, out_dtype=torch.float32)
    assert torch.equal(sample, out[rows])


@pytest.mark.parametrize("out_dtype,activation", [(torch.bfloat16, "gelu"), (torch.float16, "gelu"), (torch.bfloat16, "silu"), (torch.float16, "relu"),
                                                  (torch.float32, "silu")])
@pytest.mark.parametrize("recipe", ["tensor", "mxfp8"])
def test_large_tile_gated_gemms_equal_the_small_tile_kernels(recipe, out_dtype, activation):
    """m = 8256, h = 6208: with [g, u] kept, the gated forward and backward products run as the plain GEMM on 256-row
    tiles plus one elementwise pass (backward in place in the up half of dz); without it the per-tensor forward runs
    the gated epilogue on 256-row tiles and the MXFP8 one on 128 x 128; a 96-row sample of the same operands runs
    the gated epilogues of the 128 x 128 kernel. Same products in the same K order and the epilogue's activation expression in the passes:
    bit-equal, for h, [g, u] and dz, and for the MXFP8 codes of h handed to the down projection in either form."""
    import types
    from viola_amd.nn import _grouped_kernels as g, _linear_kernels as lk, _mlp_kernels as mk
    m, h, k, k2 = 8192 + 64, 6208, 256, 384
    torch.manual_seed(12)
    x = (torch.randn(m, k, device="cuda") * torch.exp2(torch.randint(-2, 3, (m, 1), device="cuda").float())).bfloat16()
    w = torch.empty(2 * h, k, device="cuda").uniform_(-1 / 16, 1 / 16)
    dy = torch.randn(m, k2, device="cuda").bfloat16()
    w2 = torch.empty(h, k2, device="cuda").uniform_(-1 / 16, 1 / 16)
    bias = torch.randn(2 * h, device="cuda").to(out_dtype)
    rows = torch.arange(0, m, 83, device="cuda")[:96]
    if recipe == "mxfp8":
        layer = types.SimpleNamespace(_native_scaling=True, _grouped_scaling=True, input_group_shape=(1, 32), weight_group_shape=(32, 32),
                                      fp8_dtype=E4, _group_limit=lambda *a, **kw: None)
        (qx, sx), (qw, sw) = g.quantize(x, E4, (1, 32), native=True), g.quantize(w, E4, (32, 32), native=True)
        (qg, sg), (qw2, sw2) = g.quantize(dy, E4, (1, 32), native=True), g.quantize(w2, E4, (32, 32), native=True)
        pick = lambda q, s: (q[rows].contiguous(), s[rows].contiguous())
        extra = dict(group_a=(1, 32), group_b=(32, 32))
    else:
        layer = types.SimpleNamespace(_native_scaling=False, _grouped_scaling=False)
        sx, sw, sg, sw2 = (lk.tensor_scale(t) for t in (x, w, dy, w2))
        qx, qw, qg, qw2 = (lk.quantize(t, s)[0] for t, s in ((x, sx), (w, sw), (dy, sg), (w2, sw2)))
        pick = lambda q, s: (q[rows].contiguous(), s)
        extra = {}
    out, aux, _ = mk.gemm(qx, qw, sx, sw, layer=layer, out_dtype=out_dtype, bias=bias, activation=activation, save=True)
    small_out, small_aux, _ = mk.gemm(*pick(qx, sx)[:1], qw, pick(qx, sx)[1], sw, layer=layer, out_dtype=out_dtype, bias=bias,
                                      activation=activation, save=True)
    assert torch.equal(out[rows], small_out) and torch.equal(aux[rows], small_aux)
    unsaved, _, _ = mk.gemm(qx, qw, sx, sw, layer=layer, out_dtype=out_dtype, bias=bias, activation=activation, save=False)
    assert torch.equal(unsaved, out)
    dz, _, _ = mk.gemm(qg, qw2, sg, sw2, layer=layer, out_dtype=out_dtype, activation=activation, backward=True, aux=aux, **extra)
    small_dz, _, _ = mk.gemm(pick(qg, sg)[0], qw2, pick(qg, sg)[1], sw2, layer=layer, out_dtype=out_dtype, activation=activation,
                             backward=True, aux=small_aux, **extra)
    assert torch.equal(dz[rows], small_dz)
    if recipe == "mxfp8":
        codes, _, (scale, codes_t, scale_t) = mk.gemm(qx, qw, sx, sw, layer=layer, out_dtype=out_dtype, bias=bias, activation=activation,
                                                      save=False, encode_output=True, save_output_transpose=True)
        want = g.quantize_dual(out, E4, (1, 32), native=True)
        for got, expected in zip((codes, scale, codes_t, scale_t), want):
            assert torch.equal(got.view(torch.uint8), expected.view(torch.uint8))
        codes, kept, (scale, codes_t, scale_t) = mk.gemm(qx, qw, sx, sw, layer=layer, out_dtype=out_dtype, bias=bias, activation=activation,
                                                         save=True, encode_output=True, save_output_transpose=True)
        assert torch.equal(kept, aux)
        for got, expected in zip((codes, scale, codes_t, scale_t), want):
            assert torch.equal(got.view(torch.uint8), expected.view(torch.uint8))
