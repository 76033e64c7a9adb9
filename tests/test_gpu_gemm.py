"""GPU parity: grouped-scale FP8 GEMM, gated GEMMs and the variable-group GEMMs vs the CPU oracle."""

import pytest
import torch

from oracle import grouped as og, linear as ol
from conftest import rel_l2
from viola_amd import _lib

pytestmark = pytest.mark.gpu
E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2


def _operands(m, k, n, ga, gb, fa, fb, seed=2041, spread=5):
    torch.manual_seed(seed)
    a = (torch.randn(m, k) * torch.exp2(torch.randint(-spread, spread + 1, (m, 1)).float())).bfloat16()
    b = (torch.randn(n, k) * torch.exp2(torch.randint(-spread, spread + 1, (n, 1)).float())).bfloat16()
    return og.quantize(a, fa, ga), og.quantize(b, fb, gb)


# shapes and group/format mixes of checks/check_grouped_linear.py:123-126, plus tile-edge and wgrad-like cases
CASES = [((1, 32), (32, 32), (E4, E4), (65, 96, 128)), ((1, 64), (32, 64), (E5, E4), (96, 65, 64)),
         ((32, 64), (64, 32), (E4, E5), (64, 160, 96)), ((1, 32), (32, 32), (E5, E4), (65, 4096, 128)),
         ((1, 32), (1, 32), (E4, E4), (130, 256, 200)), ((1, 32), (32, 32), (E4, E4), (256, 1024, 384)),
         ((1, 32), (1, 32), (E5, E5), (96, 8192, 64)), ((1, 32), (32, 32), (E4, E4), (1, 32, 1)),
         ((1, 32), (32, 32), (E4, E4), (129, 48, 257))]


@pytest.mark.parametrize("ga,gb,formats,shape", CASES)
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_group_gemm(ga, gb, formats, shape, out_dtype):
    from viola_amd.nn import _grouped_kernels as g
    m, k, n = shape
    (qa, sa), (qb, sb) = _operands(m, k, n, ga, gb, *formats)
    bias = torch.randn(n)
    actual = g.gemm(qa.cuda(), qb.cuda(), sa.cuda(), sb.cuda(), ga, gb, out_dtype=out_dtype, bias=bias.cuda())
    expected = og.gemm(qa, qb, sa, sb, ga, gb, bias=bias, witness=True, out_dtype=torch.float64)
    assert actual.dtype == out_dtype and torch.isfinite(actual).all()
    # fp32 out: the reference's own bound (checks/check_grouped_linear.py:41); bf16 out adds half a bf16 ulp
    assert rel_l2(actual, expected) < (2e-5 if out_dtype == torch.float32 else 3e-3)
    for _ in range(2):                                                        # bit-identical on repeat (:43-46)
        again = g.gemm(qa.cuda(), qb.cuda(), sa.cuda(), sb.cuda(), ga, gb, out_dtype=out_dtype, bias=bias.cuda())
        assert torch.equal(again, actual)
    nobias = g.gemm(qa.cuda(), qb.cuda(), sa.cuda(), sb.cuda(), ga, gb, out_dtype=torch.float32)
    assert rel_l2(nobias, og.gemm(qa, qb, sa, sb, ga, gb, witness=True, out_dtype=torch.float64)) < 2e-5


@pytest.mark.parametrize("gb", [(32, 32), (1, 32)])
@pytest.mark.parametrize("k", [96, 160, 224, 288, 32])
def test_group_gemm_scales_past_the_k_range_do_not_leak(gb, k):
    """Scales are stored [rows, k / 32], so what follows a row's last scale in memory is the next row's first one. The
    kernel fetches scales in 16-byte pieces; when k / 32 is not a multiple of four, the last piece of a row reaches into
    the next row, and a NaN or an Inf there (the scale of a group that holds one) must not reach this row's sums."""
    from viola_amd.nn import _grouped_kernels as g
    m, n = 130, 128
    (qa, sa), (qb, sb) = _operands(m, k, n, (1, 32), gb, E4, E4, seed=77)
    qa, sa, qb, sb = qa.cuda(), sa.cuda(), qb.cuda(), sb.cuda()
    clean = g.gemm(qa, qb, sa, sb, (1, 32), gb, out_dtype=torch.float32)
    sa2, sb2 = sa.clone(), sb.clone()
    sa2[5, 0], sa2[77, 0], sa2[129, 0] = float("nan"), float("inf"), float("nan")
    bad_columns = []
    if gb == (1, 32):
        sb2[9, 0] = float("nan")
        bad_columns = [9]
    dirty = g.gemm(qa, qb, sa2, sb2, (1, 32), gb, out_dtype=torch.float32)
    rows = torch.tensor([r for r in range(m) if r not in (5, 77, 129)], device="cuda")
    columns = torch.tensor([c for c in range(n) if c not in bad_columns], device="cuda")
    assert torch.equal(dirty[rows][:, columns], clean[rows][:, columns])
    assert not torch.isfinite(dirty[5]).any() and not torch.isfinite(dirty[129]).any()


@pytest.mark.parametrize("gb", [(1, 32), (32, 32)])
@pytest.mark.parametrize("m,n", [(1930, 1100), (130, 200)])                  # 16 x 9 tiles of 128 x 128; 2 x 4 of 128 x 64
@pytest.mark.parametrize("k,formats", [(2048, (E4, E4)), (2064, (E5, E4)), (2336, (E4, E4)), (4000, (E4, E5)), (6176, (E5, E5))])
def test_group_gemm_long_k_few_tiles(k, formats, m, n, gb):
    """A long k and fewer than 512 output tiles of 128 x 128 (a weight gradient; a small-batch dgrad): the kernel splits
    the k range of a tile (128 x 128 from 129 tiles up, 128 x 64 below) over two teams of waves and adds their sums. k
    values around the split's granularity (256) and with a ragged last scale piece; a NaN / Inf scale in a neighbouring
    row must stay in its row."""
    from viola_amd.nn import _grouped_kernels as g
    (qa, sa), (qb, sb) = _operands(m, k, n, (1, 32), gb, *formats, seed=k, spread=2)    # sums stay inside fp16
    bias = torch.randn(n)
    rows = torch.cat([torch.arange(0, min(m, 140)), torch.arange(min(m, 1900), m)])   # the oracle on row samples: first tiles and the ragged last
    expected = og.gemm(qa[rows], qb, sa[rows], sb, (1, 32), gb, bias=bias, witness=True, out_dtype=torch.float64)
    qa, sa, qb, sb = qa.cuda(), sa.cuda(), qb.cuda(), sb.cuda()
    for out_dtype, bound in ((torch.float32, 2e-5), (torch.bfloat16, 3e-3), (torch.float16, 1e-3)):
        actual = g.gemm(qa, qb, sa, sb, (1, 32), gb, out_dtype=out_dtype, bias=bias.cuda())
        assert actual.dtype == out_dtype and rel_l2(actual[rows.cuda()], expected) < bound
        assert torch.equal(actual, g.gemm(qa, qb, sa, sb, (1, 32), gb, out_dtype=out_dtype, bias=bias.cuda()))
    # every row against an FP32 matmul of the dequantized operands (sums of a different order)
    reference = g.dequantize(qa, sa, (1, 32)).float() @ g.dequantize(qb, sb, gb).float().t() + bias.cuda()
    assert rel_l2(g.gemm(qa, qb, sa, sb, (1, 32), gb, out_dtype=torch.float32, bias=bias.cuda()), reference) < 2e-5
    clean = g.gemm(qa, qb, sa, sb, (1, 32), gb, out_dtype=torch.float32)
    sa2, sb2 = sa.clone(), sb.clone()
    sa2[5, 0], sa2[m - 1, 0] = float("nan"), float("inf")
    bad_columns = []
    if gb == (1, 32):
        sb2[9, 0] = float("nan")
        bad_columns = [9]
    dirty = g.gemm(qa, qb, sa2, sb2, (1, 32), gb, out_dtype=torch.float32)
    keep = torch.tensor([r for r in range(m) if r not in (5, m - 1)], device="cuda")
    columns = torch.tensor([c for c in range(n) if c not in bad_columns], device="cuda")
    assert torch.equal(dirty[keep][:, columns], clean[keep][:, columns])
    assert not torch.isfinite(dirty[5]).any() and not torch.isfinite(dirty[m - 1]).any()


def test_group_gemm_special_structure():
    """Identity-like operands make the expected value exact: catches a transposed operand or a wrong scale index."""
    from viola_amd.nn import _grouped_kernels as g
    m = n = k = 128
    a = torch.eye(m, k) * torch.arange(1, m + 1).float()[:, None]
    b = torch.randn(n, k).bfloat16().float()
    qa, sa = og.quantize(a, E4, (1, 32))
    qb, sb = og.quantize(b, E4, (32, 32))
    out = g.gemm(qa.cuda(), qb.cuda(), sa.cuda(), sb.cuda(), (1, 32), (32, 32), out_dtype=torch.float32).cpu()
    expect = og.dequantize(qa, sa, (1, 32)) @ og.dequantize(qb, sb, (32, 32)).T
    assert torch.allclose(out, expect, rtol=1e-6, atol=0)
    assert not torch.allclose(out, expect.T, rtol=1e-3, atol=0)


class _Layer:
    """The attributes the gated GEMM wrapper reads from a Linear."""
    _grouped_scaling, _native_scaling = True, False
    input_group_shape, weight_group_shape = (1, 32), (32, 32)


@pytest.mark.parametrize("activation", ["silu", "gelu", "relu"])
@pytest.mark.parametrize("m,h,k", [(66, 160, 128), (130, 64, 96), (64, 40, 64)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gated_gemm_forward_backward(activation, m, h, k, dtype):
    from viola_amd.nn import _mlp_kernels as mk
    gw = (32, 32) if h % 32 == 0 else (1, 32)
    layer = _Layer()
    layer.weight_group_shape = gw
    spread = 5 if dtype == torch.bfloat16 else 1                              # keep g*u inside fp16's range
    (qa, sa), (qb, sb) = _operands(m, k, 2 * h, (1, 32), gw, E4, E4, seed=131, spread=spread)
    bias = torch.randn(2 * h).to(dtype)
    out, aux, _ = mk.gemm(qa.cuda(), qb.cuda(), sa.cuda(), sb.cuda(), layer=layer, out_dtype=dtype, bias=bias.cuda(),
                          activation=activation, save=True)
    z = og.gemm(qa, qb, sa, sb, (1, 32), gw, bias=bias.float()).to(dtype)
    assert rel_l2(aux, z) < 4e-3
    expect = ol.gated_forward(aux.cpu()[:, :h], aux.cpu()[:, h:], activation).to(dtype)     # from the saved g, u
    assert rel_l2(out, expect) < 4e-3
    nosave, aux2, _ = mk.gemm(qa.cuda(), qb.cuda(), sa.cuda(), sb.cuda(), layer=layer, out_dtype=dtype, bias=bias.cuda(),
                              activation=activation, save=False)
    assert aux2.numel() == 0 and torch.equal(nosave, out)
    # backward: d = a2 . w2^T with w2 [h, k2]
    k2 = 96
    (qg, sg), (qw, sw) = _operands(m, k2, h, (1, 32), (32, 32), E4, E4, seed=17, spread=spread)
    dz, _, _ = mk.gemm(qg.cuda(), qw.cuda(), sg.cuda(), sw.cuda(), layer=layer, out_dtype=dtype, backward=True,
                       activation=activation, aux=aux, group_a=(1, 32), group_b=(32, 32))
    d = og.gemm(qg, qw, sg, sw, (1, 32), (32, 32)).to(dtype)
    dg, du = ol.gated_backward(d, aux.cpu()[:, :h], aux.cpu()[:, h:], activation)
    assert dz.shape == (m, 2 * h) and rel_l2(dz, torch.cat([dg, du], 1).to(dtype)) < 6e-3


class _TensorLayer:
    _grouped_scaling, _native_scaling = False, False


class _NativeLayer(_Layer):
    _native_scaling = True


@pytest.mark.parametrize("recipe", ["tensor", "mxfp8"])
@pytest.mark.parametrize("activation,formats", [("silu", (E4, E4)), ("gelu", (E5, E4)), ("relu", (E4, E5))])
@pytest.mark.parametrize("m,h,k,k2", [(66, 160, 128, 256), (130, 64, 96, 96), (64, 40, 64, 128), (300, 256, 384, 128)])
def test_gated_gemm_other_recipes(recipe, activation, formats, m, h, k, k2):
    """viola_tensor_gated_gemm / viola_mx_gated_gemm (viola/nn/_mlp_kernels.py:157-194 with `grouped` false or native
    scales): aux = the plain GEMM's [g, u], out = act(g) * u, and the backward pair, for aligned shapes (the fused
    kernels) and others (generic kernel, or plain GEMM + elementwise kernels)."""
    from viola_amd.nn import _mlp_kernels as mk
    from oracle import tensor as ot
    dtype = torch.bfloat16
    native = recipe == "mxfp8"
    torch.manual_seed(7)
    a = (torch.randn(m, k) * torch.exp2(torch.randint(-3, 4, (m, 1)).float())).bfloat16()
    w = (torch.randn(2 * h, k) * torch.exp2(torch.randint(-3, 4, (2 * h, 1)).float())).bfloat16()
    dy = (torch.randn(m, k2) * torch.exp2(torch.randint(-3, 4, (m, 1)).float())).bfloat16()
    w2 = (torch.randn(h, k2) * torch.exp2(torch.randint(-3, 4, (h, 1)).float())).bfloat16()
    bias = torch.randn(2 * h).to(dtype)
    if native:
        gw = (32, 32) if h % 32 == 0 else (1, 32)
        layer = _NativeLayer()
        layer.weight_group_shape = gw
        (qa, sa), (qb, sb) = og.quantize(a, formats[0], (1, 32), native=True), og.quantize(w, formats[1], gw, native=True)
        (qg, sg), (qw, sw) = og.quantize(dy, formats[0], (1, 32), native=True), og.quantize(w2, formats[1], (32, 32), native=True)
        z = og.gemm(qa, qb, og.decode_scale(sa), og.decode_scale(sb), (1, 32), gw, bias=bias.float()).to(dtype)
        d = og.gemm(qg, qw, og.decode_scale(sg), og.decode_scale(sw), (1, 32), (32, 32)).to(dtype)
        extra = dict(group_a=(1, 32), group_b=(32, 32))
    else:
        layer = _TensorLayer()
        zero = torch.zeros(1)
        sa, sb = ot.tensor_scale(a, zero, 0, limit=torch.finfo(formats[0]).max)[0], ot.tensor_scale(w, zero, 0, limit=torch.finfo(formats[1]).max)[0]
        sg, sw = ot.tensor_scale(dy, zero, 0, limit=torch.finfo(formats[0]).max)[0], ot.tensor_scale(w2, zero, 0, limit=torch.finfo(formats[1]).max)[0]
        qa, qb, qg, qw = ot.quantize(a, sa, formats[0]), ot.quantize(w, sb, formats[1]), ot.quantize(dy, sg, formats[0]), ot.quantize(w2, sw, formats[1])
        z = ot.gemm(qa, qb, sa, sb, bias=bias, out_dtype=dtype)
        d = ot.gemm(qg, qw, sg, sw, out_dtype=dtype)
        extra = {}
    out, aux, _ = mk.gemm(qa.cuda(), qb.cuda(), sa.cuda(), sb.cuda(), layer=layer, out_dtype=dtype, bias=bias.cuda(),
                          activation=activation, save=True)
    assert aux.shape == (m, 2 * h) and rel_l2(aux, z) < 4e-3
    assert rel_l2(out, ol.gated_forward(aux.cpu()[:, :h], aux.cpu()[:, h:], activation).to(dtype)) < 4e-3
    nosave, aux2, _ = mk.gemm(qa.cuda(), qb.cuda(), sa.cuda(), sb.cuda(), layer=layer, out_dtype=dtype, bias=bias.cuda(),
                              activation=activation, save=False)
    assert aux2.numel() == 0 and torch.equal(nosave, out)
    dz, _, _ = mk.gemm(qg.cuda(), qw.cuda(), sg.cuda(), sw.cuda(), layer=layer, out_dtype=dtype, backward=True,
                       activation=activation, aux=aux, **extra)
    dg, du = ol.gated_backward(d, aux.cpu()[:, :h], aux.cpu()[:, h:], activation)
    assert dz.shape == (m, 2 * h) and rel_l2(dz, torch.cat([dg, du], 1).to(dtype)) < 6e-3


@pytest.mark.parametrize("activation", ["silu", "gelu", "relu"])
def test_gated_elementwise(activation):
    from viola_amd.nn._gated_kernels import GatedActivation
    torch.manual_seed(3)
    z = torch.randn(5, 33, 2 * 72).bfloat16().cuda().requires_grad_()
    out = GatedActivation.apply(z, activation, False)
    dy = torch.randn_like(out)
    out.backward(dy)
    g, u = z.detach().cpu()[..., :72], z.detach().cpu()[..., 72:]
    assert rel_l2(out, ol.gated_forward(g, u, activation).bfloat16()) < 3e-3
    dg, du = ol.gated_backward(dy.cpu(), g, u, activation)
    assert rel_l2(z.grad, torch.cat([dg, du], -1).bfloat16()) < 4e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("activation", ["silu", "gelu", "relu"])
def test_gated_elementwise_pieces_equal_the_scalar_kernel(dtype, activation):
    """Rows of 16-byte pieces take the vectorised kernels, anything else the element-wise ones: the same values bit
    for bit (hidden 160 against the same data at hidden 160 behind a one-element pointer offset), and against the
    oracle at an odd hidden size."""
    from viola_amd.nn import _gated_kernels as gk
    torch.manual_seed(11)
    rows, hidden = 77, 160
    z = (torch.randn(rows, 2 * hidden) * 3).to(dtype).cuda()
    dy = torch.randn(rows, hidden).to(dtype).cuda()
    _, out = gk.gated_forward(z, activation)
    dz = gk.gated_backward(z, dy, activation)
    shifted_z = torch.empty(z.numel() + 1, device="cuda", dtype=dtype)[1:].view_as(z).copy_(z)      # 2- or 4-byte aligned only
    shifted_dy = torch.empty(dy.numel() + 1, device="cuda", dtype=dtype)[1:].view_as(dy).copy_(dy)
    assert shifted_z.data_ptr() % 16 != 0 and shifted_z.is_contiguous()
    _, out_scalar = gk.gated_forward(shifted_z, activation)
    dz_scalar = gk.gated_backward(shifted_z, shifted_dy, activation)
    assert torch.equal(out, out_scalar) and torch.equal(dz, dz_scalar)
    g, u = z.cpu()[:, :hidden], z.cpu()[:, hidden:]
    assert rel_l2(out, ol.gated_forward(g, u, activation).to(dtype)) < 4e-3
    dg, du = ol.gated_backward(dy.cpu(), g, u, activation)
    assert rel_l2(dz, torch.cat([dg, du], -1).to(dtype)) < 4e-3
    odd = (torch.randn(9, 2 * 37) * 3).to(dtype).cuda()
    _, out_odd = gk.gated_forward(odd, activation)
    assert rel_l2(out_odd, ol.gated_forward(odd.cpu()[:, :37], odd.cpu()[:, 37:], activation).to(dtype)) < 4e-3


@pytest.mark.parametrize("counts", [[130, 0, 3, 64, 1, 200], [5], [0, 0, 7]])
def test_varlen_group_gemm_and_wgrad(counts):
    from viola_amd.nn import _varlen as v
    groups, k, n = len(counts), 128, 96
    total = sum(counts)
    torch.manual_seed(5)
    x = torch.randn(total, k).bfloat16()
    dy = torch.randn(total, n).bfloat16()
    w = torch.randn(groups, n, k) / 11
    qw = torch.stack([og.quantize(w[g], E4, (32, 32))[0] for g in range(groups)])
    sw = torch.stack([og.quantize(w[g], E4, (32, 32))[1] for g in range(groups)])
    wreal = [og.dequantize(qw[g], sw[g], (32, 32)) for g in range(groups)]
    expect = ol.varlen_linear(x, wreal, counts, dy, grad_dtype=torch.float32)
    xg = x.cuda().requires_grad_()
    wparam = torch.nn.Parameter(qw.cuda())
    wparam.grad_dtype = torch.float32
    y = v.grouped_linear(xg, wparam, sw.cuda(), counts)
    y.backward(dy.cuda())
    assert rel_l2(y, expect["y"]) < 3e-3 and rel_l2(xg.grad, expect["dx"]) < 3e-3
    assert wparam.grad.shape == (groups, n, k) and rel_l2(wparam.grad, expect["dw"]) < 2e-5
    for g, c in enumerate(counts):
        if c == 0:
            assert wparam.grad[g].count_nonzero() == 0


@pytest.mark.parametrize("counts", [[130, 0, 3, 64, 1, 200], [31, 33], [96, 64, 0, 160, 7]])
@pytest.mark.parametrize("cols", [136, 192])                                # rows of codes not / all 16-byte aligned
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_varlen_segmented_quantizer_rowwise_byproduct(counts, cols, dtype):
    """The segmented transposed quantizer can emit the plain row-wise codes from the same read: both outputs must be the
    ones the separate kernels give. Groups that fill whole 64-token tiles and groups that end inside one; a NaN and an Inf
    send their wavefronts down the exact route."""
    from viola_amd.nn import _varlen as v, _grouped_kernels as g
    torch.manual_seed(12)
    x = (torch.randn(sum(counts), cols) * 3).to(dtype)
    x[counts[0] // 2, 5], x[sum(counts) - 1, cols - 3] = float("nan"), float("inf")
    x = x.cuda()
    offsets, padded, offsets_dev, padded_dev = v._offsets(counts, x.device)
    qt, st = v.quantize_transposed_segmented(x, E4, offsets_dev, padded_dev, len(counts), padded[-1])
    qt2, st2, q, s = v.quantize_transposed_segmented(x, E4, offsets_dev, padded_dev, len(counts), padded[-1], rowwise=True)
    rq, rs = g.quantize(x, E4, (1, 32))
    assert torch.equal(qt.view(torch.uint8), qt2.view(torch.uint8)) and torch.equal(st, st2)
    assert torch.equal(q.view(torch.uint8), rq.view(torch.uint8)) and torch.equal(s, rs)
    # against the oracle, group by group: the transposed block of a group is the quantized transpose of its rows
    for group, count in enumerate(counts):
        if count:
            oq, os_ = og.quantize(x[offsets[group]:offsets[group + 1]].cpu(), E4, (1, 32), transposed=True)
            got = qt[:, padded[group]:padded[group] + count].cpu().view(torch.uint8)
            assert torch.equal(got, oq.view(torch.uint8))
            assert torch.equal(st[:, padded[group] // 32:padded[group] // 32 + (count + 31) // 32].cpu(), os_)
        # the padding behind a group's rows (to 32 tokens, and to 128 at the very end) holds zero codes
        assert qt[:, padded[group] + count:padded[group + 1]].view(torch.uint8).count_nonzero() == 0
    assert padded[-1] % 128 == 0 and qt.shape == (cols, padded[-1])

