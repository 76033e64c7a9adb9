"""Linear with the reference's accumulation options (accum_dtype="fp16", accum_block_size, accum_reduce_dtype):
the quantization limits they imply are the reference's (viola/nn/linear.py:232-253), so codes and scales match the
oracle bit for bit; the GEMMs follow the FP16-accumulator model of the reference's kernels (oracle.grouped.gemm_half,
oracle.tensor.gemm_half) and stay inside the bounds the reference holds its FP16 sums to
(checks/check_grouped_linear.py:41 < .01 per kernel, :73 < .012 per layer)."""

import math

import pytest
import torch

from oracle import grouped as og, linear as ol, tensor as ot
from conftest import rel_l2

pytestmark = pytest.mark.gpu
E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2


@pytest.fixture
def bf16_gradients():
    import viola_amd
    viola_amd.set_master_weight_dtype("fp32")
    viola_amd.set_gradient_dtype("bf16")
    yield
    viola_amd.precision._settings.update(master_weight_dtype=torch.float32, gradient_dtype=None,
                                         master_rounding="nearest", master_rounding_seed=0)


@pytest.mark.parametrize("options,gw,gx,gg,expected", [
    (dict(accum_dtype="fp16"), (32, 32), (1, 32), (1, 32), (32.0, 32.0, 32.0)),           # sqrt(32768 / 32) = 32
    (dict(accum_dtype="fp16", accum_block_size=32), (32, 64), (1, 64), (1, 128), (32.0, 32.0, 32.0)),
    (dict(accum_dtype="fp16"), (32, 64), (1, 64), (1, 128), (16.0, 16.0, 16.0)),          # sqrt(512) -> 16, sqrt(256) = 16
    (dict(accum_dtype="fp16"), (64, 32), (1, 32), (1, 256), (32.0, 16.0, 8.0)),           # weight: max side; sqrt(128) -> 8
    (dict(accum_dtype="fp16", quantization_limit=6.0), (32, 32), (1, 32), (1, 32), (6.0, 6.0, 6.0)),
    (dict(accum_dtype="fp32", accum_block_size=128, accum_reduce_dtype="bf16"), (32, 32), (1, 32), (1, 32), (None, None, None)),
    (dict(quantization_limit=1e9), (32, 32), (1, 32), (1, 32), (448.0, 448.0, 57344.0))])
def test_group_limits_follow_the_reference(options, gw, gx, gg, expected):
    """linear.py:244-253 evaluated by hand for each row."""
    import viola_amd
    layer = viola_amd.nn.Linear(128, 256, device="cuda", scaling="grouped", weight_group_shape=gw, input_group_shape=gx,
                                grad_group_shape=gg, **options)
    got = (layer._group_limit(gx, layer.fp8_dtype), layer._group_limit(gw, layer.fp8_dtype, weight=True),
           layer._group_limit(gg, layer.backward_fp8_dtype))
    assert got == expected


@pytest.mark.parametrize("options,reduction,fp8,expected", [
    (dict(accum_dtype="fp16"), 4096, E4, 2.0), (dict(accum_dtype="fp16"), 8192, E5, 2.0), (dict(accum_dtype="fp16"), 512, E4, 8.0),
    (dict(accum_dtype="fp16", accum_block_size=128), 4096, E4, 16.0), (dict(accum_dtype="fp16", accum_block_size=32), 4096, E5, 32.0),
    (dict(accum_dtype="fp16", quantization_limit=1000.0), 4096, E4, 448.0), (dict(), 4096, E4, None)])
def test_tensor_limits_follow_the_reference(options, reduction, fp8, expected):
    """linear.py:232-242 evaluated by hand for each row."""
    import viola_amd
    layer = viola_amd.nn.Linear(64, 64, device="cuda", scaling="current", **options)
    assert layer._quantization_limit(reduction, fp8) == expected


def test_kernel_with_the_half_sum_limit():
    """checks/check_grouped_linear.py:23-46 with half=True: limit 8 on both operands, (1,32) x (32,32), e5m2 x e4m3."""
    from viola_amd.nn import _grouped_kernels as g
    torch.manual_seed(2041)
    m, n, k = 65, 96, 128
    a = (torch.randn(m, k) * torch.exp2(torch.randint(-5, 6, (m, 1)))).bfloat16()
    b = (torch.randn(n, k) * torch.exp2(torch.randint(-5, 6, (n, 1)))).bfloat16()
    qa, sa = g.quantize(a.cuda(), E5, (1, 32), limit=8.0)
    qb, sb = g.quantize(b.cuda(), E4, (32, 32), limit=8.0)
    ra, rsa = og.quantize(a, E5, (1, 32), limit=8.0)
    rb, rsb = og.quantize(b, E4, (32, 32), limit=8.0)
    assert torch.equal(qa.cpu().view(torch.uint8), ra.view(torch.uint8)) and torch.equal(sa.cpu(), rsa)
    assert torch.equal(qb.cpu().view(torch.uint8), rb.view(torch.uint8)) and torch.equal(sb.cpu(), rsb)
    assert ra.float().abs().max() == 8.0 and rb.float().abs().max() == 8.0
    bias = torch.randn(n)
    actual = g.gemm(qa, qb, sa, sb, (1, 32), (32, 32), out_dtype=torch.float32, bias=bias.cuda(), accum_dtype="fp16")
    expected = og.dequantize(ra, rsa, (1, 32)) @ og.dequantize(rb, rsb, (32, 32)).T + bias
    assert torch.isfinite(actual).all()
    assert rel_l2(actual, expected) < .01                                     # the reference's FP16 bound (:41)
    model = og.gemm_half(ra, rb, rsa, rsb, (1, 32), (32, 32), bias=bias)
    # not to the bit: the MFMA aligns the products of a step to the largest before adding them, so its sum and the exact
    # one sometimes land on different sides of an FP16 rounding boundary (one part in 2048 of that element)
    assert rel_l2(actual, model) < 3e-4 and (actual.cpu() == model).float().mean() > .9
    again = g.gemm(qa, qb, sa, sb, (1, 32), (32, 32), out_dtype=torch.float32, bias=bias.cuda(), accum_dtype="fp16")
    assert torch.equal(again, actual)
    fp32 = g.gemm(qa, qb, sa, sb, (1, 32), (32, 32), out_dtype=torch.float32, bias=bias.cuda())
    assert rel_l2(fp32, expected) < 2e-5 and not torch.equal(fp32, actual)


def _codes(rows, k, dtype, seed, limit):
    torch.manual_seed(seed)
    x = (torch.randn(rows, k) * torch.exp2(torch.randint(-5, 6, (rows, 1)))).bfloat16()
    return x


@pytest.mark.parametrize("m,n,k", [(65, 96, 128), (96, 65, 64), (64, 160, 96), (130, 70, 200)])
@pytest.mark.parametrize("groups", [((1, 32), (32, 32)), ((1, 32), (1, 32)), ((1, 64), (32, 64)), ((1, 128), (32, 32))])
@pytest.mark.parametrize("block,reduce", [(0, "fp32"), (32, "fp32"), (0, "bf16"), (64, "bf16")])
def test_grouped_gemm_follows_the_half_accumulator_model(m, n, k, groups, block, reduce):
    """viola_group_gemm_half against oracle.grouped.gemm_half (the reference's kernel text with a 32-k step that sums
    exactly and rounds to FP16 once): identical except where the MFMA's FP32 sum of the 32 products and the exact sum
    land on different sides of an FP16 (or bf16) rounding boundary. That happens for 2-3 % of the 32-k steps (the MFMA
    aligns a step's products to the largest before adding), so with four to seven steps per output 5-15 % of the outputs
    differ, each by one part in 2048 of one step's partial sum: rel-L2 below 1e-4."""
    from viola_amd.nn import _grouped_kernels as g
    ga, gb = groups
    a, b = _codes(m, k, E5, 1, 8.0), _codes(n, k, E4, 2, 8.0)
    ra, rsa = og.quantize(a, E5, ga, limit=8.0)
    rb, rsb = og.quantize(b, E4, gb, limit=8.0)
    bias = torch.randn(n)
    dtype = torch.bfloat16 if reduce == "bf16" else torch.float32
    want = og.gemm_half(ra, rb, rsa, rsb, ga, gb, accum_block_size=block, reduce_dtype=dtype, bias=bias)
    got = g.gemm(ra.cuda(), rb.cuda(), rsa.cuda(), rsb.cuda(), ga, gb, out_dtype=torch.float32, bias=bias.cuda(), accum_dtype="fp16",
                 accum_block_size=block, accum_reduce_dtype=reduce).cpu()
    assert (got == want).float().mean() > .7 and rel_l2(got, want) < (2e-3 if reduce == "bf16" else 3e-4)
    exact = og.gemm(ra, rb, rsa, rsb, ga, gb, bias=bias)
    assert rel_l2(got, exact) < .01 and not torch.equal(got, exact)


@pytest.mark.parametrize("m,n,k", [(65, 96, 128), (64, 160, 96), (130, 70, 328)])
@pytest.mark.parametrize("formats", [(E4, E4), (E5, E4)])
@pytest.mark.parametrize("block,reduce", [(0, "fp32"), (32, "fp32"), (64, "fp32"), (128, "bf16"), (96, "bf16")])
def test_tensor_gemm_follows_the_half_accumulator_model(m, n, k, formats, block, reduce):
    """viola_tensor_gemm_half against oracle.tensor.gemm_half; 96 = one whole 64-k chunk per block, as in the reference."""
    from viola_amd.nn import _linear_kernels as lk
    limit = 2.0
    a, b = _codes(m, k, formats[0], 3, limit), _codes(n, k, formats[1], 4, limit)
    zero = torch.zeros(1)
    sa, sb = ot.tensor_scale(a, zero, 0, limit=limit)[0], ot.tensor_scale(b, zero, 0, limit=limit)[0]
    qa, qb = ot.quantize(a, sa, formats[0], limit=limit), ot.quantize(b, sb, formats[1], limit=limit)
    bias = torch.randn(n)
    dtype = torch.bfloat16 if reduce == "bf16" else torch.float32
    want = ot.gemm_half(qa, qb, sa, sb, accum_block_size=block, reduce_dtype=dtype, bias=bias)
    got = lk.gemm(qa.cuda(), qb.cuda(), sa.cuda(), sb.cuda(), out_dtype=torch.float32, bias=bias.cuda(), accum_dtype="fp16",
                  accum_block_size=block, accum_reduce_dtype=reduce).cpu()
    assert (got == want).float().mean() > .7 and rel_l2(got, want) < (2e-3 if reduce == "bf16" else 3e-4)
    assert rel_l2(got, ot.gemm(qa, qb, sa, sb, bias=bias)) < .01


def test_half_accumulator_cases_worked_out_by_hand():
    """The hand cases of the CPU pin on the device: fp16(2049) = 2048 per group, one running partial per tensor,
    a bf16 total."""
    from viola_amd.nn import _grouped_kernels as g, _linear_kernels as lk
    a, b = torch.zeros(1, 64), torch.zeros(1, 64)
    a[0, 0], b[0, 0], a[0, 1], b[0, 1], a[0, 32], b[0, 32] = 64, 32, 1, 1, 2, 3
    qa, qb = a.to(E4).cuda(), b.to(E4).cuda()
    sa, sb = torch.tensor([[.5, 2.]]).cuda(), torch.tensor([[1., 1.]]).cuda()
    run = lambda **kw: g.gemm(qa, qb, sa, sb, (1, 32), (32, 32), out_dtype=torch.float32, **kw).item()
    assert run() == 2049 * .5 + 12 and run(accum_dtype="fp16") == 2048 * .5 + 12
    one, half = torch.ones(1).cuda(), torch.tensor([.5]).cuda()
    tensor = lambda **kw: lk.gemm(qa, qb, half, one, out_dtype=torch.float32, accum_dtype="fp16", **kw).item()
    assert tensor() == 2054 * .5 and tensor(accum_block_size=32) == 2054 * .5
    assert tensor(accum_block_size=32, accum_reduce_dtype="bf16") == 2048 * .5


def test_grouped_layer_with_fp16_accumulation_options(bf16_gradients):
    """checks/check_grouped_linear.py:134 = check_layer('grouped', 'memory', (32,32), (1,32), (1,32), half=True):
    accum_dtype='fp16', accum_block_size=32 -> every group limit is 32."""
    import viola_amd
    torch.manual_seed(2041)
    gw, gx, gg = (32, 32), (1, 32), (1, 32)
    source = torch.nn.Linear(128, 96, dtype=torch.bfloat16)
    source.weight.data[:, ::17] *= 16
    options = dict(scaling="grouped", mode="memory", weight_group_shape=gw, input_group_shape=gx, grad_group_shape=gg,
                   saved_input_dtype="fp8", accum_dtype="fp16", accum_block_size=32)
    layer = viola_amd.nn.Linear.from_float(source.cuda(), **options)
    assert layer._group_limit(gx, E4) == 32.0
    rq, rs = og.quantize(source.weight.detach().float().cpu(), E4, gw, limit=32.0)
    assert torch.equal(layer.weight.detach().cpu().view(torch.uint8), rq.view(torch.uint8)) and torch.equal(layer.weight_scale.cpu(), rs)
    assert rq.float().abs().max() == 32.0
    x = torch.randn(65, 128).bfloat16()
    dy = torch.randn(65, 96).bfloat16()
    xg = x.cuda().requires_grad_()
    y = layer(xg)
    y.backward(dy.cuda())
    expect = ol.linear(x, og.dequantize(rq, rs, gw), source.bias.detach().cpu(), dy, fp8=E4, bwd_fp8=E5, gx=gx, gw=gw, gg=gg,
                       limits=(32.0, 32.0, 32.0))
    actual = dict(y=y, dx=xg.grad, dw=layer.weight.grad, db=layer.bias.grad)
    errors = {key: rel_l2(actual[key], expect[key]) for key in actual}
    assert max(errors.values()) < .012, errors                                # the reference's bound for FP16 accumulation (:73)
    # the limit costs accuracy against the unquantized layer, but not much (5 binades of e4m3 remain below 32)
    plain = ol.linear(x, og.dequantize(*og.quantize(source.weight.detach().float().cpu(), E4, gw), gw), source.bias.detach().cpu(), dy,
                      fp8=E4, bwd_fp8=E5, gx=gx, gw=gw, gg=gg)
    assert rel_l2(actual["y"], plain["y"]) < .05
    restored = viola_amd.nn.Linear(128, 96, device="cuda", dtype=torch.bfloat16, **options)
    restored.load_state_dict(layer.state_dict())
    restored.bfloat16()
    with torch.no_grad():
        assert torch.equal(restored(xg), y)
    # optimizer writeback re-encodes under the same limit (:88-97)
    optimizer = viola_amd.optim.bind_optimizer(layer, torch.optim.SGD(layer.parameters(), lr=.001))
    before = layer.weight.detach().clone()
    for _ in range(3):
        optimizer.zero_grad()
        layer(xg).float().square().mean().backward()
        optimizer.step()
    assert torch.isfinite(layer.dequantize_weight()).all()
    assert not torch.equal(before.view(torch.uint8), layer.weight.view(torch.uint8))
    assert layer.weight.detach().float().abs().max() <= 32.0


@pytest.mark.parametrize("block", [0, 128])
def test_tensor_layer_with_fp16_accumulation_options(bf16_gradients, block):
    """Linear(scaling='current', accum_dtype='fp16'[, accum_block_size]) (checks/benchmark_block_linear.py:58):
    per-tensor limits 2^floor(log2(sqrt(32768 / reduction))) on every operand, FP16 partial sums as in the reference's kernel."""
    import viola_amd
    torch.manual_seed(77)
    source = torch.nn.Linear(256, 192, dtype=torch.bfloat16)
    layer = viola_amd.nn.Linear.from_float(source.cuda(), scaling="current", accum_dtype="fp16", accum_block_size=block,
                                           backward_dtype="e5m2")
    x = torch.randn(130, 256).bfloat16()
    dy = torch.randn(130, 192).bfloat16()
    lx = lw = 2.0 ** math.floor(math.log2(math.sqrt(32768.0 / (block or 256))))
    lg = 2.0 ** math.floor(math.log2(math.sqrt(32768.0 / (block or 192))))
    zero = torch.zeros(1)
    sw = ot.tensor_scale(source.weight.detach().float().cpu(), zero, 0, limit=lw)[0]
    qw = ot.quantize(source.weight.detach().float().cpu(), sw, E4, limit=lw)
    assert torch.equal(layer.weight.detach().cpu().view(torch.uint8), qw.view(torch.uint8))
    assert torch.equal(layer.weight_scale.cpu().reshape(()), sw.reshape(()))
    assert qw.float().abs().max() == lw
    xg = x.cuda().requires_grad_()
    y = layer(xg)
    y.backward(dy.cuda())
    sx = ot.tensor_scale(x, zero, 0, limit=lx)[0]
    sg = ot.tensor_scale(dy, zero, 0, limit=lg)[0]
    qx, qg = ot.quantize(x, sx, E4, limit=lx), ot.quantize(dy, sg, E5, limit=lg)
    ey = ot.gemm(qx, qw, sx, sw, bias=source.bias.detach().cpu(), out_dtype=torch.bfloat16)
    edx = ot.gemm(qg, qw.T.contiguous(), sg, sw, out_dtype=torch.bfloat16)
    edw = ot.gemm(qg.T.contiguous(), qx.T.contiguous(), sg, sx, out_dtype=torch.bfloat16)
    for got, want in ((y, ey), (xg.grad, edx), (layer.weight.grad, edw)):
        assert rel_l2(got, want) < .012                                       # against FP32 sums: the reference's FP16 bound
    block_args = dict(accum_block_size=block, out_dtype=torch.bfloat16)
    assert rel_l2(y, ot.gemm_half(qx, qw, sx, sw, bias=source.bias.detach().cpu(), **block_args)) < 3e-3
    assert rel_l2(xg.grad, ot.gemm_half(qg, qw.T.contiguous(), sg, sw, **block_args)) < 3e-3
    assert rel_l2(layer.weight.grad, ot.gemm_half(qg.T.contiguous(), qx.T.contiguous(), sg, sx, **block_args)) < 3e-3


@pytest.mark.parametrize("scaling", ["grouped", "current"])
def test_mlp_with_fp16_accumulation(bf16_gradients, scaling):
    """MLP passes the accumulation options to both projections (viola/nn/mlp.py:80, _mlp_kernels.py:252-268). The
    FP16-accumulator model exists for the plain product, so the gated projections run as that product plus the
    elementwise activation kernels: every GEMM of the step is a *_gemm_half call, and the result stays within the
    reference's MLP bar (checks/mlp.py:42, .025) of the float model evaluated on the dequantized weights."""
    import viola_amd
    from viola_amd import _lib
    torch.manual_seed(131)
    mlp = viola_amd.nn.MLP(128, 160, 96, activation="silu", scaling=scaling, accum_dtype="fp16", accum_block_size=32,
                           device="cuda", dtype=torch.bfloat16)
    x = torch.randn(2, 33, 128, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    dy = torch.randn(2, 33, 96, device="cuda", dtype=torch.bfloat16)
    _lib.timeline = []
    try:
        y = mlp(x)
        y.backward(dy)
        torch.cuda.synchronize()
        calls = [name for name, _, _ in _lib.timeline]
    finally:
        _lib.timeline = None
    half = "viola_group_gemm_half" if scaling == "grouped" else "viola_tensor_gemm_half"
    assert calls.count(half) == 6 and not any("gemm" in name and name != half for name in calls)
    w1, w2 = mlp.gate_up.dequantize_weight(), mlp.down.dequantize_weight()
    xf = x.detach().float().requires_grad_()
    z = xf @ w1.T + mlp.gate_up.bias.float()
    yf = (torch.nn.functional.silu(z[..., :160]) * z[..., 160:]) @ w2.T + mlp.down.bias.float()
    yf.backward(dy.float())
    assert rel_l2(y, yf.detach()) < .05 and rel_l2(x.grad, xf.grad) < .08       # FP8 operands with limit 32 against float math
    assert torch.isfinite(mlp.gate_up.weight.grad).all() and torch.isfinite(mlp.down.weight.grad).all()

