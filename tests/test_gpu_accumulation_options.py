"""Linear with the reference's accumulation options (accum_dtype="fp16", accum_block_size, accum_reduce_dtype):
the quantization limits they imply are the reference's (viola/nn/linear.py:232-253), so codes and scales match the
oracle bit for bit, and the GEMMs (FP32 sums on the MFMA) stay inside the bounds the reference holds its FP16 sums to
(checks/check_grouped_linear.py:41 < .01 per kernel, :73 < .012 per layer) — here they meet the FP32 bounds."""

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
    assert rel_l2(actual, expected) < 2e-5                                    # the FP32 bound (:41); the FP16 one is .01
    again = g.gemm(qa, qb, sa, sb, (1, 32), (32, 32), out_dtype=torch.float32, bias=bias.cuda(), accum_dtype="fp16")
    assert torch.equal(again, actual)


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
    assert max(errors.values()) < .003, errors                                # the FP32 bound (:73); the FP16 one is .012
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
    per-tensor limits 2^floor(log2(sqrt(32768 / reduction))) on every operand, FP32 sums."""
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
        assert rel_l2(got, want) < .003
