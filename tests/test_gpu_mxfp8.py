"""MXFP8 on the GPU: E8M0 group scales (viola/nn/_grouped_kernels.py native=True, :72,81-85) from every quantizer
layout, and the GEMM on the block-scaled MFMA (`viola_mx_gemm`). Scale bytes and codes bit-exact against the
oracle; the GEMM < 2e-5 (fp32 out) / < 3e-3 (bf16 out) against the dequantized matmul, exact on integer data, and
equal to the FP32-scale grouped GEMM fed the decoded scales up to summation order."""

import pytest
import torch

from conftest import rel_l2
from oracle import grouped as og

pytestmark = pytest.mark.gpu
E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2


def _g():
    from viola_amd.nn import _grouped_kernels as g
    return g


def _same(q, s, rq, rs):
    assert s.dtype == torch.uint8 and torch.equal(s.cpu(), rs)
    assert torch.equal(q.view(torch.uint8).cpu(), rq.view(torch.uint8))


def _input(shape, dtype, seed):
    torch.manual_seed(seed)
    x = torch.randn(shape) * torch.exp2(torch.randint(-8, 9, (shape[0], 1)).float())
    x[::7, ::5] *= 37
    return x.to(dtype)


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("fp8", [E4, E5])
@pytest.mark.parametrize("group,shape", [((1, 32), (65, 96)), ((1, 32), (256, 1024)), ((1, 64), (96, 136)), ((32, 32), (96, 128)),
                                          ((32, 32), (70, 45)), ((32, 32), (257, 1000)), ((64, 32), (130, 96)), ((1, 32), (7, 33))])
def test_native_quantize_layouts(in_dtype, fp8, group, shape):
    g = _g()
    x = _input(shape, in_dtype, 80)
    q, s = g.quantize(x.cuda(), fp8, group, native=True)
    _same(q, s, *og.quantize(x, fp8, group, native=True))
    assert torch.equal(g.dequantize(q, s, group).cpu(), og.dequantize(q.cpu(), s.cpu(), group))
    qt, st = g.quantize(x.cuda(), fp8, group, native=True, transposed=True)
    _same(qt, st, *og.quantize(x, fp8, group, native=True, transposed=True))
    # transposes of stored codes: exact for 2-D blocks, a re-encode from the bytes for 1-D groups
    t, ts = g.transpose(q, s, group, native=True)
    _same(t, ts, *og.transpose(q.cpu(), s.cpu(), group, native=True))


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(65, 128), (300, 200), (129, 72), (8192, 1024)])
def test_native_quantize_dual(in_dtype, shape):
    g = _g()
    x = _input(shape, in_dtype, 81)
    q, s, qt, st, total = g.quantize_dual(x.cuda(), E4, (1, 32), native=True, column_sum_dtype=torch.float32)
    _same(q, s, *og.quantize(x, E4, (1, 32), native=True))
    _same(qt, st, *og.quantize(x, E4, (1, 32), native=True, transposed=True))
    assert rel_l2(total, x.double().sum(0)) < 1e-5


def test_native_scale_edges():
    """amax exactly limit * 2^k keeps 2^k, one ulp more doubles it; an all-zero group gets the 1e-30 floor's power;
    NaN members stay NaN without touching the group's scale."""
    g = _g()
    x = torch.zeros(64, 64)
    x[0, 0] = 448 * 2. ** -9
    x[0, 32] = torch.nextafter(torch.tensor(448 * 2. ** -9), torch.tensor(float("inf")))
    x[1, 1], x[1, 2] = float("nan"), 3.0
    q, s = g.quantize(x.cuda(), E4, (1, 32), native=True)
    _same(q, s, *og.quantize(x, E4, (1, 32), native=True))
    assert s[0, 0].item() == 118 and s[0, 1].item() == 119 and s[5, 0].item() == og.quantize(torch.zeros(1, 32), E4, (1, 32), native=True)[1].item()


@pytest.mark.parametrize("a_fp8,b_fp8", [(E4, E4), (E5, E4), (E4, E5)])
@pytest.mark.parametrize("m,n,k,gb", [(65, 96, 128, (32, 32)), (128, 128, 1024, (32, 32)), (300, 257, 384, (32, 32)), (130, 70, 256, (1, 32)),
                                      (96, 65, 64, (32, 32)), (64, 160, 96, (1, 32))])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_mx_gemm(a_fp8, b_fp8, m, n, k, gb, out_dtype):
    """k % 128 == 0 runs on the block-scaled MFMA, the other shapes on the FP32-scale kernel with decoded scales."""
    g = _g()
    # the reference's own test distribution (checks/check_grouped_linear.py:111-116): rows differ by powers of two,
    # members of a group do not (the FP8 MFMA aligns the products of one instruction to the largest with ~13 bits,
    # so outliers inside a K group cost ~1e-4 on either vendor's matrix unit, whatever the scale format)
    torch.manual_seed(82)
    a = torch.randn(m, k) * torch.exp2(torch.randint(-5, 6, (m, 1)).float())
    b = torch.randn(n, k) * torch.exp2(torch.randint(-5, 6, (n, 1)).float())
    qa, sa = og.quantize(a, a_fp8, (1, 32), native=True)
    qb, sb = og.quantize(b, b_fp8, gb, native=True)
    bias = torch.randn(n)
    out = g.gemm(qa.cuda(), qb.cuda(), sa.cuda(), sb.cuda(), (1, 32), gb, out_dtype=out_dtype, native=True, bias=bias.cuda())
    expected = og.gemm(qa, qb, sa, sb, (1, 32), gb, out_dtype=out_dtype, bias=bias)
    assert rel_l2(out, expected) < (2e-5 if out_dtype == torch.float32 else 3e-3)
    plain = g.gemm(qa.cuda(), qb.cuda(), g.decode_scale(sa.cuda()), g.decode_scale(sb.cuda()), (1, 32), gb, out_dtype=torch.float32)
    hw = g.gemm(qa.cuda(), qb.cuda(), sa.cuda(), sb.cuda(), (1, 32), gb, out_dtype=torch.float32, native=True)
    assert rel_l2(hw, plain) < 1e-6


def test_mx_gemm_exact_on_integers():
    """Integer codes and power-of-two scales that differ per row and per K group: every product and sum is exact, so
    the scaled MFMA must give the integer matmul of the scaled operands bit for bit."""
    g = _g()
    torch.manual_seed(84)
    m, n, k = 256, 384, 1024
    a = torch.randint(-4, 5, (m, k)).float()
    b = torch.randint(-4, 5, (n, k)).float()
    sa = torch.randint(120, 131, (m, k // 32), dtype=torch.uint8)
    sb = torch.randint(124, 129, (n // 32, k // 32), dtype=torch.uint8)
    out = g.gemm(a.to(E4).cuda(), b.to(E5).cuda(), sa.cuda(), sb.cuda(), (1, 32), (32, 32), out_dtype=torch.float32, native=True)
    da = a * og.decode_scale(sa).repeat_interleave(32, 1)
    db = b * og.decode_scale(sb).repeat_interleave(32, 0).repeat_interleave(32, 1)
    assert torch.equal(out.cpu(), (da.double() @ db.double().T).float())
