"""Per-tensor FP8 scaling on the GPU (viola/nn/_linear_kernels.py:33-104,124-293): amax + scale with history,
quantizer with row-wise and transposed outputs, epilogue-scaled GEMM, all through the C-ABI against oracle.tensor.
Scales and codes bit-exact; GEMM rel-L2 < 2e-5 for fp32 outputs and < 3e-3 for bf16 (the reference's bars,
checks/linear.py:38-39)."""

import pytest
import torch

from conftest import rel_l2
from oracle import tensor as ot

pytestmark = pytest.mark.gpu
E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2


def _k():
    from viola_amd.nn import _linear_kernels as k
    return k


def _codes(t):
    return t.view(torch.uint8).cpu()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n", [1, 7, 2048, 2049, 65536 * 3 + 5, 8192 * 1024])
def test_tensor_scale_current_and_delayed(dtype, n):
    k = _k()
    torch.manual_seed(60)
    x = (torch.randn(n) * 3).to(dtype)
    if n > 7:
        x[n // 2] = float("nan")                                               # ignored by the reduction
    for fp8 in (E4, E5):
        scale = k.tensor_scale(x.cuda(), fp8_dtype=fp8)
        expected, _ = ot.tensor_scale(x, torch.zeros(1), 0, limit=torch.finfo(fp8).max)
        assert torch.equal(scale.cpu(), expected)
    # an unaligned view takes the element-wise head and tail
    if n > 7:
        view = x.cuda()[3:]
        assert torch.equal(k.tensor_scale(view, fp8_dtype=E4).cpu(), ot.tensor_scale(x[3:], torch.zeros(1), 0)[0])
    history, reference = torch.zeros(4, device="cuda"), torch.zeros(4)
    for index in range(6):
        y = x * (.5 ** index if index % 2 else 2. ** index)
        scale = k.tensor_scale(y.cuda(), history=history, index=index, delayed=True, quantization_limit=240.0)
        expected, reference = ot.tensor_scale(y, reference, index, delayed=True, limit=240.0)
        assert torch.equal(scale.cpu(), expected) and torch.equal(history.cpu(), reference)


@pytest.mark.parametrize("in_dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("fp8", [E4, E5])
@pytest.mark.parametrize("shape", [(65, 96), (64, 64), (70, 45), (1, 33), (300, 200), (129, 1024), (8192, 1024)])
def test_tensor_quantize_rowwise_and_transposed(in_dtype, fp8, shape):
    k = _k()
    torch.manual_seed(61)
    x = (torch.randn(shape) * torch.logspace(-4, 2, shape[1])).to(in_dtype)
    x[0, 0] = float("nan")
    scale, _ = ot.tensor_scale(x, torch.zeros(1), 0, limit=torch.finfo(fp8).max)
    q, qt = k.quantize(x.cuda(), scale.cuda(), transpose=True, fp8_dtype=fp8)
    assert torch.equal(_codes(q), _codes(ot.quantize(x, scale, fp8)))
    assert torch.equal(_codes(qt), _codes(ot.quantize(x, scale, fp8, transpose=True)))
    q_only, none = k.quantize(x.cuda(), scale.cuda(), fp8_dtype=fp8)
    assert torch.equal(_codes(q_only), _codes(q)) and none.shape == (0, 0)
    none, qt_only = k.quantize(x.cuda(), scale.cuda(), rowwise=False, transpose=True, fp8_dtype=fp8)
    assert torch.equal(_codes(qt_only), _codes(qt)) and none.shape == (0, 0)
    # a smaller scale saturates at a reduced limit; tiny and huge scales take the division path
    for s, limit in ((scale / 8, 16.0), (torch.tensor([1e-33]), None), (torch.tensor([3e38]), None)):
        q, qt = k.quantize(x.cuda(), s.cuda(), transpose=True, fp8_dtype=fp8, quantization_limit=limit)
        assert torch.equal(_codes(q), _codes(ot.quantize(x, s, fp8, limit=limit)))
        assert torch.equal(_codes(qt), _codes(ot.quantize(x, s, fp8, limit=limit, transpose=True)))


def test_tensor_quantize_ties_and_nonfinite():
    """Values exactly on FP8 rounding ties relative to the scale, and Inf / NaN members (the scale is then infinite)."""
    k = _k()
    torch.manual_seed(62)
    scale = torch.tensor([0.37])
    grid = torch.arange(256, dtype=torch.uint8).view(E4).float()
    grid = grid[grid.isfinite()].sort().values
    ties = (grid[:-1] + grid[1:]) / 2
    x = torch.cat([ties, grid, -ties]).repeat(8)[: 64 * 44].reshape(64, 44) * scale
    q, qt = k.quantize(x.cuda(), scale.cuda(), transpose=True)
    assert torch.equal(_codes(q), _codes(ot.quantize(x, scale, E4))) and torch.equal(_codes(qt), _codes(ot.quantize(x, scale, E4, transpose=True)))
    y = torch.randn(130, 70)
    y[5, 6], y[77, 3], y[128, 69] = float("inf"), float("nan"), float("-inf")
    s = k.tensor_scale(y.cuda())
    expected, _ = ot.tensor_scale(y, torch.zeros(1), 0)
    assert torch.equal(s.cpu(), expected) and torch.isinf(s).all()
    q, qt = k.quantize(y.cuda(), s, transpose=True)
    assert torch.equal(_codes(q), _codes(ot.quantize(y, expected, E4))) and torch.equal(_codes(qt), _codes(ot.quantize(y, expected, E4, transpose=True)))
    # with a finite scale Inf saturates and NaN stays NaN, next to ordinary values in the same wavefront
    q, _ = k.quantize(y.cuda(), scale.cuda())
    assert torch.equal(_codes(q), _codes(ot.quantize(y, scale, E4)))


@pytest.mark.parametrize("a_fp8,b_fp8", [(E4, E4), (E5, E4), (E4, E5), (E5, E5)])
@pytest.mark.parametrize("m,n,k", [(65, 96, 128), (96, 65, 64), (64, 160, 96), (128, 128, 1024), (300, 257, 208), (33, 70, 40), (256, 192, 72)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_tensor_gemm(a_fp8, b_fp8, m, n, k, out_dtype):
    kk = _k()
    torch.manual_seed(63)
    a = (torch.randn(m, k) * 4).to(a_fp8)
    b = (torch.randn(n, k) * 4).to(b_fp8)
    sa, sb = torch.tensor([.013]), torch.tensor([2.7])
    bias = torch.randn(n)
    for use_bias in (None, bias):
        out = kk.gemm(a.cuda(), b.cuda(), sa.cuda(), sb.cuda(), out_dtype=out_dtype, bias=None if use_bias is None else use_bias.cuda())
        expected = ot.gemm(a, b, sa, sb, bias=use_bias, out_dtype=out_dtype)
        assert rel_l2(out, expected) < (2e-5 if out_dtype == torch.float32 else 3e-3)
    again = kk.gemm(a.cuda(), b.cuda(), sa.cuda(), sb.cuda(), out_dtype=out_dtype, bias=bias.cuda())
    assert torch.equal(out, again)


def test_tensor_gemm_exact_on_small_integers():
    """Integer-valued codes with power-of-two scales: every product and partial sum is exact in fp32, so the kernel
    must return the integer matmul bit for bit (K = 1024 covers sixteen 64-wide MFMA steps and the chunk ring)."""
    kk = _k()
    torch.manual_seed(64)
    for m, n, k in ((256, 384, 1024), (130, 70, 208)):
        a = torch.randint(-8, 9, (m, k)).float()
        b = torch.randint(-8, 9, (n, k)).float()
        out = kk.gemm(a.to(E4).cuda(), b.to(E5).cuda(), torch.tensor([.5], device="cuda"), torch.tensor([4.], device="cuda"),
                      out_dtype=torch.float32)
        assert torch.equal(out.cpu(), (a @ b.T) * 2)
