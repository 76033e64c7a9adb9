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


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 8), (65, 96), (300, 200), (8192, 4096), (7, 2056), (33, 45)])
def test_tensor_scale_with_column_sums(dtype, shape):
    """The amax pass that also returns x.sum(0): same scale and history as the plain pass, sums equal to fp32 column
    sums within summation-order error (the reference compares db with torch's default closeness, checks/linear.py:40)."""
    k = _k()
    torch.manual_seed(65)
    x = (torch.randn(shape) * 2).to(dtype)
    x[0, 0] = float("nan") if shape[0] > 1 else x[0, 0]
    history = torch.zeros(2, device="cuda")
    scale, total = k.tensor_scale_and_column_sum(x.cuda(), torch.float32, history=history, index=0, fp8_dtype=E5)
    expected, after = ot.tensor_scale(x, torch.zeros(2), 0, limit=torch.finfo(E5).max)
    assert torch.equal(scale.cpu(), expected) and torch.equal(history.cpu(), after)
    reference = x.double().sum(0)
    keep = ~reference.isnan()
    assert torch.equal(total.cpu().isnan(), reference.isnan())
    magnitude = x.double().abs().nan_to_num(0).sum(0)
    assert ((total.cpu().double() - reference)[keep].abs() <= 1e-6 * magnitude[keep] + 1e-30).all()
    low = k.tensor_scale_and_column_sum(x.cuda(), torch.bfloat16)[1]
    assert low.dtype == torch.bfloat16
    if shape[1] % (16 // x.element_size()) == 0:                               # one read: the fp32 sums, rounded once
        assert torch.equal(low[keep.cuda()], total.bfloat16()[keep.cuda()])
    else:                                                                       # two passes: torch's own sum(0, dtype)
        assert torch.equal(low, x.cuda().sum(0, dtype=torch.bfloat16)) or shape[0] > 1 and bool(x[0, 0].isnan())


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


@pytest.mark.parametrize("m,n", [(1930, 1100), (130, 200)])                  # 16 x 9 tiles of 128 x 128; 2 x 4 of 128 x 64
@pytest.mark.parametrize("k,a_fp8,b_fp8", [(2048, E4, E4), (2112, E5, E4), (4000, E4, E5), (6160, E4, E4)])
def test_tensor_gemm_long_k_few_tiles(k, a_fp8, b_fp8, m, n):
    """Fewer than 512 tiles of 128 x 128 and a long k (a weight gradient): the kernel splits a tile's k range (128 x 128
    from 129 tiles up, 128 x 64 below) over two teams of waves and adds their sums. Against the oracle on row samples, and
    bit for bit on integer-valued operands, whose sums are exact in any order."""
    kk = _k()
    torch.manual_seed(k)
    a = (torch.randn(m, k) * 4).to(a_fp8)
    b = (torch.randn(n, k) * 4).to(b_fp8)
    sa, sb = torch.tensor([.013]), torch.tensor([2.7])
    bias = torch.randn(n)
    rows = torch.cat([torch.arange(0, min(m, 140)), torch.arange(min(m, 1900), m)])
    for out_dtype, bound in ((torch.float32, 2e-5), (torch.bfloat16, 3e-3)):
        out = kk.gemm(a.cuda(), b.cuda(), sa.cuda(), sb.cuda(), out_dtype=out_dtype, bias=bias.cuda())
        assert rel_l2(out[rows.cuda()], ot.gemm(a[rows], b, sa, sb, bias=bias, out_dtype=out_dtype)) < bound
        assert torch.equal(out, kk.gemm(a.cuda(), b.cuda(), sa.cuda(), sb.cuda(), out_dtype=out_dtype, bias=bias.cuda()))
    ia = torch.randint(-8, 9, (m, k)).float()
    ib = torch.randint(-8, 9, (n, k)).float()
    exact = kk.gemm(ia.to(a_fp8).cuda(), ib.to(b_fp8).cuda(), torch.tensor([.5], device="cuda"), torch.tensor([4.], device="cuda"),
                    out_dtype=torch.float32)
    assert torch.equal(exact, (ia.cuda() @ ib.cuda().T) * 2)


# ----------------------------------------------------------------------------- Linear(scaling="current" | "delayed")
@pytest.fixture
def precision_policy():
    import viola_amd
    saved = dict(viola_amd.precision._settings)
    yield viola_amd
    viola_amd.precision._settings.clear()
    viola_amd.precision._settings.update(saved)


@pytest.mark.parametrize("fmt,backward,mode", [("e4m3", "e5m2", "memory"), ("e4m3", "e5m2", "fast"), ("e4m3", "e4m3", "memory"),
                                               ("e5m2", "e5m2", "fast")])
@pytest.mark.parametrize("shape,gradient", [((65, 128, 96), "bf16"), ((256, 512, 384), "fp32"), ((100, 72, 40), "bf16")])
def test_linear_current_scaling_numerics(precision_policy, fmt, backward, mode, shape, gradient):
    """checks/linear.py:23-39: y, dx, dw against the matmul of the per-tensor-quantized operands (< .003 for bf16
    results, < 2e-5 for fp32), db exact; the stored codes and scale are the oracle's quantize of the initial weight."""
    viola = precision_policy
    viola.set_master_weight_dtype("fp32")
    viola.set_gradient_dtype(gradient)
    m, k, n = shape
    torch.manual_seed(127)
    layer = viola.nn.Linear(k, n, mode=mode, forward_dtype=fmt, backward_dtype=backward, device="cuda", dtype=torch.bfloat16)
    assert layer.weight_quantizer.scaling == "current" and layer.weight_scale.shape == (1,)
    fp8, bwd = layer.fp8_dtype, layer.backward_fp8_dtype
    master = layer._initial_weight.detach().cpu()
    sw, _ = ot.tensor_scale(master, torch.zeros(1), 0, limit=torch.finfo(fp8).max)
    assert torch.equal(layer.weight_scale.cpu(), sw) and torch.equal(_codes(layer.weight), _codes(ot.quantize(master, sw, fp8)))
    if mode == "fast":
        assert torch.equal(_codes(layer.weight_transpose), _codes(ot.quantize(master, sw, fp8, transpose=True)))
    else:
        assert layer.weight_transpose.numel() == 0
    x = torch.randn(m, k, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    dy = torch.randn(m, n, device="cuda", dtype=torch.bfloat16)
    y = layer(x)
    y.backward(dy)
    grad_dtype = torch.bfloat16 if gradient == "bf16" else torch.float32
    ry, rdx, rdw, rdb = ot.linear(x.detach().cpu(), layer.weight.detach().cpu(), sw, layer.bias.detach().cpu(), dy.cpu(), fp8=fp8,
                                  bwd_fp8=bwd, out_dtype=torch.bfloat16, grad_dtype=grad_dtype)
    assert rel_l2(y, ry) < 3e-3 and rel_l2(x.grad, rdx) < 3e-3
    assert layer.weight.grad.dtype == grad_dtype and rel_l2(layer.weight.grad, rdw) < (3e-3 if gradient == "bf16" else 2e-5)
    torch.testing.assert_close(layer.bias.grad.cpu(), rdb)
    # and against the float model: FP8 noise only
    w = layer.dequantize_weight().cpu()
    assert rel_l2(y, x.detach().float().cpu() @ w.T + layer.bias.detach().float().cpu()) < .08
    assert torch.equal(w, layer.weight.detach().float().cpu() * sw)


@pytest.mark.parametrize("weight_dtype", ["bf16", "fp16"])
def test_linear_current_scaling_float_storage(precision_policy, weight_dtype):
    """BF16/FP16 storage quantizes the weight per call with its own scale; frozen weights and no-grad calls work."""
    viola = precision_policy
    viola.set_gradient_dtype("bf16")
    torch.manual_seed(128)
    layer = viola.nn.Linear(96, 80, weight_dtype=weight_dtype, backward_dtype="e4m3", device="cuda", dtype=torch.bfloat16,
                            saved_input_dtype="bf16", cache_weight_transpose=True)
    assert layer.weight_scale.shape == (0,)
    x = torch.randn(3, 50, 96, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    dy = torch.randn(3, 50, 80, device="cuda", dtype=torch.bfloat16)
    y = layer(x)
    y.backward(dy)
    w = layer.weight.detach().float().cpu()
    sw, _ = ot.tensor_scale(w, torch.zeros(1), 0)
    ry, rdx, rdw, rdb = ot.linear(x.detach().cpu().reshape(-1, 96), ot.quantize(w, sw, E4), sw, layer.bias.detach().cpu(),
                                  dy.cpu().reshape(-1, 80), bwd_fp8=E4)
    assert rel_l2(y.reshape(-1, 80), ry) < 3e-3 and rel_l2(x.grad.reshape(-1, 96), rdx) < 3e-3 and rel_l2(layer.weight.grad, rdw) < 3e-3
    with torch.no_grad():
        assert torch.equal(layer(x), y)
    layer.weight.requires_grad_(False)
    x.grad = None
    layer(x).backward(dy)
    assert rel_l2(x.grad.reshape(-1, 96), rdx) < 3e-3 and layer.weight.grad is not None


def test_linear_delayed_scaling_history(precision_policy):
    """scaling="delayed": call n > 0 of each quantizer scales with the maximum of its amax history (linear.py:20-26,
    _scale_kernel :49-71), the backward does not advance the weight history, state_dict round-trips the counters."""
    viola = precision_policy
    viola.set_gradient_dtype("bf16")
    torch.manual_seed(129)
    layer = viola.nn.Linear(64, 48, scaling="delayed", history_len=3, device="cuda", dtype=torch.bfloat16)
    assert layer.weight_quantizer.index == 1                                    # the construction-time refresh
    history = torch.zeros(3)
    for index, gain in enumerate((1., 4., .25, .125, .0625)):
        x = (torch.randn(32, 64) * gain).bfloat16()
        expected_scale, history = ot.tensor_scale(x, history, index, delayed=True)
        y = layer(x.cuda().requires_grad_())
        assert torch.equal(layer.input_quantizer.history.cpu(), history) and layer.input_quantizer.index == index + 1
        qx = ot.quantize(x, expected_scale, E4)
        ry = ot.gemm(qx, layer.weight.detach().cpu(), expected_scale, layer.weight_scale.cpu(), bias=layer.bias.detach().cpu(),
                     out_dtype=torch.bfloat16)
        assert rel_l2(y, ry) < 3e-3
        y.backward(torch.randn_like(y))
        assert layer.grad_quantizer.index == index + 1 and layer.weight_quantizer.index == 1
    state = layer.state_dict()
    other = viola.nn.Linear(64, 48, scaling="delayed", history_len=3, device="cuda", dtype=torch.bfloat16)
    other.load_state_dict(state)
    assert other.input_quantizer.index == 5 and torch.equal(other.input_quantizer.history, layer.input_quantizer.history)
    x = torch.randn(8, 64, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        assert torch.equal(other(x), layer(x))


@pytest.mark.parametrize("fmt,mode,scaling,gradient", [("e4m3", "memory", "current", "bf16"), ("e4m3", "fast", "delayed", "fp32"),
                                                       ("e5m2", "fast", "current", "bf16")])
def test_linear_update_and_resume(precision_policy, fmt, mode, scaling, gradient):
    """checks/linear.py:50-97: AdamW under bind_optimizer, three micro-batches per step; after a step the stored codes
    are exactly quantize(master, stored scale); a restored model + optimizer repeats the next step bit for bit."""
    import copy
    viola = precision_policy
    viola.set_master_weight_dtype("fp32")
    viola.set_gradient_dtype(gradient)
    torch.manual_seed(130)
    make = lambda: viola.nn.Linear(256, 192, mode=mode, forward_dtype=fmt, scaling=scaling, device="cuda", dtype=torch.bfloat16)
    layer = make()
    optimizer = viola.optim.bind_optimizer(layer, torch.optim.AdamW(layer.parameters(), lr=.002))
    assert layer._initial_weight is None
    batches = [torch.randn(64, 256, device="cuda", dtype=torch.bfloat16) for _ in range(3)]

    def step(model, opt):
        opt.zero_grad()
        for batch in batches:
            model(batch).float().square().mean().div(len(batches)).backward()
        before = model.weight.detach().view(torch.uint8).clone()
        opt.step()
        assert not torch.equal(before, model.weight.view(torch.uint8))
        master = model._master_ref().detach().cpu()
        assert torch.equal(_codes(model.weight), _codes(ot.quantize(master, model.weight_scale.cpu(), model.fp8_dtype)))
        assert model.weight.grad.dtype == {"fp32": torch.float32, "bf16": torch.bfloat16}[gradient]
        if model.cache_weight_transpose:
            assert torch.equal(model.weight.T.contiguous().view(torch.uint8), model.weight_transpose.view(torch.uint8))
        else:
            assert model.weight_transpose.numel() == 0

    step(layer, optimizer)
    state = copy.deepcopy({"model": layer.state_dict(), "optimizer": optimizer.state_dict()})
    restored = make()
    restored.load_state_dict(state["model"])
    second = viola.optim.bind_optimizer(restored, torch.optim.AdamW(restored.parameters(), lr=.002))
    second.load_state_dict(state["optimizer"])
    step(layer, optimizer)
    step(restored, second)
    assert torch.equal(layer.weight.view(torch.uint8), restored.weight.view(torch.uint8))
    assert torch.equal(layer.bias, restored.bias) and torch.equal(layer.weight_scale, restored.weight_scale)
    for p, q in zip(optimizer.param_groups[0]["params"], second.param_groups[0]["params"]):
        assert torch.equal(p, q)
    optimizer.zero_grad(set_to_none=False)
    assert layer.weight.grad.count_nonzero() == 0
    optimizer.zero_grad()
    assert layer.weight.grad is None
