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


@pytest.mark.parametrize("k,gb,a_fp8,b_fp8", [(2048, (1, 32), E4, E4), (2176, (32, 32), E5, E4), (4224, (1, 32), E4, E5), (6272, (32, 32), E4, E4)])
@pytest.mark.parametrize("m,n", [(1930, 1120), (130, 192)])                  # 16 x 9 tiles of 128 x 128; 2 x 3 of 128 x 64
def test_mx_gemm_long_k_few_tiles(k, gb, a_fp8, b_fp8, m, n):
    """Fewer than 512 tiles of 128 x 128 and a long k (a weight gradient): the kernel splits a tile's k range (at a
    multiple of 512, one block of scale bytes; 128 x 128 tiles from 129 up, 128 x 64 below) over two teams of waves and
    adds their sums. Against the oracle on row samples, and bit for bit on integer codes with power-of-two scales, whose
    sums are exact in any order."""
    g = _g()
    torch.manual_seed(k)
    a = torch.randn(m, k) * torch.exp2(torch.randint(-3, 4, (m, 1)).float())
    b = torch.randn(n, k) * torch.exp2(torch.randint(-3, 4, (n, 1)).float())
    qa, sa = og.quantize(a, a_fp8, (1, 32), native=True)
    qb, sb = og.quantize(b, b_fp8, gb, native=True)
    bias = torch.randn(n)
    rows = torch.cat([torch.arange(0, min(m, 140)), torch.arange(min(m, 1900), m)])
    for out_dtype, bound in ((torch.float32, 2e-5), (torch.bfloat16, 3e-3)):
        out = g.gemm(qa.cuda(), qb.cuda(), sa.cuda(), sb.cuda(), (1, 32), gb, out_dtype=out_dtype, native=True, bias=bias.cuda())
        assert rel_l2(out[rows.cuda()], og.gemm(qa[rows], qb, sa[rows], sb, (1, 32), gb, out_dtype=out_dtype, bias=bias)) < bound
        assert torch.equal(out, g.gemm(qa.cuda(), qb.cuda(), sa.cuda(), sb.cuda(), (1, 32), gb, out_dtype=out_dtype, native=True, bias=bias.cuda()))
    ia = torch.randint(-4, 5, (m, k)).float()
    ib = torch.randint(-4, 5, (n, k)).float()
    isa = torch.randint(125, 129, (m, k // 32), dtype=torch.uint8)           # few enough exponents for exact fp32 sums over this k
    isb = torch.randint(126, 129, ((n + gb[0] - 1) // gb[0], k // 32), dtype=torch.uint8)
    exact = g.gemm(ia.to(a_fp8).cuda(), ib.to(b_fp8).cuda(), isa.cuda(), isb.cuda(), (1, 32), gb, out_dtype=torch.float32, native=True)
    da = ia.cuda() * og.decode_scale(isa).cuda().repeat_interleave(32, 1)
    db = ib.cuda() * og.decode_scale(isb).cuda().repeat_interleave(gb[0], 0)[:n].repeat_interleave(32, 1)
    assert torch.equal(exact, (da.double() @ db.double().T).float())


# ----------------------------------------------------------------------------- Linear(scaling="mxfp8")
@pytest.fixture
def precision_policy():
    import viola_amd
    saved = dict(viola_amd.precision._settings)
    yield viola_amd
    viola_amd.precision._settings.clear()
    viola_amd.precision._settings.update(saved)


@pytest.mark.parametrize("mode,storage,backward", [("memory", "fp8", "e4m3"), ("fast", "fp8", "e5m2"), ("memory", "bf16", "e4m3")])
@pytest.mark.parametrize("shape", [(65, 128, 96), (256, 512, 384), (3 * 40, 160, 72)])
def test_linear_mxfp8(precision_policy, mode, storage, backward, shape):
    """checks/check_grouped_linear.py:50-107 with native scales: uint8 scale buffers, codes and bytes of the stored
    weight equal the oracle's, y / dx / dw within .003 of the dequantized-operand matmuls, db exact, state_dict reload
    reproduces the forward bit for bit."""
    from oracle import linear as ol
    viola = precision_policy
    viola.set_gradient_dtype("bf16")
    m, k, n = shape
    torch.manual_seed(90)
    layer = viola.nn.Linear(k, n, device="cuda", dtype=torch.bfloat16, scaling="mxfp8", mode=mode, weight_dtype=storage,
                            backward_dtype=backward)
    bwd = E4 if backward == "e4m3" else E5
    if storage == "fp8":
        assert layer.weight_scale.dtype == torch.uint8 and layer.weight_scale.shape == og.scale_shape((n, k), (32, 32))
        master = layer._initial_weight.detach().cpu()
        rq, rs = og.quantize(master, E4, (32, 32), native=True)
        assert torch.equal(layer.weight.detach().view(torch.uint8).cpu(), rq.view(torch.uint8)) and torch.equal(layer.weight_scale.cpu(), rs)
        if mode == "fast":
            assert layer.weight_transpose_scale.dtype == torch.uint8 and torch.equal(layer.weight_transpose_scale.cpu(), rs.T)
        w_real = og.dequantize(rq, rs, (32, 32))
    else:
        q, s = og.quantize(layer.weight.detach().float().cpu(), E4, (32, 32), native=True)
        w_real = og.dequantize(q, s, (32, 32))
    assert torch.equal(layer.dequantize_weight().cpu(), w_real if storage == "fp8" else layer.weight.detach().float().cpu())
    x = (torch.randn(m, k) * torch.exp2(torch.randint(-5, 6, (m, 1)).float())).bfloat16().cuda().requires_grad_()
    dy = torch.randn(m, n, device="cuda", dtype=torch.bfloat16)
    y = layer(x)
    y.backward(dy)
    expected = ol.linear(x.detach().cpu(), w_real, layer.bias.detach().cpu(), dy.cpu(), fp8=E4, bwd_fp8=bwd, native=True)
    assert rel_l2(y, expected["y"]) < 3e-3 and rel_l2(x.grad, expected["dx"]) < 3e-3 and rel_l2(layer.weight.grad, expected["dw"]) < 3e-3
    assert rel_l2(layer.bias.grad, expected["db"]) < 4e-3
    if storage == "fp8":
        other = viola.nn.Linear(k, n, device="cuda", dtype=torch.bfloat16, scaling="mxfp8", mode=mode, weight_dtype=storage,
                                backward_dtype=backward)
        other.load_state_dict(layer.state_dict())
        with torch.no_grad():
            assert torch.equal(other(x), y)


def test_linear_mxfp8_under_bind_optimizer(precision_policy):
    """A bound AdamW step re-quantizes the master into codes and E8M0 bytes that equal the oracle's."""
    viola = precision_policy
    viola.set_master_weight_dtype("fp32")
    viola.set_gradient_dtype("bf16")
    torch.manual_seed(91)
    layer = viola.nn.Linear(256, 192, device="cuda", dtype=torch.bfloat16, scaling="mxfp8", mode="fast")
    opt = viola.optim.bind_optimizer(layer, torch.optim.AdamW(layer.parameters(), lr=.01))
    x = torch.randn(64, 256, device="cuda", dtype=torch.bfloat16)
    for _ in range(2):
        opt.zero_grad()
        layer(x).float().square().mean().backward()
        before = layer.weight.detach().view(torch.uint8).clone()
        opt.step()
        assert not torch.equal(before, layer.weight.view(torch.uint8))
        rq, rs = og.quantize(layer._master_ref().detach().cpu(), E4, (32, 32), native=True)
        assert torch.equal(layer.weight.detach().view(torch.uint8).cpu(), rq.view(torch.uint8)) and torch.equal(layer.weight_scale.cpu(), rs)
        assert torch.equal(layer.weight_transpose.view(torch.uint8), layer.weight.T.contiguous().view(torch.uint8))
        assert torch.equal(layer.weight_transpose_scale, layer.weight_scale.T)


RECIPES = ([dict(weight_dtype="bf16", scaling=s) for s in ("current", "delayed", "grouped", "mxfp8")]
           + [dict(weight_dtype="fp8", scaling=s, mode="fast", activation="gelu") for s in ("current", "grouped", "mxfp8")]
           + [dict(weight_dtype="fp16", scaling="current", forward_dtype="e5m2", backward_dtype="e4m3", activation="relu"),
              dict(weight_dtype="bf16", scaling="grouped", accum_dtype="fp16", accum_block_size=32),
              dict(weight_dtype="bf16", scaling="current", accum_dtype="fp16", accum_block_size=32),
              dict(weight_dtype="bf16", scaling="mxfp8", bias=False, saved_input_dtype="bf16"),
              dict(weight_dtype="fp8", scaling="delayed", activation="relu", backward_dtype="e4m3")])


@pytest.mark.parametrize("dims", [(128, 160, 96), (128, 256, 128), (256, 384, 256)])
@pytest.mark.parametrize("options", RECIPES, ids=lambda o: "-".join(str(v) for v in o.values()))
def test_mlp_recipes_match_their_unfused_composition(precision_policy, options, dims):
    """checks/mlp.py:12-52 with its recipe list (:63-68): y, dx and every parameter gradient of the MLP, whose GEMMs
    carry the gating in their epilogues, against the model written out with its own two Linears and a float gated
    activation; the reference's bound is .025. (128, 160, 96) is the reference's shape, where the MXFP8 recipe takes
    the plain GEMM plus the elementwise kernels (k = 96 is no multiple of 128); the other two run its fused path."""
    import torch.nn.functional as F
    viola = precision_policy
    viola.set_gradient_dtype("bf16")
    torch.manual_seed(131)
    dtype = torch.float16 if options["weight_dtype"] == "fp16" else torch.bfloat16
    activation = options.get("activation", "silu")
    d_in, hidden, d_out = dims
    model = viola.nn.MLP(d_in, hidden, d_out, device="cuda", dtype=dtype, **options)
    x = torch.randn(2, 33, d_in, device="cuda", dtype=dtype, requires_grad=True)
    dy = torch.randn(2, 33, d_out, device="cuda", dtype=dtype)
    y = model(x)
    y.backward(dy)
    got = [y.detach().clone(), x.grad.clone()] + [p.grad.clone() for p in model.parameters()]
    x.grad = None
    for p in model.parameters():
        p.grad = None
    for layer in (model.gate_up, model.down):                                  # delayed scaling: replay the same history slots
        for quantizer in (layer.input_quantizer, layer.grad_quantizer):
            quantizer.index = 0
            quantizer.history.zero_()
    act = {"silu": F.silu, "relu": F.relu, "gelu": lambda t: F.gelu(t, approximate="tanh")}[activation]
    z = model.gate_up(x)
    g, u = z[..., :hidden], z[..., hidden:]
    reference = model.down((act(g.float()) * u.float()).to(z.dtype))
    reference.backward(dy)
    want = [reference.detach(), x.grad] + [p.grad for p in model.parameters()]
    for a, b in zip(got, want):
        assert a.dtype == b.dtype and rel_l2(a, b) < .025
    # same GEMM sums, same rounding points: the fused epilogue gives the composition's y to bf16 / fp16 rounding
    assert rel_l2(got[0], want[0]) < 2e-3


@pytest.mark.parametrize("fmt", [E4, E5])
@pytest.mark.parametrize("m,h,k,transpose,dtype", [(128, 64, 128, True, torch.bfloat16), (96, 160, 256, True, torch.bfloat16),
                                                   (320, 256, 128, False, torch.float16), (64, 96, 384, True, torch.float32),
                                                   (66, 64, 128, True, torch.bfloat16), (64, 64, 96, True, torch.bfloat16)])
def test_gate_up_gemm_hands_h_over_as_mxfp8_codes(fmt, m, h, k, transpose, dtype):
    """viola/nn/_mlp_kernels.py:195-230 (encode_output, save_output_transpose): the codes and E8M0 bytes of h in both
    layouts equal the oracle's quantization of the h the plain fused kernel writes, bit for bit; [g, u] is unchanged.
    The last two shapes (m not a multiple of 32, k not of 128) take the quantizer after the GEMM instead."""
    import types
    from viola_amd.nn import _mlp_kernels as mk
    torch.manual_seed(23)
    spread = 1 if dtype == torch.float16 else 3                               # keep g * u inside fp16's range
    a = (torch.randn(m, k) * torch.exp2(torch.randint(-spread, spread + 1, (m, 1)).float())).bfloat16()
    w = (torch.randn(2 * h, k) / 8 * torch.exp2(torch.randint(-spread, spread + 1, (2 * h, 1)).float())).bfloat16()
    (qa, sa), (qb, sb) = og.quantize(a, E4, (1, 32), native=True), og.quantize(w, E4, (32, 32), native=True)
    bias = torch.randn(2 * h).to(dtype)
    layer = types.SimpleNamespace(_native_scaling=True, _grouped_scaling=True, input_group_shape=(1, 32), weight_group_shape=(32, 32),
                                  fp8_dtype=fmt, _group_limit=lambda *args, **kwargs: None)
    args = (qa.cuda(), qb.cuda(), sa.cuda(), sb.cuda())
    plain, aux, _ = mk.gemm(*args, layer=layer, out_dtype=dtype, bias=bias.cuda(), activation="silu", save=True)
    codes, aux2, (scale, codes_t, scale_t) = mk.gemm(*args, layer=layer, out_dtype=dtype, bias=bias.cuda(), activation="silu",
                                                     save=True, encode_output=True, save_output_transpose=transpose)
    assert torch.equal(aux2, aux)
    want_q, want_s = og.quantize(plain.cpu(), fmt, (1, 32), native=True)
    assert codes.dtype == fmt and scale.dtype == torch.uint8
    assert torch.equal(scale.cpu(), want_s) and torch.equal(codes.cpu().view(torch.uint8), want_q.view(torch.uint8))
    if transpose:
        want_qt, want_st = og.quantize(plain.cpu(), fmt, (1, 32), native=True, transposed=True)
        assert torch.equal(scale_t.cpu(), want_st) and torch.equal(codes_t.cpu().view(torch.uint8), want_qt.view(torch.uint8))
    else:
        assert codes_t.numel() == 0 and scale_t.numel() == 0
    nosave = mk.gemm(*args, layer=layer, out_dtype=dtype, bias=bias.cuda(), activation="silu", save=False, encode_output=True)
    assert nosave[1].numel() == 0 and torch.equal(nosave[0].view(torch.uint8), codes.view(torch.uint8))


@pytest.mark.parametrize("dims,tokens", [((128, 256, 128), 128), ((256, 384, 256), 96), ((128, 160, 96), 64)])
@pytest.mark.parametrize("options", [dict(weight_dtype="fp8", mode="fast", activation="gelu"), dict(weight_dtype="bf16"),
                                     dict(weight_dtype="bf16", bias=False, saved_input_dtype="bf16")],
                         ids=lambda o: "-".join(str(v) for v in o.values()))
def test_mxfp8_mlp_with_encoded_h_matches_its_unfused_composition(precision_policy, options, dims, tokens):
    """The MXFP8 MLP at token counts that are multiples of 32, where h travels from the gate/up GEMM to the down
    projection as codes (mlp.py:103-107), against the two Linears with a float activation between them."""
    import torch.nn.functional as F
    viola = precision_policy
    viola.set_gradient_dtype("bf16")
    torch.manual_seed(131)
    activation = options.get("activation", "silu")
    d_in, hidden, d_out = dims
    model = viola.nn.MLP(d_in, hidden, d_out, device="cuda", dtype=torch.bfloat16, scaling="mxfp8", **options)
    x = torch.randn(tokens, d_in, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    dy = torch.randn(tokens, d_out, device="cuda", dtype=torch.bfloat16)
    y = model(x)
    y.backward(dy)
    got = [y.detach().clone(), x.grad.clone()] + [p.grad.clone() for p in model.parameters()]
    x.grad = None
    for p in model.parameters():
        p.grad = None
    act = {"silu": F.silu, "relu": F.relu, "gelu": lambda t: F.gelu(t, approximate="tanh")}[activation]
    z = model.gate_up(x)
    g, u = z[..., :hidden], z[..., hidden:]
    reference = model.down((act(g.float()) * u.float()).to(z.dtype))
    reference.backward(dy)
    want = [reference.detach(), x.grad] + [p.grad for p in model.parameters()]
    for a, b in zip(got, want):
        assert a.dtype == b.dtype and rel_l2(a, b) < .025
    assert rel_l2(got[0], want[0]) < 2e-3
    # frozen down weight: no transposed codes are produced, the forward still runs on codes
    model.down.weight.requires_grad_(False)
    with torch.no_grad():
        assert torch.equal(model(x), y)
