"""GPU parity: group quantize / dequantize / transpose through the C ABI vs the CPU oracle, bit-exact."""

import pytest
import torch

from oracle import grouped as og
from conftest import rel_l2

pytestmark = pytest.mark.gpu
E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2


def _gpu():
    from viola_amd.nn import _grouped_kernels as g
    return g


def _input(shape, dtype, seed=2041):
    torch.manual_seed(seed)
    x = torch.randn(*shape) * torch.exp2(torch.randint(-5, 6, (shape[0], 1)).float())
    return x.to(dtype)


def _same(q, s, rq, rs):
    assert q.dtype == rq.dtype and tuple(q.shape) == tuple(rq.shape) and tuple(s.shape) == tuple(rs.shape)
    assert torch.equal(s.cpu(), rs), "scales differ"
    assert torch.equal(q.cpu().view(torch.uint8), rq.view(torch.uint8)), "codes differ"


def test_hardware_fp8_conversions_vs_software():
    """Exhaustive: every fp32 bit pattern in range through v_cvt_pk_{fp8,bf8}_f32, all 256 codes back."""
    from viola_amd import _lib
    counts = torch.zeros(4, dtype=torch.int64, device="cuda")
    _lib.call("viola_selftest_fp8", _lib.ptr(counts))
    torch.cuda.synchronize()
    # [e4m3 encode, e5m2 encode, e4m3 decode, e5m2 decode]: every fast quantizer path relies on all four being zero
    assert counts.tolist() == [0, 0, 0, 0], f"hardware vs software FP8 conversion mismatches {counts.tolist()}"


def test_software_codecs_all_codes():
    """dequantize of every code with unit scale == torch's decode; quantize of every finite value is the identity."""
    g = _gpu()
    for dtype in (E4, E5):
        codes = torch.arange(256, dtype=torch.uint8).view(dtype).reshape(8, 32)
        out = g.dequantize(codes.cuda(), torch.ones(8, 1, device="cuda"), (1, 32)).cpu()
        ref = codes.float()
        assert torch.equal(out.isnan(), ref.isnan()) and torch.equal(out.nan_to_num(1.0, 2.0, 3.0), ref.nan_to_num(1.0, 2.0, 3.0))
        finite = ref.flatten()[ref.flatten().isfinite()]
        x = finite.repeat(2)[:256 + 64].reshape(-1, 32).contiguous()
        x[:, 0] = torch.finfo(dtype).max                                     # unit scale in every row tile
        q, s = g.quantize(x.cuda(), dtype, (1, 32))
        assert torch.equal(s.cpu(), torch.ones_like(s.cpu())) and torch.equal(q.float().cpu(), x)


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("fp8", [E4, E5])
@pytest.mark.parametrize("group,shape", [((1, 32), (65, 96)), ((1, 32), (256, 1024)), ((1, 64), (96, 136)), ((1, 128), (33, 256)),
                                          ((32, 32), (96, 128)), ((32, 32), (70, 45)), ((32, 32), (70, 132)), ((32, 32), (257, 1000)), ((32, 64), (64, 160)), ((64, 32), (130, 96)),
                                          ((1, 32), (7, 33)), ((1, 512), (9, 1024))])
def test_quantize_rowwise_and_blocks(in_dtype, fp8, group, shape):
    g = _gpu()
    x = _input(shape, in_dtype)
    q, s = g.quantize(x.cuda(), fp8, group)
    _same(q, s, *og.quantize(x, fp8, group))
    deq = g.dequantize(q, s, group)
    assert torch.equal(deq.cpu(), og.dequantize(q.cpu(), s.cpu(), group))


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("fp8", [E4, E5])
@pytest.mark.parametrize("group,shape", [((1, 32), (65, 96)), ((1, 32), (300, 200)), ((1, 32), (128, 64)), ((1, 32), (31, 7)),
                                          ((32, 32), (96, 70)), ((1, 64), (96, 65)), ((64, 32), (64, 160))])
def test_quantize_transposed(in_dtype, fp8, group, shape):
    g = _gpu()
    x = _input(shape, in_dtype, seed=7)
    q, s = g.quantize(x.cuda(), fp8, group, transposed=True)
    _same(q, s, *og.quantize(x, fp8, group, transposed=True))


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(65, 128), (128, 64), (300, 200), (1, 32), (129, 72), (8192, 1024), (176, 200), (16, 64), (144, 72), (272, 136),
                                   (2064, 4104), (1048, 8200)])     # the last two: ragged on both sides at sizes that take the XCD-contiguous walk
def test_quantize_dual_equals_two_passes(in_dtype, shape):
    g = _gpu()
    x = _input(shape, in_dtype, seed=11)
    q, s, qt, st = g.quantize_dual(x.cuda(), E4, (1, 32))
    _same(q, s, *og.quantize(x, E4, (1, 32)))
    _same(qt, st, *og.quantize(x, E4, (1, 32), transposed=True))


@pytest.mark.parametrize("fp8", [E4, E5])
@pytest.mark.parametrize("limit", [None, 240.0])
def test_quantize_rounding_ties_over_all_magnitudes(fp8, limit):
    """The kernels replace v / s by a reciprocal and two FMAs where that is provably the same quotient.
    Values sitting exactly on FP8 rounding ties (where a one-ulp error in the quotient flips the code),
    groups from 1e-36 to 1e30 in magnitude (tiny scales fall back to true division) and groups with
    NaN / Inf members must all give the oracle's codes and scales."""
    g = _gpu()
    torch.manual_seed(77)
    rows, cols = 512, 256
    top = torch.finfo(fp8).max if limit is None else limit
    amax = torch.exp(torch.empty(rows, cols // 32, 1).uniform_(-83., 69.))               # 1e-36 .. 1e30
    scale = amax.clamp_min(1e-30) / top
    mant = 3 if fp8 == E4 else 2
    k = torch.randint(2 ** mant, 2 ** (mant + 1), (rows, cols // 32, 32)).float()
    j = torch.randint(-12 if fp8 == E4 else -19, 7 if fp8 == E4 else 14, (rows, cols // 32, 32)).float()
    tie = (k + .5) / 2 ** mant * torch.exp2(j)
    x = scale * tie * torch.where(torch.rand_like(tie) < .5, -1., 1.)
    x = torch.where(x.abs() > amax, amax, x)
    x[..., 0] = amax[..., 0]
    x = x.reshape(rows, cols).contiguous()
    x[5, 40] = float("nan")
    x[6, 70] = float("inf")
    x[7, 100:132] = 0
    x[9, ::3] = -0.0
    for transposed in (False, True):
        q, sc = g.quantize(x.cuda(), fp8, (1, 32), limit=limit, transposed=transposed)
        rq, rs = og.quantize(x, fp8, (1, 32), limit=limit, transposed=transposed)
        _same(q, sc, rq, rs)
    q, sc, qt, st = g.quantize_dual(x.cuda(), fp8, (1, 32), limit=limit)
    _same(q, sc, *og.quantize(x, fp8, (1, 32), limit=limit))
    _same(qt, st, *og.quantize(x, fp8, (1, 32), limit=limit, transposed=True))
    q, sc = g.quantize(x.cuda(), fp8, (32, 32), limit=limit)
    _same(q, sc, *og.quantize(x, fp8, (32, 32), limit=limit))


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(65, 128), (300, 200), (129, 72), (8192, 1024), (32, 64), (176, 200), (144, 72), (2064, 4104)])
def test_quantize_dual_column_sums(in_dtype, shape):
    """x.sum(0) from the quantizer's own read: fp32 accumulation in a fixed order, same codes as without it."""
    g = _gpu()
    x = _input(shape, in_dtype, seed=13)
    plain = g.quantize_dual(x.cuda(), E4, (1, 32))
    for out_dtype in (torch.float32, in_dtype):
        *codes, total = g.quantize_dual(x.cuda(), E4, (1, 32), column_sum_dtype=out_dtype)
        for a, b in zip(codes, plain):
            assert torch.equal(a.view(torch.uint8) if a.dtype == E4 else a, b.view(torch.uint8) if b.dtype == E4 else b)
        ref = x.double().sum(0)
        assert total.dtype == out_dtype and total.shape == (shape[1],)
        # fp32 partial sums: error well below one rounding of the widest term per 32 rows
        bound = x.double().abs().sum(0) * 2.0 ** -22 + (ref.abs() * torch.finfo(out_dtype).eps)
        assert ((total.cpu().double() - ref).abs() <= bound + 1e-30).all()
    again = g.quantize_dual(x.cuda(), E4, (1, 32), column_sum_dtype=torch.float32)[-1]
    assert torch.equal(again, g.quantize_dual(x.cuda(), E4, (1, 32), column_sum_dtype=torch.float32)[-1])    # deterministic


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float16])
def test_quantize_dual_nonfinite_tiny_and_huge_groups(in_dtype):
    """Groups that leave the quotient route in either layout: a NaN, an Inf, magnitudes whose scale underflows the route's
    domain, the format's largest values, all-zero groups; next to ordinary groups of the same wavefront and tile."""
    g = _gpu()
    torch.manual_seed(17)
    x = torch.randn(200, 136)
    x[3, 5], x[70, 100], x[130, 40] = float("nan"), float("inf"), float("-inf")
    x[10:12, :64] = 0.0
    x[20:52, 32:64] *= 1e-30 if in_dtype == torch.bfloat16 else 6e-8         # subnormal in fp16
    x[64:96, 64:96] *= 3e38 if in_dtype == torch.bfloat16 else 6e4
    x[100, 0:32] = torch.finfo(in_dtype).max
    x = x.to(in_dtype)
    q, s, qt, st = g.quantize_dual(x.cuda(), E4, (1, 32))
    for got, got_scale, transposed in ((q, s, False), (qt, st, True)):
        rq, rs = og.quantize(x, E4, (1, 32), transposed=transposed)
        assert torch.equal(got_scale.cpu().isnan(), rs.isnan()) and torch.equal(got_scale.cpu().nan_to_num(7.0), rs.nan_to_num(7.0))
        # code bytes, the NaN codes included: 0x7f | sign from the software encoder, never the hardware converters' 0xff
        assert torch.equal(got.cpu().view(torch.uint8), rq.view(torch.uint8))


def test_quantize_limit_and_out_arguments():
    g = _gpu()
    x = _input((64, 96), torch.float32, seed=3)
    q, s = g.quantize(x.cuda(), E4, (32, 32), limit=8.0)
    _same(q, s, *og.quantize(x, E4, (32, 32), limit=8.0))
    out = torch.empty((64, 96), device="cuda", dtype=E4)
    scale_out = torch.empty((2, 3), device="cuda")
    q2, s2 = g.quantize(x.cuda(), E4, (32, 32), out=out, scale_out=scale_out)
    assert q2 is out and s2 is scale_out
    _same(out, scale_out, *og.quantize(x, E4, (32, 32)))


def test_quantize_nonfinite_and_zero():
    g = _gpu()
    x = torch.ones(4, 64)
    x[0, 3], x[1, 40], x[2] = float("nan"), float("inf"), 0.0
    for transposed in (False, True):
        q, s = g.quantize(x.cuda(), E4, (1, 32), transposed=transposed)
        rq, rs = og.quantize(x, E4, (1, 32), transposed=transposed)
        assert torch.equal(s.cpu(), rs)
        a, b = q.float().cpu(), rq.float()
        assert torch.equal(a.isnan(), b.isnan()) and torch.equal(a.nan_to_num(9.0), b.nan_to_num(9.0))
    q, s = g.quantize(torch.zeros(0, 32, device="cuda"), E4, (1, 32))
    assert q.numel() == 0 and s.numel() == 0


@pytest.mark.parametrize("group", [(32, 32), (1, 32), (64, 32)])
def test_transpose_of_codes(group):
    g = _gpu()
    w = _input((96, 160), torch.float32, seed=5)
    q, s = og.quantize(w, E4, group)
    qt, st = g.transpose(q.cuda(), s.cuda(), group)
    _same(qt, st, *og.transpose(q, s, group))
    from viola_amd.nn._linear_kernels import transpose
    raw = torch.randint(0, 255, (70, 45), dtype=torch.uint8).view(E4)
    assert torch.equal(transpose(raw.cuda()).cpu().view(torch.uint8), raw.view(torch.uint8).T)


def test_full_size_properties():
    """C2-sized inputs: properties that need no CPU oracle at that size."""
    g = _gpu()
    torch.manual_seed(1)
    dy = (torch.randn(8192, 4096) * 1e-2).bfloat16().cuda()
    q, s, qt, st = g.quantize_dual(dy, E4, (1, 32))
    assert q.float().abs().reshape(8192, 128, 32).amax(2).eq(448).all()          # every tile reaches the limit
    assert qt.float().abs().reshape(4096, 256, 32).amax(2).eq(448).all()
    assert rel_l2(g.dequantize(q, s, (1, 32)), dy.float()) < 0.04
    assert rel_l2(g.dequantize(qt, st, (1, 32)).T, dy.float()) < 0.04
    q1, s1 = g.quantize(dy, E4, (1, 32))
    q2, s2 = g.quantize(dy, E4, (1, 32), transposed=True)
    assert torch.equal(q1.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s1, s)
    assert torch.equal(q2.view(torch.uint8), qt.view(torch.uint8)) and torch.equal(s2, st)
    # idempotence: quantizing the dequantized tensor reproduces codes and scales
    q3, s3 = g.quantize(g.dequantize(q, s, (1, 32)), E4, (1, 32))
    assert torch.equal(q3.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s3, s)


@pytest.mark.parametrize("native", [False, True])
@pytest.mark.parametrize("shape,group", [((96, 128), (32, 32)), ((4096, 1024), (32, 32)), ((65, 100), (32, 64)), ((130, 33), (64, 32)),
                                         ((7, 5), (32, 32))])
def test_block_transpose_moves_codes_and_scale_grid_in_one_launch(shape, group, native):
    """viola/nn/_grouped_kernels.py:161-164: a 2-D-block-scaled matrix transposes exactly, payload and scale grid."""
    from viola_amd.nn import _grouped_kernels as g
    torch.manual_seed(19)
    x = torch.randn(shape) * torch.logspace(-3, 3, shape[1])
    q, s = og.quantize(x, E4, group, native=native)
    qt, st = g.transpose(q.cuda(), s.cuda(), group, native=native)
    want_q, want_s = og.transpose(q, s, group, native=native)
    assert qt.shape == (shape[1], shape[0]) and st.dtype == s.dtype
    assert torch.equal(qt.cpu().view(torch.uint8), want_q.view(torch.uint8)) and torch.equal(st.cpu(), want_s)
    assert torch.equal(st.cpu(), s.T) and torch.equal(qt.cpu().view(torch.uint8), q.view(torch.uint8).T)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("activation", ["silu", "gelu", "relu"])
@pytest.mark.parametrize("native", [False, True])
def test_gated_quantize_dual_equals_activation_then_quantize(dtype, activation, native):
    """h = act(g) * u quantized in both layouts straight from [g | u] is, bit for bit, the dual quantizer run on the
    stored h of the activation kernel; ragged rows and a width that is not a multiple of the 64-column tile. (silu:
    the kernel uses the gated GEMM epilogue's g * (1 / (1 + exp(-g))), the activation operator g / (1 + exp(-g)); h
    may differ in its last place there, so codes are compared after decoding; the exact silu check is the large-tile
    test of the gated GEMMs.)"""
    from viola_amd.nn import _gated_kernels as gk, _grouped_kernels as g
    torch.manual_seed(5)
    for rows, h in ((100, 72), (256, 128), (33, 8), (176, 72)):
        z = (torch.randn(rows, 2 * h, device="cuda") * torch.exp2(torch.randint(-6, 5, (rows, 1), device="cuda").float())).to(dtype)
        z[3, 5] = float("nan")
        for fp8 in (torch.float8_e4m3fn, torch.float8_e5m2):
            got = g.gated_quantize_dual(z, activation, fp8, native=native)
            assert got is not None
            _, hidden = gk.gated_forward(z, activation)
            want = g.quantize_dual(hidden, fp8, (1, 32), native=native)
            if activation == "silu":
                keep = ~torch.isnan(hidden.float())
                group = (1, 32)
                assert rel_l2(torch.where(keep, g.dequantize(got[0], got[1], group), 0), torch.where(keep, g.dequantize(want[0], want[1], group), 0)) < 2e-2
                assert (got[0].view(torch.uint8) == want[0].view(torch.uint8)).float().mean() > 0.98
                continue
            for a, b in zip(got, want):
                assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    assert g.gated_quantize_dual(torch.zeros(4, 2 * 12, device="cuda", dtype=dtype), activation, torch.float8_e4m3fn) is None
    assert g.gated_quantize_dual(torch.zeros(4, 64, device="cuda"), activation, torch.float8_e4m3fn) is None
