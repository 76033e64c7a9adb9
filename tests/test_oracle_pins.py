"""Pins for the CPU oracle itself: every check here is something the oracle's own formula does not
decide (golden vectors held by the reference, an independent implementation, a closed form, an
invariant), so that a dropped term / wrong index / wrong sign in the oracle fails. No GPU."""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import comm, fp8, grouped, linear, ns, optim
from conftest import rel_l2

E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2


# ----------------------------------------------------------------------------- FP8 casts
@pytest.mark.parametrize("name,dtype", [("e4m3", E4), ("e5m2", E5)])
def test_decode_table_matches_torch(name, dtype):
    table = fp8.decode_table(name)
    ours = torch.from_numpy(table)
    theirs = torch.arange(256, dtype=torch.uint8).view(dtype).float()
    assert torch.equal(ours.isnan(), theirs.isnan())
    assert torch.equal(ours.nan_to_num(7.0), theirs.nan_to_num(7.0))


@pytest.mark.parametrize("name,dtype", [("e4m3", E4), ("e5m2", E5)])
def test_torch_cast_is_rne_on_the_grid(name, dtype):
    """torch's CPU cast (what the reference's CPU oracles call) == exact nearest-even search."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(200000, generator=g) * torch.exp2(torch.randint(-20, 18, (200000,), generator=g).float())
    table = torch.from_numpy(fp8.decode_table(name))
    finite = table[table.isfinite()]
    mids = (finite.sort().values[:-1] + finite.sort().values[1:]) / 2             # every tie point
    special = torch.tensor([0.0, -0.0, 447.9, 448.0, 463.9, 464.0, 464.1, 479.9, 480.0, 500.0, 57344.0, 61439.0,
                            61440.0, 65536.0, 1e30, -1e30, float("inf"), -float("inf"), float("nan"), 2.0 ** -10,
                            2.0 ** -9, 1.5 * 2.0 ** -10, 2.0 ** -17, 2.0 ** -16, 3 * 2.0 ** -17])
    x = torch.cat([x, finite, mids, torch.nextafter(mids, mids + 1), torch.nextafter(mids, mids - 1), special])
    ours = torch.from_numpy(fp8.encode(x.numpy(), name))
    theirs = x.to(dtype).view(torch.uint8)
    nan_ours = torch.from_numpy(np.isnan(fp8.decode_table(name)))[ours.long()]
    nan_theirs = torch.from_numpy(np.isnan(fp8.decode_table(name)))[theirs.long()]
    assert torch.equal(nan_ours, nan_theirs)
    keep = ~nan_ours
    assert torch.equal(ours[keep], theirs[keep])


def test_cast_cases_the_quantizers_rely_on():
    x = torch.tensor([447.9, 448.0, 464.0, float("nan"), -float("nan")])
    codes = x.to(E4).view(torch.uint8)
    assert codes[:3].tolist() == [0x7E, 0x7E, 0x7E] and (codes[3] & 0x7F) == 0x7F
    assert torch.tensor([500.0]).clamp(-448, 448).to(E4).view(torch.uint8).item() == 0x7E
    assert torch.tensor([float("nan")]).clamp(-448, 448).isnan().item()          # clamp keeps NaN


# ----------------------------------------------------------------------------- group quantize
@pytest.mark.parametrize("dtype", [E4, E5])
@pytest.mark.parametrize("group,shape", [((1, 32), (65, 96)), ((32, 32), (96, 70)), ((1, 64), (33, 130)), ((32, 64), (64, 160))])
def test_quantize_invariants(dtype, group, shape):
    torch.manual_seed(1)
    x = (torch.randn(*shape) * torch.exp2(torch.randint(-5, 6, (shape[0], 1)).float())).bfloat16()
    q, s = grouped.quantize(x, dtype, group)
    assert q.shape == x.shape and tuple(s.shape) == grouped.scale_shape(shape, group)
    limit = torch.finfo(dtype).max
    # the largest element of each group maps to +-limit and the scale is amax/limit exactly
    gr, gc = group
    pad = F.pad(x.float(), (0, s.shape[1] * gc - shape[1], 0, s.shape[0] * gr - shape[0]))
    amax = pad.reshape(s.shape[0], gr, s.shape[1], gc).abs().amax((1, 3))
    assert torch.equal(s, amax.clamp_min(1e-30) / limit)
    qpad = F.pad(q.float(), (0, s.shape[1] * gc - shape[1], 0, s.shape[0] * gr - shape[0]))
    assert torch.equal(qpad.reshape(s.shape[0], gr, s.shape[1], gc).abs().amax((1, 3))[amax > 0],
                       torch.full_like(amax, limit)[amax > 0])
    # element-wise against a scalar loop on a sample of positions (independent indexing)
    table = fp8.decode_table("e4m3" if dtype == E4 else "e5m2")
    for r, c in [(0, 0), (shape[0] - 1, shape[1] - 1), (shape[0] // 2, shape[1] // 3), (1, shape[1] - 1)]:
        sc = s[r // gr, c // gc].item()
        v = np.float32(x[r, c].float().item()) / np.float32(sc)
        expect = fp8.encode(np.clip(np.array([v], dtype=np.float32), -limit, limit), "e4m3" if dtype == E4 else "e5m2")[0]
        assert q.view(torch.uint8)[r, c].item() == expect
    # quantization error bound: half a grid step at the element's magnitude
    deq = grouped.dequantize(q, s, group)
    mant = 3 if dtype == E4 else 2
    assert rel_l2(deq, x.float()) < 2.0 ** -(mant + 1)


def test_quantize_exact_roundtrip_and_transpose():
    """Representable values times a power-of-two scale come back exactly; transposed == quantize(x.T)."""
    torch.manual_seed(2)
    codes = torch.randint(0, 0x7F, (64, 64), dtype=torch.uint8)
    codes[::32, ::32] = 0x7E                                   # every (32,32) block and (1,32) row tile holds 448
    codes[:, ::32] = 0x7E
    value = codes.view(E4).float() * 0.25
    for group in ((1, 32), (32, 32)):
        q, s = grouped.quantize(value, E4, group)
        assert torch.equal(grouped.dequantize(q, s, group), value)
    x = torch.randn(70, 45).bfloat16()
    qt, st = grouped.quantize(x, E4, (1, 32), transposed=True)
    q2, s2 = grouped.quantize(x.T.contiguous(), E4, (1, 32))
    assert torch.equal(qt.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(st, s2)
    assert qt.shape == (45, 70) and st.shape == (45, 3)


def test_quantize_nan_inf_follow_the_device_kernel():
    x = torch.ones(2, 64)
    x[0, 3], x[1, 40] = float("nan"), float("inf")
    q, s = grouped.quantize(x, E4, (1, 32))
    d = q.float()
    assert d[0, 3].isnan() and d[0, :3].eq(448).all() and s[0, 0] == 1 / 448     # NaN stays local
    assert s[1, 1].isinf() and d[1, 40].isnan() and d[1, 33] == 0                  # inf/inf = NaN, finite/inf = 0


def test_reencode_and_transpose_rules():
    torch.manual_seed(3)
    w = torch.randn(64, 96)
    q, s = grouped.quantize(w, E4, (32, 32))
    qt, st = grouped.transpose(q, s, (32, 32))
    assert torch.equal(grouped.dequantize(qt, st, (32, 32)), grouped.dequantize(q, s, (32, 32)).T)
    q1, s1 = grouped.quantize(w, E4, (1, 32))
    qt1, st1 = grouped.transpose(q1, s1, (1, 32))               # 1-D groups must be re-encoded
    again, sa = grouped.quantize(grouped.dequantize(q1, s1, (1, 32)), E4, (1, 32), transposed=True)
    assert torch.equal(qt1.view(torch.uint8), again.view(torch.uint8)) and torch.equal(st1, sa)


# ----------------------------------------------------------------------------- grouped GEMM
@pytest.mark.parametrize("ga,gb,fa,fb,shape", [((1, 32), (32, 32), E4, E4, (65, 96, 128)), ((1, 64), (32, 64), E5, E4, (96, 65, 64)),
                                                ((32, 64), (64, 32), E4, E5, (64, 160, 96))])
def test_gemm_oracle_vs_fp64_and_kernel_order(ga, gb, fa, fb, shape):
    """fp32 dequantize-matmul == fp64 witness == the device kernel's per-K-group order, to fp32 rounding."""
    m, k, n = shape
    torch.manual_seed(2041)
    a = (torch.randn(m, k) * torch.exp2(torch.randint(-5, 6, (m, 1)).float())).bfloat16()
    b = (torch.randn(n, k) * torch.exp2(torch.randint(-5, 6, (n, 1)).float())).bfloat16()
    qa, sa = grouped.quantize(a, fa, ga)
    qb, sb = grouped.quantize(b, fb, gb)
    bias = torch.randn(n)
    plain = grouped.gemm(qa, qb, sa, sb, ga, gb, bias=bias)
    witness = grouped.gemm(qa, qb, sa, sb, ga, gb, bias=bias, witness=True, out_dtype=torch.float64)
    ordered = grouped.gemm_kgroup_order(qa, qb, sa, sb, ga, gb, bias=bias) if ga[1] % 32 == 0 and k % 32 == 0 else plain
    assert rel_l2(plain, witness) < 2e-6 and rel_l2(ordered, witness) < 2e-6
    # brute force on a few entries, written with scalar indexing
    da, db = qa.float().double(), qb.float().double()
    for i, j in [(0, 0), (m - 1, n - 1), (m // 2, n // 3)]:
        total = sum(da[i, kk] * sa[i // ga[0], kk // ga[1]].double() * db[j, kk] * sb[j // gb[0], kk // gb[1]].double()
                    for kk in range(k)) + bias[j].double()
        assert abs(witness[i, j] - total) <= 1e-6 * max(1.0, abs(total))   # dequantize rounds code*scale to fp32


# ----------------------------------------------------------------------------- Philox / stochastic rounding
def test_philox_known_answers():
    """Random123 kat_vectors for philox4x32-10, word 0 (held by the reference, checks/quantization.py:77-81)."""
    triples = [(0, 0, 0), (0xffffffffffffffff,) * 3, (0x85a308d3243f6a88, 0x0370734413198a2e, 0x299f31d0a4093822)]
    answers = [int(optim.philox(np.array([e], dtype=np.uint64), s, k)[0]) for e, s, k in triples]
    assert answers == [0x6627e8d5, 0x408f276d, 0xd16cfe09]


def test_stochastic_round_probability_and_adjacency():
    n = 256 * 1024
    x = np.full(n, 1 + .27 * .125, dtype=np.float32)
    out = optim.stochastic_round_e4m3(x, np.arange(n, dtype=np.uint64), 7, 42)
    assert set(np.unique(out)) == {np.float32(1.0), np.float32(1.125)}
    assert abs((out == 1.125).mean() - .27) < .005                                # checks/quantization.py:114-136
    assert not np.array_equal(out, optim.stochastic_round_e4m3(x, np.arange(n, dtype=np.uint64), 8, 42))
    table = fp8.decode_table("e4m3")[:127]
    values = np.tile(table[:-1] * .7 + table[1:] * .3, 64).astype(np.float32)
    both = np.concatenate([values, -values, np.tile(table, 64)])
    out = optim.stochastic_round_e4m3(both, np.arange(both.size, dtype=np.uint64), 0, 0)
    idx = np.searchsorted(table, np.abs(both)).clip(max=126)
    lower, upper = table[np.maximum(idx - 1, 0)], table[idx]
    assert (((np.abs(out) == lower) | (np.abs(out) == upper))).all()              # checks/quantization.py:138-153
    assert ((np.sign(out) == np.sign(both)) | (out == 0)).all()


@pytest.mark.parametrize("fn,spacing", [(optim.stochastic_bf16, 2.0 ** -8), (optim.stochastic_fp16, 2.0 ** -11)])
def test_stochastic_storage_rounding_fraction(fn, spacing):
    """One quarter of a grid step below 1: kept about 25 % of the time (checks/precision_kernels.py:48-58)."""
    n = 131072
    x = np.full(n, 1.0 - spacing / 4, dtype=np.float32)
    out = fn(x, np.arange(n, dtype=np.uint64), 17, 29)
    assert set(np.unique(out)) <= {np.float32(1.0), np.float32(1.0 - spacing)}
    assert abs((out != 1.0).mean() - .25) < .005
    cut = 13001
    replay = np.concatenate([fn(x[:cut], np.arange(cut, dtype=np.uint64), 17, 29),
                             fn(x[cut:], np.arange(n - cut, dtype=np.uint64) + np.uint64(cut), 17, 29)])
    assert np.array_equal(out, replay)


# ----------------------------------------------------------------------------- momentum / weight / adam
@pytest.mark.parametrize("granularity,size", [("tile", 64), ("tile", 256), ("tile", 1024), ("block", (8, 8)), ("block", (16, 32)), ("block", (64, 64))])
@pytest.mark.parametrize("shape", [(17, 31), (2, 33, 67)])
def test_momentum_against_the_reference_checks(granularity, size, shape):
    """The closed forms of checks/quantization.py:27-53,83-112 written independently of oracle.optim's body."""
    torch.manual_seed(79)
    quant = dict(granularity=granularity, tile_size=size if granularity == "tile" else 256,
                 block_shape=size if granularity == "block" else (16, 16))
    qn, sn = optim.state_sizes(shape, **quant)
    n = math.prod(shape)
    q, scale = torch.zeros(qn, dtype=torch.uint8), torch.ones(sn)
    for step in range(4):
        g = torch.randn(n) * (1e-8 if step < 1 else 1.)
        old = optim.dequantize(q, scale, shape, **quant)
        fresh = .95 * old.double() + .05 * g.double()
        q, scale, u = optim.momentum_update(g, q, scale, beta=.95, shape=shape, **quant)
        if granularity == "tile":
            tiles = F.pad(fresh, (0, qn - n)).view(-1, size)
        else:
            rows, cols = shape[-2:]
            tr, tc = size
            p = F.pad(fresh.view(-1, rows, cols), (0, (-cols) % tc, 0, (-rows) % tr))
            tiles = p.view(-1, p.shape[1] // tr, tr, p.shape[2] // tc, tc).permute(0, 1, 3, 2, 4).reshape(-1, tr * tc)
        expected_scale = (tiles.abs().amax(1).clamp_min(1e-30) / 448).float()
        torch.testing.assert_close(scale, expected_scale, rtol=2e-6, atol=1e-30)
        torch.testing.assert_close(u.float(), (.05 * g.double() + .95 * fresh).float().bfloat16().float(), rtol=.01, atol=2e-7)
        current = optim.dequantize(q, scale, shape, **quant)
        assert ((current - fresh).norm() / fresh.norm()).item() < .06
        assert q.numel() == qn and scale.numel() == sn


def test_momentum_zero_stays_zero_and_loss_scale():
    q, scale, u = optim.momentum_update(torch.zeros(300), torch.zeros(512, dtype=torch.uint8), torch.ones(2), beta=.95,
                                        shape=(300,), tile_size=256)
    assert q.count_nonzero() == 0 and u.count_nonzero() == 0 and torch.equal(scale, torch.full((2,), 1e-30) / 448)
    g = torch.randn(257).half()
    _, _, u = optim.momentum_update(g, torch.zeros(512, dtype=torch.uint8), torch.ones(2), beta=.95, shape=(257,),
                                    tile_size=256, loss_scale=32.0, nesterov=False)
    torch.testing.assert_close(u.float(), (.05 * g.float() / 32).bfloat16().float(), rtol=.01, atol=2e-7)


def test_weight_and_adam_closed_forms():
    torch.manual_seed(107)
    for wdtype in (torch.float32, torch.bfloat16, torch.float16):
        w = (torch.randn(1025) * .1).to(wdtype)
        g = (torch.randn(1025) * .01)
        new = optim.weight_update(w, g, .001, .01, update_scale=3.0)
        target = w.double() * (1 - .001 * .01) - .001 * 3.0 * g.double()
        assert (new.double() - target).abs().max() <= 1.01 * (torch.finfo(wdtype).eps * target.abs().max())
        m, v = torch.zeros(1025), torch.zeros(1025)
        cur = w
        for step in range(1, 4):
            rm = .9 * m.double() + .1 * g.double()
            rv = .95 * v.double() + .05 * g.double().square()
            value = cur.double() * (1 - .001 * .01) - .001 * (rm / (1 - .9 ** step)) / ((rv / (1 - .95 ** step)).sqrt() + 1e-8)
            cur, m, v = optim.adam_update(cur, g, m, v, lr=.001, weight_decay=.01, betas=(.9, .95), eps=1e-8, step=step)
            torch.testing.assert_close(m.double(), rm, rtol=2e-6, atol=1e-12)
            torch.testing.assert_close(v.double(), rv, rtol=2e-6, atol=1e-12)
            assert (cur.double() - value).abs().max() <= 1.01 * torch.finfo(wdtype).eps * value.abs().max()
    out = optim.copy_scaled(torch.arange(20.).bfloat16(), torch.zeros(30), 11, 3, 5, 3.2)
    assert torch.equal(out[3:8], torch.arange(11., 16.) * torch.tensor(3.2)) and out[:3].eq(0).all() and out[8:].eq(0).all()


# ----------------------------------------------------------------------------- wire codec
@pytest.mark.parametrize("tile,n", [(64, 1), (64, 31), (256, 513), (1024, 8193), (256, 65539)])
@pytest.mark.parametrize("dtype", [E4, E5])
def test_comm_roundtrip_matches_reference_formula(tile, n, dtype):
    """pack -> unpack == pad / amax / cast / multiply back (checks/fp8_communication.py:32-38)."""
    torch.manual_seed(300)
    x = torch.randn(n) * torch.logspace(-5, 5, n)
    x[::31] *= 64
    groups = math.ceil(n / tile)
    packet = comm.pack(x, 1, groups, tile, dtype)
    assert packet.shape == (1, comm.packet_bytes(groups, tile)) and packet.shape[1] % 16 == 0
    out = comm.unpack(packet, n, tile, dtype)
    assert torch.equal(out, comm.roundtrip(x, tile, dtype))
    # rows = R with reduce: the sum of the R single-row decodes, rank order
    rows = 3
    g3 = math.ceil(n / (rows * tile))
    packet3 = comm.pack(x, rows, g3, tile, dtype)
    parts = F.pad(x, (0, rows * g3 * tile - n)).view(rows, -1)
    expect = sum(comm.roundtrip(parts[r], tile, dtype) for r in range(rows))
    assert torch.allclose(comm.unpack(packet3, g3 * tile, tile, dtype, reduce=True), expect, rtol=1e-6, atol=0)


def test_comm_nonfinite_survive():
    x = torch.ones(1025)
    x[3], x[600] = float("nan"), float("inf")
    for dtype in (E4, E5):
        out = comm.unpack(comm.pack(x, 1, 5, 256, dtype), 1025, 256, dtype)
        assert not out[3].isfinite() and not out[600].isfinite() and out[900].isfinite()     # fp8_communication.py:80-92


def test_packet_layout_constants():
    assert comm.packet_bytes(25600, 256) == 6656000 and comm.packet_bytes(1, 64) == 80


# ----------------------------------------------------------------------------- Newton-Schulz
def test_ns_matches_reference_golden(golden_dir):
    """Vectors written by tests/golden/make_ns_golden.py from the reference's own eager recipe."""
    rows = torch.load(golden_dir / "ns_golden.pt", weights_only=True)
    assert len(rows) >= 8
    for row in rows:
        out = ns.METHODS[row["method"]](row["input"], steps=row["steps"])
        assert out.dtype == row["output"].dtype and torch.equal(out, row["output"]), (row["method"], row["input"].shape)


@pytest.mark.parametrize("method", ["standard", "gram"])
def test_ns_matches_reference_golden_at_1024x4096(method, golden_dir):
    """The benchmark's single-matrix configuration (viola/optim/_orthogonalize.py:10-54 on one 1024 x 4096 Gaussian
    matrix, seed 1, 5 steps): a strided sample of the reference's output and its singular values, written by
    tests/golden/make_ns_golden.py. The input is regenerated from the seed and checked against the stored sample."""
    golden = torch.load(golden_dir / "ns_golden_1024x4096.pt", weights_only=True)
    torch.manual_seed(golden["seed"])
    matrix = torch.randn(*golden["shape"])
    stride = golden["stride"]
    assert torch.equal(matrix[::stride, ::stride], golden["input_sample"]) and matrix.double().sum() == golden["input_sum"]
    out = ns.METHODS[method](matrix, steps=golden["steps"])
    assert torch.equal(out[::stride, ::stride], golden[method]["sample"])
    sigma = torch.linalg.svdvals(out.float())
    assert torch.allclose(sigma, golden[method]["singular_values"], atol=1e-4)
    assert sigma.max() < 1.25 and sigma.min() > .6                                  # the quintic's band


@pytest.mark.parametrize("method", ["standard", "gram"])
@pytest.mark.parametrize("shape", [(64, 256), (192, 64), (96, 96)])
def test_ns_invariants_and_chain(method, shape):
    torch.manual_seed(1)
    g = torch.randn(*shape)
    out = ns.METHODS[method](g, steps=5).float()
    sv = torch.linalg.svdvals(out)
    assert sv.max() < 1.3 and .6 < sv.median() < 1.25                             # singular values pushed towards 1
    if shape[0] != shape[1]:
        assert sv.min() > .45                                                     # (a square Gaussian matrix is nearly singular)
    u, _, vh = torch.linalg.svd(g, full_matrices=False)
    assert F.cosine_similarity(out.flatten(), (u @ vh).flatten(), dim=0) > .97      # same singular vectors as G
    transposed = ns.METHODS[method](g.T.contiguous(), steps=5).float()
    # ns(A^T) = ns(A)^T: exact when the recipe transposes the tall case itself, approximate for a square input
    assert rel_l2(transposed.T, out) < (1e-6 if shape[0] != shape[1] else .08)
    # fp64 evaluation of the same polynomial (loose: half-precision trajectory)
    x = g.double() if shape[0] <= shape[1] else g.double().T
    x = x / (x.norm() + 1e-7)
    for _ in range(5):
        a = x @ x.T
        x = 3.4445 * x + (-4.7750 * a + 2.0315 * a @ a) @ x
    x = x if shape[0] <= shape[1] else x.T
    assert rel_l2(out, x) < (.05 if method == "standard" else .01)
    chain = ns.chain(g, 5, method).float()
    assert rel_l2(chain, out) < (.06 if method == "standard" else .01)       # eager vs fused-epilogue rounding points


# ----------------------------------------------------------------------------- composition
def test_linear_oracle_against_float_math():
    torch.manual_seed(4)
    x = torch.randn(65, 128).bfloat16()
    w = torch.randn(96, 128) / 11
    dy = torch.randn(65, 96).bfloat16()
    qw, sw = grouped.quantize(w, E4, (32, 32))
    r = linear.linear(x, grouped.dequantize(qw, sw, (32, 32)), torch.zeros(96), dy)
    assert rel_l2(r["y"], x.float() @ w.T) < .06 and rel_l2(r["dx"], dy.float() @ w) < .06
    assert rel_l2(r["dw"], dy.float().T @ x.float()) < .06 and torch.equal(r["db"], dy.sum(0, dtype=torch.bfloat16))
    g, u = torch.randn(33, 40), torch.randn(33, 40)
    for name in ("silu", "gelu", "relu"):
        gg = g.clone().requires_grad_(); uu = u.clone().requires_grad_()
        out = linear.activation(name)(gg) * uu
        d = torch.randn(33, 40)
        out.backward(d)
        assert rel_l2(linear.gated_forward(g, u, name), out.detach()) < 1e-6
        dg, du = linear.gated_backward(d, g, u, name)
        assert rel_l2(dg, gg.grad) < 1e-5 and rel_l2(du, uu.grad) < 1e-6


def _fake_quantize_rows(x, dtype=E4):
    """Row-wise (1, 32) fake quantization written out with scalar loops over tiles: amax -> scale -> torch cast."""
    limit = torch.finfo(dtype).max
    out = torch.zeros(x.shape)
    for r in range(x.shape[0]):
        for c0 in range(0, x.shape[1], 32):
            tile = x[r, c0:c0 + 32].float()
            scale = tile.abs().max().clamp_min(1e-30) / limit
            out[r, c0:c0 + 32] = (tile / scale).clamp(-limit, limit).to(dtype).float() * scale
    return out


@pytest.mark.parametrize("name", ["silu", "gelu", "relu"])
def test_mlp_oracle_against_float_autograd_and_hand_composition(name):
    """oracle.linear.mlp, pinned two ways. (1) Autograd of the float model down(act(gate(x)) * up(x))
    (checks/mlp.py:12-16): a swapped gate/up half, dy used where the down projection's dx belongs, or a missing
    term moves y / dx / a weight gradient by far more than FP8 quantization noise. (2) Every intermediate rebuilt by
    hand from per-tile scalar-loop fake quantization and plain matmuls, bit for bit: z = [g | u] in that column order
    and rounded to bf16, h = bf16(act(g) * u) from the ROUNDED g and u, dz = bf16([d*u*act'(g) | d*act(g)]) from the
    rounded dH."""
    torch.manual_seed(131)
    rows, d_in, hidden, d_out = 33, 64, 96, 64
    x = torch.randn(rows, d_in).bfloat16()
    dy = torch.randn(rows, d_out).bfloat16()
    w_gu = (torch.randn(2 * hidden, d_in) / d_in ** .5)
    w_dn = (torch.randn(d_out, hidden) / hidden ** .5)
    b_gu, b_dn = torch.randn(2 * hidden) * .1, torch.randn(d_out) * .1
    # the oracle takes dequantized weights: put them on the (32, 32) FP8 grid first
    w_gu = grouped.dequantize(*grouped.quantize(w_gu, E4, (32, 32)), (32, 32))
    w_dn = grouped.dequantize(*grouped.quantize(w_dn, E4, (32, 32)), (32, 32))
    r = linear.mlp(x, w_gu, b_gu, w_dn, b_dn, dy, name=name)

    # (1) float autograd
    xf = x.float().requires_grad_()
    wg, wd = w_gu.clone().requires_grad_(), w_dn.clone().requires_grad_()
    bg, bd = b_gu.clone().requires_grad_(), b_dn.clone().requires_grad_()
    zf = xf @ wg.T + bg
    yf = (linear.activation(name)(zf[:, :hidden]) * zf[:, hidden:]) @ wd.T + bd
    yf.backward(dy.float())
    bar = .12                                                        # two to three FP8 + bf16 roundings in a row (relu: kinks flip)
    assert rel_l2(r["y"], yf.detach()) < bar and rel_l2(r["dx"], xf.grad) < bar
    assert rel_l2(r["dw_gate_up"], wg.grad) < bar and rel_l2(r["dw_down"], wd.grad) < bar
    assert rel_l2(r["db_gate_up"], bg.grad) < bar and torch.equal(r["db_down"], dy.sum(0, dtype=torch.bfloat16))
    # the two halves are not interchangeable: the swapped model is far outside the bar
    swapped = (linear.activation(name)(zf[:, hidden:]) * zf[:, :hidden]) @ wd.T + bd
    assert rel_l2(r["y"], swapped.detach()) > 3 * bar

    # (2) by hand
    z = (_fake_quantize_rows(x) @ w_gu.T + b_gu).bfloat16()
    assert r["z"].dtype == torch.bfloat16 and torch.equal(r["z"], z)
    g, u = z[:, :hidden].float(), z[:, hidden:].float()
    act = {"silu": lambda t: t * (1 / (1 + torch.exp(-t))), "relu": lambda t: t.clamp_min(0),
           "gelu": lambda t: .5 * t * (1 + torch.tanh(0.7978845608028654 * (t + 0.044715 * t * t * t)))}[name]
    h = (act(g) * u).bfloat16()
    assert r["h"].dtype == torch.bfloat16 and torch.equal(r["h"], h)
    assert torch.equal(r["y"], (_fake_quantize_rows(h) @ w_dn.T + b_dn).bfloat16())
    dh = (_fake_quantize_rows(dy) @ w_dn).bfloat16().float()          # dgrad of the down projection, rounded
    gg = g.clone().requires_grad_()
    act(gg).sum().backward()
    dz = torch.cat([dh * u * gg.grad, dh * act(g)], 1).bfloat16()
    assert rel_l2(r["dz"], dz) < 2e-3                                  # autograd's derivative vs the closed form: last-place
    assert (r["dz"].float() - dz.float()).abs().max() <= 2 ** -7 * dz.float().abs().max()
    assert torch.equal(r["dx"], (_fake_quantize_rows(r["dz"]) @ w_gu).bfloat16())
    # weight gradients contract over tokens: groups of 32 along the token axis of the transposed operands
    gt, ht = _fake_quantize_rows(dy.T.contiguous()), _fake_quantize_rows(h.T.contiguous())
    assert torch.equal(r["dw_down"], (gt @ ht.T).bfloat16())
    zt, xt = _fake_quantize_rows(r["dz"].T.contiguous()), _fake_quantize_rows(x.T.contiguous())
    assert torch.equal(r["dw_gate_up"], (zt @ xt.T).bfloat16())
    assert torch.equal(r["db_gate_up"], r["dz"].sum(0, dtype=torch.bfloat16))


def test_varlen_linear_oracle_against_brute_force():
    """oracle.linear.varlen_linear on tiny inputs (groups of 0, 1, 37 and 3 rows), against loops that know nothing of
    oracle.linear: rows of group g see weight g only, token tiles of the weight gradient restart at each group's first
    row, an empty group contributes no rows and a zero gradient."""
    torch.manual_seed(77)
    counts, d_in, d_out = [0, 1, 37, 3, 0], 64, 32
    total = sum(counts)
    x = torch.randn(total, d_in).bfloat16()
    dy = (torch.randn(total, d_out) * .1).bfloat16()
    weights = [grouped.dequantize(*grouped.quantize(torch.randn(d_out, d_in) / 8, E4, (32, 32)), (32, 32)) for _ in counts]
    r = linear.varlen_linear(x, weights, counts, dy)
    assert r["y"].shape == (total, d_out) and r["dx"].shape == (total, d_in) and r["dw"].shape == (len(counts), d_out, d_in)
    fx, fg = _fake_quantize_rows(x).double(), _fake_quantize_rows(dy).double()
    offset = 0
    for group, count in enumerate(counts):
        w = weights[group].double()
        for row in range(offset, offset + count):
            y_row = torch.tensor([sum(fx[row, k] * w[n, k] for k in range(d_in)) for n in range(d_out)])
            dx_row = torch.tensor([sum(fg[row, n] * w[n, k] for n in range(d_out)) for k in range(d_in)])
            assert torch.equal(r["y"][row], y_row.float().bfloat16()) or rel_l2(r["y"][row], y_row) < 4e-3
            assert torch.equal(r["dx"][row], dx_row.float().bfloat16()) or rel_l2(r["dx"][row], dx_row) < 4e-3
        if count == 0:
            assert r["dw"][group].abs().max() == 0
        else:
            # tiles of 32 tokens counted from the group's own first row
            gt = _fake_quantize_rows(dy[offset:offset + count].T.contiguous()).double()
            xt = _fake_quantize_rows(x[offset:offset + count].T.contiguous()).double()
            assert rel_l2(r["dw"][group], gt @ xt.T) < 4e-3
            if count > 1:                                            # tiles counted from row 0 of the batch differ
                wrong = _fake_quantize_rows(dy.T.contiguous())[:, offset:offset + count].double() @ _fake_quantize_rows(x.T.contiguous())[:, offset:offset + count].double().T
                assert rel_l2(wrong, gt @ xt.T) > 1e-3 or count % 32 == 0 and offset % 32 == 0
        offset += count
    # a group's rows depend on no other group: recomputing with the other weights zeroed changes nothing for group 2
    zeroed = [w if g == 2 else torch.zeros_like(w) for g, w in enumerate(weights)]
    r2 = linear.varlen_linear(x, zeroed, counts, dy)
    assert torch.equal(r2["y"][1:38], r["y"][1:38]) and torch.equal(r2["dw"][2], r["dw"][2]) and r2["y"][0].abs().max() == 0


def test_half_accumulator_oracles_by_hand():
    """oracle.grouped.gemm_half / oracle.tensor.gemm_half (the reference's accum_dtype='fp16' loops) on cases worked out
    by hand: 2049 is a tie between the FP16 neighbours 2048 and 2050 and goes to 2048; the partial is cleared per scale
    group (grouped recipe) or runs on (per-tensor, no block); a bf16 total rounds after every addition; sums that FP16
    holds exactly reproduce the FP32 product; and on the reference's test distribution with its half-sum limit the
    result stays inside the bound of checks/check_grouped_linear.py:41 while differing from the FP32 sums."""
    from oracle import tensor
    a, b = torch.zeros(1, 64), torch.zeros(1, 64)
    a[0, 0], b[0, 0], a[0, 1], b[0, 1] = 64, 32, 1, 1                              # first 32 k: 2048 + 1
    a[0, 32], b[0, 32] = 2, 3                                                      # second 32 k: 6
    qa, qb = a.to(E4), b.to(E4)
    sa, sb = torch.tensor([[.5, 2.]]), torch.tensor([[1., 1.]])
    assert grouped.gemm(qa, qb, sa, sb, (1, 32), (32, 32)).item() == 2049 * .5 + 12
    assert grouped.gemm_half(qa, qb, sa, sb, (1, 32), (32, 32)).item() == 2048 * .5 + 12       # per group: fp16(2049) = 2048
    one, half = torch.tensor([1.]), torch.tensor([.5])
    assert tensor.gemm_half(qa, qb, half, one).item() == 2054 * .5                 # one running partial: fp16(2048 + 6) = 2054
    assert tensor.gemm_half(qa, qb, half, one, accum_block_size=32).item() == 2054 * .5      # fp32 total of 2048 and 6
    # a bf16 total: 2048 + 6 = 2054 rounds to 2048 (bf16 spacing 16 there)
    assert tensor.gemm_half(qa, qb, half, one, accum_block_size=32, reduce_dtype=torch.bfloat16).item() == 2048 * .5
    assert grouped.gemm_half(qa, qb, torch.ones(1, 2), sb, (1, 32), (32, 32), reduce_dtype=torch.bfloat16).item() == 2048
    # (1, 64) groups: one partial spans both 32-k steps, fp16(2048 + 6); an accumulation block of 32 splits it again
    wide = torch.tensor([[.5]])
    assert grouped.gemm_half(qa, qb, wide, torch.ones(1, 1), (1, 64), (32, 64)).item() == 2054 * .5
    assert grouped.gemm_half(qa, qb, wide, torch.ones(1, 1), (1, 64), (32, 64), accum_block_size=32).item() == 2054 * .5
    # small integers: every partial sum is an integer below 2048, exact in FP16
    torch.manual_seed(60)
    ia, ib = torch.randint(-3, 4, (9, 96)).float().to(E4), torch.randint(-3, 4, (7, 96)).float().to(E4)
    isa, isb = torch.exp2(torch.randint(-2, 3, (9, 3)).float()), torch.exp2(torch.randint(-2, 3, (1, 3)).float())
    assert torch.equal(grouped.gemm_half(ia, ib, isa, isb, (1, 32), (32, 32)), grouped.gemm(ia, ib, isa, isb, (1, 32), (32, 32)))
    assert torch.equal(tensor.gemm_half(ia, ib, one, one), tensor.gemm(ia, ib, one, one))
    # the reference's own check (check_grouped_linear.py:23-46, half=True): limit 8, bound .01
    torch.manual_seed(2041)
    x = (torch.randn(65, 128) * torch.exp2(torch.randint(-5, 6, (65, 1)))).bfloat16()
    w = (torch.randn(96, 128) * torch.exp2(torch.randint(-5, 6, (96, 1)))).bfloat16()
    (qx, sx), (qw, sw) = grouped.quantize(x, E5, (1, 32), limit=8.0), grouped.quantize(w, E4, (32, 32), limit=8.0)
    exact = grouped.gemm(qx, qw, sx, sw, (1, 32), (32, 32))
    model = grouped.gemm_half(qx, qw, sx, sw, (1, 32), (32, 32))
    assert 0 < rel_l2(model, exact) < .01
    assert 0 < rel_l2(grouped.gemm_half(qx, qw, sx, sw, (1, 32), (32, 32), reduce_dtype=torch.bfloat16), exact) < .01


# ----------------------------------------------------------------------------- per-tensor scaling
@pytest.mark.parametrize("dtype", [E4, E5])
def test_tensor_oracle_matches_the_reference_cpu_definitions(dtype):
    """checks/linear.py:17-20 `quantized` and viola/nn/linear.py:298-312 (CPU refresh_weight) written out here,
    independently of oracle.tensor: same scale, same codes; delayed scaling reads the history as it was."""
    from oracle import tensor
    torch.manual_seed(51)
    x = torch.randn(70, 45) * torch.logspace(-3, 2, 45)
    limit = torch.finfo(dtype).max
    expected_scale = x.float().abs().max().clamp_min(1e-30) / limit
    scale, history = tensor.tensor_scale(x, torch.zeros(4), 0, limit=limit)
    assert torch.equal(scale, expected_scale.reshape(1)) and history.tolist() == [x.abs().max().item(), 0, 0, 0]
    expected = (x.float() / expected_scale).clamp(-limit, limit).to(dtype)
    assert torch.equal(tensor.quantize(x, scale, dtype).view(torch.uint8), expected.view(torch.uint8))
    assert torch.equal(tensor.quantize(x, scale, dtype, transpose=True).view(torch.uint8), expected.T.contiguous().view(torch.uint8))
    assert tensor.quantize(x, scale, dtype).float().abs().max() == limit            # the largest element maps to the limit
    # delayed: index 0 uses the tensor itself, later calls the history's maximum before the new amax is written
    history = torch.zeros(3)
    amaxes = [2.0, 8.0, 1.0, 0.5, 0.25, 0.125]
    for index, a in enumerate(amaxes):
        y = torch.full((5,), a)
        y[2] = float("nan")                                                          # dropped by the reduction
        before = history.clone()
        scale, history = tensor.tensor_scale(y, history, index, delayed=True, limit=limit)
        basis = a if index == 0 else before.max().item()
        assert scale.item() == torch.tensor(basis) / limit and history[index % 3] == a
    # all-zero tensor: the 1e-30 floor
    assert tensor.tensor_scale(torch.zeros(9), torch.zeros(1), 0, limit=limit)[0].item() == (torch.tensor(1e-30) / limit).item()
    # a reduced quantization limit clamps
    q = tensor.quantize(x, scale=torch.tensor([x.abs().max().item() / 64]), dtype=dtype, limit=16.0)
    assert q.float().abs().max() == 16.0


def test_tensor_gemm_oracle_against_brute_force():
    from oracle import tensor
    torch.manual_seed(52)
    a = torch.randn(5, 48).to(E5)
    b = torch.randn(7, 48).to(E4)
    sa, sb, bias = torch.tensor([.37]), torch.tensor([1.9]), torch.randn(7)
    out = tensor.gemm(a, b, sa, sb, bias=bias)
    for m in range(5):
        for n in range(7):
            acc = sum(float(a[m, k].float()) * float(b[n, k].float()) for k in range(48))
            assert abs(out[m, n].item() - (acc * .37 * 1.9 + bias[n].item())) < 1e-4 * (1 + abs(acc))


# ----------------------------------------------------------------------------- MXFP8 (E8M0 scales)
@pytest.mark.parametrize("dtype", [E4, E5])
@pytest.mark.parametrize("group,shape", [((1, 32), (9, 96)), ((32, 32), (70, 45)), ((1, 32), (33, 64))])
def test_native_quantize_matches_the_reference_cpu_branch(dtype, group, shape):
    """viola/nn/_grouped_kernels.py:135-151 with native=True, written out with its own log2 / ceil / exp2: bytes and
    codes equal the oracle's (random data does not sit within an ulp of a power of two, where the two could differ)."""
    torch.manual_seed(70)
    x = torch.randn(shape) * torch.logspace(-6, 4, shape[1])
    limit = torch.finfo(dtype).max
    gr, gc = group
    nr, nc = grouped.scale_shape(shape, group)
    blocks = F.pad(x, (0, nc * gc - shape[1], 0, nr * gr - shape[0])).reshape(nr, gr, nc, gc)
    scales = blocks.abs().amax((1, 3)).clamp_min(1e-30) / limit
    exponent = scales.log2().ceil()
    expected_bytes = (exponent + 127).to(torch.uint8)
    expected = (blocks / exponent.exp2()[:, None, :, None]).clamp(-limit, limit).reshape(nr * gr, nc * gc)[:shape[0], :shape[1]].to(dtype)
    q, s = grouped.quantize(x, dtype, group, native=True)
    assert s.dtype == torch.uint8 and torch.equal(s, expected_bytes)
    assert torch.equal(q.view(torch.uint8), expected.view(torch.uint8))
    assert torch.equal(grouped.decode_scale(s), exponent.exp2())
    # the scale is the smallest power of two >= amax / limit: nothing clamps, and half of it would
    assert (q.float().abs() <= limit).all() and (grouped.decode_scale(s) >= scales).all() and (grouped.decode_scale(s) < 2 * scales).all()
    # an amax that is exactly limit * 2^k keeps the scale 2^k
    y = torch.zeros(32, 32)
    y[3, 5] = limit * 2. ** -9
    assert grouped.quantize(y, dtype, (32, 32), native=True)[1].item() == 127 - 9
    y[3, 5] = torch.nextafter(torch.tensor(limit * 2. ** -9), torch.tensor(float("inf")))
    assert grouped.quantize(y, dtype, (32, 32), native=True)[1].item() == 127 - 8
    # dequantize and the re-encoding transpose read the bytes
    assert torch.equal(grouped.dequantize(q, s, group), q.float() * grouped.decode_scale(s).repeat_interleave(gr, 0).repeat_interleave(gc, 1)[:shape[0], :shape[1]])


# ----------------------------------------------------------------------------- Hadamard-64 rotation
def test_rotation_is_the_kronecker_hadamard_matrix():
    """The staged butterflies of oracle.rotation.rotate against the matrix the reference defines the rotation by
    (rotate_cpu, viola/nn/_rotation_kernels.py:126-130): equal bit for bit on small integers (every sum exact), to
    rounding otherwise; H64 is symmetric, orthogonal and has entries +-1/8; rotating twice gives the input back; a
    group cut off by the matrix edge is completed with zeros. A wrong stride, digit or sign fails the first check."""
    from oracle import rotation
    h = rotation.hadamard64()
    assert torch.equal(h, h.T) and torch.equal(h.abs(), torch.full((64, 64), 0.125))
    assert torch.equal(h @ h, torch.eye(64))
    torch.manual_seed(9)
    k = torch.randint(-50, 51, (7, 192)).float()
    assert torch.equal(rotation.rotate(k), (k.reshape(-1, 64) @ h).reshape(k.shape))
    assert torch.equal(rotation.rotate(rotation.rotate(k)), k)
    # one-hot rows pick out the rows of H64: every output position and sign is checked
    assert torch.equal(rotation.rotate(torch.eye(64)), h)
    x = torch.randn(5, 128)
    exact = (x.double().reshape(-1, 64) @ h.double()).reshape(x.shape)
    assert (rotation.rotate(x).double() - exact).abs().max() < 1e-6
    z = torch.randn(3, 100)
    padded = torch.zeros(3, 128)
    padded[:, :100] = z
    assert torch.equal(rotation.rotate(z), rotation.rotate(padded)[:, :100])
    # the norm of every group is preserved (orthogonality), which is why one scale serves the rotated tensor
    assert torch.allclose(rotation.rotate(x).reshape(-1, 64).norm(dim=1), x.reshape(-1, 64).norm(dim=1), rtol=1e-5)
    n = x.clone()
    n[2, 5] = float("nan")
    assert rotation.amax(n) == rotation.rotate(x)[torch.arange(5) != 2].abs().max().maximum(rotation.rotate(x)[2, 64:].abs().max())
