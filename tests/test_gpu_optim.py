"""GPU parity: FP8Muon kernels (momentum codec, Philox SR, weight / AdamW updates, copy_scaled) vs the CPU oracle.
FP8 payloads, scales and fp32 results are compared bit for bit."""

import itertools
import math

import numpy as np
import pytest
import torch

from oracle import optim as oo

pytestmark = pytest.mark.gpu


def _k():
    from viola_amd.optim import _kernels
    return _kernels


def test_philox_known_answers_on_device():
    from viola_amd import _lib
    triples = [(0, 0, 0), (0xffffffffffffffff,) * 3, (0x85a308d3243f6a88, 0x0370734413198a2e, 0x299f31d0a4093822)]
    rng = np.random.default_rng(0)
    extra = rng.integers(0, 2 ** 63, size=(200, 3), dtype=np.uint64)
    table = np.concatenate([np.array(triples, dtype=np.uint64), extra])
    dev = torch.from_numpy(table.view(np.int64).copy()).cuda()
    out = torch.zeros(len(table), dtype=torch.int32, device="cuda")
    _lib.call("viola_selftest_philox", _lib.ptr(dev), _lib.ptr(out), len(table))
    got = out.cpu().numpy().view(np.uint32)
    assert got[:3].tolist() == [0x6627e8d5, 0x408f276d, 0xd16cfe09]          # Random123 kat_vectors
    expect = np.array([oo.philox(np.array([e], dtype=np.uint64), int(s), int(k))[0] for e, s, k in table], dtype=np.uint32)
    assert np.array_equal(got, expect)


CONFIGS = [("tile", b) for b in (64, 128, 256, 512, 1024)] + [("block", t) for t in ((8, 8), (8, 32), (16, 16), (16, 32), (32, 32), (64, 64))]


@pytest.mark.parametrize("granularity,size", CONFIGS)
@pytest.mark.parametrize("shape", [(17, 31), (2, 33, 67)])
@pytest.mark.parametrize("rounding", ["nearest", "stochastic"])
def test_momentum_update_bit_exact(granularity, size, shape, rounding):
    """The sweep of checks/quantization.py:83-112 (tile sizes, block shapes, ragged shapes, unaligned buffers,
    in-place state), held to bit equality with the oracle instead of the reference's rtol 2e-6."""
    k = _k()
    torch.manual_seed(79)
    quant = dict(granularity=granularity, tile_size=size if granularity == "tile" else 256,
                 block_shape=size if granularity == "block" else (16, 16))
    qn, sn = k.state_sizes(shape, **quant)
    assert (qn, sn) == oo.state_sizes(shape, **quant)
    n = math.prod(shape)
    q = torch.zeros(qn + 1, dtype=torch.uint8, device="cuda")[1:]            # element-aligned views only
    scale = torch.ones(sn + 1, device="cuda")[1:]
    u = torch.empty(n + 1, dtype=torch.bfloat16, device="cuda")[1:]
    rq, rs = torch.zeros(qn, dtype=torch.uint8), torch.ones(sn)
    for step in range(6):
        g = torch.randn(n + 1)[1:] * (1e-8 if step < 2 else 1.)
        gd = torch.empty(n + 1, device="cuda")[1:].copy_(g)
        nesterov = step % 2 == 0
        k.momentum_update(gd, q, scale, q, scale, u, beta=.95, matrix_shape=shape, nesterov=nesterov,
                          rounding=rounding, rounding_step=step, rounding_key=123, **quant)
        rq, rs, ru = oo.momentum_update(g, rq, rs, beta=.95, shape=shape, nesterov=nesterov, rounding=rounding,
                                        rounding_step=step, rounding_key=123, **quant)
        assert torch.equal(scale.cpu(), rs), f"scales differ at step {step}"
        assert torch.equal(q.cpu(), rq), f"payload differs at step {step}"
        assert torch.equal(u.cpu().view(torch.int16), ru.view(torch.int16)), f"update differs at step {step}"
        assert torch.equal(k.dequantize(q, scale, shape, **quant).cpu(), oo.dequantize(rq, rs, shape, **quant))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tile_size,n", [(128, 13), (256, 257), (512, 1537), (256, 8192)])
def test_momentum_out_of_place_loss_scale(dtype, tile_size, n):
    """checks/numerics.py:18-49: separate next buffers, fp16 gradients with loss scaling."""
    k = _k()
    torch.manual_seed(42)
    blocks = -(-n // tile_size)
    q, scales = torch.zeros(blocks * tile_size, dtype=torch.uint8, device="cuda"), torch.ones(blocks, device="cuda")
    nq, ns_ = torch.empty_like(q), torch.empty_like(scales)
    out = torch.empty(n, dtype=torch.bfloat16, device="cuda")
    rq, rs = q.cpu(), scales.cpu()
    loss_scale = 32.0 if dtype == torch.float16 else 1.0
    for step in range(4):
        grad = torch.randn(n).to(dtype)
        k.momentum_update(grad.cuda(), q, scales, nq, ns_, out, beta=.95, tile_size=tile_size, nesterov=step % 2 == 0,
                          loss_scale=loss_scale)
        rq, rs, ru = oo.momentum_update(grad, rq, rs, beta=.95, shape=(n,), tile_size=tile_size, nesterov=step % 2 == 0,
                                        loss_scale=loss_scale)
        assert torch.equal(nq.cpu(), rq) and torch.equal(ns_.cpu(), rs) and torch.equal(out.cpu().view(torch.int16), ru.view(torch.int16))
        q, nq, scales, ns_ = nq, q, ns_, scales
    zero = torch.zeros(n, device="cuda", dtype=dtype)
    q.zero_(); scales.fill_(1)
    k.momentum_update(zero, q, scales, nq, ns_, out, beta=.95, tile_size=tile_size)
    assert nq.count_nonzero() == 0 and out.count_nonzero() == 0                # zero stays zero (numerics.py:51-55)


def test_stochastic_rounding_statistics_and_replay():
    """checks/quantization.py:114-153 on the device."""
    k = _k()
    n = 256 * 1024
    g = torch.full((n,), 1 + .27 * .125, device="cuda")
    g[::256] = 448
    q, scales = torch.zeros(n, dtype=torch.uint8, device="cuda"), torch.ones(n // 256, device="cuda")
    out = torch.empty(n, dtype=torch.bfloat16, device="cuda")

    def draw(step=7, key=42):
        q.zero_(); scales.fill_(1)
        k.momentum_update(g, q, scales, q, scales, out, beta=0., rounding="stochastic", rounding_step=step,
                          rounding_key=key, nesterov=False)
        return q.clone()

    rng_state = torch.cuda.get_rng_state()
    first = draw()
    assert torch.equal(first, draw()) and not torch.equal(first, draw(step=8)) and not torch.equal(first, draw(key=43))
    assert torch.equal(rng_state, torch.cuda.get_rng_state())
    values = first.view(torch.float8_e4m3fn).float().view(-1, 256)[:, 1:]
    assert ((values == 1.) | (values == 1.125)).all()
    assert abs((values == 1.125).float().mean().item() - .27) < .005
    table = torch.arange(127, dtype=torch.uint8).view(torch.float8_e4m3fn).float().cuda()
    mids = (table[:-1] * .7 + table[1:] * .3).repeat(1024)
    g2 = torch.cat((mids, -mids, table.repeat(1024)))
    g2[::256] = 448
    qn, sn = k.state_sizes(g2.shape)
    q2, s2 = torch.zeros(qn, dtype=torch.uint8, device="cuda"), torch.ones(sn, device="cuda")
    o2 = torch.empty(g2.numel(), dtype=torch.bfloat16, device="cuda")
    torch.cuda.synchronize()
    allocated = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    k.momentum_update(g2, q2, s2, q2, s2, o2, beta=0., rounding="stochastic", nesterov=False)
    torch.cuda.synchronize()
    assert torch.cuda.max_memory_allocated() - allocated == 0                  # kernels allocate nothing (:155-161)
    actual = k.dequantize(q2, s2, g2.shape)
    idx = torch.searchsorted(table, g2.abs()).clamp_max(126)
    lower, upper = table[(idx - 1).clamp_min(0)], table[idx]
    assert ((actual.abs() == lower) | (actual.abs() == upper)).all()
    assert ((actual.sign() == g2.sign()) | (actual == 0)).all()


DTYPES = (torch.float32, torch.bfloat16, torch.float16)


@pytest.mark.parametrize("wdtype,gdtype", list(itertools.product(DTYPES, repeat=2)))
def test_weight_and_adam_bit_exact(wdtype, gdtype):
    """The dtype sweep of checks/precision_kernels.py:26-46 on unaligned views; bit equality with the oracle."""
    k = _k()
    torch.manual_seed(107)
    w = (torch.randn(1030) * .1).to(wdtype)[1:1026]
    g = (torch.randn(1030) * .01).to(gdtype)[1:1026]
    wd = (torch.zeros(1030, device="cuda", dtype=wdtype))[1:1026].copy_(w)
    gd = (torch.zeros(1030, device="cuda", dtype=gdtype))[1:1026].copy_(g)
    k.weight_update(wd, gd, .001, .01, update_scale=6.4)
    ref = oo.weight_update(w, g, .001, .01, update_scale=6.4)
    assert torch.equal(wd.cpu().view(torch.uint8), ref.contiguous().view(torch.uint8))
    for sdtype in DTYPES:
        m, v = torch.zeros(1025, device="cuda", dtype=sdtype), torch.zeros(1025, device="cuda", dtype=sdtype)
        rm, rv, rw = m.cpu(), v.cpu(), ref
        for step in range(1, 4):
            k.adam_update(wd, gd, m, v, lr=.001, weight_decay=.01, betas=(.9, .95), eps=1e-8, step=step)
            rw, rm, rv = oo.adam_update(rw, g, rm, rv, lr=.001, weight_decay=.01, betas=(.9, .95), eps=1e-8, step=step)
            assert torch.equal(m.cpu().view(torch.uint8), rm.contiguous().view(torch.uint8))
            assert torch.equal(v.cpu().view(torch.uint8), rv.contiguous().view(torch.uint8))
            assert torch.equal(wd.cpu().view(torch.uint8), rw.contiguous().view(torch.uint8)), (sdtype, step)
        ref = rw


def test_adam_variants():
    k = _k()
    torch.manual_seed(1)
    w, g = torch.randn(300), torch.randn(300)
    for adamw, maximize, bias_correction in itertools.product((True, False), repeat=3):
        wd, m, v = w.cuda(), torch.zeros(300, device="cuda"), torch.zeros(300, device="cuda")
        k.adam_update(wd, g.cuda(), m, v, lr=.01, weight_decay=.1, betas=(.9, .999), eps=1e-8, step=3, adamw=adamw,
                      maximize=maximize, bias_correction=bias_correction)
        rw, rm, rv = oo.adam_update(w, g, torch.zeros(300), torch.zeros(300), lr=.01, weight_decay=.1, betas=(.9, .999),
                                    eps=1e-8, step=3, adamw=adamw, maximize=maximize, bias_correction=bias_correction)
        assert torch.equal(wd.cpu(), rw) and torch.equal(m.cpu(), rm) and torch.equal(v.cpu(), rv)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_stochastic_master_rounding(dtype):
    """checks/precision_kernels.py:48-65: 25 % of sub-ulp updates survive; a split call with `offset` replays exactly."""
    k = _k()
    n = 131072
    spacing = 2. ** (-8 if dtype == torch.bfloat16 else -11)
    w = torch.ones(n, device="cuda", dtype=dtype)
    g = torch.ones(n, device="cuda")
    k.weight_update(w, g, spacing / 4, 0., rounding="stochastic", step=17, key=29)
    assert abs((w != 1).float().mean().item() - .25) < .005
    ref = oo.weight_update(torch.ones(n, dtype=dtype), torch.ones(n), spacing / 4, 0., rounding="stochastic", step=17, key=29)
    assert torch.equal(w.cpu(), ref)
    replay = torch.ones_like(w)
    cut = 13001
    k.weight_update(replay[:cut], g[:cut], spacing / 4, 0., rounding="stochastic", step=17, key=29)
    k.weight_update(replay[cut:], g[cut:], spacing / 4, 0., rounding="stochastic", step=17, key=29, offset=cut)
    assert torch.equal(w, replay)
    m, v = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    w2 = torch.ones(n, device="cuda", dtype=dtype)
    k.adam_update(w2, g * 1e-3, m, v, lr=1e-4, weight_decay=0., betas=(.9, .95), eps=1e-8, step=1, rounding="stochastic", key=5)
    rw, _, _ = oo.adam_update(torch.ones(n, dtype=dtype), torch.ones(n) * 1e-3, torch.zeros(n), torch.zeros(n), lr=1e-4,
                              weight_decay=0., betas=(.9, .95), eps=1e-8, step=1, rounding="stochastic", key=5)
    assert torch.equal(w2.cpu(), rw)


@pytest.mark.parametrize("wdtype,rounding", [(torch.float32, "nearest"), (torch.bfloat16, "nearest"), (torch.bfloat16, "stochastic"),
                                             (torch.float16, "stochastic")])
def test_adam_table_equals_per_tensor_and_oracle(wdtype, rounding):
    """One launch over a pointer table == one adam_update per tensor (viola/optim/muon.py:137-140), bit for bit,
    ragged sizes from 1 element to beyond one grid stride, own rounding key per tensor."""
    k = _k()
    torch.manual_seed(31)
    sizes = [1, 7, 256, 1152, 3 * 1152 + 5, 300001]
    hyper = dict(lr=1e-3, weight_decay=.01, betas=(.9, .95), eps=1e-8)
    weights = [(torch.randn(n) * .1).to(wdtype) for n in sizes]
    grads = [torch.randn(n) * 1e-2 for n in sizes]
    many = [(w.cuda(), g.cuda(), torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda"), 1000 + i, 3 * i)
            for i, (w, g, n) in enumerate(zip(weights, grads, sizes))]
    single = [(w.cuda(), g.cuda(), torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda"), 1000 + i, 3 * i)
              for i, (w, g, n) in enumerate(zip(weights, grads, sizes))]
    cache = {}
    for step in (1, 2):
        k.adam_update_many(many, step=step, rounding=rounding, cache=cache, **hyper)
        for w, g, m, v, key, offset in single:
            k.adam_update(w, g, m, v, step=step, rounding=rounding, key=key, offset=offset, **hyper)
    assert len(cache["rows"]) == len(sizes)
    for a, b in zip(many, single):
        for x, y in zip(a[:4], b[:4]):
            assert torch.equal(x, y)
    rw, rm, rv = weights[4], torch.zeros(sizes[4]), torch.zeros(sizes[4])
    for step in (1, 2):
        rw, rm, rv = oo.adam_update(rw, grads[4], rm, rv, step=step, rounding=rounding, key=1004, offset=12, **hyper)
    assert torch.equal(many[4][0].cpu(), rw) and torch.equal(many[4][2].cpu(), rm) and torch.equal(many[4][3].cpu(), rv)


@pytest.mark.parametrize("gdtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rounding", ["nearest", "stochastic"])
@pytest.mark.parametrize("tile_size", [256, 1024])
def test_momentum_and_weight_tables_equal_per_tensor(gdtype, rounding, tile_size):
    """One launch over a pointer table == one momentum_update / weight_update per matrix (viola/optim/muon.py:104-106,
    131-132), bit for bit: codes, scales, bf16 update and fp32 weights, over two steps (the second starts from state)."""
    k = _k()
    torch.manual_seed(41)
    n, tensors = 12 * 1024, 5
    grads = [(torch.randn(n, device="cuda") * 10. ** (i - 2)).to(gdtype) for i in range(tensors)]
    grads[2][5] = float("inf")                                                  # a poisoned tile takes the division path
    def state():
        return [(torch.zeros(n, dtype=torch.uint8, device="cuda"), torch.ones(n // tile_size, device="cuda"),
                 torch.empty(n, dtype=torch.bfloat16, device="cuda")) for _ in range(tensors)]
    many, single = state(), state()
    w_many = [torch.randn(n, device="cuda") for _ in range(tensors)]
    w_single = [w.clone() for w in w_many]
    caches = ({}, {})
    for step in (0, 1):
        assert k.momentum_update_many([(g, q, s, out, 77 + i) for i, (g, (q, s, out)) in enumerate(zip(grads, many))], beta=.95,
                                      tile_size=tile_size, rounding=rounding, rounding_step=step, cache=caches[0])
        assert k.weight_update_many([(w, out) for w, (_, _, out) in zip(w_many, many)], 1e-3, .01, update_scale=.7, cache=caches[1])
        for i, (g, (q, s, out)) in enumerate(zip(grads, single)):
            k.momentum_update(g, q, s, q, s, out, beta=.95, tile_size=tile_size, rounding=rounding, rounding_step=step, rounding_key=77 + i)
            k.weight_update(w_single[i], out, 1e-3, .01, update_scale=.7)
    for a, b in zip(many, single):
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
        assert torch.equal(a[2].view(torch.int16), b[2].view(torch.int16))
    for a, b in zip(w_many, w_single):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    # shapes the table kernels decline are reported, not mangled
    assert not k.momentum_update_many([(grads[0][:300], many[0][0], many[0][1], many[0][2], 0)], beta=.95, tile_size=256)
    assert not k.weight_update_many([(w_many[0][:6], many[0][2][:6])], 1e-3, .01)


def test_copy_scaled():
    k = _k()
    matrix = torch.randn(17, 31).bfloat16().T
    partition = torch.zeros(257, device="cuda")
    k.copy_scaled(matrix.cuda(), partition, 11, 3, 251, 3.2)
    assert torch.equal(partition.cpu(), oo.copy_scaled(matrix, torch.zeros(257), 11, 3, 251, 3.2))   # numerics.py:74-77


def test_full_size_momentum_properties():
    """DiT-XL qkv-sized state: replay determinism, payload/scales consistent with the bf16 update it emitted."""
    k = _k()
    torch.manual_seed(3)
    n = 3456 * 1152
    g = (torch.randn(n, device="cuda") * 1e-3)
    q, s = torch.zeros(n, dtype=torch.uint8, device="cuda"), torch.ones(n // 256, device="cuda")
    u = torch.empty(n, dtype=torch.bfloat16, device="cuda")
    k.momentum_update(g, q, s, q, s, u, beta=.95, tile_size=256, nesterov=False)
    m = k.dequantize(q, s, (n,))
    assert ((m - u.float()).norm() / u.float().norm()).item() < .04
    assert q.view(torch.float8_e4m3fn).float().abs().view(-1, 256).amax(1).eq(448).all()
    q2, s2 = torch.zeros_like(q), torch.ones_like(s)
    k.momentum_update(g, q2, s2, q2, s2, u, beta=.95, tile_size=256, nesterov=False)
    assert torch.equal(q, q2) and torch.equal(s, s2)


@pytest.mark.parametrize("method", ["standard", "gram"])
def test_fp8muon_buckets_on_several_streams_equal_one_stream(method):
    """FP8Muon.step spreads independent shape buckets over streams; a shape that is split into several buckets (batch
    limit) gives those their own pointer tables. Parameters and states after three steps are bit-equal to the
    single-stream, unsplit optimizer."""
    import viola_amd
    shapes = [(256, 128)] * 6 + [(128, 384)] * 3 + [(192, 192)] * 2 + [(64,)] * 4
    def build(lanes, limit):
        torch.manual_seed(5)
        params = [torch.nn.Parameter(torch.randn(*shape, device="cuda") * .05) for shape in shapes]
        opt = viola_amd.optim.FP8Muon(params, lr=2e-3, weight_decay=.01, tile_size=64, ns_method=method, rounding="stochastic",
                                      rounding_seed=9)
        opt._LANES, opt._BATCH_ELEMENTS = lanes, limit
        return params, opt
    many, opt_many = build(4, 2 * 256 * 128 + 1)                              # (256, 128) goes in three buckets of two
    one, opt_one = build(1, 1 << 28)
    for step in range(3):
        torch.manual_seed(100 + step)
        grads = [torch.randn(*shape, device="cuda") * 1e-2 for shape in shapes]
        for params, opt in ((many, opt_many), (one, opt_one)):
            for p, g in zip(params, grads):
                p.grad = g.clone()
            opt.step()
    torch.cuda.synchronize()
    assert len(opt_many._streams[many[0].device]) == 4
    for a, b in zip(many, one):
        assert torch.equal(a, b)
        for key in ("momentum_q", "momentum_scale", "exp_avg", "exp_avg_sq"):
            if key in opt_many.state[a]:
                assert torch.equal(opt_many.state[a][key], opt_one.state[b][key])
