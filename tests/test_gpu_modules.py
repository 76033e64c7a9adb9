"""GPU parity: viola_amd.nn.Linear / MLP and viola_amd.optim.FP8Muon end to end vs the CPU oracle."""

import copy

import pytest
import torch

from oracle import grouped as og, linear as ol, ns as ons, optim as oo
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


@pytest.mark.parametrize("mode,gw,gx,gg,saved,bwd,storage", [
    ("memory", (32, 32), (1, 32), (1, 32), "fp8", "e5m2", "fp8"), ("memory", (32, 32), (1, 32), (1, 32), "fp8", "e4m3", "fp8"),
    ("fast", (32, 64), (32, 32), (1, 64), "bf16", "e5m2", "fp8"), ("fast", (1, 32), (1, 32), (1, 32), "fp8", "e5m2", "fp8"),
    ("memory", (32, 32), (1, 32), (1, 32), "fp8", "e4m3", "bf16"), ("fast", (32, 32), (1, 32), (1, 32), "fp32", "e5m2", "bf16")])
def test_linear_layer(mode, gw, gx, gg, saved, bwd, storage, bf16_gradients):
    """checks/check_grouped_linear.py:48-87: Linear(128, 96) with scaled weight columns, x [65, 128]."""
    import viola_amd
    torch.manual_seed(2041)
    source = torch.nn.Linear(128, 96, dtype=torch.bfloat16)
    source.weight.data[:, ::17] *= 16
    layer = viola_amd.nn.Linear.from_float(source.cuda(), scaling="grouped", mode=mode, weight_group_shape=gw,
                                           input_group_shape=gx, grad_group_shape=gg, saved_input_dtype=saved,
                                           backward_dtype=bwd, weight_dtype=storage)
    x = torch.randn(65, 128).bfloat16()
    dy = torch.randn(65, 96).bfloat16()
    xg = x.cuda().requires_grad_()
    y = layer(xg)
    y.backward(dy.cuda())
    bwd_dtype = E5 if bwd == "e5m2" else E4
    if storage == "fp8":
        assert layer.weight.dtype == E4 and layer.weight_scale.shape == og.scale_shape((96, 128), gw)
        rq, rs = og.quantize(source.weight.detach().float().cpu(), E4, gw)
        assert torch.equal(layer.weight.detach().cpu().view(torch.uint8), rq.view(torch.uint8)) and torch.equal(layer.weight_scale.cpu(), rs)
        w_real = og.dequantize(rq, rs, gw)
        assert torch.equal(layer.dequantize_weight().cpu(), w_real)
    else:
        assert layer.weight.dtype == torch.bfloat16 and layer.weight_scale.numel() == 0
        w_real = og.dequantize(*og.quantize(source.weight.detach().cpu(), E4, gw), gw)
    expect = ol.linear(x, w_real, source.bias.detach().cpu(), dy, fp8=E4, bwd_fp8=bwd_dtype, gx=gx, gw=gw, gg=gg)
    actual = dict(y=y, dx=xg.grad, dw=layer.weight.grad, db=layer.bias.grad)
    assert layer.weight.grad.dtype == torch.bfloat16 and layer.bias.grad.dtype == torch.bfloat16
    errors = {key: rel_l2(actual[key], expect[key]) for key in actual}
    assert max(errors.values()) < .003, errors                                 # the reference's bound (:76-77)
    assert torch.equal(layer.bias.grad.cpu(), expect["db"])
    # state-dict reload reproduces the forward bit for bit (:82-87)
    restored = viola_amd.nn.Linear(128, 96, device="cuda", dtype=torch.bfloat16, scaling="grouped", mode=mode,
                                   weight_group_shape=gw, input_group_shape=gx, grad_group_shape=gg,
                                   saved_input_dtype=saved, backward_dtype=bwd, weight_dtype=storage)
    restored.load_state_dict(layer.state_dict())
    restored.bfloat16()
    assert restored.weight.dtype == layer.weight.dtype and restored.weight_scale.dtype == torch.float32
    with torch.no_grad():
        assert torch.equal(restored(xg), y)
    assert (restored.weight_transpose.numel() > 0) == (mode == "fast" and storage == "fp8")


def test_linear_host_construction_then_move_and_no_grad_paths():
    import viola_amd
    torch.manual_seed(5)
    layer = viola_amd.nn.Linear(64, 32, scaling="grouped", backward_dtype="e4m3")   # built on the host
    master = layer._initial_weight.clone()
    layer = layer.cuda()
    rq, rs = og.quantize(master, E4, (32, 32))
    assert torch.equal(layer.weight.detach().cpu().view(torch.uint8), rq.view(torch.uint8)) and torch.equal(layer.weight_scale.cpu(), rs)
    x = torch.randn(3, 5, 64, device="cuda")
    with torch.no_grad():
        y = layer(x)
    assert y.shape == (3, 5, 32) and y.dtype == torch.float32
    with pytest.raises(AssertionError):
        layer(x.cpu())
    with pytest.raises(AssertionError):
        viola_amd.nn.Linear(64, 64, scaling="grouped", rotation_size=64)         # linear.py:183
    with pytest.raises(AssertionError):
        viola_amd.nn.Linear(96, 64, scaling="current", rotation_size=64)         # linear.py:200
    with pytest.raises(AssertionError):
        viola_amd.nn.Linear(64, 32, scaling="mxfp8", accum_dtype="fp16")         # linear.py:187-188
    layer.weight.requires_grad_(False)
    layer.bias.requires_grad_(False)
    xg = x.clone().requires_grad_()
    layer(xg).sum().backward()
    assert xg.grad is not None and layer.weight.grad is None


@pytest.mark.parametrize("options", [dict(weight_dtype="bf16"), dict(weight_dtype="fp8", mode="fast", activation="gelu"),
                                     dict(weight_dtype="fp8", activation="relu", backward_dtype="e5m2"),
                                     dict(weight_dtype="fp8", bias=False)])
def test_mlp_fused_vs_oracle(options, bf16_gradients):
    """checks/mlp.py:19-52: MLP(128, 160, 96), x [2, 33, 128], all of y, dx and every parameter gradient."""
    import viola_amd
    torch.manual_seed(131)
    options = dict(backward_dtype="e4m3", **options) if "backward_dtype" not in options else options
    model = viola_amd.nn.MLP(128, 160, 96, device="cuda", dtype=torch.bfloat16, scaling="grouped", **options)
    x = torch.randn(2, 33, 128).bfloat16()
    dy = torch.randn(2, 33, 96).bfloat16()
    xg = x.cuda().requires_grad_()
    y = model(xg)
    y.backward(dy.cuda())
    name = options.get("activation", "silu")
    bwd = E5 if options.get("backward_dtype") == "e5m2" else E4
    def real(layer):
        if layer.weight_dtype == "fp8":
            return layer.dequantize_weight().cpu()
        return og.dequantize(*og.quantize(layer.weight.detach().cpu(), E4, (32, 32)), (32, 32))
    bias = lambda layer: None if layer.bias is None else layer.bias.detach().cpu()
    expect = ol.mlp(x, real(model.gate_up), bias(model.gate_up), real(model.down), bias(model.down), dy, name=name, bwd_fp8=bwd)
    errors = dict(y=rel_l2(y, expect["y"]), dx=rel_l2(xg.grad, expect["dx"]),
                  dw_gate_up=rel_l2(model.gate_up.weight.grad, expect["dw_gate_up"]),
                  dw_down=rel_l2(model.down.weight.grad, expect["dw_down"]))
    if model.down.bias is not None:
        errors["db_down"] = rel_l2(model.down.bias.grad, expect["db_down"])
        errors["db_gate_up"] = rel_l2(model.gate_up.bias.grad, expect["db_gate_up"])
    assert max(errors.values()) < .025, errors                                 # the reference's bound (checks/mlp.py:42)
    # two pending forwards + accumulation use distinct contexts (:49-51)
    model.zero_grad(); xg.grad = None
    (model(xg).float().square().mean() + model(xg * .7).float().square().mean()).backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in model.parameters() if p.requires_grad)


def test_mlp_frozen_gate_up(bf16_gradients):
    import viola_amd
    torch.manual_seed(131)
    model = viola_amd.nn.MLP(128, 160, 96, device="cuda", dtype=torch.bfloat16, scaling="grouped", weight_dtype="bf16", backward_dtype="e4m3")
    model.gate_up.requires_grad_(False)
    x = torch.randn(2, 33, 128, device="cuda", dtype=torch.bfloat16)
    model(x).backward(torch.randn(2, 33, 96, device="cuda", dtype=torch.bfloat16))
    assert model.gate_up.weight.grad is None and model.down.weight.grad is not None


class _Probe:
    def __init__(self):
        self.updates, self.momenta = {}, 0

    def momentum(self, p, grad, old_q, old_scale, q, scale, matrix, group, loss_scale, quant):
        self.momenta += 1

    def update(self, p, update, group, fn):
        self.updates[id(p)] = update.float().reshape_as(p).clone()


@pytest.mark.parametrize("granularity,rounding,method", [("tile", "nearest", "standard"), ("block", "stochastic", "standard"),
                                                          ("tile", "stochastic", "gram")])
def test_fp8muon_step_state_and_resume(granularity, rounding, method):
    """checks/optimizer.py:45-92: routing, state layout, the weight formula, exact resume, grad=None skip; plus an
    oracle replay of the momentum state and AdamW weights."""
    import viola_amd
    torch.manual_seed(31)
    shapes = ((32, 64), (4, 4, 3, 3), (2, 16, 32), (32,))
    params = [torch.nn.Parameter(torch.randn(*s, device="cuda")) for s in shapes]
    groups = [dict(params=params[:1], use_muon=True), dict(params=params[1:2], use_muon=True, nesterov=False),
              dict(params=params[2:3], batched=True), dict(params=params[3:], use_muon=False)]
    opt = viola_amd.optim.FP8Muon(groups, lr=.003, weight_decay=.07, tile_size=64, granularity=granularity,
                                  rounding=rounding, rounding_seed=17, ns_method=method, adam_state_dtype="bf16")
    probe = _Probe()
    opt.observer = probe
    quant = dict(granularity=granularity, tile_size=64, block_shape=(16, 16))
    mshape = lambda p: tuple(p.shape) if p is params[2] else (p.shape[0], p.numel() // p.shape[0])
    ref_q = [torch.zeros(oo.state_sizes(mshape(p), **quant)[0], dtype=torch.uint8) for p in params[:3]]
    ref_s = [torch.ones(oo.state_sizes(mshape(p), **quant)[1]) for p in params[:3]]
    ref_vec = [params[3].detach().cpu().clone(), torch.zeros(32, dtype=torch.bfloat16), torch.zeros(32, dtype=torch.bfloat16)]
    for step in range(3):
        before = [p.detach().clone() for p in params]
        for p in params:
            p.grad = torch.randn_like(p)
        opt.step()
        for i, (p, previous) in enumerate(zip(params[:3], before)):
            shape = mshape(p)
            scale = .2 * max(shape[-2:]) ** .5
            expected = previous * (1 - .003 * .07) - .003 * scale * probe.updates[id(p)]
            torch.testing.assert_close(p.detach(), expected, rtol=2e-6, atol=5e-7)
            state = opt.state[p]
            assert set(state) == {"step", "momentum_q", "momentum_scale"} and state["step"] == step + 1
            assert state["momentum_q"].dtype == torch.uint8 and state["momentum_scale"].dtype == torch.float32
            key = (17 + i * 0x9E3779B97F4A7C15) & ((1 << 63) - 1)
            ref_q[i], ref_s[i], _ = oo.momentum_update(p.grad.cpu(), ref_q[i], ref_s[i], beta=.95, shape=shape,
                                                       nesterov=i != 1, rounding=rounding, rounding_step=step, rounding_key=key, **quant)
            assert torch.equal(state["momentum_q"].cpu(), ref_q[i]) and torch.equal(state["momentum_scale"].cpu(), ref_s[i])
        ref_vec = list(oo.adam_update(ref_vec[0], params[3].grad.cpu(), ref_vec[1], ref_vec[2], lr=.003, weight_decay=.07,
                                      betas=(.9, .95), eps=1e-8, step=step + 1))
        assert torch.equal(params[3].detach().cpu(), ref_vec[0]) and opt.state[params[3]]["exp_avg"].dtype == torch.bfloat16
    assert probe.momenta == 9
    saved_weights, saved = [p.detach().clone() for p in params], copy.deepcopy(opt.state_dict())
    opt.observer = None
    opt.step()
    expected_weights, expected_state = [p.detach().clone() for p in params], copy.deepcopy(opt.state_dict())
    with torch.no_grad():
        for p, value in zip(params, saved_weights):
            p.copy_(value)
    opt.load_state_dict(saved)
    assert opt.state[params[0]]["momentum_q"].dtype == torch.uint8 and opt.state[params[3]]["exp_avg"].dtype == torch.bfloat16
    opt.step()
    for p, value in zip(params, expected_weights):
        assert torch.equal(p.detach(), value)
    for (ka, va), (kb, vb) in zip(sorted(opt.state_dict()["state"].items()), sorted(expected_state["state"].items())):
        for name in va:
            assert torch.equal(torch.as_tensor(va[name]), torch.as_tensor(vb[name])), name
    before, step = params[0].detach().clone(), opt.state[params[0]]["step"]
    params[0].grad = None
    opt.step()
    assert torch.equal(params[0].detach(), before) and opt.state[params[0]]["step"] == step


def test_fp8muon_update_matches_oracle_ns():
    """One matrix, one step: the weight equals w(1 - lr wd) - lr 0.2 sqrt(max) NS(momentum update), NS from the oracle chain."""
    import viola_amd
    torch.manual_seed(2)
    w = torch.nn.Parameter(torch.randn(96, 256, device="cuda"))
    before = w.detach().cpu().clone()
    w.grad = torch.randn_like(w) * 1e-3
    for method in ("standard", "gram"):
        with torch.no_grad():
            w.copy_(before)
        opt = viola_amd.optim.FP8Muon([w], lr=1e-3, weight_decay=.01, tile_size=256, ns_method=method)
        opt.step()
        _, _, u = oo.momentum_update(w.grad.cpu(), torch.zeros(96 * 256, dtype=torch.uint8), torch.ones(96), beta=.95, shape=(96, 256))
        update = ons.chain(u.view(96, 256), 5, method)
        expect = oo.weight_update(before, update, 1e-3, .01, update_scale=.2 * 256 ** .5)
        assert rel_l2(w.detach() - before.cuda(), expect - before) < (.07 if method == "standard" else .03)


def test_skip_nonfinite():
    import viola_amd
    w = torch.nn.Parameter(torch.randn(32, 64, device="cuda"))
    opt = viola_amd.optim.FP8Muon([w], tile_size=64, skip_nonfinite=True)
    w.grad = torch.full_like(w, float("nan"))
    before = w.detach().clone()
    opt.step()
    assert opt.step_was_skipped and not opt.state and torch.equal(w.detach(), before)
    opt.skip_nonfinite = False
    opt.step()
    assert not opt.step_was_skipped and torch.isnan(w).any()
