"""Hadamard-64 rotation (viola/nn/_rotation_kernels.py) through the C ABI: rotated amax / scale, rotated quantize
(row-wise and transposed) and the in-place rotation, bit for bit against the oracle's staged restatement; then
Linear(rotation_size=64) against the reference's own definition of the recipe, rotate = x.reshape(-1, 64) @ H64
(checks/floating_weight_storage.py:74-87, bound .004) and MLP with that recipe (checks/mlp.py:67, bound .025)."""

import pytest
import torch
import torch.nn.functional as F

from oracle import rotation as orot, tensor as ot
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


def outliers(rows, cols, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g)
    x[:, ::37] *= 30                                                             # channel outliers: what the rotation spreads
    return x.to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(64, 64), (65, 128), (130, 192), (7, 100), (200, 24), (1, 64)])
def test_rotated_scale_and_codes_match_the_oracle(dtype, shape):
    from viola_amd.nn import _rotation_kernels as rotation
    x = outliers(*shape, dtype, 3)
    rotated = orot.rotate(x)
    history = torch.zeros(4, device="cuda")
    scale = rotation.tensor_scale(x.cuda(), history=history, index=0, delayed=False, fp8_dtype=E4)
    want_scale, after = ot.tensor_scale(rotated, torch.zeros(4), 0, limit=448.0)
    assert torch.equal(scale.cpu().reshape(()), want_scale.reshape(()))
    assert history[0].item() == orot.amax(x).item() == after[0].item()
    for fp8 in (E4, E5):
        q, qt = rotation.quantize(x.cuda(), scale, transpose=True, fp8_dtype=fp8)
        want = ot.quantize(rotated, want_scale, fp8)
        assert torch.equal(q.cpu().view(torch.uint8), want.view(torch.uint8))
        assert torch.equal(qt.cpu().view(torch.uint8), want.T.contiguous().view(torch.uint8))
        only_t = rotation.quantize(x.cuda(), scale, rowwise=False, transpose=True, fp8_dtype=fp8)
        assert only_t[0].numel() == 0 and torch.equal(only_t[1], qt)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(64, 64), (65, 128), (96, 4096), (7, 100), (33, 8)])
def test_inplace_rotation_matches_the_oracle_and_undoes_itself(dtype, shape):
    from viola_amd.nn import _rotation_kernels as rotation
    x = outliers(*shape, dtype, 5)
    got = rotation.inverse_(x.cuda().clone())
    assert torch.equal(got.cpu(), orot.rotate(x).to(dtype))
    # on small integers every fp32 sum is exact: the rotation is an involution bit for bit (whole groups only: a
    # group cut off by the matrix edge loses its tail)
    if dtype == torch.float32 and shape[1] % 64 == 0:
        k = torch.randint(-40, 41, shape).float()
        assert torch.equal(rotation.inverse_(rotation.inverse_(k.cuda().clone())).cpu(), k)


def test_rotated_quantize_keeps_nan_and_spreads_it_over_its_group():
    from viola_amd.nn import _rotation_kernels as rotation
    x = torch.randn(4, 128)
    x[1, 70] = float("nan")
    scale = torch.tensor([0.01], device="cuda")
    q, _ = rotation.quantize(x.cuda(), scale, fp8_dtype=E4)
    want = ot.quantize(orot.rotate(x), torch.tensor(0.01), E4)
    # the sign of a NaN that went through additions is the arithmetic unit's choice: compare NaN-ness there, bits elsewhere
    bad = want.float().isnan()
    assert torch.equal(q.cpu().float().isnan(), bad) and bad[1, 64:].all() and bad.sum() == 64
    assert torch.equal(q.cpu().view(torch.uint8)[~bad], want.view(torch.uint8)[~bad])


def reference_rotate(x):
    """rotate_cpu, the reference's definition (_rotation_kernels.py:126-130)."""
    return (x.float().reshape(-1, 64) @ orot.hadamard64()).reshape(x.shape)


def fake_quantize(x, scale, fp8, limit=None):
    limit = torch.finfo(fp8).max if limit is None else limit
    return (x.float() / scale).clamp(-limit, limit).to(fp8).float() * scale


@pytest.mark.parametrize("storage,mode,saved", [("bf16", "memory", "bf16"), ("fp8", "fast", "fp8"), ("fp8", "memory", "fp32")])
def test_linear_with_rotation(bf16_gradients, storage, mode, saved):
    """checks/floating_weight_storage.py:30-93 with rotate=64: Linear(128, 96), x [65, 128]."""
    import viola_amd
    torch.manual_seed(121)
    source = torch.nn.Linear(128, 96, dtype=torch.bfloat16)
    source.weight.data[:, ::19] *= 12
    weight, bias = source.weight.detach().clone(), source.bias.detach().clone()
    layer = viola_amd.nn.Linear.from_float(source.cuda(), weight_dtype=storage, mode=mode, scaling="current",
                                           saved_input_dtype=saved, rotation_size=64)
    x = torch.randn(65, 128).bfloat16()
    dy = torch.randn(65, 96).bfloat16()
    xg = x.cuda().requires_grad_()
    captured = []
    with torch.autograd.graph.saved_tensors_hooks(lambda t: (captured.append(t), t)[1], lambda t: t):
        y = layer(xg)
    y.backward(dy.cuda())
    sx, sw = captured[1].cpu(), captured[3].cpu()
    rx, rw = reference_rotate(x), reference_rotate(weight)
    assert torch.equal(sx.reshape(()), (orot.amax(x) / 448.0).reshape(()))
    qx, qw = fake_quantize(rx, sx, E4), fake_quantize(rw, sw, E4)
    sg = dy.float().abs().max() / 57344.0
    qg = fake_quantize(dy, sg, E5)
    expected = dict(y=qx @ qw.T + bias.float(), dx=reference_rotate((qg @ qw).bfloat16()),
                    dw=reference_rotate((qg.T @ qx).bfloat16()))
    actual = dict(y=y, dx=xg.grad, dw=layer.weight.grad)
    errors = {name: rel_l2(actual[name], expected[name].bfloat16()) for name in actual}
    assert max(errors.values()) < .004, errors
    assert torch.equal(layer.bias.grad.cpu(), dy.sum(0, dtype=torch.bfloat16))
    # against the unquantized layer the rotated recipe is an ordinary FP8 Linear
    plain = dict(y=F.linear(x.float(), weight.float(), bias.float()), dx=dy.float() @ weight.float(), dw=dy.float().T @ x.float())
    assert max(rel_l2(actual[name], plain[name]) for name in actual) < .08
    if storage == "fp8":
        # the stored codes are those of the rotated weight; dequantize_weight returns original coordinates
        want_scale = ot.tensor_scale(orot.rotate(weight), torch.zeros(1), 0, limit=448.0)[0]
        assert torch.equal(layer.weight_scale.cpu().reshape(()), want_scale.reshape(()))
        assert torch.equal(layer.weight.detach().cpu().view(torch.uint8), ot.quantize(orot.rotate(weight), want_scale, E4).view(torch.uint8))
        assert rel_l2(layer.dequantize_weight(), weight) < .04
        if mode == "fast":
            assert torch.equal(layer.weight_transpose.cpu().view(torch.uint8), layer.weight.detach().cpu().view(torch.uint8).T)


def test_mlp_with_rotation(bf16_gradients):
    """checks/mlp.py:19-45 with the recipe of :67 (hidden 192): the MLP against its own two Linears around the
    activation computed by PyTorch."""
    import viola_amd
    torch.manual_seed(131)
    model = viola_amd.nn.MLP(128, 192, 96, device="cuda", dtype=torch.bfloat16, weight_dtype="bf16", scaling="current",
                             rotation_size=64, saved_input_dtype="bf16")
    x = torch.randn(2, 33, 128, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    dy = torch.randn(2, 33, 96, device="cuda", dtype=torch.bfloat16)
    y = model(x)
    y.backward(dy)
    actual = [y.detach().clone(), x.grad.clone()] + [p.grad.clone() for p in model.parameters()]
    model.zero_grad(set_to_none=True)
    x.grad = None
    g, u = model.gate_up(x).chunk(2, -1)
    target = model.down((F.silu(g.float()) * u.float()).to(x.dtype))
    target.backward(dy)
    expected = [target.detach(), x.grad] + [p.grad for p in model.parameters()]
    for a, b in zip(actual, expected):
        assert rel_l2(a, b) < .025
