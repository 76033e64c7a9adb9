"""viola.optim.bind_optimizer on the GPU: master weights behind FP8 / BF16 / FP16 weight storage
(viola/optim/master_weights.py, pinned by checks/optimizer.py:111-152). The write-back after a step is the
(32, 32)-block quantizer, held bit for bit to the oracle's quantize of the master."""

import copy

import pytest
import torch

from oracle import grouped as og, optim as oo

pytestmark = pytest.mark.gpu
E4 = torch.float8_e4m3fn
DTYPES = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}


@pytest.fixture
def precision_policy():
    import viola_amd
    saved = dict(viola_amd.precision._settings)
    yield viola_amd
    viola_amd.precision._settings.clear()
    viola_amd.precision._settings.update(saved)


def _equal(a, b):
    if isinstance(a, torch.Tensor):
        assert a.dtype == b.dtype and torch.equal(a.view(torch.uint8) if a.dtype.itemsize == 1 else a, b.view(torch.uint8) if b.dtype.itemsize == 1 else b)
    elif isinstance(a, dict):
        assert a.keys() == b.keys()
        for key in a:
            _equal(a[key], b[key])
    elif isinstance(a, (list, tuple)):
        assert len(a) == len(b)
        for x, y in zip(a, b):
            _equal(x, y)
    else:
        assert a == b


@pytest.mark.parametrize("master,gradient,weight_dtype", [("fp32", "bf16", "fp8"), ("bf16", "fp32", "fp8"), ("fp16", "bf16", "fp8"),
                                                          (None, "fp32", "bf16"), (None, "bf16", "fp16")])
def test_linear_integration_exact_resume(precision_policy, master, gradient, weight_dtype):
    """checks/optimizer.py:111-139: two micro-batches per update, three updates, save, one more update; reloading the
    saved model + optimizer state and repeating that update reproduces model and optimizer state bit for bit."""
    viola = precision_policy
    viola.set_master_weight_dtype(master, rounding="nearest" if master in (None, "fp32") else "stochastic", seed=37)
    viola.set_gradient_dtype(gradient)
    torch.manual_seed(5)
    model = viola.nn.Linear(64, 32, device="cuda", dtype=torch.bfloat16, weight_dtype=weight_dtype, scaling="grouped")
    opt = viola.optim.bind_optimizer(model, viola.optim.FP8Muon(model.parameters(), lr=.01, tile_size=64))
    x = torch.randn(128, 64, device="cuda", dtype=torch.bfloat16)

    def update():
        opt.zero_grad()
        for micro in x.chunk(2):
            (model(micro).float().square().mean() / 2).backward()
        opt.step()

    for _ in range(3):
        update()
    saved = copy.deepcopy(dict(model=model.state_dict(), optimizer=opt.state_dict()))
    update()
    expected = copy.deepcopy(dict(model=model.state_dict(), optimizer=opt.state_dict()))
    model.load_state_dict(saved["model"])
    opt.load_state_dict(saved["optimizer"])
    update()
    _equal(model.state_dict(), expected["model"])
    _equal(opt.state_dict(), expected["optimizer"])
    assert model.weight.grad.dtype == DTYPES[gradient]
    if master is None:
        assert model._master_ref() is model.weight
        assert all(value is None for value in opt.state_dict()["viola_masters"]["weights"])
    else:
        assert model._master_ref().dtype == DTYPES[master]
    assert not torch.equal(saved["model"]["weight"].view(torch.uint8) if weight_dtype == "fp8" else saved["model"]["weight"],
                           expected["model"]["weight"].view(torch.uint8) if weight_dtype == "fp8" else expected["model"]["weight"])


def test_bound_step_equals_unbound_master_and_oracle_requantize(precision_policy):
    """One bound step on an FP8-stored Linear: the master moves exactly as an unbound FP8Muon moves a plain fp32
    parameter given the same gradient, and the stored codes / scales are the oracle's (32, 32) quantize of it."""
    viola = precision_policy
    viola.set_master_weight_dtype("fp32")
    viola.set_gradient_dtype("bf16")
    torch.manual_seed(6)
    model = viola.nn.Linear(256, 160, bias=False, device="cuda", dtype=torch.bfloat16, weight_dtype="fp8", scaling="grouped")
    start = model._initial_weight.detach().clone()
    opt = viola.optim.bind_optimizer(model, viola.optim.FP8Muon(model.parameters(), lr=.01, weight_decay=.1, tile_size=256))
    assert model._initial_weight is None and torch.equal(model._master_ref().detach(), start)
    x = torch.randn(96, 256, device="cuda", dtype=torch.bfloat16)
    for _ in range(2):
        opt.zero_grad()
        model(x).float().square().mean().backward()
        opt.step()
        assert model._master_ref().grad is None and model.weight.grad is not None
        master = model._master_ref().detach()
        q, s = og.quantize(master.cpu(), E4, (32, 32))
        assert torch.equal(model.weight.detach().view(torch.uint8).cpu(), q.view(torch.uint8)) and torch.equal(model.weight_scale.cpu(), s)
    # the same two updates on free-standing fp32 parameters (fresh state each time would differ: replay both steps)
    torch.manual_seed(6)
    again = viola.nn.Linear(256, 160, bias=False, device="cuda", dtype=torch.bfloat16, weight_dtype="fp8", scaling="grouped")
    free = torch.nn.Parameter(again._initial_weight.detach().clone())
    free.grad_dtype = torch.bfloat16
    plain = viola.optim.FP8Muon([free], lr=.01, weight_decay=.1, tile_size=256)
    for _ in range(2):
        with torch.no_grad():
            again.refresh_weight(free)
        again.zero_grad()
        again(x).float().square().mean().backward()
        free.grad = again.weight.grad
        plain.step()
    assert torch.equal(free.detach(), model._master_ref().detach())


def test_nonfinite_policy(precision_policy):
    """checks/optimizer.py:142-152: a skipped step leaves model and optimizer untouched; the default propagates NaN."""
    viola = precision_policy
    model = viola.nn.Linear(64, 32, device="cuda", scaling="grouped", weight_dtype="fp8")
    opt = viola.optim.bind_optimizer(model, viola.optim.FP8Muon(model.parameters(), tile_size=64, skip_nonfinite=True))
    model.weight.grad = torch.full(model.weight.shape, float("nan"), device="cuda", dtype=model.weight.grad_dtype)
    before = copy.deepcopy(model.state_dict())
    opt.step()
    _equal(model.state_dict(), before)
    assert opt.step_was_skipped and not opt.state
    opt.skip_nonfinite = False
    opt.step()
    assert not opt.step_was_skipped and torch.isnan(model._master_ref()).any()


@pytest.mark.parametrize("rounding", ["nearest", "stochastic"])
def test_mixed_adamw_goes_through_the_kernel(precision_policy, rounding):
    """torch.optim.AdamW bound to bf16 storage: the master takes the kernel's AdamW (viola/optim/master_weights.py:13-43),
    bit for bit the oracle's, and the model receives the rounded copy."""
    viola = precision_policy
    master = "fp32" if rounding == "nearest" else "bf16"
    viola.set_master_weight_dtype(master, rounding=rounding, seed=11)
    viola.set_gradient_dtype("bf16")
    torch.manual_seed(8)
    model = torch.nn.Linear(48, 24, bias=False, device="cuda", dtype=torch.bfloat16 if master == "fp32" else torch.float16)
    opt = viola.optim.bind_optimizer(model, torch.optim.AdamW(model.parameters(), lr=1e-2, weight_decay=.1, betas=(.9, .95)))
    w = model.weight.detach().cpu().to(DTYPES[master])
    m, v = torch.zeros(24, 48), torch.zeros(24, 48)
    m, v = m.to(w.dtype), v.to(w.dtype)
    for step in (1, 2, 3):
        grad = (torch.randn(24, 48) * .1).bfloat16()
        model.weight.grad = grad.cuda()
        opt.step()
        w, m, v = oo.adam_update(w, grad, m, v, lr=1e-2, weight_decay=.1, betas=(.9, .95), eps=1e-8, step=step,
                                 rounding=rounding, key=11)
        w, m, v = w.view(24, 48), m.view(24, 48), v.view(24, 48)
        held = opt.param_groups[0]["params"][0]
        assert held is not model.weight and held.dtype == DTYPES[master]
        assert torch.equal(held.detach().cpu(), w)
        assert torch.equal(model.weight.detach().cpu(), w.to(model.weight.dtype))
        assert model.weight.grad is not None and held.grad is None
    state = opt.state_dict()
    assert state["viola_masters"]["weights"][0].dtype == DTYPES[master]


def test_block_quantizer_at_weight_size():
    """The write-back kernel at the benchmark layer's size (4096 x 1024, fp32 and bf16 masters): oracle codes and scales."""
    from viola_amd.nn import _grouped_kernels as g
    torch.manual_seed(9)
    for dtype in (torch.float32, torch.bfloat16):
        x = ((torch.rand(4096, 1024) - .5) / 16).to(dtype)
        x[100, 200] = 3.0
        x[4000, 1000:1024] = 0
        q, s = g.quantize(x.cuda(), E4, (32, 32))
        rq, rs = og.quantize(x, E4, (32, 32))
        assert torch.equal(q.view(torch.uint8).cpu(), rq.view(torch.uint8)) and torch.equal(s.cpu(), rs)
