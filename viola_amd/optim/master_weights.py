"""`bind_optimizer(model, optimizer)`: the optimizer updates a higher-precision master of every parameter while the
model keeps its storage format (drop-in for viola/optim/master_weights.py:168-179; behaviour pinned by the reference's
checks/optimizer.py:111-152: micro-batch accumulation, exact resume from model + optimizer state dicts, gradient and
master dtypes, masters switched off, the non-finite skip).

Organisation here: each optimizer slot gets a `_Slot` that knows three things about its parameter: where the master
comes from, how a finished step flows back into the model (FP8 codes + (32, 32) scales from the HIP block quantizer,
or a plain copy), and how it is restored from a checkpoint. The binding itself only walks the slots from five
optimizer hooks. The `viola_masters` state-dict entry has the reference's keys, so checkpoints move between the two."""

import weakref

import torch
from torch import nn

from ..nn import Linear
from ..precision import settings
from ._kernels import adam_update
from .matrix import MatrixOptimizer


class _Slot:
    """One model parameter, the tensor the optimizer really updates for it, and the Linear that owns it (if any)."""

    __slots__ = ("param", "master", "layer", "lent")

    def __init__(self, param, layer, master_dtype, gradient_dtype):
        self.param, self.layer, self.lent = param, layer, None
        fp8_storage = layer is not None and layer.weight_dtype == "fp8"
        if fp8_storage:
            assert master_dtype is not None, "Disabling the master requires BF16/FP16/FP32 weight storage."
            # the values the codes were made from, while the module still has them; a module restored from a
            # model-only checkpoint does not, and starts from what its codes decode to
            start = layer._initial_weight if layer._initial_weight is not None else layer.dequantize_weight()
            self.master = nn.Parameter(start.to(master_dtype), requires_grad=param.requires_grad)
        elif master_dtype is None or param.dtype == master_dtype:
            self.master = param
        else:
            self.master = nn.Parameter(param.detach().to(master_dtype), requires_grad=param.requires_grad)
        self.master.grad_dtype = param.grad_dtype = gradient_dtype
        if layer is not None:
            layer._initial_weight, layer._master_ref = None, weakref.ref(self.master)

    @property
    def aliased(self):
        return self.master is self.param

    def lend(self):
        """Hand the model's gradient accumulator to the master for one step (no second buffer). False: nothing to step."""
        self.lent = self.param.grad
        if self.lent is not None:
            self.master.grad = self.lent
        return self.lent is not None

    def settle(self, write_back):
        """After the step: push the master into the model's storage and undo `lend`."""
        if self.lent is None:
            return
        if write_back:
            if self.layer is not None:
                self.layer.refresh_weight(self.master)
            elif not self.aliased:
                self.param.copy_(self.master)
        if self.aliased:
            self.param.grad = self.lent          # the mixed-dtype AdamW route may have hidden it from the stock step
        else:
            self.master.grad = None
        self.lent = None

    def clear_model_grad(self, set_to_none):
        if self.aliased or self.param.grad is None:
            return
        if set_to_none:
            self.param.grad = None
        else:
            self.param.grad.detach_().zero_()

    def saved(self):
        return None if self.aliased else self.master.detach()        # an aliased master travels with the model

    def restore(self, value):
        if value is not None:
            self.master.copy_(value)

    def after_restore(self):
        # FP8 codes and scales come back verbatim with the model's own state dict: quantizing the master again would
        # round a second time what is already exact. Other storage formats are re-derived from the master.
        if not self.aliased and not (self.layer is not None and self.layer.weight_dtype == "fp8"):
            self.param.copy_(self.master)


def _mixed_precision_adamw(optimizer, rounding, seed):
    """Stock torch optimizers refuse a gradient whose dtype differs from the parameter's and cannot round
    stochastically (viola/optim/master_weights.py:13-43). For torch.optim.AdamW such parameters take the AdamW
    kernel here and are hidden from the stock step by taking their `.grad` away; torch.optim.SGD is sent down its
    single-tensor path, which accepts mixed dtypes."""
    kind = type(optimizer)
    if kind not in (torch.optim.AdamW, torch.optim.SGD):
        return
    for group in optimizer.param_groups:
        odd = [p for p in group["params"] if p.grad is not None and (p.grad.dtype != p.dtype or rounding != "nearest")]
        if not odd:
            continue
        if kind is torch.optim.SGD:
            assert rounding == "nearest"
            group["foreach"] = False
            continue
        assert not any(group.get(flag, False) for flag in ("amsgrad", "capturable", "differentiable", "fused"))
        for p in odd:
            state = optimizer.state[p]
            if "step" not in state:
                state.update(step=torch.tensor(0.), exp_avg=torch.zeros_like(p), exp_avg_sq=torch.zeros_like(p))
            state["step"] += 1
            adam_update(p, p.grad, state["exp_avg"], state["exp_avg_sq"], lr=group["lr"], weight_decay=group["weight_decay"],
                        betas=group["betas"], eps=group["eps"], step=int(state["step"]), rounding=rounding, key=seed,
                        maximize=group.get("maximize", False))
            p.grad = None


class _Binding:
    def __init__(self, model, optimizer):
        assert not optimizer.state, "Bind the optimizer before its first step or load_state_dict."
        policy = settings()
        self.master_dtype = policy["master_weight_dtype"]
        self.gradient_dtype = policy["gradient_dtype"] or torch.float32
        self.rounding, self.seed = policy["master_rounding"], policy["master_rounding_seed"]
        self.matrix = isinstance(optimizer, MatrixOptimizer)
        layer_of = {id(m.weight): m for m in model.modules() if isinstance(m, Linear)}
        by_param = {}
        for group in optimizer.param_groups:
            if self.matrix:
                group.update(master_rounding=self.rounding, master_rounding_seed=self.seed)
            params = group["params"]
            for position, p in enumerate(params):
                slot = by_param.get(id(p))
                if slot is None:
                    slot = by_param[id(p)] = _Slot(p, layer_of.get(id(p)), self.master_dtype, self.gradient_dtype)
                params[position] = slot.master
        self.slots = list(by_param.values())
        if self.matrix:
            optimizer._partition = None
        optimizer.register_step_pre_hook(self._before_step)
        optimizer.register_step_post_hook(self._after_step)
        optimizer.register_state_dict_post_hook(self._on_save)
        optimizer.register_load_state_dict_pre_hook(self._on_load)
        optimizer.register_load_state_dict_post_hook(self._after_load)
        stock_zero_grad = optimizer.zero_grad

        def zero_grad(set_to_none=True):
            stock_zero_grad(set_to_none=set_to_none)
            for slot in self.slots:
                slot.clear_model_grad(set_to_none)
        optimizer.zero_grad = zero_grad

    @torch.no_grad()
    def _before_step(self, optimizer, args, kwargs):
        assert len(args) == 1 and kwargs.get("closure") is None, \
            "The master binding uses explicit forward/backward, without an optimizer closure."
        for slot in self.slots:
            slot.lend()
        _mixed_precision_adamw(optimizer, self.rounding, self.seed)

    @torch.no_grad()
    def _after_step(self, optimizer, args, kwargs):
        write_back = not (self.matrix and optimizer.step_was_skipped)
        for slot in self.slots:
            slot.settle(write_back)

    def _on_save(self, optimizer, state):
        state["viola_masters"] = {"weights": [slot.saved() for slot in self.slots], "gradient_dtype": self.gradient_dtype,
                                  "master_dtype": self.master_dtype, "rounding": self.rounding, "seed": self.seed}

    @torch.no_grad()
    def _on_load(self, optimizer, state):
        rest = {key: value for key, value in state.items() if key != "viola_masters"}
        entry = state["viola_masters"]
        assert (entry["master_dtype"], entry["gradient_dtype"]) == (self.master_dtype, self.gradient_dtype)
        assert len(entry["weights"]) == len(self.slots)
        self.rounding, self.seed = entry["rounding"], entry["seed"]
        for slot, value in zip(self.slots, entry["weights"]):
            slot.restore(value)
        return rest

    @torch.no_grad()
    def _after_load(self, optimizer):
        for slot in self.slots:
            slot.after_restore()
        optimizer.zero_grad()


def bind_optimizer(model, optimizer):
    """Install the master write-back on `optimizer` and return it. Move the model to the GPU and call the precision
    setters (`set_master_weight_dtype`, `set_gradient_dtype`) first; for an exact resume save and load both the
    model's and the optimizer's state dict. `set_master_weight_dtype(None)` makes every parameter its own master
    (BF16/FP16/FP32 storage only)."""
    assert not hasattr(optimizer, "_viola_linear_masters"), "This optimizer is already bound."
    optimizer._viola_linear_masters = _Binding(model, optimizer)
    return optimizer
