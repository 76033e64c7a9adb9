"""Master weights behind a model whose storage precision differs from the precision the optimizer updates in
(viola/optim/master_weights.py:13-179). `bind_optimizer(model, optimizer)` swaps every bound parameter of the
optimizer for its master (an FP32/BF16/FP16 copy, or the parameter itself when masters are disabled), lends the
model's gradient to the master for the duration of `step()`, and writes the result back: FP8-stored Linear weights
are re-quantized from the master by the (32, 32)-block HIP quantizer, BF16/FP16 parameters are copied.

State dict layout matches the reference (`viola_masters` entry with weights / dtypes / rounding / seed), so a
checkpoint moves between the two implementations."""

import weakref

import torch
from torch import nn

from ..nn import Linear
from ..precision import settings
from .matrix import MatrixOptimizer
from ._kernels import adam_update

_PLAIN_ADAMW_FLAGS = ("amsgrad", "capturable", "differentiable", "fused")


@torch.no_grad()
def step_mixed_adamw(optimizer, precision):
    """torch.optim.AdamW cannot step a parameter whose gradient has another dtype, nor round stochastically: such
    entries are stepped here by the AdamW kernel and hidden from the stock step (viola/optim/master_weights.py:13-43).
    Returns the (parameter, gradient) pairs whose `.grad` was taken away."""
    taken = []
    rounding = precision["master_rounding"]
    for group in optimizer.param_groups:
        for parameter in group["params"]:
            gradient = parameter.grad
            if gradient is None or (gradient.dtype == parameter.dtype and rounding == "nearest"):
                continue
            if type(optimizer) is torch.optim.AdamW:
                assert not any(group.get(flag, False) for flag in _PLAIN_ADAMW_FLAGS)
                state = optimizer.state[parameter]
                if not state:
                    state["step"] = torch.tensor(0.)
                    state["exp_avg"] = torch.zeros_like(parameter)
                    state["exp_avg_sq"] = torch.zeros_like(parameter)
                state["step"] += 1
                adam_update(parameter, gradient, state["exp_avg"], state["exp_avg_sq"], lr=group["lr"],
                            weight_decay=group["weight_decay"], betas=group["betas"], eps=group["eps"],
                            step=int(state["step"]), rounding=rounding, key=precision["master_rounding_seed"],
                            maximize=group.get("maximize", False))
                taken.append((parameter, gradient))
                parameter.grad = None
            elif type(optimizer) is torch.optim.SGD:
                assert rounding == "nearest"
                group["foreach"] = False                # the single-tensor path accepts mixed dtypes
    return taken


class _MasterWeights:
    """One binding of (model, optimizer): `pairs` holds (model parameter, master, owning Linear or None)."""

    def __init__(self, model, optimizer):
        assert not optimizer.state, "Bind the optimizer before its first step or load_state_dict."
        policy = settings()
        self.master_dtype = policy["master_weight_dtype"]
        self.gradient_dtype = policy["gradient_dtype"] or torch.float32
        self.rounding, self.seed = policy["master_rounding"], policy["master_rounding_seed"]
        self.optimizer = optimizer
        self.pairs, self.active = [], []
        owner = {id(layer.weight): layer for layer in model.modules() if isinstance(layer, Linear)}
        master_of = {}
        for group in optimizer.param_groups:
            if isinstance(optimizer, MatrixOptimizer):
                group["master_rounding"], group["master_rounding_seed"] = self.rounding, self.seed
            for slot, param in enumerate(group["params"]):
                param.grad_dtype = self.gradient_dtype
                if id(param) not in master_of:
                    master_of[id(param)] = self._adopt(param, owner.get(id(param)))
                group["params"][slot] = master_of[id(param)]
        if isinstance(optimizer, MatrixOptimizer):
            optimizer._partition = None
        optimizer.register_step_pre_hook(self.before_step)
        optimizer.register_step_post_hook(self.after_step)
        optimizer.register_state_dict_post_hook(self.save_masters)
        optimizer.register_load_state_dict_pre_hook(self.load_masters)
        optimizer.register_load_state_dict_post_hook(self.after_load)
        self._stock_zero_grad = optimizer.zero_grad
        optimizer.zero_grad = self.zero_grad

    def _adopt(self, param, layer):
        """The master for one model parameter (viola/optim/master_weights.py:66-87)."""
        if layer is not None and layer.weight_dtype == "fp8":
            assert self.master_dtype is not None, "Disabling the master requires BF16/FP16/FP32 weight storage."
            # a module restored from a model-only checkpoint has no initial weight left: start from its codes
            source = layer._initial_weight if layer._initial_weight is not None else layer.dequantize_weight()
            master = nn.Parameter(source.to(self.master_dtype), requires_grad=param.requires_grad)
        elif self.master_dtype is not None and param.dtype != self.master_dtype:
            master = nn.Parameter(param.detach().to(self.master_dtype), requires_grad=param.requires_grad)
        else:
            master = param
        if layer is not None:
            layer._initial_weight = None
            layer._master_ref = weakref.ref(master)
        master.grad_dtype = self.gradient_dtype
        self.pairs.append((param, master, layer))
        return master

    def zero_grad(self, set_to_none=True):
        self._stock_zero_grad(set_to_none=set_to_none)
        for param, master, _ in self.pairs:
            if param is master or param.grad is None:
                continue
            if set_to_none:
                param.grad = None
            else:
                param.grad.detach_()
                param.grad.zero_()

    @torch.no_grad()
    def before_step(self, optimizer, args, kwargs):
        assert len(args) == 1 and kwargs.get("closure") is None, \
            "The master binding uses explicit forward/backward, without an optimizer closure."
        self.active = []
        for param, master, layer in self.pairs:
            if param.grad is not None:
                master.grad = param.grad            # the same accumulator: no second gradient buffer
                self.active.append((param, master, layer, param.grad))
        step_mixed_adamw(optimizer, dict(master_rounding=self.rounding, master_rounding_seed=self.seed))

    @torch.no_grad()
    def after_step(self, optimizer, args, kwargs):
        skipped = isinstance(optimizer, MatrixOptimizer) and optimizer.step_was_skipped
        for param, master, layer, gradient in self.active:
            if not skipped:
                if layer is not None:
                    layer.refresh_weight(master)
                elif param is not master:
                    param.copy_(master)
            if param is master:
                param.grad = gradient               # step_mixed_adamw may have hidden it from the stock step
            else:
                master.grad = None
        self.active.clear()

    def save_masters(self, optimizer, state):
        # aliased masters are the model's own parameters and travel with the model checkpoint
        state["viola_masters"] = dict(weights=[None if master is param else master.detach() for param, master, _ in self.pairs],
                                      gradient_dtype=self.gradient_dtype, master_dtype=self.master_dtype,
                                      rounding=self.rounding, seed=self.seed)

    @torch.no_grad()
    def load_masters(self, optimizer, state):
        state = dict(state)
        saved = state.pop("viola_masters")
        assert saved["master_dtype"] == self.master_dtype and saved["gradient_dtype"] == self.gradient_dtype
        assert len(saved["weights"]) == len(self.pairs)
        self.rounding, self.seed = saved["rounding"], saved["seed"]
        for (_, master, _), value in zip(self.pairs, saved["weights"]):
            if value is not None:
                master.copy_(value)
        return state

    @torch.no_grad()
    def after_load(self, optimizer):
        # FP8 payloads and scales come back verbatim with the model's state dict; quantizing the master again here
        # would be a second rounding of state that is already exact
        for param, master, layer in self.pairs:
            if param is not master and (layer is None or layer.weight_dtype != "fp8"):
                param.copy_(master)
        optimizer.zero_grad()


def bind_optimizer(model, optimizer):
    """Install the master write-back hooks on `optimizer` and return it (viola/optim/master_weights.py:166-179).

    Move the model to the GPU and call the precision setters (`set_master_weight_dtype`, `set_gradient_dtype`) first;
    save and load both the model's and the optimizer's state dict for an exact resume.
    `set_master_weight_dtype(None)` makes the model parameter its own master (BF16/FP16/FP32 storage only)."""
    assert not hasattr(optimizer, "_viola_linear_masters"), "This optimizer is already bound."
    optimizer._viola_linear_masters = _MasterWeights(model, optimizer)
    return optimizer
