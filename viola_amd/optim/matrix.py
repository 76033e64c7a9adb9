"""Base class for optimizers whose update needs a whole logical matrix
(viola/optim/matrix.py:14-135, plain-tensor path). One GPU: DTensor parameters, owner
gather/scatter and mesh all-reduces of the reference are not part of this build."""

import torch


class MatrixOptimizer(torch.optim.Optimizer):
    """Subclasses implement `_step_local(parameter, gradient, state, group, index)` on full tensors;
    `index` is the parameter's stable position over all groups."""

    def __init__(self, params, defaults, *, shard_state=True, skip_nonfinite=False):
        self.shard_state = shard_state
        self.skip_nonfinite = skip_nonfinite
        self.step_was_skipped = False
        self._partition = None
        super().__init__(params, defaults)
        self.register_load_state_dict_pre_hook(self._before_load)
        self.register_load_state_dict_post_hook(self._after_load)

    def _step_local(self, parameter, gradient, state, group, index):
        raise NotImplementedError

    def _has_nonfinite(self):
        return any(not torch.isfinite(p.grad).all() for g in self.param_groups for p in g["params"] if p.grad is not None)

    @torch.no_grad()
    def step(self, closure=None):
        self.step_was_skipped = False
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        if self.skip_nonfinite and self._has_nonfinite():
            self.step_was_skipped = True
            return loss
        index = 0
        work = []
        for group in self.param_groups:
            stable = group.get("viola_parameter_indices")
            for local, param in enumerate(group["params"]):
                position = stable[local] if stable is not None else index
                index += 1
                if param.grad is None:          # no decay, no state advance for a missing gradient
                    continue
                work.append((param, param.grad, self.state[param], group, position))
        self._step_all(work)
        return loss

    def _step_all(self, work):
        """All (parameter, gradient, state, group, index) of one step; subclasses may batch equal shapes."""
        for item in work:
            self._step_local(*item)

    # Optimizer.load_state_dict casts floating state tensors to the parameter's dtype, which would
    # destroy the raw uint8 FP8 payload / fp32 scales / bf16 moments. Tensors are therefore set
    # aside before the stock loader runs and put back verbatim afterwards.
    def _before_load(self, optimizer, saved):
        saved = dict(saved)
        is_tensor = lambda v: isinstance(v, torch.Tensor)
        self._held = {pid: {k: v for k, v in state.items() if is_tensor(v)} for pid, state in saved["state"].items()}
        self._held_groups = saved["param_groups"]
        saved["state"] = {pid: {k: v for k, v in state.items() if not is_tensor(v)} for pid, state in saved["state"].items()}
        return saved

    def _after_load(self, optimizer):
        for old, group in zip(self._held_groups, self.param_groups):
            for pid, param in zip(old["params"], group["params"]):
                for name, value in self._held.get(pid, {}).items():
                    self.state[param][name] = value.to(device=param.device)
        del self._held, self._held_groups
