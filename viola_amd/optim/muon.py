"""FP8Muon: Muon with one e4m3 momentum buffer + FP32 tile scales per matrix, AdamW for vectors
(viola/optim/muon.py:14-141). Every arithmetic step is a HIP kernel: fused momentum/codec,
Newton-Schulz GEMM chain, weight update, AdamW."""

import os
import warnings

import torch

from .matrix import MatrixOptimizer
from ..precision import _resolve as _dtype, settings
from ._kernels import adam_update, adam_update_many, momentum_update, momentum_update_many, weight_update_many, state_sizes, weight_update
from ._orthogonalize import METHODS

_MODES = {"fast": (256, 3), "balanced": (256, 5), "stable": (128, 5)}
_MASK63 = (1 << 63) - 1


def _shape(param, group):
    """Conv filters flatten to [out, -1]; batched=True keeps the leading dims as independent matrices."""
    return tuple(param.shape) if group["batched"] else (param.shape[0], param.numel() // param.shape[0])


def _use_muon(param, group):
    return param.ndim >= 2 if group["use_muon"] is None else group["use_muon"]


class FP8Muon(MatrixOptimizer):
    """Matrices use Muon, vectors AdamW; `use_muon=False` on a group forces AdamW (embeddings, heads).

    State per matrix: {"step", "momentum_q" uint8 payload, "momentum_scale" fp32}; per vector:
    {"step", "exp_avg", "exp_avg_sq"}.
    """

    def __init__(self, params, lr=1e-3, *, weight_decay=0., momentum=.95, nesterov=True, mode="balanced",
                 granularity="tile", tile_size=None, block_shape=None, rounding="nearest", rounding_seed=0,
                 ns_steps=None, ns_method="standard", ns_backend="torch", ns_autotune=True,
                 adjust_lr_fn="match_rms_adamw", betas=(.9, .95), eps=1e-8, adam_state_dtype="fp32",
                 skip_nonfinite=False, shard_state=True):
        tile_default, steps_default = _MODES[mode]
        policy = settings()
        defaults = dict(
            lr=lr, weight_decay=weight_decay, momentum=momentum, nesterov=nesterov, use_muon=None, batched=False,
            granularity=granularity, tile_size=tile_default if tile_size is None else tile_size,
            block_shape=(16, 16) if block_shape is None else tuple(block_shape),
            rounding=rounding, rounding_seed=rounding_seed,
            ns_steps=steps_default if ns_steps is None else ns_steps, ns_method=ns_method,
            ns_backend=ns_backend, ns_autotune=ns_autotune, adjust_lr_fn=adjust_lr_fn, betas=betas, eps=eps,
            adam_state_dtype=_dtype(adam_state_dtype), master_rounding=policy["master_rounding"],
            master_rounding_seed=policy["master_rounding_seed"])
        self.observer = None
        self._workspace = {}
        self._streams = {}
        self._adam_tables = {}
        self._bucket_tables = {}
        super().__init__(params, defaults, shard_state=shard_state, skip_nonfinite=skip_nonfinite)

    def add_param_group(self, group):
        super().add_param_group(group)
        group = self.param_groups[-1]
        assert group["lr"] >= 0 and group["weight_decay"] >= 0
        assert 0 <= group["momentum"] < 1 and group["ns_steps"] > 0
        assert group["ns_method"] in METHODS
        # both backends of the reference ("torch" = torch.compile, "tilelang") map to the HIP GEMM chain
        assert group["ns_backend"] in ("torch", "tilelang", "hip")
        assert group["adjust_lr_fn"] in ("original", "match_rms_adamw")
        assert group["granularity"] in ("tile", "block") and group["rounding"] in ("nearest", "stochastic")
        assert 0 <= group["rounding_seed"] < (1 << 63)
        assert group["tile_size"] in (64, 128, 256, 512, 1024)
        assert len(group["block_shape"]) == 2 and all(v in (8, 16, 32, 64) for v in group["block_shape"])
        group["adam_state_dtype"] = _dtype(group["adam_state_dtype"])
        grad_dtype = settings()["gradient_dtype"]
        ragged = []
        for param in group["params"]:
            if grad_dtype is not None:
                param.grad_dtype = grad_dtype
            if _use_muon(param, group):
                assert param.ndim >= 2
                shape = _shape(param, group)
                if group["granularity"] == "tile":
                    partial = shape[-1] % group["tile_size"]
                else:
                    partial = shape[-2] % group["block_shape"][0] or shape[-1] % group["block_shape"][1]
                if partial:
                    ragged.append(shape)
        if ragged and int(os.environ.get("RANK", "0")) == 0:
            warnings.warn(f"FP8Muon: {len(ragged)} matrices have partial {group['granularity']} groups "
                          f"(e.g. {ragged[:3]}). Original matrix shapes are kept; edge groups use valid elements.",
                          stacklevel=3)

    def _momentum(self, param, grad, state, group, key, out=None):
        """Advance the FP8 momentum in place and return the bf16 update as a matrix view of the workspace
        (or of `out`, a flat bf16 buffer of the parameter's size)."""
        shape = _shape(param, group)
        quant = dict(granularity=group["granularity"], tile_size=group["tile_size"], block_shape=group["block_shape"])
        if "momentum_q" not in state:
            payload, scales = state_sizes(shape, **quant)
            state["momentum_q"] = torch.zeros(payload, device=param.device, dtype=torch.uint8)
            state["momentum_scale"] = torch.ones(scales, device=param.device, dtype=torch.float32)
        if out is None:
            out = self._workspace.get(param.device)
            if out is None or out.numel() < param.numel():
                out = self._workspace[param.device] = torch.empty(param.numel(), device=param.device, dtype=torch.bfloat16)
        matrix = out[:param.numel()].view(shape)
        q, scale = state["momentum_q"], state["momentum_scale"]
        before = (q.clone(), scale.clone()) if self.observer is not None else None
        momentum_update(grad, q, scale, q, scale, matrix.view(-1), beta=group["momentum"], nesterov=group["nesterov"],
                        matrix_shape=shape, rounding=group["rounding"], rounding_step=state["step"], rounding_key=key,
                        **quant)
        if self.observer is not None:
            self.observer.momentum(param, grad, *before, q, scale, matrix, group, 1., quant)
        return matrix

    # Equal-shaped matrices of one step go through Newton-Schulz as ONE batched GEMM chain: every matrix of
    # the batch sees exactly the arithmetic it would see alone, and the launches fill the GPU.
    _BATCH_ELEMENTS = 1 << 28

    def _step_all(self, work):
        if self.observer is not None:
            return super()._step_all(work)
        buckets, vectors, ready = {}, {}, []
        for item in work:
            param, grad, state, group, index = item
            if not _use_muon(param, group):
                state.setdefault("step", 0)
                key = (param.device, param.dtype, grad.dtype, group["adam_state_dtype"], group["lr"], group["weight_decay"],
                       tuple(group["betas"]), group["eps"], state["step"], group["master_rounding"])
                vectors.setdefault(key, []).append(item)
                continue
            shape = _shape(param, group)
            key = (shape, param.device, group["ns_method"], group["ns_steps"])
            bucket = buckets.setdefault(key, [])
            bucket.append(item)
            if (len(bucket) + 1) * param.numel() > self._BATCH_ELEMENTS:
                ready.append(buckets.pop(key))
        ready.extend(buckets.values())
        self._step_buckets(ready)
        for key, bucket in vectors.items():
            self._step_vectors(key, bucket)

    # The chains of different buckets are independent, and a single chain leaves the GPU partly idle at every launch
    # boundary (a Newton-Schulz GEMM of 28 matrices is ~590 tiles for 512 tile slots: its second round is nearly
    # empty). Buckets therefore go to up to _LANES streams of default priority, each with its own workspace, so the
    # blocks of one chain fill the tails of the others; the caller's stream waits for all of them at the end.
    _LANES = 4

    def _step_buckets(self, ready):
        devices = {bucket[0][0].device for bucket in ready}
        # buckets of one shape and size (a shape split because it exceeds _BATCH_ELEMENTS) each keep their own pointer
        # tables: a table must not be rewritten while another stream's launch still reads it
        seen, ordinals = {}, []
        for bucket in ready:
            key = (_shape(bucket[0][0], bucket[0][3]), len(bucket))
            ordinals.append(seen.get(key, 0))
            seen[key] = ordinals[-1] + 1
        if len(ready) < 2 or self._LANES < 2 or len(devices) != 1 or not ready[0][0][0].is_cuda:
            for bucket, ordinal in zip(ready, ordinals):
                self._step_bucket(bucket, ordinal=ordinal)
            return
        device = ready[0][0][0].device
        lanes = self._streams.setdefault(device, [])
        while len(lanes) < min(self._LANES, len(ready)):
            lanes.append(torch.cuda.Stream(device=device))
        main = torch.cuda.current_stream(device)
        start = torch.cuda.Event()
        start.record(main)
        # largest chains first, one lane after the other: the long ones start together and the short ones pack behind
        order = sorted(range(len(ready)), key=lambda i: -len(ready[i]) * ready[i][0][0].numel())
        for slot, i in enumerate(order):
            lane = slot % len(lanes)
            lanes[lane].wait_event(start)
            with torch.cuda.stream(lanes[lane]):
                self._step_bucket(ready[i], lane=lane, ordinal=ordinals[i])
        for stream in lanes:
            done = torch.cuda.Event()
            done.record(stream)
            main.wait_event(done)

    # Vectors (biases, norms, modulation tables) are a few thousand elements each: those that share dtypes,
    # hyper-parameters and step count take AdamW in one launch over a table of their pointers.
    def _step_vectors(self, key, bucket):
        if len(bucket) == 1 or any(not item[1].is_contiguous() or not item[0].is_contiguous() for item in bucket):
            for item in bucket:
                self._step_local(*item)
            return
        items = []
        for param, grad, state, group, index in bucket:
            assert param.is_cuda and not grad.is_sparse
            assert param.dtype in (torch.float32, torch.bfloat16, torch.float16), \
                "Bind FP8 modules with viola.optim.bind_optimizer before stepping."
            if "exp_avg" not in state:
                state["exp_avg"] = torch.zeros_like(param, dtype=group["adam_state_dtype"])
                state["exp_avg_sq"] = torch.zeros_like(param, dtype=group["adam_state_dtype"])
            master_key = (group["master_rounding_seed"] + index * 0x517CC1B727220A95) & _MASK63
            items.append((param, grad, state["exp_avg"], state["exp_avg_sq"], master_key, 0))
        param, grad, state, group, index = bucket[0]
        adam_update_many(items, lr=group["lr"], weight_decay=group["weight_decay"], betas=group["betas"], eps=group["eps"],
                         step=state["step"] + 1, rounding=group["master_rounding"],
                         cache=self._adam_tables.setdefault(key[:4] + (len(bucket),), {}))
        for _, _, state, _, _ in bucket:
            state["step"] += 1

    def _step_bucket(self, bucket, lane=0, ordinal=0):
        param, _, _, group, _ = bucket[0]
        shape = _shape(param, group)
        count = param.numel()
        work = self._workspace.get((param.device, lane))
        if work is None or work.numel() < len(bucket) * count:
            work = self._workspace[(param.device, lane)] = torch.empty(len(bucket) * count, device=param.device, dtype=torch.bfloat16)
        # keyed by lane as well: a table is only ever rewritten on the stream whose launches read it
        tables = self._bucket_tables.setdefault((shape, param.device, len(bucket), ordinal, lane), ({}, {}))
        # one launch for the momentum of the whole bucket when its members share the recipe, else one per matrix
        uniform = lambda *names: all(all(item[3][name] == group[name] for name in names) for item in bucket)
        items = []
        for slot, (param, grad, state, group_, index) in enumerate(bucket):
            assert param.is_cuda and not grad.is_sparse
            assert param.dtype in (torch.float32, torch.bfloat16, torch.float16), \
                "Bind FP8 modules with viola.optim.bind_optimizer before stepping."
            state.setdefault("step", 0)
            if "momentum_q" not in state:
                payload, scales = state_sizes(shape, granularity=group_["granularity"], tile_size=group_["tile_size"],
                                              block_shape=group_["block_shape"])
                state["momentum_q"] = torch.zeros(payload, device=param.device, dtype=torch.uint8)
                state["momentum_scale"] = torch.ones(scales, device=param.device, dtype=torch.float32)
            key = (group_["rounding_seed"] + index * 0x9E3779B97F4A7C15) & _MASK63
            items.append((grad, state["momentum_q"], state["momentum_scale"], work[slot * count:(slot + 1) * count], key))
        step = bucket[0][2]["step"]
        together = (group["granularity"] == "tile" and all(item[2]["step"] == step for item in bucket)
                    and uniform("granularity", "tile_size", "momentum", "nesterov", "rounding")
                    and momentum_update_many(items, beta=group["momentum"], tile_size=group["tile_size"],
                                             nesterov=group["nesterov"], rounding=group["rounding"], rounding_step=step,
                                             cache=tables[0]))
        if not together:
            for (param, grad, state, group_, index), item in zip(bucket, items):
                self._momentum(param, grad, state, group_, item[4], out=item[3])
        stacked = work[:len(bucket) * count].view(len(bucket), -1, *shape[-2:])
        updates = METHODS[group["ns_method"]](stacked, steps=group["ns_steps"]).reshape(len(bucket), count)
        rows, cols = shape[-2:]
        scale_of = lambda g: .2 * max(rows, cols) ** .5 if g["adjust_lr_fn"] == "match_rms_adamw" else max(1., rows / cols) ** .5
        together = (uniform("lr", "weight_decay", "adjust_lr_fn") and all(item[3]["master_rounding"] == "nearest" or
                                                                          item[0].dtype == torch.float32 for item in bucket)
                    and weight_update_many([(item[0], updates[slot]) for slot, item in enumerate(bucket)], group["lr"],
                                           group["weight_decay"], update_scale=scale_of(group), cache=tables[1]))
        for slot, (param, grad, state, group_, index) in enumerate(bucket):
            if not together:
                master_key = (group_["master_rounding_seed"] + index * 0x517CC1B727220A95) & _MASK63
                weight_update(param, updates[slot], group_["lr"], group_["weight_decay"], update_scale=scale_of(group_),
                              rounding=group_["master_rounding"], step=state["step"], key=master_key)
            state["step"] += 1

    def _step_local(self, param, grad, state, group, index):
        key = (group["rounding_seed"] + index * 0x9E3779B97F4A7C15) & _MASK63
        master_key = (group["master_rounding_seed"] + index * 0x517CC1B727220A95) & _MASK63
        assert param.is_cuda and not grad.is_sparse
        assert param.dtype in (torch.float32, torch.bfloat16, torch.float16), \
            "Bind FP8 modules with viola.optim.bind_optimizer before stepping."
        state.setdefault("step", 0)
        if _use_muon(param, group):
            matrix = self._momentum(param, grad, state, group, key)
            orthogonalize = METHODS[group["ns_method"]]
            update = orthogonalize(matrix, steps=group["ns_steps"])
            if self.observer is not None:
                self.observer.update(param, update, group, orthogonalize)
            rows, cols = matrix.shape[-2:]
            scale = .2 * max(rows, cols) ** .5 if group["adjust_lr_fn"] == "match_rms_adamw" else max(1., rows / cols) ** .5
            weight_update(param, update, group["lr"], group["weight_decay"], update_scale=scale,
                          rounding=group["master_rounding"], step=state["step"], key=master_key)
        else:
            if "exp_avg" not in state:
                state["exp_avg"] = torch.zeros_like(param, dtype=group["adam_state_dtype"])
                state["exp_avg_sq"] = torch.zeros_like(param, dtype=group["adam_state_dtype"])
            adam_update(param, grad, state["exp_avg"], state["exp_avg_sq"], lr=group["lr"],
                        weight_decay=group["weight_decay"], betas=group["betas"], eps=group["eps"],
                        step=state["step"] + 1, rounding=group["master_rounding"], key=master_key)
        state["step"] += 1
