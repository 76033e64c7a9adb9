"""Headline benchmark on ONE MI355X: viola.nn.Linear FP8 forward+backward at 8192 x 1024 -> 4096
(e4m3, FP32 tile/block scales, bf16 outputs) in TFLOP/s, with the FP8Muon step time on the DiT-XL
parameter set, the wire codec and quantizer bandwidths, a roofline object for the dominant kernel
(the grouped-scale FP8 GEMM) and the CPU oracle timed on this host's cores.

    python bench.py --gpus 1 --steps 200 --warmup 50

Before a leg is sampled the device runs that leg's own step back to back for about 100 ms, outside the step and
warm-up counts (the reference's benchmarks warm for about 30 ms before sampling, checks/benchmark_linear.py:41-52): a
GPU that has idled through set-up needs some tens of milliseconds of work to reach its sustained clock, and a
20-step run would otherwise read that ramp instead of the steady state a training loop sees.

A step is one `y = layer(x); y.backward(dy)` including every quantize / transpose launch, inputs
resident in HBM. TFLOP/s = 6*M*K*N / t (the reference's definition, checks/benchmark_linear.py:165).
"""

import argparse
import json
import math
import os
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

M, K, N = 8192, 1024, 4096
PEAK = {"fp8_tflops": 5000.0, "bf16_tflops": 2500.0, "hbm_gbs": 8000.0}
# L2<->fabric bytes per grouped-scale GEMM launch, mean of the step's three launches (fwd, dgrad, wgrad), from two
# `rocprofv3 --pmc` runs of `bench.py --skip-cpu --skip-muon --steps 5 --warmup 3 --calibrate` (FETCH_SIZE, then WRITE_SIZE, KiB per
# dispatch), each scaled by the same counter's reading for the 256 MiB copy_scaled_kernel launch (factors 2.00 and 1.00):
# fetch (2 * 58.3 + 113.5) / 3 MB, write (2 * 41.9 + 8.4) / 3 MB. The algorithmic figure is 65 MB per launch.
GEMM_TRAFFIC_BYTES = 76.7e6 + 30.8e6
WARM_MS = 100.0


def log(message):
    """Progress on stderr (the JSON line is the only thing on stdout)."""
    print(f"[bench] {message}", file=sys.stderr, flush=True)


def device_warm(fn, target_ms=WARM_MS):
    """Run fn back to back for about target_ms of device time (probe one call, then repeat; at most 4096 calls)."""
    import torch
    fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    fn()
    end.record()
    end.synchronize()
    for _ in range(min(4096, math.ceil(target_ms / max(start.elapsed_time(end), 1e-3)))):
        fn()
    torch.cuda.synchronize()


def timed(fn, steps, warmup, warm=True):
    import torch
    if warm:
        device_warm(fn)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    begin = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - begin) * 1e3
    return max(start.elapsed_time(end), 0.0) / steps, wall / steps


def kernel_breakdown(fn, steps):
    """Second, instrumented pass: HIP events around every C-ABI call on the stream it is launched on."""
    import torch
    from viola_amd import _lib
    _lib.timeline = []
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    rows, _lib.timeline = _lib.timeline, None
    table = {}
    for name, start, end in rows:
        table.setdefault(name, []).append(start.elapsed_time(end))
    return {name: dict(launches_per_step=len(v) / steps, avg_ms=sum(v) / len(v)) for name, v in table.items()}


def linear_case():
    import torch
    import viola_amd
    torch.manual_seed(20261125)
    viola_amd.set_gradient_dtype("bf16")
    layer = viola_amd.nn.Linear(K, N, device="cuda", dtype=torch.bfloat16, scaling="grouped", forward_dtype="e4m3",
                                backward_dtype="e4m3", mode="memory", weight_dtype="fp8")
    viola_amd.precision._settings["gradient_dtype"] = None
    x = torch.randn(M, K).bfloat16().cuda().requires_grad_()
    dy = (torch.randn(M, N) * 1e-2).bfloat16().cuda()

    def step():
        x.grad = layer.weight.grad = layer.bias.grad = None
        layer(x).backward(dy)

    return layer, x, dy, step


def muon_case(method="standard", rounding="nearest", blocks=28, d=1152):
    """DiT-XL-shaped parameter set: per block qkv [3d, d], proj [d, d], fc1 [4d, d], fc2 [d, 4d] + vectors."""
    import torch
    import viola_amd
    torch.manual_seed(7)
    params = []
    for _ in range(blocks):
        for shape in ((3 * d, d), (d, d), (4 * d, d), (d, 4 * d), (3 * d,), (d,), (4 * d,), (d,), (d,), (d,)):
            p = torch.nn.Parameter(torch.randn(*shape, device="cuda") * .02)
            p.grad = torch.randn_like(p) * 1e-3
            params.append(p)
    opt = viola_amd.optim.FP8Muon(params, lr=1e-3, weight_decay=.01, mode="balanced", tile_size=256, ns_method=method,
                                  rounding=rounding, rounding_seed=42, adjust_lr_fn="match_rms_adamw")
    elements = sum(p.numel() for p in params if p.ndim >= 2)
    return opt, params, elements


def _median_time(fn, repeats=3):
    fn()                                                                          # warm-up
    times = []
    for _ in range(repeats):
        begin = time.perf_counter()
        fn()
        times.append(time.perf_counter() - begin)
    return statistics.median(times)


def _bounded(fn, seconds):
    """fn() in a daemon thread; its result, or None when it has not returned after `seconds`."""
    import threading
    box = []
    worker = threading.Thread(target=lambda: box.append(fn()), daemon=True)
    worker.start()
    worker.join(seconds)
    return box[0] if box else None


def cpu_baseline():
    """The oracle's Linear forward+backward (dequantized-FP32 matmuls) on this host's cores, one full C2 step, plus
    the other CPU legs (eager Newton-Schulz on one 1024 x 4096 matrix, the wire codec on one 25 MB bucket, the momentum
    codec on one qkv-sized matrix) under `others`."""
    import torch
    from oracle import comm as oc, grouped as og, linear as ol, ns as ons, optim as oo
    torch.manual_seed(20261125)
    # threads: this job's share of the host (the GPU boxes give a one-GPU job 16 of the host's cores, whatever
    # os.cpu_count() reports for the whole machine); both numbers go into the record
    host_cpus = os.cpu_count() or 1
    cores = min(host_cpus, 16)
    torch.set_num_threads(cores)
    x = torch.randn(M, K).bfloat16()
    dy = (torch.randn(M, N) * 1e-2).bfloat16()
    w = torch.empty(N, K).uniform_(-1 / 32, 1 / 32)
    qw, sw = og.quantize(w, torch.float8_e4m3fn, (32, 32))
    w_real = og.dequantize(qw, sw, (32, 32))
    best = _median_time(lambda: ol.linear(x, w_real, torch.zeros(N), dy), repeats=2)
    log(f"cpu linear: {best * 1e3:.0f} ms")
    others = {}
    n = 6553600
    bucket = torch.randn(n) * 1e-3
    t_pack = _median_time(lambda: oc.pack(bucket, 1, n // 256, 256, torch.float8_e4m3fn))
    packet = oc.pack(bucket, 1, n // 256, 256, torch.float8_e4m3fn)
    t_unpack = _median_time(lambda: oc.unpack(packet, n, 256, torch.float8_e4m3fn))
    others["comm_codec_25MB"] = dict(pack_ms=t_pack * 1e3, unpack_ms=t_unpack * 1e3, pack_gbs=5.016 * n / t_pack / 1e9,
                                     unpack_gbs=5.016 * n / t_unpack / 1e9, sample="one 6 553 600-element fp32 bucket, tile 256")
    shape = (3456, 1152)
    grad = torch.randn(shape) * 1e-3
    count = shape[0] * shape[1]
    q0, s0 = torch.zeros(count, dtype=torch.uint8), torch.ones(count // 256)
    t_mom = _median_time(lambda: oo.momentum_update(grad, q0, s0, beta=.95, shape=shape))
    others["momentum_3456x1152"] = dict(ms=t_mom * 1e3, gbs=8.03 * count / t_mom / 1e9, sample="one qkv-sized matrix, tile 256, nearest")
    # the eager Newton-Schulz recipes last, each under a time limit: a host without fast half-precision matmuls
    # can take minutes (or not come back) on them; a leg that misses its limit is reported as such
    g = torch.randn(1024, 4096)
    small = torch.randn(256, 1024)
    small_flops = {"standard": 5 * (4 * 256 ** 2 * 1024 + 2 * 256 ** 3), "gram": 8 * 256 ** 2 * 1024 + 28 * 256 ** 3}
    for method in ("standard", "gram"):
        # a 256 x 1024 matrix first (1/64 of the work): the fp16 chain of `gram` runs on the host's scalar half-precision
        # matmul and does not finish the full matrix within the limit; its full-size figure is then this one scaled
        t_small = _bounded(lambda: _median_time(lambda: ons.METHODS[method](small, steps=5)), 30.0)
        if t_small is None:
            others[f"ns_{method}_256x1024"] = dict(ms=None, tflops=None, sample="one 256 x 1024 matrix, 5 steps, eager torch on the host: not finished within 30 s")
            break                                                                 # its threads may still be busy
        others[f"ns_{method}_256x1024"] = dict(ms=t_small * 1e3, tflops=small_flops[method] / t_small / 1e12,
                                               sample="one 256 x 1024 matrix, 5 steps, eager torch on the host")
        scaled_ms = t_small * 1e3 * NS_C1_FLOPS[method] / small_flops[method]
        if scaled_ms > 20e3:
            log(f"cpu ns {method}: 256 x 1024 in {t_small * 1e3:.0f} ms; full size not run (about {scaled_ms / 1e3:.0f} s by flop count)")
            others[f"ns_{method}_1024x4096"] = dict(ms=scaled_ms, tflops=small_flops[method] / t_small / 1e12, scaled=True,
                                                   sample="not run: the 256 x 1024 time scaled by the flop ratio (x%.1f)" % (NS_C1_FLOPS[method] / small_flops[method]))
            continue
        t = _bounded(lambda: _median_time(lambda: ons.METHODS[method](g, steps=5)), 60.0)
        log(f"cpu ns {method}: {'no result within 60 s' if t is None else f'{t * 1e3:.0f} ms'}")
        if t is None:
            others[f"ns_{method}_1024x4096"] = dict(ms=scaled_ms, tflops=small_flops[method] / t_small / 1e12, scaled=True,
                                                   sample="not finished within 60 s: the 256 x 1024 time scaled by the flop ratio")
            break
        others[f"ns_{method}_1024x4096"] = dict(ms=t * 1e3, tflops=NS_C1_FLOPS[method] / t / 1e12, scaled=False,
                                               sample="one matrix, 5 steps, eager torch on the host")
    return dict(value=6 * M * K * N / best / 1e12, unit="TFLOP/s", cores=cores, host_cpus=host_cpus,
                cores_note=f"{cores} torch threads = this job's share of the host's {host_cpus} logical CPUs", kind="port",
                sample=f"one full {M}x{K}->{N} forward+backward per run, median of 2 after 1 warm-up "
                       f"({best * 1e3:.0f} ms per step)", others=others)


# Newton-Schulz on one 1024 x 4096 matrix, 5 steps: standard 5 (4 m^2 n + 2 m^3), gram 8 m^2 n + 28 m^3
NS_C1_FLOPS = {"standard": 5 * (4 * 1024 ** 2 * 4096 + 2 * 1024 ** 3), "gram": 8 * 1024 ** 2 * 4096 + 28 * 1024 ** 3}


def ns_single_case(steps, warmup):
    """Config 1: one [1024, 4096] fp32 gradient through each Newton-Schulz method, with the per-launch breakdown."""
    import torch
    from viola_amd.optim._orthogonalize import METHODS
    torch.manual_seed(1)
    g = torch.randn(1024, 4096, device="cuda")
    out = {}
    for method in ("standard", "gram"):
        fn = lambda: METHODS[method](g, steps=5)
        ms, _ = timed(fn, steps, warmup)
        b = kernel_breakdown(fn, min(steps, 20))
        gemm_ms = b["viola_ns_gemm"]["avg_ms"] * b["viola_ns_gemm"]["launches_per_step"]
        out[method] = dict(ms=ms, tflops=NS_C1_FLOPS[method] / (ms * 1e-3) / 1e12, gemm_launches=b["viola_ns_gemm"]["launches_per_step"],
                           gemm_ms=gemm_ms, gemm_tflops=NS_C1_FLOPS[method] / (gemm_ms * 1e-3) / 1e12,
                           gemm_frac_peak=NS_C1_FLOPS[method] / (gemm_ms * 1e-3) / 1e12 / PEAK["bf16_tflops"])
    out["note"] = ("gemm_ms sums HIP-event pairs around 15-18 launches of 5-18 us each in a second, instrumented pass: the pairs' own "
                   "cost makes it exceed ms, the chain timed without them")
    return out


def varlen_case(steps, warmup):
    """Config 4: 16 groups sharing K = 4096, N = 1024, 32768 rows split by a seeded multinomial with one empty and
    one 3-row group; forward + backward of the variable-group linear, 3 x 2 x 32768 x 4096 x 1024 flop."""
    import torch
    from viola_amd.nn import _varlen as v
    groups, k, n, total = 16, 4096, 1024, 32768
    generator = torch.Generator().manual_seed(6)
    counts = torch.bincount(torch.multinomial(torch.ones(groups) / groups, total, replacement=True, generator=generator), minlength=groups)
    counts[3] += counts[5] - 3
    counts[5] = 3
    counts[7] += counts[9]
    counts[9] = 0
    counts = counts.tolist()
    torch.manual_seed(7)
    x = torch.randn(total, k, device="cuda").bfloat16().requires_grad_()
    dy = torch.randn(total, n, device="cuda").bfloat16()
    experts = v.GroupedExperts(groups, k, n, device="cuda")

    def step():
        x.grad = experts.weight.grad = None
        experts(x, counts).backward(dy)
    ms, wall = timed(step, steps, warmup)
    flops = 3 * 2 * total * k * n
    b = kernel_breakdown(step, min(steps, 10))
    gemm_ms = sum(v_["avg_ms"] * v_["launches_per_step"] for name, v_ in b.items() if "gemm" in name)
    return dict(step_ms=ms, wall_ms=wall, flops=flops, tflops=flops / (ms * 1e-3) / 1e12, counts=counts, kernels=b,
                gemm_ms=gemm_ms, gemm_tflops=flops / (gemm_ms * 1e-3) / 1e12, gemm_frac_fp8_peak=flops / (gemm_ms * 1e-3) / 1e12 / PEAK["fp8_tflops"])


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=200)
    parser.add_argument("--warmup", type=int, default=50)
    parser.add_argument("--skip-cpu", action="store_true", help="leave out the CPU baseline leg")
    parser.add_argument("--skip-muon", action="store_true", help="leave out the FP8Muon / codec legs")
    parser.add_argument("--skip-mlp", action="store_true", help="leave out the gated MLP leg")
    parser.add_argument("--skip-varlen", action="store_true", help="leave out the variable-group (MoE) leg")
    parser.add_argument("--muon-streams", type=int, default=0, help="streams FP8Muon.step spreads its shape buckets over "
                        "(0: the optimizer's default; 1 keeps a kernel trace free of overlapping launches)")
    parser.add_argument("--calibrate", action="store_true",
                        help="also launch copy_scaled_kernel once over 64 Mi floats (256 MiB read, 256 MiB written): "
                             "the known-size kernel that FETCH_SIZE / WRITE_SIZE readings are scaled by")
    parser.add_argument("--only", default="", help="comma-separated legs to run besides the Linear step (muon, bound, recipes, mlp, "
                        "ns1, varlen); default: all that are not skipped. For profiling one leg at a time")
    args = parser.parse_args()
    skipped = {"muon": args.skip_muon, "bound": args.skip_muon, "recipes": args.skip_muon, "ns1": args.skip_muon,
               "mlp": args.skip_mlp, "varlen": args.skip_varlen}
    only = {leg for leg in args.only.split(",") if leg}
    assert only <= set(skipped), f"unknown leg in --only: {sorted(only - set(skipped))}"

    def want(leg):
        return leg in only if only else not skipped[leg]
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    import torch
    from viola_amd import _lib
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    _lib.library()

    log("linear step")
    layer, x, dy, step = linear_case()
    ms, wall_ms = timed(step, args.steps, args.warmup)
    flops = 6 * M * K * N
    value = flops / (ms * 1e-3) / 1e12
    breakdown = kernel_breakdown(step, args.steps)
    gemm = breakdown["viola_group_gemm"]
    gemm_tflops = 2 * M * K * N / (gemm["avg_ms"] * 1e-3) / 1e12
    roofline = dict(bound="mfma", kernel="group_gemm_fast (viola_group_gemm: fwd, dgrad, wgrad)",
                    achieved=gemm_tflops, peak=PEAK["fp8_tflops"], unit="TFLOP/s", frac=gemm_tflops / PEAK["fp8_tflops"],
                    avg_launch_ms=gemm["avg_ms"], traffic=GEMM_TRAFFIC_BYTES,
                    traffic_source="stored calibration (two rocprofv3 --pmc runs, profiles/linear_step_8192x1024x4096_hbm_traffic.txt), not read in this run")
    quant = {}
    if "viola_group_quantize_dual" in breakdown:
        # X [M, K] and dY [M, N] each once per step: 4.25 B per element (bf16 in, two FP8 layouts + scales out)
        per_step = 4.25 * (M * K + M * N) / 2
        q = breakdown["viola_group_quantize_dual"]
        quant = dict(kernel="quantize_dual16_tile64 (row-wise + transposed + column partials, one read)", avg_ms=q["avg_ms"],
                     gbs=per_step / (q["avg_ms"] * 1e-3) / 1e9, frac_hbm=per_step / (q["avg_ms"] * 1e-3) / 1e9 / PEAK["hbm_gbs"])

    extra = {}
    if want("muon"):
        for method in ("standard", "gram"):
            log(f"FP8Muon step, {method}")
            opt, params, elements = muon_case(method)
            if args.muon_streams:
                opt._LANES = args.muon_streams
            step_ms, step_wall = timed(opt.step, 5, 3)
            # the step runs its shape buckets on several streams; for per-launch durations that do not overlap each
            # other the instrumented pass (and one timing next to it) keeps them on one
            lanes, opt._LANES = opt._LANES, 1
            serial_ms, _ = timed(opt.step, 3, 1)
            b = kernel_breakdown(opt.step, 2)
            ns_flops = 0.0
            for p in params:
                if p.ndim >= 2:
                    m_, n_ = min(p.shape), max(p.shape)
                    if method == "standard":
                        ns_flops += 5 * (4 * m_ * m_ * n_ + 2 * m_ ** 3)
                    else:
                        ns_flops += 5 * 6 * m_ ** 3 if m_ == n_ else 8 * m_ * m_ * n_ + 28 * m_ ** 3
            ns_ms = b["viola_ns_gemm"]["avg_ms"] * b["viola_ns_gemm"]["launches_per_step"]
            mom = b.get("viola_momentum_update_table") or b["viola_momentum_update"]
            upd = b.get("viola_weight_update_table") or b["viola_weight_update"]
            extra[f"muon_{method}"] = dict(step_ms=step_ms, step_wall_ms=step_wall, streams=lanes, step_one_stream_ms=serial_ms,
                                           muon_elements=elements,
                                           ns_gemm_ms=ns_ms, ns_tflops=ns_flops / (ns_ms * 1e-3) / 1e12,
                                           ns_frac_bf16_peak=ns_flops / (ns_ms * 1e-3) / 1e12 / PEAK["bf16_tflops"],
                                           momentum_gbs=8.03 * elements / (mom["avg_ms"] * mom["launches_per_step"] * 1e-3) / 1e9,
                                           weight_update_gbs=10 * elements / (upd["avg_ms"] * upd["launches_per_step"] * 1e-3) / 1e9,
                                           launches_per_step=sum(v["launches_per_step"] for v in b.values()))
            del opt, params
            torch.cuda.empty_cache()
        from viola_amd.distributed import _fp8_kernels as codec, packet_bytes
        log("comm codec")
        n = 6553600
        bucket = torch.randn(n, device="cuda") * 1e-3
        packet = torch.empty((1, packet_bytes(n // 256, 256)), dtype=torch.uint8, device="cuda")
        out = torch.empty_like(bucket)
        pack_ms, _ = timed(lambda: codec.pack(bucket, packet, 256, torch.float8_e4m3fn), 50, 5)
        unpack_ms, _ = timed(lambda: codec.unpack(packet, out, 256, torch.float8_e4m3fn), 50, 5)
        extra["comm_codec"] = dict(bucket_elements=n, pack_ms=pack_ms, unpack_ms=unpack_ms,
                                   pack_gbs=5.016 * n / (pack_ms * 1e-3) / 1e9, unpack_gbs=5.016 * n / (unpack_ms * 1e-3) / 1e9)
        # the DiT-XL gradients are 68 such buckets; 16 of them through the table entry points, one launch each way
        many = 16
        buckets = [torch.randn(n, device="cuda") * 1e-3 for _ in range(many)]
        packets = [torch.empty((1, packet_bytes(n // 256, 256)), dtype=torch.uint8, device="cuda") for _ in range(many)]
        outs = [torch.empty_like(b) for b in buckets]
        tables = ({}, {})
        pack_many_ms, _ = timed(lambda: codec.pack_many(buckets, packets, 256, torch.float8_e4m3fn, cache=tables[0]), 20, 5)
        unpack_many_ms, _ = timed(lambda: codec.unpack_many(packets, outs, 256, torch.float8_e4m3fn, cache=tables[1]), 20, 5)
        extra["comm_codec"].update(buckets_per_launch=many, pack_many_ms=pack_many_ms, unpack_many_ms=unpack_many_ms,
                                   pack_many_gbs=5.016 * n * many / (pack_many_ms * 1e-3) / 1e9,
                                   unpack_many_gbs=5.016 * n * many / (unpack_many_ms * 1e-3) / 1e9,
                                   pack_many_frac_hbm=5.016 * n * many / (pack_many_ms * 1e-3) / 1e9 / PEAK["hbm_gbs"],
                                   unpack_many_frac_hbm=5.016 * n * many / (unpack_many_ms * 1e-3) / 1e9 / PEAK["hbm_gbs"])
        del buckets, packets, outs

    if want("bound"):
        # the training loop closed: the same Linear under bind_optimizer (fp32 master, bf16 gradients), one
        # forward + backward + FP8Muon step + write-back of the master as FP8 codes and (32, 32) scales
        import viola_amd
        from viola_amd.nn import _grouped_kernels as gk
        log("bound training step")
        viola_amd.set_master_weight_dtype("fp32")
        viola_amd.set_gradient_dtype("bf16")
        torch.manual_seed(1)
        bound = viola_amd.nn.Linear(K, N, device="cuda", dtype=torch.bfloat16, scaling="grouped", forward_dtype="e4m3",
                                    backward_dtype="e4m3", mode="memory", weight_dtype="fp8")
        opt = viola_amd.optim.bind_optimizer(bound, viola_amd.optim.FP8Muon(bound.parameters(), lr=1e-3, weight_decay=.01))
        xb = torch.randn(M, K, device="cuda").bfloat16().requires_grad_()

        def train_step():
            opt.zero_grad()
            bound(xb).backward(dy)
            opt.step()
        train_ms, _ = timed(train_step, min(args.steps, 50), min(args.warmup, 10))
        master = bound._master_ref().detach()
        codes, scales = torch.empty_like(bound.weight), torch.empty_like(bound.weight_scale)
        refresh_ms, _ = timed(lambda: gk.quantize(master, torch.float8_e4m3fn, (32, 32), out=codes, scale_out=scales), 100, 20)
        extra["bound_training_step"] = dict(step_ms=train_ms, optimizer="FP8Muon standard, fp32 master, bf16 gradients",
                                            refresh_quantize_ms=refresh_ms,
                                            refresh_gbs=(4 + 1 + 4 / 1024) * K * N / (refresh_ms * 1e-3) / 1e9)
        viola_amd.precision._settings.update(master_weight_dtype=torch.float32, gradient_dtype=None)

    if want("recipes"):
        # the reference's default recipe on the same layer: one scale per tensor, epilogue scaling (the GEMM runs on
        # the K = 64 f8f6f4 MFMA, the kernel the 5 PFLOP/s figure belongs to)
        import viola_amd
        log("per-tensor and MXFP8 linear steps")
        viola_amd.set_gradient_dtype("bf16")
        torch.manual_seed(2)
        current = viola_amd.nn.Linear(K, N, device="cuda", dtype=torch.bfloat16, scaling="current", forward_dtype="e4m3",
                                      backward_dtype="e5m2", mode="memory", weight_dtype="fp8")
        viola_amd.precision._settings["gradient_dtype"] = None
        xc = torch.randn(M, K, device="cuda").bfloat16().requires_grad_()

        def current_step():
            xc.grad = current.weight.grad = current.bias.grad = None
            current(xc).backward(dy)
        c_ms, _ = timed(current_step, args.steps, args.warmup)
        cb = kernel_breakdown(current_step, min(args.steps, 50))
        cg = cb["viola_tensor_gemm"]
        # and the grouped recipe with E8M0 scales: same groups as the headline, the scaling done by the block-scaled MFMA
        viola_amd.set_gradient_dtype("bf16")
        mx = viola_amd.nn.Linear(K, N, device="cuda", dtype=torch.bfloat16, scaling="mxfp8", forward_dtype="e4m3",
                                 backward_dtype="e4m3", mode="memory", weight_dtype="fp8")
        viola_amd.precision._settings["gradient_dtype"] = None

        def mx_step():
            xc.grad = mx.weight.grad = mx.bias.grad = None
            mx(xc).backward(dy)
        m_ms, _ = timed(mx_step, args.steps, args.warmup)
        mb = kernel_breakdown(mx_step, min(args.steps, 50))
        mg = mb["viola_mx_gemm"]
        extra["linear_mxfp8"] = dict(step_ms=m_ms, tflops=flops / (m_ms * 1e-3) / 1e12, gemm_avg_ms=mg["avg_ms"],
                                     gemm_tflops=2 * M * K * N / (mg["avg_ms"] * 1e-3) / 1e12,
                                     gemm_frac_fp8_peak=2 * M * K * N / (mg["avg_ms"] * 1e-3) / 1e12 / PEAK["fp8_tflops"],
                                     launches_per_step=sum(v["launches_per_step"] for v in mb.values()))
        extra["linear_current_scaling"] = dict(step_ms=c_ms, tflops=flops / (c_ms * 1e-3) / 1e12, gemm_avg_ms=cg["avg_ms"],
                                               gemm_tflops=2 * M * K * N / (cg["avg_ms"] * 1e-3) / 1e12,
                                               gemm_frac_fp8_peak=2 * M * K * N / (cg["avg_ms"] * 1e-3) / 1e12 / PEAK["fp8_tflops"],
                                               launches_per_step=sum(v["launches_per_step"] for v in cb.values()))

    if want("mlp"):
        # the gated MLP of the reference's MLP benchmark shape (16384 tokens, 4096 -> 11008 -> 4096, SwiGLU), forward +
        # backward, under the three recipes: gating fused into the gate/up GEMM's and the down dgrad GEMM's epilogues
        import viola_amd
        Mm, Dm, Hm = 16384, 4096, 11008
        mlp_flops = 3 * (2 * Mm * Dm * 2 * Hm + 2 * Mm * Hm * Dm)
        xm = torch.randn(Mm, Dm, device="cuda").bfloat16().requires_grad_()
        dym = torch.randn(Mm, Dm, device="cuda").bfloat16()
        extra["mlp_step"] = {"shape": [Mm, Dm, Hm], "flops": mlp_flops}
        for scaling in ("grouped", "current", "mxfp8"):
            log(f"MLP step, {scaling}")
            viola_amd.set_gradient_dtype("bf16")
            torch.manual_seed(4)
            mlp = viola_amd.nn.MLP(Dm, Hm, activation="silu", weight_dtype="fp8", scaling=scaling, mode="memory", backward_dtype="e4m3",
                                   device="cuda", dtype=torch.bfloat16)
            viola_amd.precision._settings["gradient_dtype"] = None

            def mlp_step():
                xm.grad = None
                for parameter in mlp.parameters():
                    parameter.grad = None
                mlp(xm).backward(dym)
            mlp_ms, _ = timed(mlp_step, min(args.steps, 20), min(args.warmup, 5))
            gated = {k: v for k, v in kernel_breakdown(mlp_step, 3).items() if "gated" in k}
            extra["mlp_step"][scaling] = dict(step_ms=mlp_ms, tflops=mlp_flops / (mlp_ms * 1e-3) / 1e12, gated_gemm=gated)
            del mlp
        del xm, dym

    if want("ns1"):
        log("Newton-Schulz, one 1024 x 4096 matrix")
        extra["ns_1024x4096"] = ns_single_case(min(args.steps, 50), min(args.warmup, 10))
    if want("varlen"):
        log("variable-group step")
        extra["varlen_step"] = varlen_case(min(args.steps, 20), min(args.warmup, 5))

    if args.calibrate:
        from viola_amd.optim import _kernels as ok
        src = torch.ones(1 << 26, device="cuda")
        dst = torch.empty_like(src)
        ok.copy_scaled(src, dst, 0, 0, src.numel(), 1.0)
        torch.cuda.synchronize()

    result = {
        "metric": "FP8 Linear fwd+bwd TFLOPS (8192x1024->4096) + FP8Muon step ms; % of roofline",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "wall_ms_per_step": wall_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "e4m3 operands, fp32 accumulate", "data": "synthetic",
        "config": {"workload": "viola.nn.Linear(1024, 4096, scaling='grouped', e4m3/e4m3, fp8 weight storage, mode='memory') "
                               "forward+backward on 8192 tokens, bf16 activations and gradients"},
        "frac_of_fp8_peak": value / PEAK["fp8_tflops"],
        "roofline": roofline, "quantize": quant, "kernels": breakdown, **extra,
    }
    if not args.skip_cpu:
        log("CPU baselines")
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result), flush=True)
    others = result.get("cpu_baseline", {}).get("others", {})
    if any(leg.get("ms", 0) is None or "not finished" in leg.get("sample", "") for leg in others.values()):
        os._exit(0)                                                  # a CPU leg is still running in its thread: do not wait for it


if __name__ == "__main__":
    main()
