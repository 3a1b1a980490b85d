#!/usr/bin/env python3
"""Benchmark of the MI355X SOAP step: steps/s on one GPU for one parameter shape.

    python bench.py [--gpus 1] [--steps 50] [--warmup 11] [--shape 4096x11008] [--rank 128]

A "step" is one call of the public ``soap_tp_amd.soap_step`` on a synthetic low-rank-plus-noise
gradient that is already resident in HBM (generated on the CPU by the oracle's generator, so the
CPU baseline consumes the same bits, and copied over before anything is timed).  The warm-up
contains the initialising call (Gram matrices + both eigensolves) and, by default, ten more steps
including one basis refresh, so that the timed region is the steady-state schedule of the
benchmark configuration: K steps with a refresh every 10.  One JSON line is printed; ``value`` is K
divided by the time of the timed region: device synchronisation, HIP event, K ``soap_step`` calls,
HIP event, device synchronisation (the reference times its step the same way,
scripts/run_soap_tp_timing_gpu.py:139-165).

Stage times come from a second pass over the same schedule that issues the step's library calls
one by one with event marks between them.  ``roofline`` describes the dominant kernel, the fp32 MFMA
product behind the four rotation products of a step (algorithmic flops 4 m n (m+n) per step,
2 m n k per launch), from that pass's events.  After the timed passes one more step is checked
against the CPU oracle conditionally on the device's bases (``parity_check``: update, moments and both
Gram matrices; also for every other shape reported and for one parameter per distinct shape of the
layer).  ``cpu_baseline``
times the CPU oracle (torch/MKL on the host cores) on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import statistics
import sys
import time

import torch

FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix peak
HBM_PEAK_GBS = 8000.0
GRID = (1, 1)
HYPER = dict(preconditioner_beta=0.95, beta1=0.95, beta2=0.95, eps=1e-8, basis_refresh_interval=10)

def measured_traffic_bytes(rows, columns):
    """Memory bytes per launch of the rotation product (mean of the four launches of a step) for this
    shape, read from the committed counter summary profiles/rotate_adam_rotate_<rows>x<columns>_memory_traffic.txt
    (two rocprofv3 --pmc runs, FETCH_SIZE and WRITE_SIZE, of tests/native/abi_probe.bin, each scaled by what
    the same counter reads for a layout copy of known size), with the file it came from; (None, None)
    for a shape that has not been measured."""
    import re
    from pathlib import Path

    path = Path(__file__).resolve().parent / "profiles" / f"rotate_adam_rotate_{rows}x{columns}_memory_traffic.txt"
    if not path.exists():
        return None, None
    match = re.search(r"traffic per launch ([0-9.]+e[0-9]+) bytes", path.read_text())
    return (float(match.group(1)), f"profiles/{path.name}") if match else (None, None)



def gradient_pool(rows, columns, rank, count, device, seed0=42):
    """`count` gradients from the oracle's CPU generator (seed0 + i), copied to the device."""
    from oracle import soap_oracle as oracle

    pool = [oracle.low_rank_plus_noise(rows, columns, rank, seed=seed0 + i).to(device) for i in range(count)]
    torch.cuda.synchronize()
    return pool


class StepTimer:
    """HIP events on the current stream around sub-stages of a step (no synchronisation)."""

    def __init__(self):
        self.records = []

    def mark(self):
        event = torch.cuda.Event(enable_timing=True)
        event.record(torch.cuda.current_stream())
        return event


def run_schedule(shape, rank, steps, warmup, device, pool_size=6, interval=10, shard_dim=1, detail=True,
                 parity=False):
    """Initialising call + warm-up, then `steps` timed calls of the public soap_step (the headline),
    then, with `detail`, the same number of steps again through the step's individual library calls
    with event marks between them (stage times), then, with `parity`, one checked step."""
    import soap_tp_amd
    from soap_tp_amd import soap as soap_module
    from soap_tp_amd.ops import refresh_bases_and_transport_optimizer_state_

    rows, columns = shape
    gradients = gradient_pool(rows, columns, rank, pool_size, device)
    state = {}
    hyper = dict(HYPER, basis_refresh_interval=interval)
    kwargs = dict(global_shape=shape, shard_dim=shard_dim, block_size=128, process_grid_shape=GRID, **hyper)

    init_start = time.perf_counter()
    soap_tp_amd.soap_step(gradients[0], state, **kwargs)
    torch.cuda.synchronize()
    init_ms = (time.perf_counter() - init_start) * 1e3
    for w in range(1, warmup):
        soap_tp_amd.soap_step(gradients[w % pool_size], state, **kwargs)
    torch.cuda.synchronize()

    # ---- headline: the public entry point, nothing else inside the timed region
    timer = StepTimer()
    first_step = int(state["step"]) + 1
    wall_start = time.perf_counter()
    begin = timer.mark()
    for k in range(steps):
        soap_tp_amd.soap_step(gradients[(warmup + k) % pool_size], state, **kwargs)
    end = timer.mark()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - wall_start) * 1e3
    total_ms = begin.elapsed_time(end)
    refreshes = sum(1 for step in range(first_step, first_step + steps) if step % interval == 0)
    result = {"total_ms": total_ms, "wall_ms": wall_ms, "init_ms": init_ms, "refreshes": refreshes}

    # ---- stage times: the same library calls soap_step makes, with event marks between them
    if detail:
        marks = []
        begin = timer.mark()
        for k in range(steps):
            gradient = gradients[(warmup + steps + k) % pool_size]
            step = int(state["step"]) + 1
            t0 = timer.mark()
            soap_module._fused_update(gradient, state, rows, columns, step, hyper["beta1"], hyper["beta2"], hyper["eps"])
            t1 = timer.mark()
            soap_module._fused_gram_pair(gradient, state, rows, columns, hyper["preconditioner_beta"], False)
            t2 = timer.mark()
            refreshed = step % interval == 0
            if refreshed:
                refresh_bases_and_transport_optimizer_state_(
                    state["momentum"], state["variance"], state["left_preconditioner"],
                    state["right_preconditioner"], state["left_basis"], state["right_basis"], state["left_work"],
                    state["right_work"], shape, 128, GRID, symmetrize=True)
            t3 = timer.mark()
            state["step"] = step
            marks.append((t0, t1, t2, t3, refreshed))
        end = timer.mark()
        torch.cuda.synchronize()
        rotate = [a.elapsed_time(b) for a, b, _, _, _ in marks]
        gram = [b.elapsed_time(c) for _, b, c, _, _ in marks]
        refresh = [c.elapsed_time(d) for _, _, c, d, r in marks if r]
        result.update(rotate_ms=statistics.mean(rotate), gram_ms=statistics.mean(gram),
                      refresh_ms=statistics.mean(refresh) if refresh else None, detail_refreshes=len(refresh),
                      detail_total_ms=begin.elapsed_time(end))

    if parity:
        result["parity_check"] = checked_step(gradients[1], state, kwargs, dict(hyper))
    del state
    return result


def _lower_to_full(matrix):
    """The symmetric matrix whose lower triangle (diagonal included) `matrix` holds."""
    lower = torch.tril(matrix)
    return lower + torch.tril(matrix, -1).T


def checked_step(gradient, state, kwargs, hyper, step_function=None):
    """One more soap_step on the state the timed passes left, compared with the CPU oracle's
    arithmetic for that step on the same bits, conditionally on the device's bases: the update, both
    moments and both Gram matrices (their lower triangles: the step keeps only those up to date
    between refreshes).  `step_function(gradient)` makes the step and returns the update; by default it
    is soap_tp_amd.soap_step on `state`."""
    import soap_tp_amd
    from oracle import soap_oracle as oracle

    if step_function is None:
        def step_function(g):
            return soap_tp_amd.soap_step(g, state, **kwargs)

    step = int(state["step"]) + 1
    if step % hyper["basis_refresh_interval"] == 0:  # keep the checked step a plain one
        step_function(gradient)
        step += 1
    momentum, variance = state["momentum"].cpu().clone(), state["variance"].cpu().clone()
    q_left, q_right = state["left_basis"].cpu(), state["right_basis"].cpu()
    grams = {side: _lower_to_full(state[f"{side}_preconditioner"].cpu()) for side in ("left", "right")}
    update = step_function(gradient).cpu()
    gradient = gradient.cpu().to(torch.float32)
    start = time.perf_counter()
    projected = oracle.rotate(gradient, q_left, q_right, "forward")
    coordinate = oracle.adam_update(projected, momentum, variance, step, hyper["beta1"], hyper["beta2"],
                                    hyper["eps"] / math.sqrt(1.0 - hyper["beta2"] ** step))
    expected = oracle.rotate(coordinate, q_left, q_right, "backward")
    cpu_ms = (time.perf_counter() - start) * 1e3

    def relative(actual, reference):
        return ((actual.double() - reference.double()).norm() / reference.double().norm()).item()

    errors = {"update": relative(update, expected), "momentum": relative(state["momentum"].cpu(), momentum),
              "variance": relative(state["variance"].cpu(), variance)}
    for side in ("left", "right"):
        expected_gram = oracle.gram_ema(grams[side], gradient, hyper["preconditioner_beta"], side)
        errors[f"{side}_gram"] = relative(torch.tril(state[f"{side}_preconditioner"].cpu()), torch.tril(expected_gram))
        del expected_gram
    ok = all(math.isfinite(e) and e <= 1e-4 for e in errors.values())
    return {"step": step, "relative_frobenius_error": errors, "tolerance": 1e-4, "ok": ok,
            "what": "the step after the timed passes against the CPU oracle, given the device's bases: update, "
                    "moments, lower triangles of both Gram matrices",
            "cpu_ms": cpu_ms}


def cpu_baseline(shape, rank, sample_plain_steps=2, with_refresh=True, full_init=True, interval=10):
    """The CPU oracle on a bounded sample: `sample_plain_steps` steady-state steps and one refresh."""
    from oracle import soap_oracle as oracle

    rows, columns = shape
    torch.set_num_threads(os.cpu_count() or 1)
    cores = torch.get_num_threads()
    generator = torch.Generator().manual_seed(7)
    # orthonormal bases and Gram matrices of the right size; their values do not change the cost
    state = {
        "left_basis": torch.linalg.qr(torch.randn(rows, rows, generator=generator))[0],
        "right_basis": torch.linalg.qr(torch.randn(columns, columns, generator=generator))[0],
        "momentum": torch.zeros(rows, columns), "variance": torch.zeros(rows, columns), "step": 0,
    }
    gradient = oracle.low_rank_plus_noise(rows, columns, rank, seed=42)
    state["left_preconditioner"] = 0.05 * gradient @ gradient.T
    state["right_preconditioner"] = 0.05 * gradient.T @ gradient
    kwargs = dict(HYPER)
    kwargs["basis_refresh_interval"] = 10**9  # plain steps only
    oracle.soap_step(gradient, state, **kwargs)  # warm-up
    start = time.perf_counter()
    for _ in range(sample_plain_steps):
        oracle.soap_step(gradient, state, **kwargs)
    plain_ms = (time.perf_counter() - start) * 1e3 / sample_plain_steps
    refresh_ms = None
    if with_refresh:
        start = time.perf_counter()
        oracle.refresh(state)
        refresh_ms = (time.perf_counter() - start) * 1e3
    # the two eigensolves of the initialising call (fp64 solve of -P as the "elpa" variant does); the
    # larger side (about 20 s at 11008) can be left out with --cpu-small-init
    init_sizes = [min(rows, columns)] + ([max(rows, columns)] if full_init and rows != columns else [])
    init_ms = {}
    for size in init_sizes:
        matrix = state["left_preconditioner"] if size == rows else state["right_preconditioner"]
        start = time.perf_counter()
        oracle.eigh_descending(matrix, "elpa")
        init_ms[str(size)] = (time.perf_counter() - start) * 1e3
    per_step_ms = plain_ms + (refresh_ms / interval if refresh_ms is not None else 0.0)
    return {
        "value": 1e3 / per_step_ms, "unit": "steps/s", "cores": cores, "kind": "port",
        "sample": f"{sample_plain_steps} steady-state steps" + (" + 1 basis refresh" if with_refresh else "")
                  + f" of the {rows}x{columns} workload on the CPU oracle (torch/MKL), refresh cost spread over "
                  + f"{interval} steps; plus the initialising fp64 eigensolve of size(s) {', '.join(init_ms)} "
                  + "(reported, not part of value)",
        "plain_step_ms": plain_ms, "refresh_ms": refresh_ms, "init_eigensolve_ms_by_size": init_ms,
    }


def run_layer(device, steps=30, rank=64):
    """One transformer layer's seven matrices (q, k, v, o, gate, up, down), each with its own state,
    stepped together by the optimizer wrapper: whole-layer time per optimizer step."""
    from soap_tp_amd import SOAP

    shapes = [(4096, 4096)] * 4 + [(4096, 14336)] * 2 + [(14336, 4096)]
    parameters = [torch.nn.Parameter(torch.zeros(shape, device=device)) for shape in shapes]
    gradients = {shape: gradient_pool(shape[0], shape[1], rank, 2, device, seed0=42 + 1000 * i)
                 for i, shape in enumerate(dict.fromkeys(shapes))}
    optimizer = SOAP(parameters, lr=3e-3, betas=(HYPER["beta1"], HYPER["beta2"]),
                     shampoo_beta=HYPER["preconditioner_beta"], eps=HYPER["eps"], weight_decay=0.0,
                     precondition_frequency=HYPER["basis_refresh_interval"])

    def one_step(t):
        for parameter in parameters:
            parameter.grad = gradients[tuple(parameter.shape)][t % 2]
        optimizer.step()

    torch.cuda.synchronize()
    start = time.perf_counter()
    one_step(0)
    torch.cuda.synchronize()
    init_ms = (time.perf_counter() - start) * 1e3
    interval = HYPER["basis_refresh_interval"]
    for t in range(1, interval + 1):  # up to and including the first refresh
        one_step(t)
    torch.cuda.synchronize()
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    begin.record()
    for t in range(steps):
        one_step(interval + 1 + t)
    end.record()
    torch.cuda.synchronize()
    total_ms = begin.elapsed_time(end)
    if not all(bool(torch.isfinite(parameter).all()) for parameter in parameters):
        raise RuntimeError("a parameter of the layer run is not finite")
    # one more step per distinct shape, checked against the CPU oracle: that parameter alone receives a
    # gradient, so the wrapper steps only it, and its update is read off the parameter (lr * update)
    hyper = dict(HYPER)
    checks = {}
    lr = optimizer.param_groups[0]["lr"]
    for shape in dict.fromkeys(shapes):
        parameter = next(p for p in parameters if tuple(p.shape) == shape)
        soap_state = optimizer.state[parameter]["soap"]

        def step_function(gradient, parameter=parameter):
            for other in parameters:
                other.grad = None
            before = parameter.detach().clone()
            parameter.grad = gradient
            optimizer.step()
            return (before - parameter.detach()) / lr

        check = checked_step(gradients[shape][1], soap_state, None, hyper, step_function=step_function)
        # the update passed through p -= lr * update: two more roundings on values of the parameter's size
        checks[f"{shape[0]}x{shape[1]}"] = check
    flops = sum(5.0 * m * n * (m + n) for m, n in shapes)
    return {"parity_check": checks, "workload": "4 x 4096x4096, 2 x 4096x14336, 1 x 14336x4096, rank 64, refresh every 10, "
                        "optimizer wrapper with 2 side streams", "steps": steps,
            "ms_per_layer_step": total_ms / steps, "layer_steps_per_s": steps / (total_ms * 1e-3),
            "initialisation_ms": init_ms, "plain_step_mfma_flops": flops}


def hbm_stages(rows, columns, device, repeats=10):
    """The bandwidth-bound kernels of the path, each timed alone with HIP events over `repeats` launches:
    achieved GB/s over their algorithmic bytes against the 8 TB/s HBM peak."""
    from soap_tp_amd.ops import (adam_update, allocate_2d_block_cyclic, permute_2d_block_cyclic_,
                                 redistribute_tp_shard_to_2d_block_cyclic)

    def timed(function):
        function()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        for _ in range(repeats):
            function()
        end.record()
        torch.cuda.synchronize()
        return begin.elapsed_time(end) / repeats

    shape = (rows, columns)
    gradient = allocate_2d_block_cyclic(shape, 128, GRID, device=device)
    gradient.normal_()
    momentum = allocate_2d_block_cyclic(shape, 128, GRID, device=device)
    variance = allocate_2d_block_cyclic(shape, 128, GRID, device=device)
    row_major = torch.randn(rows, columns, device=device)
    row_order = torch.randperm(rows, device=device)
    column_order = torch.randperm(columns, device=device)
    stages = {
        "adam_kernel": (24.0 * rows * columns,
                        lambda: adam_update(gradient, momentum, variance, 3, 0.95, 0.95, 1e-8)),
        "layout_copy": (8.0 * rows * columns,
                        lambda: redistribute_tp_shard_to_2d_block_cyclic(row_major, shape, 128, GRID, shard_dim=1)),
        "variance_permute": (16.0 * rows * columns,  # gather into a temporary, copy back
                             lambda: permute_2d_block_cyclic_(variance, shape, row_order, column_order, 128, GRID,
                                                              validate=False)),
    }
    result = {}
    for name, (nbytes, function) in stages.items():
        ms = timed(function)
        rate = nbytes / (ms * 1e-3) / 1e9
        result[name] = {"bytes": nbytes, "ms": ms, "GB/s": rate, "frac_of_hbm_peak": rate / HBM_PEAK_GBS}
    return result


def calibration_copies(rows, columns, count, device):
    """Row-major to column-major copies of a rows x columns fp32 matrix through the library."""
    from soap_tp_amd.ops import redistribute_tp_shard_to_2d_block_cyclic

    source = torch.randn(rows, columns, device=device)
    for _ in range(count):
        redistribute_tp_shard_to_2d_block_cyclic(source, (rows, columns), 128, GRID, shard_dim=1)
    torch.cuda.synchronize()


def gpu_eigensolve_ms(sizes, rank, device):
    """The initialising eigensolve ("elpa" variant: fp64 solve of -P) of a Gram matrix of each size,
    timed alone with HIP events (second of two calls)."""
    from oracle import soap_oracle as oracle
    from soap_tp_amd.ops import allocate_2d_block_cyclic, initialize_basis_2d_block_cyclic_

    result = {}
    for size in sizes:
        gradient = oracle.low_rank_plus_noise(size, size, rank, seed=42).to(device)
        gram = allocate_2d_block_cyclic((size, size), 128, GRID, device=device)
        gram.copy_(0.05 * gradient @ gradient.T)
        basis = allocate_2d_block_cyclic((size, size), 128, GRID, device=device)
        work = allocate_2d_block_cyclic((size, size), 128, GRID, device=device)
        values = torch.empty(size, dtype=torch.float32, device=device)
        for _ in range(2):
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            begin.record()
            initialize_basis_2d_block_cyclic_(gram, basis, work, values, size, 128, GRID, implementation="elpa")
            end.record()
            torch.cuda.synchronize()
        result[str(size)] = begin.elapsed_time(end)
        del gradient, gram, basis, work
    return result


def parse_shape(text):
    rows, columns = text.lower().split("x")
    return int(rows), int(columns)


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=50)
    parser.add_argument("--warmup", type=int, default=11)
    parser.add_argument("--shape", type=parse_shape, default=(4096, 11008))
    parser.add_argument("--rank", type=int, default=128)
    parser.add_argument("--shard-dim", type=int, default=1, choices=(0, 1),
                        help="shard_dim passed to the step (same mathematics on one rank; the reference's two Gram "
                             "code paths)")
    parser.add_argument("--refresh-interval", type=int, default=HYPER["basis_refresh_interval"],
                        help="steps between two basis refreshes of the main shape (the benchmark configurations use "
                             "10, and 5 for 8192x3584)")
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--no-other-shapes", action="store_true")
    parser.add_argument("--cpu-small-init", action="store_true",
                        help="time only the smaller side's initialising eigensolve on the CPU oracle (the larger one "
                             "takes about 20 s at 11008)")
    parser.add_argument("--no-layer", action="store_true",
                        help="skip the whole-layer configuration (4 x 4096x4096, 2 x 4096x14336, 1 x 14336x4096, "
                             "rank 64, 30 steps through the optimizer wrapper), reported under 'layer'")
    parser.add_argument("--calibration-copies", type=int, default=0,
                        help="run this many layout copies of one rows x columns fp32 matrix (transpose_kernel: "
                             "4*rows*columns bytes read and as many written) before the schedule; the known-size "
                             "kernel that hardware-counter readings of a profiled run are scaled by")
    args = parser.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU's share of the SOAP step: this build has no multi-GPU path, "
                 "run it with --gpus 1.")
    if args.warmup < 1:
        sys.exit("--warmup must be at least 1: the first call initialises the state and returns zeros.")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs an MI355X: no GPU is visible.")
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    rows, columns = args.shape

    if args.calibration_copies > 0:
        calibration_copies(rows, columns, args.calibration_copies, device)
    if args.refresh_interval <= 0:
        sys.exit("--refresh-interval must be positive.")
    main_run = run_schedule(args.shape, args.rank, args.steps, args.warmup, device, shard_dim=args.shard_dim,
                            interval=args.refresh_interval, parity=True)
    if not main_run["parity_check"]["ok"]:
        sys.exit(f"bench.py: the checked step disagrees with the CPU oracle: {main_run['parity_check']}")
    ms_per_step = main_run["total_ms"] / args.steps
    rotation_flops = 4.0 * rows * columns * (rows + columns)
    gram_flops = 1.0 * rows * columns * (rows + columns)
    achieved = rotation_flops / (main_run["rotate_ms"] * 1e-3) / 1e12
    traffic, traffic_source = measured_traffic_bytes(rows, columns)
    line = {
        "metric": "SOAP steps/sec per param shape (1 GPU)",
        "value": args.steps / (main_run["total_ms"] * 1e-3),
        "unit": "steps/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": f"{rows}x{columns} fp32 parameter, rank-{args.rank} low-rank-plus-noise gradients "
                        f"(log-uniform spectrum 1e-4..1e-1, noise std 1e-4), world_size 1, shard_dim {args.shard_dim}, "
                        f"block_size 128, "
                        f"refresh every {args.refresh_interval} steps, beta1=beta2=shampoo_beta=0.95, "
                        "eps=1e-8, basis_implementation=elpa (fp64 eigensolve)",
            "schedule": f"{args.warmup} warm-up calls (initialisation + {args.warmup - 1} steps), then {args.steps} "
                        f"timed calls of soap_step ({main_run['refreshes']} of them refresh the bases)",
            "gradients": "generated on the CPU by the oracle's generator (seeds 42..47), resident in HBM before timing",
        },
        "timed_region": "sync, event, K x soap_tp_amd.soap_step, event, sync",
        "ms_per_step_in_stage_pass": main_run["detail_total_ms"] / args.steps,
        "parity_check": main_run["parity_check"],
        "stages_ms": {
            "rotate_adam_rotate": main_run["rotate_ms"],
            "gram_pair": main_run["gram_ms"],
            "plain_step": main_run["rotate_ms"] + main_run["gram_ms"],
            "refresh": main_run["refresh_ms"],
            "initialisation_call": main_run["init_ms"],
            "refreshes_timed": main_run["detail_refreshes"],
            "from": "a second pass over the same schedule, library calls issued one by one with event marks",
        },
        "roofline": {
            "bound": "mfma",
            "kernel": "gemm_kernel<float,128x128x16> (the 4 rotation products of a step, one with the Adam epilogue)",
            "achieved": achieved,
            "peak": FP32_MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / FP32_MFMA_PEAK_TFLOPS,
            "traffic": traffic,
            "traffic_unit": "bytes per launch (L2 fills + writes; compulsory 0.82e9 at 4096x11008)",
            "traffic_source": traffic_source,
            "flops_per_step": rotation_flops,
            "avg_launch_ms": main_run["rotate_ms"] / 4.0,
            "gram_pair_tflops_syrk_convention": gram_flops / (main_run["gram_ms"] * 1e-3) / 1e12,
            "step_mfma_stages_tflops": (rotation_flops + gram_flops)
                                       / ((main_run["rotate_ms"] + main_run["gram_ms"]) * 1e-3) / 1e12,
        },
    }
    if not args.no_other_shapes:
        others = {}
        for shape, rank, steps, interval in (((1024, 1024), 32, 20, 10), ((4096, 4096), 64, 50, 10),
                                             ((8192, 3584), 128, 100, 5)):
            if shape == args.shape:
                continue
            run = run_schedule(shape, rank, steps, interval + 1, device, interval=interval, parity=True)
            flops = 5.0 * shape[0] * shape[1] * (shape[0] + shape[1])
            plain = run["rotate_ms"] + run["gram_ms"]
            others[f"{shape[0]}x{shape[1]}"] = {
                "steps": steps, "refresh_every": interval, "steps_per_s": steps / (run["total_ms"] * 1e-3),
                "plain_step_ms": plain, "refresh_ms": run["refresh_ms"], "initialisation_call_ms": run["init_ms"],
                "step_mfma_stages_tflops": flops / (plain * 1e-3) / 1e12,
                "parity_check": run["parity_check"],
            }
        line["other_shapes"] = others
    line["hbm_stages"] = hbm_stages(rows, columns, device)
    if not args.no_layer:
        line["layer"] = run_layer(device)
    if not args.no_cpu_baseline:
        baseline = cpu_baseline(args.shape, args.rank, full_init=not args.cpu_small_init, interval=args.refresh_interval)
        gpu_ms = gpu_eigensolve_ms([int(size) for size in baseline["init_eigensolve_ms_by_size"]], args.rank, device)
        baseline["gpu_eigensolve_ms_by_size"] = gpu_ms
        baseline["eigensolve_speedup_by_size"] = {
            size: baseline["init_eigensolve_ms_by_size"][size] / gpu_ms[size] for size in gpu_ms}
        if baseline["refresh_ms"] is not None and main_run["refresh_ms"]:
            baseline["refresh_speedup"] = baseline["refresh_ms"] / main_run["refresh_ms"]
        line["cpu_baseline"] = baseline
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))
    failed = [name for name, entry in line.get("other_shapes", {}).items() if not entry["parity_check"]["ok"]]
    failed += [f"layer {name}" for name, entry in (line.get("layer") or {}).get("parity_check", {}).items()
               if not entry["ok"]]
    if failed:
        sys.exit(f"bench.py: the checked step disagrees with the CPU oracle for {failed}")


if __name__ == "__main__":
    main()
