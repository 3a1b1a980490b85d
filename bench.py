#!/usr/bin/env python3
"""Benchmark of the MI355X SOAP step: steps/s on one GPU for one parameter shape.

    python bench.py [--gpus 1] [--steps 50] [--warmup 11] [--shape 4096x11008] [--rank 128]

A "step" is one ``soap_step`` call on a synthetic low-rank-plus-noise gradient that is already
resident in HBM.  The warm-up contains the initialising call (Gram matrices + both eigensolves) and,
by default, ten more steps including one basis refresh, so that the timed region is the
steady-state schedule of the benchmark configuration: K steps with a refresh every 10.  One JSON line
is printed; ``value`` is K divided by the time of the timed region, taken with HIP events on the
stream the kernels run on and bracketed by device synchronisations.

``roofline`` describes the dominant kernel, the fp32 MFMA product behind the four rotation products
of a step (algorithmic flops 4 m n (m+n) per step, 2 m n k per launch); its launches are timed live
with HIP events inside the timed region.  ``cpu_baseline`` times the CPU oracle (torch/MKL on the
host cores) on a bounded sample of the same workload.
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

# Memory bytes per launch of the rotation product (mean of the four launches of a step), from two
# rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) of tests/native/abi_probe.bin, each scaled by what the
# same counter reads for a layout copy of known size; summary under profiles/.  Keyed by shape; a shape
# that has not been measured reports null.
MEASURED_TRAFFIC_BYTES = {"4096x11008": 5.33e9}


def device_low_rank_plus_noise(rows, columns, rank, seed, device, noise_std=1e-4):
    generator = torch.Generator(device=device).manual_seed(seed)
    U, _ = torch.linalg.qr(torch.randn(rows, rank, generator=generator, device=device))
    V, _ = torch.linalg.qr(torch.randn(columns, rank, generator=generator, device=device))
    low, high = math.log(1e-4), math.log(1e-1)
    s = torch.exp(torch.rand(rank, generator=generator, device=device) * (high - low) + low)
    noise = torch.randn(rows, columns, generator=generator, device=device)
    return ((U * s) @ V.T + noise_std * noise).contiguous()


class StepTimer:
    """HIP events on the current stream around sub-stages of a step (no synchronisation)."""

    def __init__(self):
        self.records = []

    def mark(self):
        event = torch.cuda.Event(enable_timing=True)
        event.record(torch.cuda.current_stream())
        return event


def run_schedule(shape, rank, steps, warmup, device, pool_size=6, detail=True, shard_dim=1):
    import soap_tp_amd
    from soap_tp_amd import soap as soap_module
    from soap_tp_amd.ops import (refresh_bases_and_transport_optimizer_state_,
                                 update_left_preconditioner_2d_block_cyclic_,
                                 update_right_preconditioner_2d_block_cyclic_)

    rows, columns = shape
    gradients = [device_low_rank_plus_noise(rows, columns, rank, 42 + i, device) for i in range(pool_size)]
    torch.cuda.synchronize()
    state = {}
    kwargs = dict(global_shape=shape, shard_dim=shard_dim, block_size=128, process_grid_shape=GRID, **HYPER)

    init_start = time.perf_counter()
    soap_tp_amd.soap_step(gradients[0], state, **kwargs)
    torch.cuda.synchronize()
    init_ms = (time.perf_counter() - init_start) * 1e3
    for w in range(1, warmup):
        soap_tp_amd.soap_step(gradients[w % pool_size], state, **kwargs)
    torch.cuda.synchronize()

    # The timed region runs the same three library calls per step as soap_step does, with event
    # marks between them so that stage times are measured on the kernels' own stream.
    timer = StepTimer()
    marks = []
    interval = HYPER["basis_refresh_interval"]
    begin = timer.mark()
    wall_start = time.perf_counter()
    for k in range(steps):
        gradient = gradients[(warmup + k) % pool_size]
        if detail:
            step = int(state["step"]) + 1
            t0 = timer.mark()
            update = soap_module._fused_update(gradient, state, rows, columns, step, HYPER["beta1"], HYPER["beta2"],
                                               HYPER["eps"])
            t1 = timer.mark()
            update_left_preconditioner_2d_block_cyclic_(gradient, state["left_preconditioner"],
                                                        HYPER["preconditioner_beta"], 128, GRID, shard_dim=shard_dim,
                                                        mirror=False)
            update_right_preconditioner_2d_block_cyclic_(gradient, state["right_preconditioner"],
                                                         HYPER["preconditioner_beta"], 128, GRID,
                                                         shard_dim=shard_dim, mirror=False)
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
        else:
            soap_tp_amd.soap_step(gradient, state, **kwargs)
    end = timer.mark()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - wall_start) * 1e3
    total_ms = begin.elapsed_time(end)
    result = {"total_ms": total_ms, "wall_ms": wall_ms, "init_ms": init_ms}
    if detail and marks:
        rotate = [a.elapsed_time(b) for a, b, _, _, _ in marks]
        gram = [b.elapsed_time(c) for _, b, c, _, _ in marks]
        refresh = [c.elapsed_time(d) for _, _, c, d, r in marks if r]
        result.update(rotate_ms=statistics.mean(rotate), gram_ms=statistics.mean(gram),
                      refresh_ms=statistics.mean(refresh) if refresh else None, refreshes=len(refresh))
    del state
    return result


def cpu_baseline(shape, rank, sample_plain_steps=2, with_refresh=True, full_init=False):
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
    # one of the two eigensolves of the initialising call (the smaller side, fp64 solve of -P as the
    # "elpa" variant does); the larger side only on request, it takes most of a minute
    init_sizes = [min(rows, columns)] + ([max(rows, columns)] if full_init and rows != columns else [])
    init_ms = {}
    for size in init_sizes:
        matrix = state["left_preconditioner"] if size == rows else state["right_preconditioner"]
        start = time.perf_counter()
        oracle.eigh_descending(matrix, "elpa")
        init_ms[str(size)] = (time.perf_counter() - start) * 1e3
    interval = HYPER["basis_refresh_interval"]
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
    gradients = {shape: [device_low_rank_plus_noise(shape[0], shape[1], rank, 42 + 1000 * i + t, device)
                         for t in range(2)] for i, shape in enumerate(dict.fromkeys(shapes))}
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
    flops = sum(5.0 * m * n * (m + n) for m, n in shapes)
    return {"workload": "4 x 4096x4096, 2 x 4096x14336, 1 x 14336x4096, rank 64, refresh every 10, "
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
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--no-other-shapes", action="store_true")
    parser.add_argument("--cpu-full-init", action="store_true",
                        help="also time the larger side's initialising eigensolve on the CPU oracle (about a minute)")
    parser.add_argument("--layer", action="store_true",
                        help="also run the whole-layer configuration (4 x 4096x4096, 2 x 4096x14336, 1 x 14336x4096, "
                             "rank 64, 30 steps) through the optimizer wrapper and report it under 'layer'")
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
    main_run = run_schedule(args.shape, args.rank, args.steps, args.warmup, device, shard_dim=args.shard_dim)
    ms_per_step = main_run["total_ms"] / args.steps
    rotation_flops = 4.0 * rows * columns * (rows + columns)
    gram_flops = 1.0 * rows * columns * (rows + columns)
    achieved = rotation_flops / (main_run["rotate_ms"] * 1e-3) / 1e12
    traffic = MEASURED_TRAFFIC_BYTES.get(f"{rows}x{columns}")
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
                        f"refresh every {HYPER['basis_refresh_interval']} steps, beta1=beta2=shampoo_beta=0.95, "
                        "eps=1e-8, basis_implementation=elpa (fp64 eigensolve)",
            "schedule": f"{args.warmup} warm-up calls (initialisation + {args.warmup - 1} steps), then {args.steps} "
                        "timed steps",
        },
        "stages_ms": {
            "rotate_adam_rotate": main_run["rotate_ms"],
            "gram_pair": main_run["gram_ms"],
            "plain_step": main_run["rotate_ms"] + main_run["gram_ms"],
            "refresh": main_run["refresh_ms"],
            "initialisation_call": main_run["init_ms"],
            "refreshes_timed": main_run["refreshes"],
        },
        "roofline": {
            "bound": "mfma",
            "kernel": "gemm_kernel<float,128x128x16> (the 4 rotation products of a step, one with the Adam epilogue)",
            "achieved": achieved,
            "peak": FP32_MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / FP32_MFMA_PEAK_TFLOPS,
            "traffic": traffic,
            "traffic_unit": "bytes per launch (L2 fills + writes; compulsory 0.82e9)",
            "flops_per_step": rotation_flops,
            "avg_launch_ms": main_run["rotate_ms"] / 4.0,
            "gram_pair_tflops_syrk_convention": gram_flops / (main_run["gram_ms"] * 1e-3) / 1e12,
            "step_mfma_stages_tflops": (rotation_flops + gram_flops)
                                       / ((main_run["rotate_ms"] + main_run["gram_ms"]) * 1e-3) / 1e12,
        },
    }
    if not args.no_other_shapes:
        others = {}
        for shape, rank in (((1024, 1024), 32), ((4096, 4096), 64), ((8192, 3584), 128)):
            if shape == args.shape:
                continue
            run = run_schedule(shape, rank, 20, 11, device)
            flops = 5.0 * shape[0] * shape[1] * (shape[0] + shape[1])
            plain = run["rotate_ms"] + run["gram_ms"]
            others[f"{shape[0]}x{shape[1]}"] = {
                "steps_per_s": 20 / (run["total_ms"] * 1e-3), "plain_step_ms": plain, "refresh_ms": run["refresh_ms"],
                "initialisation_call_ms": run["init_ms"], "step_mfma_stages_tflops": flops / (plain * 1e-3) / 1e12,
            }
        line["other_shapes"] = others
    line["hbm_stages"] = hbm_stages(rows, columns, device)
    if args.layer:
        line["layer"] = run_layer(device)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(args.shape, args.rank, full_init=args.cpu_full_init)
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
