#!/usr/bin/env python3
"""Device time per forward of the HIP extension, the eager model and ``torch.compile``.

Behaviour follows the reference workspace's profiler (agent_workdir/utils/profiling.py:29-117):
inputs are built once, each target gets 5 warm-up forwards and ``--iters`` (default 10) timed
forwards on the same tensors under ``torch.profiler`` with GPU activity only, and the figure
reported is the sum of device time of all GPU events divided by the iteration count, in
microseconds. Targets are timed in the order extension, eager, compiled; the result line has
the reference's format. ``--single-run <targets>`` runs the named targets exactly once with no
profiler, so that an external profiler (``rocprofv3 --kernel-trace --stats -- python3 -m
utils.profiling --single-run cuda_extension``) sees one forward.

If the torch profiler reports no GPU events, the time falls back to HIP events around the
timed loop (wall time on the stream, which then includes launch gaps). Which of the two produced
a figure is printed on a ``[timing]`` line per target in front of the result line.

Run from the workspace directory: ``python3 -m utils.profiling``.
"""

import argparse

import torch

from model import Model, get_inputs, get_init_inputs
from model_new import ModelNew

WARMUP_ITERS = 5
TARGETS = ("torch_baseline", "torch_compile", "cuda_extension")


def transform_tensors(tensors, fn):
    if isinstance(tensors, torch.Tensor):
        return fn(tensors)
    if isinstance(tensors, (list, tuple)):
        return [transform_tensors(item, fn) for item in tensors]
    if isinstance(tensors, dict):
        return {key: transform_tensors(item, fn) for key, item in tensors.items()}
    return tensors


def get_prof_ctx():
    return torch.profiler.profile(
        activities=[torch.profiler.ProfilerActivity.CUDA],
        record_shapes=False,
        with_stack=False,
    )


def parse_args(argv=None):
    parser = argparse.ArgumentParser(
        description="Profile cuda_extension vs torch baseline and torch.compile."
    )
    parser.add_argument("--iters", type=int, default=10, help="Benchmark iterations")
    parser.add_argument(
        "--single-run",
        type=str,
        help="Run once for targets: torch_baseline,torch_compile,cuda_extension",
    )
    return parser.parse_args(argv)


def initialize_models():
    init_inputs = get_init_inputs()
    if not isinstance(init_inputs, (list, tuple)):
        init_inputs = [init_inputs]

    torch_model = Model(*init_inputs).eval().cuda()
    cuda_model = ModelNew(*init_inputs).eval().cuda()
    cuda_model.load_state_dict(torch_model.state_dict())

    torch_inputs = get_inputs()
    if not isinstance(torch_inputs, (list, tuple)):
        torch_inputs = [torch_inputs]
    torch_inputs = transform_tensors(torch_inputs, lambda t: t.cuda())
    cuda_inputs = transform_tensors(torch_inputs, lambda t: t.clone())
    return torch_model, cuda_model, torch_inputs, cuda_inputs


def benchmark_model(model, inputs, warmup_iters, run_iters, label="model"):
    """Mean GPU time per forward in microseconds."""
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    with torch.no_grad():
        for _ in range(warmup_iters):
            model(*inputs)

        with get_prof_ctx() as prof:
            torch.cuda.synchronize()
            start.record()
            for _ in range(run_iters):
                model(*inputs)
            stop.record()
            torch.cuda.synchronize()

    device_events = [e for e in prof.events() if e.device_type.name == "CUDA"]
    device_us = sum(e.device_time for e in device_events)
    event_us = start.elapsed_time(stop) * 1e3
    if device_us > 0:
        print(f"[timing] {label}: profiler device time, {len(device_events)} GPU events "
              f"(stream time by events {event_us / run_iters:.3f}us)")
        return device_us / run_iters
    print(f"[timing] {label}: the profiler reported no GPU events, stream time by events")
    return event_us / run_iters


def print_results(torch_time, compile_time, cuda_time):
    print(
        f"Torch Baseline: {torch_time:.3f}us, "
        f"Torch Compile: {compile_time:.3f}us, "
        f"CUDA Extension: {cuda_time:.3f}us"
    )


def run_single(targets, torch_model, cuda_model, torch_inputs, cuda_inputs):
    with torch.no_grad():
        if "torch_baseline" in targets:
            torch_model(*torch_inputs)
        if "torch_compile" in targets:
            torch.compile(torch_model)(*torch_inputs)
        if "cuda_extension" in targets:
            cuda_model(*cuda_inputs)
    torch.cuda.synchronize()
    print("[DONE] single-run completed")


def main(argv=None):
    args = parse_args(argv)
    torch_model, cuda_model, torch_inputs, cuda_inputs = initialize_models()

    if args.single_run:
        targets = [name.strip() for name in args.single_run.split(",") if name.strip()]
        run_single(targets, torch_model, cuda_model, torch_inputs, cuda_inputs)
        return

    torch_compile_model = torch.compile(torch_model)

    cuda_time = benchmark_model(cuda_model, cuda_inputs, WARMUP_ITERS, args.iters, "cuda_extension")
    torch_time = benchmark_model(torch_model, torch_inputs, WARMUP_ITERS, args.iters, "torch_baseline")
    compile_time = benchmark_model(torch_compile_model, torch_inputs, WARMUP_ITERS, args.iters, "torch_compile")
    print_results(torch_time, compile_time, cuda_time)


if __name__ == "__main__":
    main()
