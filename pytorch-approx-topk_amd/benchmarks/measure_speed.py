#!/usr/bin/env python3
"""Runtime sweep of exact and approximate top-k on one GPU, written as JSON lines.

Covers the grid of the reference's benchmarks/measure_speed.py:264-327
(n in 2^12..2^16, batch in {128, 32}, k in {64, n/8}, fp32; torch.topk, the
approximate top-k at j in {1, 2, 4}, and the torch-level bucketed arg-max, the last two
also under torch.compile as there, :66-71), once
with plain launches and once with the inner loop captured in a HIP graph, timed
with events as benchmarks/measure_speed.py:98-146 does, a device-side spin queued
ahead of every timed repetition included (:141): the host gets ahead of the GPU
while the spin runs, so that the events bracket the kernels and not the time the
host needs to enqueue them.  Every line carries the
per-call durations in seconds; input bandwidth is dtype_bytes * n * batch / mean
(benchmarks/plot_bandwidth.py:41-45).

    python pytorch-approx-topk_amd/benchmarks/measure_speed.py [--out results.jsonl] [--quick]

`--shapes` times given shapes in steady state (calls back to back); `--reference-rows` times instead the
shapes of the measurements the reference keeps of itself
(fp16, batch 256 or 1, an H100 PCIe: notebooks/data/generic2/measure_speed_approx_finer_multi2.jsonl
and measure_speed_exact_finer.jsonl), for orientation beside those figures.
"""
from __future__ import annotations

import argparse
import itertools
import json
import os
import sys
from typing import Any, Callable

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from approx_topk import topk as approx_topk  # noqa: E402
from approx_topk.experimental import bucketed_argmax  # noqa: E402


def exact_topk(xs, k, dim):
    return torch.topk(xs, k, dim, sorted=False)


# Device clock ticks the GPU spins before each timed repetition (torch.cuda._sleep; the reference
# spins 10 M cycles, several milliseconds).  Long enough for the host to enqueue `n_inner` calls
# and the closing event behind it: ~100 us cover a few un-graphed calls or one graph launch.
HIDE_LAUNCH_CYCLES = 200_000


def time_calls(call: Callable[[int], Any], refresh: Callable[[], None], n_outer: int, n_inner: int,
               graph: bool, n_warmup: int = 16, hide_launch_cycles: int = HIDE_LAUNCH_CYCLES) -> list[float]:
    """Seconds per call for `n_outer` timed repetitions of `n_inner` calls each.

    `hide_launch_cycles` > 0 queues a device-side spin of that many clock ticks ahead of the
    opening event of every repetition (benchmarks/measure_speed.py:135-146 in the reference)."""
    def inner():
        return [call(i) for i in range(n_inner)]

    run = inner
    if graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            refresh()
            inner()
        torch.cuda.current_stream().wait_stream(side)
        captured = torch.cuda.CUDAGraph()
        with torch.cuda.graph(captured):
            keep = inner()  # noqa: F841  (outputs stay alive with the graph)
        run = captured.replay
    for _ in range(n_warmup):
        refresh()
        run()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
              for _ in range(n_outer)]
    for start, stop in events:
        refresh()
        if hide_launch_cycles > 0:
            torch.cuda._sleep(hide_launch_cycles)
        start.record()
        run()
        stop.record()
    torch.cuda.synchronize()
    return [start.elapsed_time(stop) / 1e3 / n_inner for start, stop in events]


def compiled_method(fn: Callable) -> Callable:
    """`fn` under torch.compile as the reference's sweep compiles its methods
    (benchmarks/measure_speed.py:66-71): mode "default", one graph, static shapes."""
    torch.compiler.reset()
    return torch.compile(fn, mode="default", fullgraph=True, dynamic=False)


# (batch, n, k, j, k_mult) of the reference's own recorded rows, fp16, and the method they timed
REFERENCE_ROWS = (
    [("approx_topk.topk", 256, 1 << 20, k, j, 1) for k in (65536, 16384) for j in (1, 2, 4)]
    + [("approx_topk.topk", 256, 65536, 4096, 4, km) for km in (1, 2, 4, 8)]
    + [("approx_topk.topk", 256, 262144, 64, 1, 8),
       ("approx_topk.topk", 1, 4194304, 16384, 4, 2),
       ("approx_topk.topk", 256, 1 << 22, 4, 1, 2),
       ("bucketed_argmax.topk_torch", 256, 1 << 20, 65536, 1, 1),
       ("bucketed_argmax.topk_triton", 256, 1 << 20, 65536, 1, 1),
       ("bucketed_argmax.topk_torch", 256, 1 << 22, 4096, 1, 1),
       ("bucketed_argmax.topk_triton", 256, 1 << 22, 4096, 1, 1),
       ("torch.topk", 256, 1 << 20, 65536, 1, 1)])


def reference_rows(out_path: str, quick: bool, only: list[int] | None = None, steady: bool = False) -> int:
    """`steady`: 30 calls back to back per repetition over the resident inputs, which are filled once,
    with no spin ahead of them: the rate of a loop of calls rather than of a call on fresh data."""
    device = torch.cuda.get_device_name()
    rows = REFERENCE_ROWS if only is None else [REFERENCE_ROWS[i] for i in only]
    with open(out_path, "w") as out:
        for name, batch, n, k, j, km in rows:
            # two or three rotating inputs: together larger than the 256 MiB last-level cache
            n_inputs = 3 if batch * n * 2 < (1 << 30) else 2
            n_inner = 30 if steady else n_inputs
            xs = torch.zeros(n_inputs, batch, n, device="cuda", dtype=torch.float16)
            xs.normal_()
            if name == "approx_topk.topk":
                call = lambda i: approx_topk(xs[i % n_inputs], k=k, dim=1, j=j, k_mult=km)[0]          # noqa: E731
            elif name == "bucketed_argmax.topk_torch":
                call = lambda i: bucketed_argmax.topk_torch(xs[i % n_inputs], k=k, dim=1, interleaved=True)[0]   # noqa: E731
            elif name == "bucketed_argmax.topk_triton":
                call = lambda i: bucketed_argmax.topk_triton(xs[i % n_inputs], k=k, dim=1, interleaved=True)[0]  # noqa: E731
            else:
                call = lambda i: exact_topk(xs[i % n_inputs], k, 1)[0]                                  # noqa: E731
            for graph in (False, True):
                if steady:
                    durations = time_calls(call, lambda: None, n_outer=4 if quick else 8, n_inner=n_inner,
                                           graph=graph, n_warmup=2, hide_launch_cycles=0)
                else:
                    durations = time_calls(call, lambda: xs.normal_(), n_outer=8 if quick else 32, n_inner=n_inner,
                                           graph=graph, n_warmup=4)
                mean = sum(durations) / len(durations)
                row = dict(method=name, args=dict(j=j, k_mult=km), batch_size=batch, topk_size=n, k=k,
                           dtype="float16", hip_graphs=graph, n_inner=n_inner, steady=steady, duration=durations,
                           input_GBps=2 * n * batch / mean / 1e9, device=device)
                print(json.dumps(row), file=out, flush=True)
                print(f"{name} fp16 [{batch}, {n}] k={k} j={j} k_mult={km} graph={graph}"
                      f"{' steady' if steady else ''}: {mean * 1e6:.1f} us, {row['input_GBps']:.0f} GB/s", flush=True)
            del xs
            torch.cuda.empty_cache()
    return 0


DTYPES = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16, "int32": torch.int32,
          "int16": torch.int16, "uint8": torch.uint8}


def time_shapes(spec: str, out_path: str) -> int:
    """Steady-state time per call of `approx_topk.topk` at given shapes, beside the planner's description.

    `spec`: shapes separated by ';', each dtype:rows:n:k:j:k_mult[:layout[:data]] with layout `interleaved`
    (default) or `contiguous` and data `normal` (default) or `sparse` (relu(N(0,1) - 2.5): 0.6 % of the elements
    are positive, the rest zeros; with buckets of around a hundred elements most candidates are zeros, and so is
    the cut: thousands of candidates of one key, told apart by their indices)."""
    from approx_topk import _native
    device = torch.cuda.get_device_name()
    with open(out_path, "w") as out:
        for item in spec.split(";"):
            f = item.strip().split(":")
            dtype, (rows, n, k, j, km) = DTYPES[f[0]], (int(v) for v in f[1:6])
            interleaved = len(f) < 7 or f[6] == "interleaved"
            data = f[7] if len(f) > 7 else "normal"
            n_inputs = max(2, min(8, (1 << 29) // max(1, rows * n * torch.empty(0, dtype=dtype).element_size())))
            base = torch.randn(n_inputs, rows, n, device="cuda")
            if data == "sparse":
                base = torch.relu(base - 2.5)
            xs = (base * (30 if not dtype.is_floating_point else 1)).to(dtype)
            del base
            call = lambda i: approx_topk(xs[i % n_inputs], k=k, dim=1, j=j, k_mult=km, interleaved=interleaved)[0]  # noqa: E731
            durations = time_calls(call, lambda: None, n_outer=8, n_inner=30, graph=False, n_warmup=2,
                                   hide_launch_cycles=0)
            mean = sum(durations) / len(durations)
            kernels = _native.describe(xs[0], k * km, j, k, layout=_native.INTERLEAVED if interleaved else 1)
            row = dict(method="approx_topk.topk", args=dict(j=j, k_mult=km, interleaved=interleaved), data=data,
                       batch_size=rows, topk_size=n, k=k, dtype=f[0], duration=durations, kernels=kernels,
                       input_GBps=xs.element_size() * n * rows / mean / 1e9, device=device)
            print(json.dumps(row), file=out, flush=True)
            print(f"{f[0]} [{rows}, {n}] k={k} j={j} k_mult={km} {'interleaved' if interleaved else 'contiguous'} "
                  f"{data}: {mean * 1e6:.1f} us, {row['input_GBps']:.0f} GB/s | {kernels}", flush=True)
            del xs
            torch.cuda.empty_cache()
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default="measure_speed.jsonl")
    ap.add_argument("--quick", action="store_true", help="fewer repetitions")
    ap.add_argument("--no-compile", action="store_true", help="leave out the torch.compile variants")
    ap.add_argument("--reference-rows", action="store_true",
                    help="the shapes of the reference's own recorded measurements (fp16) instead of the grid")
    ap.add_argument("--only", default=None,
                    help="with --reference-rows: comma-separated numbers of the rows to time (for a profiler run)")
    ap.add_argument("--steady", action="store_true",
                    help="with --reference-rows: 30 calls back to back per repetition, inputs filled once, no spin")
    ap.add_argument("--shapes", default=None,
                    help="time these shapes instead: dtype:rows:n:k:j:k_mult[:interleaved|contiguous[:normal|sparse]];...")
    args = ap.parse_args()
    if args.shapes:
        return time_shapes(args.shapes, args.out)
    if args.reference_rows:
        only = None if args.only is None else [int(i) for i in args.only.split(",")]
        return reference_rows(args.out, args.quick, only, args.steady)

    # (name, function, arguments, compiled): as the reference does (benchmarks/measure_speed.py:66-71,
    # 292-296), the approximate top-k and the torch-level arg-max are also timed under
    # torch.compile(mode="default", fullgraph=True, dynamic=False)
    methods: list[tuple[str, Callable, dict, bool]] = [("torch.topk", exact_topk, {}, False)]
    for compiled in (False, True):
        for j in (1, 2, 4):
            methods.append((f"approx_topk.topk j={j}", approx_topk, dict(j=j, k_mult=1), compiled))
        methods.append(("bucketed_argmax.topk_torch", bucketed_argmax.topk_torch, dict(interleaved=True), compiled))

    modes = [dict(graph=False, n_outer=64 if args.quick else 512, n_inner=1),
             dict(graph=True, n_outer=4 if args.quick else 16, n_inner=128)]
    device = torch.cuda.get_device_name()
    with open(args.out, "w") as out:
        for exp, batch, mode in itertools.product([16, 15, 14, 13, 12], [128, 32], modes):
            n = 2 ** exp
            xs = torch.zeros(mode["n_inner"], batch, n, device="cuda")
            for k in (64, n // 8):
                for name, fn, kwargs, compiled in methods:
                    if args.no_compile and compiled:
                        continue
                    method = compiled_method(fn) if compiled else fn
                    durations = time_calls(lambda i: method(xs[i], k=k, dim=1, **kwargs)[0],
                                           lambda: xs.normal_(), **mode)
                    mean = sum(durations) / len(durations)
                    row = dict(method=name, args=kwargs, compile="default" if compiled else None, batch_size=batch,
                               topk_size=n, k=k, dtype="float32",
                               hip_graphs=mode["graph"], n_outer=mode["n_outer"], n_inner=mode["n_inner"],
                               duration=durations, input_GBps=4 * n * batch / mean / 1e9, device=device)
                    print(json.dumps(row), file=out, flush=True)
                    print(f"n=2^{exp} batch={batch} k={k} graph={mode['graph']} {name}"
                          f"{' compiled' if compiled else ''}: "
                          f"{mean * 1e6:.1f} us, {row['input_GBps']:.0f} GB/s", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
