#!/usr/bin/env python3
"""Benchmark of the bucketed approximate top-k hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--headline-only]

A "step" is one ``approx_topk.topk`` call over one batch of synthetic input that
already sits in HBM.  The headline workload (``value``, ``roofline``) is C2: fp32
x[128, 2^20] iid N(0,1), k = 65536, j = 2, k_mult = 1 (32768 interleaved buckets
of 32).  The other benchmark configurations (C1, C3, C4, C5) are timed the same
way and reported under ``other_configs``.  Inputs rotate over several distinct
tensors so that the working set is larger than the last-level cache.  One JSON
line is printed on stdout.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "pytorch-approx-topk_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth

# HBM bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE scaled by a copy of known size), keyed by
# the kernels the planner reports for the call: a change of plan leaves the figure out (null)
# rather than stale.  Source: profiles/stream_kernel_f32_j2_c2_hbm_traffic.md.
MEASURED_TRAFFIC_BYTES = {
    "stream_kernel<f32, J=2, V=4, W=8, U=8, RUN=4, PACKED=0> grid=16384 block=512 fold=1 slabs=1": 637_658_986,
    # profiles/hbm_traffic_c1_c3_c4_c5.md (C5: the sum of its three kernels)
    "stream_kernel<f32, J=1, V=4, W=8, U=8, RUN=8, PACKED=0> grid=16 block=512 fold=1 slabs=1": 1_209_344,
    "fused_regs_kernel<f16, J=4, V=4, pos16, PACKED=1> grid=1024 block=512 tiles=8 split=1 lds=32768 staged past-cache": 88597838,
    "fused_regs_kernel<f32, J=1, V=4, pos16, PACKED=0> grid=256 block=512 tiles=2 split=4 lds=19584 staged": 134_724_608,
    "stream_kernel<f32, J=4, V=4, W=4, U=8, RUN=0, PACKED=0> grid=256 block=256 fold=1 slabs=8 + "
    "stream_merge_kernel<f32, J=4> + chain_solo_kernel<f32> grid=32 block=1024": 275_389_132,
}

# name -> (rows, n, dtype, k, j, k_mult, seed)
CONFIGS = {
    "C1": (4, 65536, "float32", 1024, 1, 1, 1001),
    "C2": (128, 1 << 20, "float32", 65536, 2, 1, 1002),
    "C3": (1024, 32768, "float16", 2048, 4, 4, 1003),
    "C4": (256, 131072, "float32", 64, 1, 8, 1004),
    "C5": (1, 1 << 26, "float32", 16384, 4, 2, 1005),
}
# closed-form expected recall for iid inputs (C4 and C5 are not iid: informative only)
EXPECTED_RECALL = {"C1": 0.6323, "C2": 0.7293, "C3": 0.9957, "C4": 0.9409, "C5": 0.9624}


def make_input(name: str, variant: int = 0):
    """Synthetic input of a config, generated on the CPU from a fixed seed."""
    import numpy as np
    import torch

    rows, n, dtype, k, j, km, seed = CONFIGS[name]
    g = torch.Generator().manual_seed(seed + 7919 * variant)
    if name == "C3":
        x = (torch.randn(rows, n, generator=g) / math.sqrt(128.0)).half()
    elif name == "C4":
        x = torch.randn(rows, n, generator=g)
        rng = np.random.default_rng(seed + 7919 * variant)
        hot = n // 100
        for r in range(rows):
            cols = torch.randperm(n, generator=g)[:hot]
            x[r, cols] += torch.from_numpy(rng.zipf(1.1, hot).astype(np.float32))
    elif name == "C5":
        x = 0.5 * torch.linspace(-1, 1, n).reshape(1, n) + torch.randn(rows, n, generator=g)
    else:
        x = torch.randn(rows, n, generator=g)
    return x


def device_inputs(name: str, n_inputs: int, distinct: bool):
    """`n_inputs` tensors of the config's workload in HBM.  `distinct`: each from its own seed;
    else the first from its seed and the others derived from it on the GPU (rows rotated, or, for a
    single row, the row rotated by a multiple of the bucket count, which keeps every bucket's
    content): the same values and statistics at other addresses, without the CPU generation time."""
    import torch

    rows, n, dtype, k, j, km, seed = CONFIGS[name]
    first = make_input(name)
    xs = [first.cuda()]
    for v in range(1, n_inputs):
        if distinct:
            xs.append(make_input(name, v).cuda())
        elif rows > 1:
            xs.append(torch.roll(xs[0], shifts=v * max(1, rows // n_inputs), dims=0).contiguous())
        else:
            xs.append(torch.roll(xs[0], shifts=v * (k * km // j) * 64, dims=1).contiguous())
    return first, xs


def recall_at_k(approx_values, exact_values, k: int) -> float:
    """mean over rows of count(approx >= k-th exact value) / k
    (definition of benchmarks/run_recall.py:31-36 in the reference)."""
    kth = exact_values.min(dim=-1, keepdim=True).values
    return float(((approx_values >= kth).sum(-1).double() / k).mean())


def settle_clocks(x, k, j, km, seconds: float = 0.05):
    """An idle GPU runs its first ~100 launches 10-25 % slower: keep it busy for a moment
    before the warm-up steps (untimed, not counted as steps)."""
    import torch

    from approx_topk import topk

    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(16):
            topk(x, k, -1, j=j, k_mult=km)
        torch.cuda.synchronize()


def time_steps(fn, xs, steps: int, warmup: int):
    """(wall seconds, device milliseconds between HIP events on the launch stream) for `steps` calls."""
    import torch

    n_inputs = len(xs)
    for s in range(warmup):
        fn(xs[s % n_inputs])
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for s in range(steps):
        fn(xs[s % n_inputs])
    stop.record()
    torch.cuda.synchronize()
    return time.perf_counter() - t0, start.elapsed_time(stop)


def time_graphed(name: str, xs, steps: int) -> float:
    """Device microseconds per call with the calls replayed from a HIP graph (one call per
    rotating input captured, replayed until at least `steps` calls have run): what a caller
    that captures its step pays, without the host's launch path between the kernels."""
    import torch

    from approx_topk import topk

    rows, n, dtype, k, j, km, seed = CONFIGS[name]
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):          # capture needs a warm allocator and a side stream
        for x in xs:
            topk(x, k, -1, j=j, k_mult=km)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for x in xs:
            topk(x, k, -1, j=j, k_mult=km)
    replays = max(2, -(-steps // len(xs)))
    for _ in range(2):
        graph.replay()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(replays):
        graph.replay()
    stop.record()
    torch.cuda.synchronize()
    us = start.elapsed_time(stop) * 1e3 / (replays * len(xs))
    del graph
    return us


def time_config(name: str, steps: int, warmup: int, n_inputs: int, distinct: bool = True):
    import torch

    from approx_topk import topk

    rows, n, dtype, k, j, km, seed = CONFIGS[name]
    esize = 2 if dtype == "float16" else 4
    # enough distinct inputs to exceed a 256 MiB last-level cache
    per = rows * n * esize
    n_inputs = max(n_inputs, min(8, -(-(600 << 20) // per)))
    first, xs = device_inputs(name, n_inputs, distinct)
    torch.cuda.synchronize()
    settle_clocks(xs[0], k, j, km)
    wall, dev_ms = time_steps(lambda x: topk(x, k, -1, j=j, k_mult=km), xs, steps, warmup)
    return first, xs, wall, dev_ms, rows * n, per


def time_int32_indices(name: str, xs, steps: int, warmup: int):
    """int32 against int64 indices, and int32 indices alone (no values written), from
    approx_topk.experimental.compact_indices, timed alike and alternately: device microseconds
    per call of each, and whether the results are equal."""
    import torch

    from approx_topk import topk
    from approx_topk.experimental.compact_indices import topk as topk_i32
    from approx_topk.experimental.compact_indices import topk_indices

    rows, n, dtype, k, j, km, seed = CONFIGS[name]
    best = {"i32": float("inf"), "i64": float("inf"), "only": float("inf")}
    for _ in range(3):
        for tag, fn in (("i64", topk), ("i32", topk_i32), ("only", topk_indices)):
            _, dev_ms = time_steps(lambda x: fn(x, k, -1, j=j, k_mult=km), xs, steps, warmup)
            best[tag] = min(best[tag], dev_ms * 1e3 / steps)
    v32, i32 = topk_i32(xs[0], k, -1, j=j, k_mult=km)
    v64, i64 = topk(xs[0], k, -1, j=j, k_mult=km)
    only = topk_indices(xs[0], k, -1, j=j, k_mult=km)
    same = bool(torch.equal(i32.long(), i64) and torch.equal(v32.view(torch.uint8), v64.view(torch.uint8))
                and torch.equal(only, i32))
    return best["i32"], best["i64"], best["only"], same


def parity_and_recall(name: str, x_cpu, x_gpu, sample_rows: int):
    """Oracle check on a few rows (bit-exact) and recall against exact torch.topk."""
    import torch

    import oracle
    from approx_topk import topk

    rows, n, dtype, k, j, km, seed = CONFIGS[name]
    v, i = topk(x_gpu, k, -1, j=j, k_mult=km)
    exact = torch.topk(x_gpu.float(), k, dim=-1).values
    rec = recall_at_k(v.float(), exact, k)
    take = min(sample_rows, rows)
    ev, ei = oracle.topk(x_cpu[:take], k, -1, j=j, k_mult=km)
    bits = torch.int16 if dtype == "float16" else torch.int32
    ok = bool(torch.equal(v[:take].cpu().view(bits), ev.view(bits)) and torch.equal(i[:take].cpu(), ei))
    return rec, ok, take


def cpu_baseline(name: str):
    """Torch-level bucketed top-k (the reference's CPU-capable algorithm, restated
    in oracle/) timed on this machine's host cores over the full workload."""
    import torch

    import oracle

    rows, n, dtype, k, j, km, seed = CONFIGS[name]
    x = make_input(name)
    oracle.torch_bucketed_topk(x, k, j, km)  # warm-up
    times = []
    for _ in range(3):
        t = time.perf_counter()
        oracle.torch_bucketed_topk(x, k, j, km)
        times.append(time.perf_counter() - t)
    med = sorted(times)[1]
    esize = x.element_size()
    return {
        "value": rows * n * esize / med / 1e9,
        "unit": "GB/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"all {rows} rows of the workload, median of 3 runs after 1 warm-up "
                  f"({med:.3f} s per pass, {rows * n / med / 1e9:.3f} G elem/s, os.cpu_count()={os.cpu_count()})",
    }


def kernels_of(name: str, x_gpu) -> str:
    from approx_topk import _native

    rows, n, dtype, k, j, km, seed = CONFIGS[name]
    return _native.describe(x_gpu, k * km, j, k)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=150, help="untimed steps before the timed ones")
    ap.add_argument("--inputs", type=int, default=5, help="distinct input tensors to rotate over")
    ap.add_argument("--workload", default="C2", choices=sorted(CONFIGS))
    ap.add_argument("--headline-only", action="store_true", help="skip the other configurations")
    ap.add_argument("--all-configs", action="store_true", help="accepted for compatibility: the default now")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-index-variants", action="store_true",
                    help="skip the int32-index and indices-only timings (they launch the same kernel "
                         "with less output, which blurs per-kernel profiles of the workload)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a 512 MiB device copy a few times (a kernel of known traffic for "
                         "scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; rows shard across GPUs with no communication, "
              "but no multi-GPU path is built or measured here. Use --gpus 1.", file=sys.stderr)
        return 2

    import torch

    from approx_topk import _native

    if not torch.cuda.is_available():
        print("bench.py: needs a GPU", file=sys.stderr)
        return 2
    if not os.path.exists(_native.library_path()):
        import __graft_entry__
        __graft_entry__.build()

    name = args.workload
    rows, n, dtype, k, j, km, seed = CONFIGS[name]
    first, xs, wall, dev_ms, elems, in_bytes = time_config(name, args.steps, args.warmup, args.inputs)
    ms_per_step = wall * 1e3 / args.steps
    launch_ms = dev_ms / args.steps  # device time between HIP events on the launch stream
    rec, ok, checked = parity_and_recall(name, first, xs[0], 4)
    kernels = kernels_of(name, xs[0])
    if not args.no_index_variants:
        i32_us, i64_us, only_us, i32_same = time_int32_indices(name, xs, max(50, args.steps // 2),
                                                               max(20, args.warmup // 3))
    esize = in_bytes // elems
    out_bytes = rows * k * (esize + 8)

    result = {
        "metric": f"input HBM GB/s at {dtype} [{rows},{n}] k={k} j={j} k_mult={km}",
        "value": in_bytes / (wall / args.steps) / 1e9,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32" if dtype == "float32" else "f16",
        "data": "synthetic",
        "config": {"workload": f"{name}: {dtype} x[{rows},{n}] iid N(0,1), k={k}, j={j}, k_mult={km}, "
                               f"interleaved buckets, {len(xs)} rotating inputs resident in HBM"},
        "elements_per_s": elems / (wall / args.steps),
        "frac_of_hbm_peak": in_bytes / (wall / args.steps) / 1e9 / HBM_PEAK_GBS,
        "input_plus_output_GBps": (in_bytes + out_bytes) / (wall / args.steps) / 1e9,
        "recall_at_k": rec,
        "oracle_bit_exact": ok,
        "oracle_rows_checked": checked,
        "kernels": kernels,
        "roofline": {
            "bound": "hbm",
            "achieved": in_bytes / (launch_ms * 1e-3) / 1e9,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": in_bytes / (launch_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "traffic": MEASURED_TRAFFIC_BYTES.get(kernels),
            "launch_us": launch_ms * 1e3,
            "algorithmic_bytes_per_launch": in_bytes,
        },
    }
    # not the metric: the operator's contract is int64 indices; shown because the index write is
    # part of what keeps this shape from the read-only rate
    if not args.no_index_variants:
        result["int32_indices"] = {
            "launch_us": i32_us,
            "int64_launch_us_same_loop": i64_us,
            "input_GBps": in_bytes / (i32_us * 1e-6) / 1e9,
            # the indices alone (values == NULL in the C ABI), for consumers that only gather by them
            "indices_only_launch_us": only_us,
            "indices_only_input_GBps": in_bytes / (only_us * 1e-6) / 1e9,
            "equal_to_int64_result": i32_same,
        }
    del xs, first
    torch.cuda.empty_cache()

    if args.calibrate_copy:
        src = torch.randn(128 << 20, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    all_ok = ok
    if not args.headline_only:
        others = {}
        for other in sorted(CONFIGS):
            if other == name:
                continue
            o_rows, o_n, o_dtype, o_k, o_j, o_km, _ = CONFIGS[other]
            o_first, oxs, o_wall, o_dev_ms, o_elems, o_bytes = time_config(
                other, args.steps, args.warmup, args.inputs, distinct=False)
            o_rec, o_ok, o_checked = parity_and_recall(other, o_first, oxs[0], 2)
            all_ok = all_ok and o_ok
            o_s = o_dev_ms * 1e-3 / args.steps
            o_graphed_us = time_graphed(other, oxs, args.steps)
            others[other] = {
                "shape": [o_rows, o_n], "dtype": o_dtype, "k": o_k, "j": o_j, "k_mult": o_km,
                "us_per_step": o_s * 1e6,
                "input_GBps": o_bytes / o_s / 1e9,
                "frac_of_hbm_peak": o_bytes / o_s / 1e9 / HBM_PEAK_GBS,
                "elements_per_s": o_elems / o_s,
                # the same calls replayed from a HIP graph (no host launch path between kernels)
                "us_per_step_in_hip_graph": o_graphed_us,
                "frac_of_hbm_peak_in_hip_graph": o_bytes / (o_graphed_us * 1e-6) / 1e9 / HBM_PEAK_GBS,
                "recall_at_k": o_rec, "recall_closed_form_iid": EXPECTED_RECALL[other],
                "oracle_bit_exact": o_ok, "oracle_rows_checked": o_checked,
                "kernels": kernels_of(other, oxs[0]),
                # HBM bytes per call measured with rocprofv3 on these very kernels, or null
                "traffic": MEASURED_TRAFFIC_BYTES.get(kernels_of(other, oxs[0])),
            }
            del oxs, o_first
            torch.cuda.empty_cache()
        result["other_configs"] = others

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(name)
    print(json.dumps(result))
    return 0 if all_ok else 1


if __name__ == "__main__":
    sys.exit(main())
