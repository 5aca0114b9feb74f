#!/usr/bin/env python3
"""Time of the second stage alone (`atk_select`: the k best of k0 candidates per row, what
`torch.topk` + `gather` do in the reference, approx_topk/priority_queue.py:85-88) on candidate
sets of different make: normal values, the zeros of a ReLU at the cut (thousands of candidates of
one key, told apart by their indices), a handful of distinct values, all equal.

    python pytorch-approx-topk_amd/benchmarks/time_select.py [--rows 1,4] [--candidates 16384,20000,32768]

Calls back to back between two events, microseconds per call; candidate indices are a random
subset of 0..2^22-1 in random order.
"""
from __future__ import annotations

import argparse
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from approx_topk import _native  # noqa: E402

INDEX_BOUND = 1 << 22


def time_select(cand_values: torch.Tensor, cand_indices: torch.Tensor, k: int, steps: int = 20) -> float:
    for _ in range(5):
        _native.select(cand_values, cand_indices, k, INDEX_BOUND)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        _native.select(cand_values, cand_indices, k, INDEX_BOUND)
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e3 / steps


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--rows", default="1,4")
    ap.add_argument("--candidates", default="16384,20000,32768")
    args = ap.parse_args()
    gen = torch.Generator().manual_seed(3)
    for rows in (int(v) for v in args.rows.split(",")):
        for k0 in (int(v) for v in args.candidates.split(",")):
            indices = torch.stack([torch.randperm(INDEX_BOUND, generator=gen)[:k0] for _ in range(rows)]).cuda()
            # (name, candidates, k): with half of the candidates zero, k = 3/4 k0 puts the cut among the zeros
            cases = [
                ("normal fp32", torch.randn(rows, k0, generator=gen), k0 // 2),
                ("relu(normal) fp32, cut among the zeros", torch.randn(rows, k0, generator=gen).clamp(min=0), 3 * k0 // 4),
                ("7 distinct values fp32", torch.randint(-3, 4, (rows, k0), generator=gen).float(), k0 // 2),
                ("all equal fp32", torch.full((rows, k0), 2.0), k0 // 2),
                ("normal fp16", torch.randn(rows, k0, generator=gen).half(), k0 // 2),
                ("relu(normal) fp16, cut among the zeros", torch.randn(rows, k0, generator=gen).clamp(min=0).half(), 3 * k0 // 4),
            ]
            for name, values, k in cases:
                us = time_select(values.cuda(), indices, k)
                print(f"rows={rows} candidates={k0} k={k} {name}: {us:.1f} us", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
