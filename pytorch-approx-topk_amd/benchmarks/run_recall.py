#!/usr/bin/env python3
"""Recall of the approximate top-k against exact torch.topk, as JSON lines.

Definitions follow the reference: top-k recall = mean over rows of
count(approx >= true k-th value) / k and top-50 recall likewise against the
true 50th value (benchmarks/run_recall.py:27-36); `coverage` at r = the
fraction of rows whose r-th best result is the true r-th best value, both
sides sorted -- what the reference plots as cumulative recall
(benchmarks/run_cumulative_recall.py:31-42: mean over rows of true_top[:, r]
== approx_top[:, r]).  `contains_top` at r, beside it, is what that script's
docstring describes: the fraction of rows whose result holds all of the true
top-r.  Same inputs as there: 100 rows of
n = 16*32*40, uniform and log-normal.  The closed form for uniformly scattered
top-k elements (notebooks/theoretical_models.py:9-12) is printed beside the
measured top-k recall.

    python pytorch-approx-topk_amd/benchmarks/run_recall.py [--out recall.jsonl]
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from approx_topk import topk as approx_topk  # noqa: E402

N_ROWS, N = 100, 16 * 32 * 40


def closed_form(k: int, buckets: int, per_bucket: int) -> float:
    from scipy.stats import binom
    return float((per_bucket + binom.cdf(per_bucket - 1, np.arange(per_bucket, k), 1.0 / buckets).sum()) / k)


def recalls(xs: torch.Tensor, k: int, j: int) -> dict:
    exact = torch.topk(xs, k, dim=-1, sorted=True).values
    approx = approx_topk(xs, k, -1, j=j)[0].sort(dim=-1, descending=True).values
    top50 = float(((approx >= exact[:, 49:50]).sum(-1) / 50).mean())
    topk = float(((approx >= exact[:, k - 1:k]).sum(-1) / k).mean())
    same = exact == approx                                    # position r holds the true r-th value
    ranks = [r for r in (1, 10, 100, k) if r <= k]
    coverage = {r: float(same[:, r - 1].float().mean()) for r in ranks}
    contains_top = {r: float(same[:, :r].all(dim=-1).float().mean()) for r in ranks}
    return dict(top50=top50, topk=topk, coverage=coverage, contains_top=contains_top)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default="recall.jsonl")
    args = ap.parse_args()
    gen = torch.Generator(device="cuda").manual_seed(0)
    inputs = {"uniform": torch.rand(N_ROWS, N, device="cuda", generator=gen),
              "log normal": torch.randn(N_ROWS, N, device="cuda", generator=gen).exp()}
    with open(args.out, "w") as out:
        for name, xs in inputs.items():
            for k in range(1024, N, 1024):
                for j in (1, 2, 4):
                    if k % j or k > N:
                        continue
                    row = dict(distribution=name, n=N, k=k, j=j, expected_topk=closed_form(k, k // j, j),
                               **recalls(xs, k, j))
                    print(json.dumps(row), file=out, flush=True)
                    print(f"{name} k={k} j={j}: top-k recall {row['topk']:.4f} (closed form "
                          f"{row['expected_topk']:.4f}), top-50 recall {row['top50']:.4f}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
