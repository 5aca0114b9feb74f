#!/usr/bin/env python3
"""Read bandwidth of every point of a measure_speed.py sweep, as a text table.

Bandwidth = dtype_bytes * n * batch / mean call duration, the quantity the
reference plots (benchmarks/plot_bandwidth.py:41-45); one table per
(batch size, k regime, HIP graphs) with a row per n and a column per method.

    python pytorch-approx-topk_amd/benchmarks/report_bandwidth.py measure_speed.jsonl
"""
from __future__ import annotations

import collections
import json
import sys

BYTES = {"float32": 4, "float16": 2, "bfloat16": 2}


def main(path: str) -> int:
    tables: dict = collections.defaultdict(lambda: collections.defaultdict(dict))
    methods: list[str] = []
    for line in open(path):
        row = json.loads(line)
        mean = sum(row["duration"]) / len(row["duration"])
        regime = "k=64" if row["k"] == 64 else f"k=n/{row['topk_size'] // row['k']}"
        key = (row["batch_size"], regime, row["hip_graphs"])
        gbps = BYTES[row["dtype"]] * row["topk_size"] * row["batch_size"] / mean / 1e9
        method = row["method"] + (" compiled" if row.get("compile") else "")  # under torch.compile: a column of its own
        tables[key][row["topk_size"]][method] = (gbps, mean * 1e6)
        if method not in methods:
            methods.append(method)
    for (batch, regime, graphs), by_n in sorted(tables.items()):
        print(f"\nbatch {batch}, {regime}, HIP graphs {'on' if graphs else 'off'}: GB/s read (us per call)")
        print("n".rjust(8) + "".join(m.replace("approx_topk.topk", "approx").replace("bucketed_argmax.", "").rjust(22) for m in methods))
        for n in sorted(by_n):
            cells = [by_n[n].get(m) for m in methods]
            print(str(n).rjust(8) + "".join(("%.0f (%.1f)" % c if c else "-").rjust(22) for c in cells))
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1] if len(sys.argv) > 1 else "measure_speed.jsonl"))
