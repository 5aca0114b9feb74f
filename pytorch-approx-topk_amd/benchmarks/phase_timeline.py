"""Where the time of one launch goes: phase boundaries per workgroup, from the clock stamps of a
library built with `python pytorch-approx-topk_amd/build.py --trace` (csrc/atk_trace.h).

    python pytorch-approx-topk_amd/benchmarks/phase_timeline.py fused  float16:1024:32768:2048:4:4
    python pytorch-approx-topk_amd/benchmarks/phase_timeline.py stream float32:1:67108864:16384:4:2
    python pytorch-approx-topk_amd/benchmarks/phase_timeline.py solo   float32:1:67108864:16384:4:2

A shape is dtype:rows:n:k:j:k_mult.  `fused` reads the stamps of fused_regs_kernel (both stages
in one kernel), `stream` those of stream_kernel (stage 1; every wave's scan and the workgroup's
end), `solo` those of chain_solo_kernel (stage 2 of few rows of up to 32768 candidates in one launch).  The call is repeated back to back and the stamps are those of the last launch; times are
microseconds since the first workgroup's start (the 100 MHz clock that every compute unit reads
alike), as minimum / median / maximum over the workgroups, then by XCD (workgroup number mod 8).
The stamps cost the kernel a little: its duration here is 1-3 % above the product library's.
"""
from __future__ import annotations

import argparse
import ctypes
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
TRACE_LIB = os.path.join(os.path.dirname(HERE), "approx_topk", "libapprox_topk_hip_trace.so")
os.environ.setdefault("APPROX_TOPK_HIP_LIB", TRACE_LIB)

import numpy as np  # noqa: E402
import torch  # noqa: E402

from approx_topk import _native, topk  # noqa: E402

SLOTS, GROUPS = 20, 16384  # csrc/atk_trace.h
SHORT = {"float16": "f16", "float32": "f32"}
SOLO_PHASES = ["start", "keys in registers, the digit's place known", "histogram counted", "cut digit found",
               "members of the cut digit listed", "list ranked, earlier survivors counted", "written"]
FUSED_PHASES = ["start", "first wave's scan done", "all waves done, histograms cleared", "first radix pass",
                "last of the later passes", "cut known", "survivors placed", "survivors staged", "written"]


def three(a):
    return "%7.2f %7.2f %7.2f" % (a.min(), np.median(a), a.max())


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("kernel", choices=["fused", "stream", "solo"])
    ap.add_argument("shape")
    ap.add_argument("--calls", type=int, default=40, help="back-to-back calls before the stamps are read")
    ap.add_argument("--contiguous", action="store_true")
    args = ap.parse_args()
    f = args.shape.split(":")
    dtype = getattr(torch, f[0])
    rows, n, k, j, k_mult = map(int, f[1:6])
    xs = [torch.randn(rows, n, device="cuda").to(dtype) for _ in range(3)]
    kw = dict(j=j, k_mult=k_mult, interleaved=not args.contiguous)
    plan = _native.describe(xs[0], k * k_mult, j, k, _native.INTERLEAVED if not args.contiguous else _native.BALANCED)
    print(plan)
    unit = {"fused": "fused_row_" + SHORT[f[0]], "stream": "stage1_stream_" + SHORT[f[0]],
            "solo": "stage2_chain_select"}[args.kernel]
    reader = getattr(_native.lib(), "atk_trace_" + unit)
    reader.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
    for s in range(args.calls):
        topk(xs[s % 3], k, -1, **kw)
    torch.cuda.synchronize()
    buf = np.zeros((GROUPS, SLOTS), dtype=np.uint64)
    rc = reader(buf.ctypes.data, buf.nbytes)
    assert rc == 0, rc
    t = buf.astype(np.float64) * 0.01  # microseconds
    if args.kernel == "fused":
        groups = rows
        t = t[:groups]
        t0 = t[:, 0].min()
        print("%-36s %7s %7s %7s" % ("us since the first workgroup's start", "min", "median", "max"))
        cols = []
        for i, name in enumerate(FUSED_PHASES):
            c = t[:, i] - t0
            if (t[:, i] == 0).all() or c.min() < 0:
                continue  # a phase this launch did not go through
            cols.append(i)
            print("%-36s %s" % (name, three(c)))
        d = np.diff(t[:, cols], axis=1)
        print("median time between them:", " ".join("%.2f" % v for v in np.median(d, axis=0)))
        first, last = 0, cols[-1]
        for x in range(8):
            s = t[x::8] - t0
            print("XCD %d: start %s | scan done %s | written %s" % (x, three(s[:, first]), three(s[:, 1]), three(s[:, last])))
        end = t[:, last] - t0
        scan = t[:, 1] - t0
        print("deciles of scan done:", np.round(np.sort(scan)[:: max(1, groups // 10)], 1))
        print("deciles of written:  ", np.round(np.sort(end)[:: max(1, groups // 10)], 1))
    elif args.kernel == "solo":
        groups = int(plan.split("chain_solo_kernel")[1].split("grid=")[1].split()[0])
        t = t[:groups]
        t0 = t[:, 0].min()
        print("%-44s %7s %7s %7s" % ("us since the first workgroup's start", "min", "median", "max"))
        for i, name in enumerate(SOLO_PHASES):
            print("%-44s %s" % (name, three(t[:, i] - t0)))
    else:
        grid = int(plan.split("grid=")[1].split()[0])
        waves = int(plan.split("block=")[1].split()[0]) // 64
        groups = min(grid, GROUPS)
        t = t[:groups]
        st, en, fin = t[:, 0:2 * waves:2], t[:, 1:2 * waves:2], t[:, 16]
        t0 = st.min()
        print("%-36s %7s %7s %7s" % ("us since the first wave's start", "min", "median", "max"))
        print("%-36s %s" % ("a wave starts its scan", three(st - t0)))
        print("%-36s %s" % ("a wave's scan is done", three(en - t0)))
        print("%-36s %s" % ("a wave's scan takes", three(en - st)))
        print("%-36s %s" % ("the workgroup's last scan is done", three(en.max(axis=1) - t0)))
        print("%-36s %s" % ("the workgroup has written", three(fin - t0)))
        print("%-36s %s" % ("... after its last scan", three(fin - en.max(axis=1))))
        for x in range(8):
            print("XCD %d: start %s | scans done %s | written %s" % (x, three(st[x::8] - t0), three(en[x::8] - t0), three(fin[x::8] - t0)))
        print("deciles of the waves' scan done:", np.round(np.sort((en - t0).ravel())[:: max(1, en.size // 10)], 1))


if __name__ == "__main__":
    main()
