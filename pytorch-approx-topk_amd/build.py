"""Builds libapprox_topk_hip.so for gfx950 with hipcc, in-tree.

    python pytorch-approx-topk_amd/build.py [--force] [--trace]

Every .hip file under csrc/ is compiled to an object (in parallel) and linked
into approx_topk/libapprox_topk_hip.so, next to the Python package that loads
it.  Nothing is linked against libtorch: the library speaks a C ABI only.

--trace builds a second library, approx_topk/libapprox_topk_hip_trace.so, whose long
kernels stamp a clock at their phase boundaries (csrc/atk_trace.h); it is what
benchmarks/phase_timeline.py loads, and nothing else does.
"""
from __future__ import annotations

import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "approx_topk", "libapprox_topk_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wextra",
    # Packed FP32 instructions are kept out of the device code on purpose.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # The float queues compare with the hardware's IEEE '>': subnormals must keep their
    # order (a flush-to-zero compare would tie them with 0 and pick other candidates).
    "-fno-gpu-flush-denormals-to-zero",
]


def _newer(target: str, deps: list[str]) -> bool:
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(d) <= t for d in deps)


def build(force: bool = False, verbose: bool = True, trace: bool = False) -> str:
    obj_dir, lib, flags = OBJ, LIB, list(FLAGS)
    if trace:
        obj_dir, lib, flags = OBJ + "_trace", LIB[:-3] + "_trace.so", flags + ["-DATK_TRACE"]
    os.makedirs(obj_dir, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    headers = sorted(glob.glob(os.path.join(CSRC, "*.h"))) + [
        os.path.join(os.path.dirname(HERE), "include", "approx_topk_hip.h")]
    jobs = []
    objects = []
    for src in sources:
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        objects.append(obj)
        if force or not _newer(obj, [src] + headers):
            jobs.append([HIPCC, *flags, "-c", src, "-o", obj])

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        return cmd, r

    # the translation units with the most kernels first (the per-type instances of the streaming
    # and the one-workgroup-per-row kernels take minutes each), so that none of them is left for the end
    def weight(cmd):
        name = os.path.basename(cmd[-3])
        heavy = ("stage1_stream_f16", "stage1_stream_bf16", "stage1_stream_i16", "fused_row_f16", "fused_row_bf16",
                 "fused_row_i16", "fused_row_", "stage1_stream_", "stage2_chain", "stage1_contig_")
        for rank, prefix in enumerate(heavy):
            if name.startswith(prefix):
                return rank
        return len(heavy)
    jobs.sort(key=weight)
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        for cmd, r in ex.map(run, jobs):
            # hipcc's host pass warns that it does not know the packed-fp32 feature.
            err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
            if r.returncode != 0:
                raise RuntimeError(f"{' '.join(cmd)}\n{r.stdout}\n{r.stderr}")
            if verbose and err.strip():
                print(err, file=sys.stderr)
    if force or jobs or not _newer(lib, objects):
        cmd, r = run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *objects])
        if r.returncode != 0:
            raise RuntimeError(f"{' '.join(cmd)}\n{r.stdout}\n{r.stderr}")
    return lib


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, trace="--trace" in sys.argv))
