"""CPU oracle for bucketed approximate top-k.  TEST INFRASTRUCTURE ONLY.

Only the tests, the smoke check and the benchmark's CPU-baseline leg may import
this package; the shipped library must never reach it.  The arithmetic lives in
``atk_oracle.c`` (scalar C, each function citing the reference lines it
restates); this module is the ctypes/torch plumbing around it plus the
host-level flow of the reference wrapper:

* ``topk``            approx_topk/priority_queue.py:51-88 (k0 = k*k_mult,
                      stage 1, optional stage 2)
* ``bucketed_argmax`` approx_topk/experimental/bucketed_argmax.py:18-42
                      (k_b = 1 over a row padded to a multiple of k)
* ``torch_bucketed_topk`` approx_topk/experimental/autobucket.py:18-74 restated
                      with torch ops; used as the timed CPU baseline only.

Tie order, NaN rank and output order are this build's choices ("parity
unpinned" against the reference, whose tests never exercise them); see the
header of ``atk_oracle.c``.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libatk_oracle.so")

INTERLEAVED, BALANCED, CEIL_CHUNK, INTERLEAVED_PADDED = 0, 1, 2, 3

_DTYPE_CODE = {
    torch.float32: 0, torch.float16: 1, torch.bfloat16: 2, torch.float64: 3,
    torch.uint8: 4, torch.int8: 5, torch.int16: 6, torch.int32: 7, torch.int64: 8,
}

_lib = None


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (``make -C oracle``)."""
    if force or not os.path.exists(_LIB_PATH):
        if force:
            subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
        subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, vp = ctypes.c_int64, ctypes.c_void_p
        L.atko_stage1.argtypes = [vp, ctypes.c_int, i64, i64, i64, i64, ctypes.c_int, vp, vp]
        L.atko_stage1.restype = ctypes.c_int
        L.atko_stage2.argtypes = [vp, vp, ctypes.c_int, i64, i64, i64, vp, vp]
        L.atko_stage2.restype = ctypes.c_int
        L.atko_bucket_geometry.argtypes = [i64, i64, i64, ctypes.c_int] + [ctypes.POINTER(i64)] * 3
        L.atko_bucket_geometry.restype = ctypes.c_int
        L.atko_key.argtypes = [vp, ctypes.c_int]
        L.atko_key.restype = ctypes.c_uint64
        _lib = L
    return _lib


def bucket_geometry(n: int, b: int, c: int, layout: int) -> tuple[int, int, int]:
    """(start, stride, count) of bucket ``c``."""
    s, st, cnt = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
    rc = lib().atko_bucket_geometry(n, b, c, layout, ctypes.byref(s), ctypes.byref(st), ctypes.byref(cnt))
    if rc:
        raise ValueError(f"bad bucket geometry arguments n={n} b={b} c={c} layout={layout}")
    return s.value, st.value, cnt.value


def key(x: torch.Tensor) -> int:
    """Order key of a one-element tensor."""
    x = x.detach().cpu().contiguous()
    return int(lib().atko_key(x.data_ptr(), _DTYPE_CODE[x.dtype]))


def _rows(x: torch.Tensor) -> tuple[torch.Tensor, int, int]:
    x = x.detach().cpu().contiguous()
    n = x.shape[-1] if x.ndim else 1
    rows = x.numel() // n if n else 0
    return x, rows, n


def stage1(x: torch.Tensor, k0: int, j: int, layout: int = INTERLEAVED):
    """Per-bucket top-``j`` along the last dim -> (values[..., k0], indices[..., k0])."""
    x, rows, n = _rows(x)
    shape = list(x.shape[:-1]) + [k0]
    values = torch.empty(shape, dtype=x.dtype)
    indices = torch.empty(shape, dtype=torch.int64)
    rc = lib().atko_stage1(x.data_ptr(), _DTYPE_CODE[x.dtype], rows, n, k0, j, layout,
                           values.data_ptr(), indices.data_ptr())
    if rc:
        raise RuntimeError(f"oracle stage1 rejected its arguments (code {rc})")
    return values, indices


def stage2(cand_values: torch.Tensor, cand_indices: torch.Tensor, k: int):
    """Exact top-``k`` of the candidates along the last dim, in candidate order."""
    cv, rows, k0 = _rows(cand_values)
    ci = cand_indices.detach().cpu().contiguous()
    shape = list(cv.shape[:-1]) + [k]
    values = torch.empty(shape, dtype=cv.dtype)
    indices = torch.empty(shape, dtype=torch.int64)
    rc = lib().atko_stage2(cv.data_ptr(), ci.data_ptr(), _DTYPE_CODE[cv.dtype], rows, k0, k,
                           values.data_ptr(), indices.data_ptr())
    if rc:
        raise RuntimeError(f"oracle stage2 rejected its arguments (code {rc})")
    return values, indices


def topk(xs: torch.Tensor, k: int, dim: int = -1, j: int = 1, k_mult: int = 1,
         interleaved: bool = True):
    """The whole operator on the CPU, same argument meaning as ``approx_topk.topk``."""
    dim = dim % xs.ndim
    moved = xs.movedim(dim, -1)
    k0 = k * k_mult
    if k0 == 0:
        shape = list(moved.shape[:-1]) + [0]
        v, i = torch.empty(shape, dtype=xs.dtype), torch.empty(shape, dtype=torch.int64)
    else:
        v, i = stage1(moved, k0, j, INTERLEAVED if interleaved else BALANCED)
        if k_mult > 1:
            v, i = stage2(v, i, k)
    return v.movedim(-1, dim), i.movedim(-1, dim)


def bucketed_argmax(xs: torch.Tensor, k: int, dim: int, interleaved: bool):
    """k_b = 1 over the row padded to a multiple of ``k`` with the dtype minimum."""
    dim = dim % xs.ndim
    moved = xs.movedim(dim, -1)
    v, i = stage1(moved, k, 1, INTERLEAVED_PADDED if interleaved else CEIL_CHUNK)
    return v.movedim(-1, dim), i.movedim(-1, dim)


def torch_bucketed_topk(xs: torch.Tensor, k: int, j: int, k_mult: int):
    """Torch-level bucketed top-k (interleaved buckets, last dim) on host cores.

    Restates the flow of approx_topk/experimental/autobucket.py:18-74 with
    ``torch.topk`` as the exact method: view the (padded) row as [L, b], take
    the top ``j`` of every column, rebase the positions to row indices, then a
    final exact top-``k`` over the ``k*k_mult`` candidates.  Used for timing the
    CPU baseline and for value-multiset checks; tie choice is torch's.
    """
    k0 = k * k_mult
    b = k0 // j
    n = xs.shape[-1]
    fill = torch.finfo(xs.dtype).min if xs.dtype.is_floating_point else torch.iinfo(xs.dtype).min
    short = (-n) % b
    grid = torch.nn.functional.pad(xs, (0, short), value=fill) if short else xs
    grid = grid.reshape(*xs.shape[:-1], -1, b)            # [.., L, b]
    val0, sub = torch.topk(grid, j, dim=-2, sorted=False)  # [.., j, b]
    idx0 = sub * b + torch.arange(b, dtype=torch.int64)
    val0, idx0 = val0.flatten(-2), idx0.flatten(-2)
    val, pick = torch.topk(val0, k, dim=-1, sorted=False)
    return val, idx0.gather(-1, pick)
