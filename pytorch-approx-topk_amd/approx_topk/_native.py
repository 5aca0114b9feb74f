"""ctypes binding of libapprox_topk_hip.so (the C ABI in include/approx_topk_hip.h).

The library is built in-tree by ``pytorch-approx-topk_amd/build.py`` and sits
next to this file.  There is no fallback: if it cannot be loaded, every call
that needs it raises.
"""
from __future__ import annotations

import ctypes
import functools
import os

import torch

INTERLEAVED, BALANCED, CEIL_CHUNK, INTERLEAVED_PADDED = 0, 1, 2, 3

DTYPE_CODE = {
    torch.float32: 0, torch.float16: 1, torch.bfloat16: 2, torch.float64: 3,
    torch.uint8: 4, torch.int8: 5, torch.int16: 6, torch.int32: 7, torch.int64: 8,
}

ABI_VERSION = 3
LIB_NAME = "libapprox_topk_hip.so"

_SIGNATURES = {
    # name: (restype, argtypes)
    "atk_version": (ctypes.c_int, []),
    "atk_strerror": (ctypes.c_char_p, [ctypes.c_int]),
    "atk_stage1_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int64] * 3 + [ctypes.c_int] * 3),
    "atk_stage1": (ctypes.c_int, [ctypes.c_void_p] + [ctypes.c_int64] * 4 + [ctypes.c_int] * 3
                   + [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                      ctypes.c_void_p]),
    "atk_stage1_i32": (ctypes.c_int, [ctypes.c_void_p] + [ctypes.c_int64] * 4 + [ctypes.c_int] * 3
                       + [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                          ctypes.c_void_p]),
    "atk_select_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int64] * 3 + [ctypes.c_int]),
    "atk_select": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int64] * 4
                   + [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                      ctypes.c_size_t, ctypes.c_void_p]),
    "atk_topk_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int64] * 3 + [ctypes.c_int, ctypes.c_int64,
                                                                          ctypes.c_int, ctypes.c_int]),
    "atk_topk_workspace_bytes_at": (ctypes.c_size_t, [ctypes.c_void_p] + [ctypes.c_int64] * 4
                                    + [ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int]),
    "atk_topk": (ctypes.c_int, [ctypes.c_void_p] + [ctypes.c_int64] * 4 + [ctypes.c_int, ctypes.c_int64,
                                                                           ctypes.c_int, ctypes.c_int]
                 + [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                    ctypes.c_void_p]),
    "atk_describe": (ctypes.c_int, [ctypes.c_void_p] + [ctypes.c_int64] * 4
                     + [ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int]
                     + [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_char_p, ctypes.c_size_t]),
    "atk_topk_noalloc": (ctypes.c_int, [ctypes.c_void_p] + [ctypes.c_int64] * 4
                         + [ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int]
                         + [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]),
    "atk_topk_i32": (ctypes.c_int, [ctypes.c_void_p] + [ctypes.c_int64] * 4 + [ctypes.c_int, ctypes.c_int64,
                                                                               ctypes.c_int, ctypes.c_int]
                     + [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                        ctypes.c_void_p]),
}


def library_path() -> str:
    return os.environ.get("APPROX_TOPK_HIP_LIB") or os.path.join(
        os.path.dirname(os.path.abspath(__file__)), LIB_NAME)


@functools.cache
def lib() -> ctypes.CDLL:
    path = library_path()
    if not os.path.exists(path):
        raise RuntimeError(
            f"approx_topk: {path} is missing. Build it with "
            "`python pytorch-approx-topk_amd/build.py` (needs hipcc); there is no fallback path.")
    handle = ctypes.CDLL(path)
    for name, (restype, argtypes) in _SIGNATURES.items():
        fn = getattr(handle, name)
        fn.restype, fn.argtypes = restype, argtypes
    if handle.atk_version() != ABI_VERSION:
        raise RuntimeError(f"approx_topk: {path} has ABI {handle.atk_version()}, expected {ABI_VERSION}")
    return handle


def check(status: int) -> None:
    if status != 0:
        raise RuntimeError(lib().atk_strerror(status).decode())


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return DTYPE_CODE[dtype]
    except KeyError:
        raise RuntimeError(f"approx_topk: unsupported dtype {dtype}") from None


def require_gpu(xs: torch.Tensor) -> None:
    if xs.device.type != "cuda":
        raise RuntimeError(
            f"approx_topk: expected a tensor on a GPU, got device {xs.device}; "
            "the HIP kernels have no CPU path")


def _stream(device: torch.device) -> int:
    """Raw handle of the current stream of `device` (no Python stream object is built)."""
    return torch._C._cuda_getCurrentRawStream(device.index)


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def _on_device(device: torch.device):
    """Makes `device` current for a native call; free when it already is."""
    return _NO_GUARD if device.index == torch.cuda.current_device() else torch.cuda.device(device)


@functools.lru_cache(maxsize=4096)
def _stage1_workspace(rows: int, n: int, k0: int, j: int, layout: int, code: int) -> int:
    return lib().atk_stage1_workspace_bytes(rows, n, k0, j, layout, code)


@functools.lru_cache(maxsize=4096)
def _topk_workspace(misalign: int, rows: int, n: int, step: int, k0: int, j: int, k: int, layout: int,
                    code: int) -> int:
    # the library only looks at the address's alignment: any address with the same one stands for it
    return lib().atk_topk_workspace_bytes_at(4096 + misalign, rows, n, step, k0, j, k, layout, code)


def rows_view(xs: torch.Tensor) -> tuple[torch.Tensor, int, int, int]:
    """(tensor, rows, n, row_stride) with the top-k dim last and unit stride.

    Rows may be spaced by any uniform stride >= n (e.g. a column slice of a
    matrix); anything else is made contiguous.
    """
    n = xs.shape[-1]
    rows = xs.numel() // n if n else 0
    if xs.is_contiguous():  # the common case, without walking the strides
        return xs, rows, n, n
    if xs.ndim == 1:
        return (xs if xs.stride(0) == 1 or n <= 1 else xs.contiguous()), rows, n, n
    uniform = xs.stride(-1) == 1 or n <= 1
    step = xs.stride(-2)
    expect = step
    for d in range(xs.ndim - 2, -1, -1):
        if xs.shape[d] != 1 and xs.stride(d) != expect:
            uniform = False
        expect *= xs.shape[d]
    if not uniform or step < n:
        xs = xs.contiguous()
        step = n
    return xs, rows, n, step


# Per-call constants of a contiguous input, keyed by everything they depend on:
# (rows, n, dtype code, output shape, bound entry point).  One dictionary lookup
# replaces the shape arithmetic on the way to the native call.
_CALLS: dict = {}


def _call_constants(xs: torch.Tensor, k_out: int, two_stage: bool, index_dtype: torch.dtype):
    key = (xs.shape, xs.dtype, k_out, two_stage, index_dtype)
    hit = _CALLS.get(key)
    if hit is None:
        L = lib()
        n = xs.shape[-1]
        rows = xs.numel() // n if n else 0
        narrow = index_dtype != torch.int64
        if two_stage:
            entry = L.atk_topk_i32 if narrow else L.atk_topk
        else:
            entry = L.atk_stage1_i32 if narrow else L.atk_stage1
        hit = (rows, n, dtype_code(xs.dtype), tuple(xs.shape[:-1]) + (k_out,), entry)
        if len(_CALLS) < 4096:
            _CALLS[key] = hit
    return hit


def stage1(xs: torch.Tensor, k0: int, j: int, layout: int, index_dtype: torch.dtype = torch.int64,
           want_values: bool = True) -> tuple[torch.Tensor | None, torch.Tensor]:
    """Per-bucket top-j along the last dim: (values[..., k0], indices[..., k0]).

    ``index_dtype``: torch.int64 (the operator's contract) or torch.int32.
    ``want_values=False``: only the indices are written; values is None."""
    require_gpu(xs)
    step = None
    if not xs.is_contiguous():
        xs, _, _, step = rows_view(xs)
    rows, n, code, shape, entry = _call_constants(xs, k0, False, index_dtype)
    device = xs.device
    values = torch.empty(shape, dtype=xs.dtype, device=device) if want_values else None
    indices = torch.empty(shape, dtype=index_dtype, device=device)
    with _on_device(device):
        need = _stage1_workspace(rows, n, k0, j, layout, code)
        ws = torch.empty(need, dtype=torch.uint8, device=device) if need else None
        status = entry(xs.data_ptr(), rows, n, n if step is None else step, k0, j, layout, code,
                       values.data_ptr() if want_values else None, indices.data_ptr(),
                       ws.data_ptr() if ws is not None else None, need, _stream(device))
    if status != 0:
        check(status)
    return values, indices


def select(cand_values: torch.Tensor, cand_indices: torch.Tensor, k: int,
           index_bound: int) -> tuple[torch.Tensor, torch.Tensor]:
    """Exact top-k of candidates along the last dim, in candidate order."""
    require_gpu(cand_values)
    L = lib()
    cv, ci = cand_values.contiguous(), cand_indices.contiguous()
    k0 = cv.shape[-1]
    rows = cv.numel() // k0 if k0 else 0
    code = dtype_code(cv.dtype)
    shape = list(cv.shape[:-1]) + [k]
    values = torch.empty(shape, dtype=cv.dtype, device=cv.device)
    indices = torch.empty(shape, dtype=torch.int64, device=cv.device)
    with _on_device(cv.device):
        need = L.atk_select_workspace_bytes(rows, k0, k, code)
        ws = torch.empty(need, dtype=torch.uint8, device=cv.device) if need else None
        check(L.atk_select(cv.data_ptr(), ci.data_ptr(), rows, k0, k, index_bound, code,
                           values.data_ptr(), indices.data_ptr(),
                           ws.data_ptr() if ws is not None else None, need, _stream(cv.device)))
    return values, indices


def topk(xs: torch.Tensor, k0: int, j: int, k: int, layout: int, index_dtype: torch.dtype = torch.int64,
         want_values: bool = True) -> tuple[torch.Tensor | None, torch.Tensor]:
    """Stage 1 (k0 candidates) and stage 2 (k survivors) along the last dim."""
    require_gpu(xs)
    step = None
    if not xs.is_contiguous():
        xs, _, _, step = rows_view(xs)
    rows, n, code, shape, entry = _call_constants(xs, k, True, index_dtype)
    device = xs.device
    values = torch.empty(shape, dtype=xs.dtype, device=device) if want_values else None
    indices = torch.empty(shape, dtype=index_dtype, device=device)
    with _on_device(device):
        pitch = n if step is None else step
        need = _topk_workspace(xs.data_ptr() % 16, rows, n, pitch, k0, j, k, layout, code)
        ws = torch.empty(need, dtype=torch.uint8, device=device) if need else None
        status = entry(xs.data_ptr(), rows, n, pitch, k0, j, k, layout, code,
                       values.data_ptr() if want_values else None, indices.data_ptr(),
                       ws.data_ptr() if ws is not None else None, need, _stream(device))
    if status != 0:
        check(status)
    return values, indices


def describe(xs: torch.Tensor, k0: int, j: int, k: int, layout: int = INTERLEAVED,
             values: torch.Tensor | None = None, indices: torch.Tensor | None = None) -> str:
    """The kernels a call on `xs` (top-k along the last dim) would launch, as text.

    The plan depends on the alignment of the output buffers as well: pass the ones the call
    will write (slices of larger buffers may be misaligned); without them the outputs are taken
    to be fresh `torch.empty` tensors, which are at least 256-byte aligned."""
    xs, rows, n, step = rows_view(xs)
    buf = ctypes.create_string_buffer(1024)
    check(lib().atk_describe(xs.data_ptr() if xs.numel() else 4096, rows, n, step, k0, j, k, layout,
                             dtype_code(xs.dtype), values.data_ptr() if values is not None else 4096,
                             indices.data_ptr() if indices is not None else 4096, buf, len(buf)))
    return buf.value.decode()
