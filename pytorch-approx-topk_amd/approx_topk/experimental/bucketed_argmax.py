"""Bucketed arg-max: the k_b = 1 special case, over a row padded to a multiple of k.

Entry points and argument meaning follow the reference's
approx_topk/experimental/bucketed_argmax.py:18-42 (``topk_torch``) and
:145-202 (``topk_triton``).  ``topk_triton`` keeps its name and signature for
drop-in use but runs the library's HIP stage-1 kernel at one element per
bucket; ``block_size`` and ``kernel`` are accepted and have no effect.
"""
from __future__ import annotations

from typing import Any, Literal

import torch
from torch import Tensor

from .. import _native


def _min_value(dtype: torch.dtype) -> Any:
    info = torch.finfo(dtype) if dtype.is_floating_point else torch.iinfo(dtype)
    return info.min


def topk_torch(xs: Tensor, k: int, dim: int, interleaved: bool) -> tuple[Tensor, Tensor]:
    """Torch-level bucketed arg-max (any device, any ``dim``).

    The slice is padded with the dtype minimum to ``k * m``, ``m = ceil(n/k)``.
    Interleaved buckets are the columns of the ``[m, k]`` view, contiguous ones
    the rows of the ``[k, m]`` view; each bucket yields its maximum and the
    position (in the padded slice) of its first occurrence.
    """
    dim %= xs.ndim
    n = xs.shape[dim]
    m = -(-n // k)
    trailing = xs.ndim - 1 - dim
    padded = torch.nn.functional.pad(xs, (0, 0) * trailing + (0, k * m - n), value=_min_value(xs.dtype))
    bucket_ids = torch.arange(k, dtype=torch.int64, device=xs.device).reshape((k,) + (1,) * trailing)
    if interleaved:
        best = padded.unflatten(dim, (m, k)).max(dim=dim)
        return best.values, best.indices * k + bucket_ids
    best = padded.unflatten(dim, (k, m)).max(dim=dim + 1)
    return best.values, best.indices + bucket_ids * m


def _batch_contiguous(x: Tensor) -> Tensor:
    """``x`` itself when one row pitch addresses the whole batch, else a copy.

    The native entry takes a base pointer, a row count and one pitch in
    elements, so every row must start ``pitch`` elements after the previous one
    in flattened batch order, with ``pitch >= n`` and unit stride inside a row.
    A [6, 5, 8] tensor sliced to ``[:, :, :7]`` qualifies (pitch 8); sliced to
    ``[:, :4]`` it does not (the rows of consecutive outer entries are 16 apart,
    not 8), nor does any view whose last stride is not 1.
    """
    if x.stride(-1) != 1:
        return x.contiguous()
    if x.ndim == 1:
        return x
    pitch = x.stride(-2)
    if pitch < x.shape[-1]:
        return x.contiguous()
    # Row (i0, .., i_{m-1}) must sit at pitch * flat(i): dimension d's stride is
    # then the pitch times the number of rows under one step of d.
    rows_under = 1
    for size, stride in zip(reversed(x.shape[:-1]), reversed(x.stride()[:-1])):
        if size > 1 and stride != pitch * rows_under:
            return x.contiguous()
        rows_under *= size
    return x


def topk_triton(
    xs: Tensor,
    k: int,
    dim: int,
    interleaved: bool,
    block_size: int = 64,
    kernel: Literal["bk", "bkn"] = "bk",
) -> tuple[Tensor, Tensor]:
    """Bucketed arg-max on the GPU through the HIP stage-1 kernel."""
    if kernel not in ("bk", "bkn"):
        raise ValueError(f"Unknown kernel {kernel!r}")
    dim %= xs.ndim
    if dim != xs.ndim - 1:
        values, indices = topk_triton(xs.movedim(dim, -1), k=k, dim=-1, interleaved=interleaved,
                                      block_size=block_size, kernel=kernel)
        return values.movedim(-1, dim), indices.movedim(-1, dim)
    layout = _native.INTERLEAVED_PADDED if interleaved else _native.CEIL_CHUNK
    return _native.stage1(_batch_contiguous(xs), k, 1, layout)


topk_hip = topk_triton
