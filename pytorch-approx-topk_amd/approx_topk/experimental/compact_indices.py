"""``approx_topk.topk`` with int32 indices, and its indices alone.

The operator returns int64 indices, as the reference does
(approx_topk/priority_queue.py:67).  On 4-byte elements the index write is two
thirds of the output traffic, and on the widest shapes (k = n/16) the output is
a sixth of all the traffic of the call; a consumer that gathers with 32-bit
offsets can ask for int32 indices here and save half of the index bytes.  Same
arguments, same values and the same indices as ``approx_topk.topk``, narrowed;
rows (padded rows, for the arg-max layouts) must be shorter than 2^31.

``topk_indices`` goes one step further for consumers that only gather other
tensors at the selected positions (the keys and values of a sparse attention
step) and never read the selected elements themselves: the kernels then write
no values at all.  At fp32 [128, 2^20], k = 65536, j = 2 the output shrinks from
96 MiB (values + int64 indices) to 32 MiB and the call from 110 to 96 us.

Neither is registered as a torch operator: call them eagerly or under a HIP graph.
"""
from __future__ import annotations

import torch
from torch import Tensor

from ..priority_queue import _topk


def topk(
    xs: Tensor,
    k: int,
    dim: int,
    j: int = 1,
    k_mult: int = 1,
    interleaved: bool = True,
    multithread_buckets: bool | None = False,
) -> tuple[Tensor, Tensor]:
    """(values, int32 indices); otherwise as ``approx_topk.topk``."""
    return _topk(xs, k, dim, j, k_mult, interleaved, multithread_buckets, index_dtype=torch.int32)


def topk_indices(
    xs: Tensor,
    k: int,
    dim: int,
    j: int = 1,
    k_mult: int = 1,
    interleaved: bool = True,
    index_dtype: torch.dtype = torch.int32,
) -> Tensor:
    """The indices ``approx_topk.topk`` would return (as ``index_dtype``: int32 or int64), and
    nothing else: no values are written."""
    return _topk(xs, k, dim, j, k_mult, interleaved, False, index_dtype=index_dtype, want_values=False)[1]
