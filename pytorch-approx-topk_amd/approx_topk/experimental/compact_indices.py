"""``approx_topk.topk`` with int32 indices.

The operator returns int64 indices, as the reference does
(approx_topk/priority_queue.py:67).  On 4-byte elements the index write is two
thirds of the output traffic, and on the widest shapes (k = n/16) the output is
a sixth of all the traffic of the call; a consumer that gathers with 32-bit
offsets can ask for int32 indices here and save half of the index bytes.  Same
arguments, same values and the same indices as ``approx_topk.topk``, narrowed;
rows (padded rows, for the arg-max layouts) must be shorter than 2^31.  Not
registered as a torch operator: call it eagerly or under a HIP graph.
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
