"""``approx_topk.topk`` with a gradient.

The reference registers no autograd formula for its operator
(approx_topk/priority_queue.py:14: ``mutates_args=()`` and nothing else), and
neither does ``approx_topk.topk`` here: an autograd kernel on the operator
costs every call about 3 us of host time, gradient or not.  This wrapper is the
opt-in: same arguments, same results, and the values' gradient flows back to
the input.  The values are a gather of the input at the returned indices, so
their gradient scatters to those positions and every other position gets zero;
the indices are distinct along ``dim``, so a plain scatter is exact.
"""
from __future__ import annotations

import torch
from torch import Tensor

from ..priority_queue import topk as _topk


class _TopkWithGradient(torch.autograd.Function):
    @staticmethod
    def forward(ctx, xs, k, dim, j, k_mult, interleaved, multithread_buckets):
        values, indices = _topk(xs, k, dim, j, k_mult, interleaved, multithread_buckets)
        ctx.dim = dim if dim >= 0 else dim + xs.ndim
        ctx.shape = xs.shape
        ctx.save_for_backward(indices)
        ctx.mark_non_differentiable(indices)
        return values, indices

    @staticmethod
    def backward(ctx, grad_values, _grad_indices):
        (indices,) = ctx.saved_tensors
        if len(ctx.shape) == 0:
            grad_xs = grad_values.reshape(()) if indices.numel() else grad_values.new_zeros(())
        else:
            grad_xs = grad_values.new_zeros(ctx.shape).scatter(ctx.dim, indices, grad_values)
        return grad_xs, None, None, None, None, None, None


def topk(
    xs: Tensor,
    k: int,
    dim: int,
    j: int = 1,
    k_mult: int = 1,
    interleaved: bool = True,
    multithread_buckets: bool | None = False,
) -> tuple[Tensor, Tensor]:
    """``approx_topk.topk`` whose values carry a gradient with respect to ``xs``."""
    return _TopkWithGradient.apply(xs, k, dim, j, k_mult, interleaved, multithread_buckets)
