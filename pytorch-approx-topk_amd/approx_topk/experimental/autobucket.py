"""Bucketing wrapper around any exact top-k, in plain torch ops.

Same entry points and argument meaning as the reference's
approx_topk/experimental/autobucket.py:10-95: ``bucket`` turns an exact method
``(xs, k, dim) -> (values, indices)`` into the bucketed approximation (split the
slice into ``k*k_mult/k_per_bucket`` buckets, keep ``k_per_bucket`` of each,
finish with an exact top-``k`` of the survivors).  It runs wherever torch runs
and launches several library kernels per call; ``approx_topk.topk`` is the
fast path on the GPU.
"""
from __future__ import annotations

import torch
from torch import Tensor

from .. import Topk


def _lowest(dtype: torch.dtype):
    return torch.finfo(dtype).min if dtype.is_floating_point else torch.iinfo(dtype).min


def _bucket_positions(n: int, buckets: int, interleaved: bool, device) -> tuple[Tensor, Tensor]:
    """positions[c, t] = index of member t of bucket c, and which of them exist.

    Interleaved: bucket c holds c, c+b, c+2b, ...  Contiguous: runs of
    floor(n/b) elements, the first n mod b runs one longer.
    """
    longest = -(-n // buckets)
    c = torch.arange(buckets, dtype=torch.int64, device=device).unsqueeze(1)
    t = torch.arange(longest, dtype=torch.int64, device=device).unsqueeze(0)
    base, extra = divmod(n, buckets)
    size = base + (c < extra).to(torch.int64)
    if interleaved:
        positions = c + t * buckets
    else:
        positions = c * base + torch.clamp(c, max=extra) + t
    return positions, t < size


def bucket(exact_method: Topk, k_mult: int, k_per_bucket: int, interleaved: bool) -> Topk:
    """Build an approximate, bucket-parallel top-k from an exact method."""

    def bucketed(xs: Tensor, k: int, dim: int) -> tuple[Tensor, Tensor]:
        candidates = k * k_mult
        if candidates % k_per_bucket != 0:
            raise NotImplementedError
        dim %= xs.ndim
        if dim != xs.ndim - 1:
            values, indices = bucketed(xs.movedim(dim, -1), k, -1)
            return values.movedim(-1, dim), indices.movedim(-1, dim)

        n = xs.shape[-1]
        buckets = candidates // k_per_bucket
        positions, exists = _bucket_positions(n, buckets, interleaved, xs.device)
        members = xs[..., positions.clamp(max=n - 1)]            # [..., b, longest]
        members = members.masked_fill(~exists, _lowest(xs.dtype))
        kept_values, kept_at = exact_method(members, k=k_per_bucket, dim=-1)
        kept_indices = positions.expand(members.shape).gather(-1, kept_at)
        kept_values, kept_indices = kept_values.flatten(-2), kept_indices.flatten(-2)
        values, pick = torch.topk(kept_values, k=k, dim=-1, sorted=False)
        return values, kept_indices.gather(-1, pick)

    return bucketed


def bucketed_torch_topk(
    xs: Tensor,
    k: int,
    dim: int,
    k_mult: int,
    k_per_bucket: int,
    interleaved: bool,
) -> tuple[Tensor, Tensor]:
    """``bucket`` around ``torch.topk(sorted=False)``."""

    def exact(xs: Tensor, k: int, dim: int) -> tuple[Tensor, Tensor]:
        return torch.topk(xs, k, dim, sorted=False)

    return bucket(exact, k_mult=k_mult, k_per_bucket=k_per_bucket, interleaved=interleaved)(xs, k, dim)
