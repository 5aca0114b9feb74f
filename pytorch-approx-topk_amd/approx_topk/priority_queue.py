"""``approx_topk.topk``: bucketed approximate top-k on AMD GPUs.

Same operator name, signature, defaults and error behaviour as the reference's
approx_topk/priority_queue.py:14-110; the body calls hand-written HIP kernels
through the C ABI of libapprox_topk_hip.so instead of a JIT-built CUDA module.

The operator is defined on a ``torch.library.Library`` and ``topk`` is its
overload object (callable like the reference's, accepted by
``torch.library.opcheck`` and traced by ``torch.compile`` through the fake
implementation below): the dispatcher then calls the Python body directly,
without the wrapper frames ``torch.library.custom_op`` puts around it, which
cost about as much host time per call as the rest of the body.
"""
from __future__ import annotations

import torch
from torch import Tensor

from . import _native


def _result_shape(xs: Tensor, k: int, dim: int) -> list[int]:
    shape = list(xs.shape)
    shape[dim] = k
    return shape


def _empty_result(xs: Tensor, k: int, dim: int) -> tuple[Tensor, Tensor]:
    shape = _result_shape(xs, k, dim)
    return (torch.empty(shape, dtype=xs.dtype, device=xs.device),
            torch.empty(shape, dtype=torch.int64, device=xs.device))


_LIBRARY = torch.library.Library("approx_topk", "DEF")
_LIBRARY.define(
    "topk(Tensor xs, SymInt k, SymInt dim, SymInt j=1, SymInt k_mult=1, bool interleaved=True, "
    "bool? multithread_buckets=False) -> (Tensor, Tensor)",
    tags=(torch.Tag.pt2_compliant_tag,))


def _topk(
    xs: Tensor,
    k: int,
    dim: int,
    j: int = 1,
    k_mult: int = 1,
    interleaved: bool = True,
    multithread_buckets: bool | None = False,
    index_dtype: torch.dtype = torch.int64,
    want_values: bool = True,
) -> tuple[Tensor | None, Tensor]:
    """Approximate top-``k`` of ``xs`` along ``dim``.

    The slice is cut into ``b = k_mult * k / j`` buckets (interleaved: bucket
    ``c`` holds positions ``c, c+b, c+2b, ...``; otherwise contiguous runs), the
    ``j`` largest of every bucket are kept, and if that leaves more than ``k``
    candidates (``k_mult > 1``) an exact top-``k`` of the candidates follows.

    Returns ``(values, indices)`` shaped like ``xs`` with ``dim`` of size ``k``;
    ``values`` has the dtype of ``xs``, ``indices`` is int64, and
    ``xs.gather(dim, indices) == values``.  The order along ``dim`` is
    deterministic but carries no meaning.  Ties between equal values go to the
    lowest index.

    :param j: elements kept per bucket, 1..4; must divide ``k * k_mult``.
    :param k_mult: factor on the number of stage-1 candidates; >= 1.
    :param multithread_buckets: accepted for compatibility; the kernels choose
        their own work split from the shape.
    """
    if dim < 0:
        dim += xs.ndim
    last = xs.ndim - 1
    if j < k and dim != last:
        raise NotImplementedError("This topk only currently works on the last dim")
    if k_mult < 1:
        raise ValueError(f"k_mult must be >=1, was {k_mult}")
    k0 = k * k_mult

    if k0 == 0:
        values, indices = _empty_result(xs, 0, dim)
        return (values if want_values else None), indices.to(index_dtype)
    if j < 1 or j > 4:
        raise RuntimeError("topk: j must 0 < j < 5")
    if k0 % j != 0:
        raise RuntimeError("topk: j must divide k")
    n = xs.shape[dim] if xs.ndim else 1
    if k0 > n:
        raise RuntimeError("topk: k must not be larger than topk size")
    _native.require_gpu(xs)
    layout = _native.INTERLEAVED if interleaved else _native.BALANCED
    if dim == last and n != 0 and xs.ndim and xs.numel():  # the common case, straight through
        if k_mult == 1:
            return _native.stage1(xs, k0, j, layout, index_dtype, want_values)
        return _native.topk(xs, k0, j, k, layout, index_dtype, want_values)
    if xs.numel() == 0:
        values, indices = _empty_result(xs, k, dim)
        return (values if want_values else None), indices.to(index_dtype)

    rows = xs if xs.ndim else xs.reshape(1)
    moved = dim != last and xs.ndim > 1
    if moved:
        rows = rows.movedim(dim, -1)
    if k_mult == 1:
        values, indices = _native.stage1(rows, k0, j, layout, index_dtype, want_values)
    else:
        values, indices = _native.topk(rows, k0, j, k, layout, index_dtype, want_values)
    if moved:
        values = values.movedim(-1, dim).contiguous() if want_values else None
        indices = indices.movedim(-1, dim).contiguous()
    if not xs.ndim:
        values, indices = (values.reshape(()) if want_values else None), indices.reshape(())
    return values, indices


_LIBRARY.impl("topk", _topk, "CompositeExplicitAutograd")


@torch.library.register_fake("approx_topk::topk", lib=_LIBRARY)
def _(
    xs: Tensor,
    k: int,
    dim: int,
    j: int | None = None,
    k_mult: int = 1,
    interleaved: bool = True,
    multithread_buckets: bool | None = False,
) -> tuple[Tensor, Tensor]:
    return _empty_result(xs, k, dim)


topk = torch.ops.approx_topk.topk.default


# The reference's ``topk`` is a ``CustomOpDef`` (approx_topk/priority_queue.py:14), whose
# ``register_fake`` (used at :91) and ``register_autograd`` methods callers may reach for; the
# overload object carries the same two names, forwarding to ``torch.library``.
def _register_fake(fn):
    """Replaces the operator's fake (meta) implementation; usable as a decorator."""
    torch.library.register_fake("approx_topk::topk", fn, lib=_LIBRARY, allow_override=True)
    return fn


def _register_autograd(backward, /, *, setup_context=None):
    """Attaches an autograd formula to the operator (``torch.library.register_autograd``).  Once
    registered, every call goes through autograd's dispatch (about 3 us more per call), which is
    why none is registered by default: ``approx_topk.experimental.differentiable.topk`` is the
    opt-in wrapper with the scatter gradient."""
    torch.library.register_autograd("approx_topk::topk", backward, setup_context=setup_context, lib=_LIBRARY)


topk.register_fake = _register_fake
topk.register_autograd = _register_autograd
