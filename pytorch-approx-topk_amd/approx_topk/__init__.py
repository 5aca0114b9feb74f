"""Bucketed approximate top-k for AMD MI355X (gfx950).

Public surface mirrors approx_topk/__init__.py:7-12 of the reference: the
``topk`` operator and the ``Topk`` call protocol.
"""
from typing import Protocol

from torch import Tensor

from .priority_queue import topk as topk


class Topk(Protocol):
    @staticmethod
    def __call__(xs: Tensor, k: int, dim: int) -> tuple[Tensor, Tensor]: ...
