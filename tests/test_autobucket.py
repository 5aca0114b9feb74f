"""The torch-level bucketing wrapper against the known answers of the reference's
tests/test_autobucket.py and against the oracle (CPU only)."""
import pytest
import torch

import oracle
from approx_topk.experimental.autobucket import bucket, bucketed_torch_topk


def _exact(xs, k, dim):
    return torch.topk(xs, k, dim, sorted=False)


def _sorted(t, dim=-1):
    return t.sort(dim=dim).values


def test_k_not_divisible_raises():
    with pytest.raises(NotImplementedError):
        bucket(_exact, k_mult=1, k_per_bucket=12, interleaved=True)(torch.randn(1024), 13, dim=0)


@pytest.mark.parametrize("interleaved,k_mult,expected", [
    (False, 1, [3, 6, 9]), (True, 1, [7, 8, 9])])
def test_arange10(interleaved, k_mult, expected):
    v, i = bucket(torch.topk, k_mult=k_mult, k_per_bucket=1, interleaved=interleaved)(torch.arange(10), k=3, dim=-1)
    assert _sorted(v).tolist() == expected and _sorted(i).tolist() == expected


@pytest.mark.parametrize("interleaved,expected", [(False, [9, 11, 13, 15]), (True, [12, 13, 14, 15])])
def test_arange16_k_mult2(interleaved, expected):
    v, i = bucket(torch.topk, k_mult=2, k_per_bucket=1, interleaved=interleaved)(torch.arange(16), k=4, dim=-1)
    assert _sorted(v).tolist() == expected and _sorted(i).tolist() == expected


def test_ideal_distribution_n1025_contiguous():
    xs = torch.zeros(2, 1025)
    for r, cells in enumerate([[(1, 10.), (2, 11.), (300, 11.), (301, 12.), (600, 11.), (601, 12.), (900, 13.), (901, 12.)],
                               [(5, 10.), (6, 11.), (302, 11.), (305, 12.), (610, 11.), (611, 12.), (920, 13.), (921, 12.)]]):
        for pos, val in cells:
            xs[r, pos] = val
    v, i = bucket(_exact, k_mult=1, k_per_bucket=2, interleaved=False)(xs, 8, dim=1)
    ev, ei = _exact(xs, 8, 1)
    assert torch.equal(_sorted(v), _sorted(ev)) and torch.equal(_sorted(i), _sorted(ei))


@pytest.mark.parametrize("interleaved", [True, False])
def test_one_bucket_is_exact(interleaved):
    xs = torch.randn(1024, generator=torch.Generator().manual_seed(1))
    v, i = bucket(_exact, k_mult=1, k_per_bucket=128, interleaved=interleaved)(xs, 128, dim=0)
    ev, ei = _exact(xs, 128, 0)
    assert torch.equal(_sorted(v), _sorted(ev)) and torch.equal(_sorted(i), _sorted(ei))


@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("k_mult", [1, 2, 4])
@pytest.mark.parametrize("k_per_bucket", [1, 2, 4])
def test_matches_oracle_on_distinct_values(interleaved, k_mult, k_per_bucket):
    xs = torch.randn(5, 32, 1000, generator=torch.Generator().manual_seed(3))
    v, i = bucketed_torch_topk(xs, 16, -1, k_mult, k_per_bucket, interleaved)
    assert v.shape == (5, 32, 16) and i.shape == (5, 32, 16)
    ev, ei = oracle.topk(xs, 16, -1, j=k_per_bucket, k_mult=k_mult, interleaved=interleaved)
    assert torch.equal(_sorted(v), _sorted(ev)) and torch.equal(_sorted(i), _sorted(ei))
    assert torch.equal(xs.gather(-1, i), v)


def test_other_dim():
    xs = torch.randn(6, 40, 7, generator=torch.Generator().manual_seed(4))
    v, i = bucketed_torch_topk(xs, 8, 1, 2, 2, True)
    ev, ei = oracle.topk(xs, 8, 1, j=2, k_mult=2)
    assert torch.equal(_sorted(v, 1), _sorted(ev, 1)) and torch.equal(_sorted(i, 1), _sorted(ei, 1))
