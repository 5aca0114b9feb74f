"""GPU parity of the bucketed arg-max entry points against the known answers of
the reference's tests/test_bucket_argmax.py, the torch-level definition and the
oracle."""
import numpy as np
import pytest
import torch

import oracle
from helpers import assert_same

pytestmark = pytest.mark.gpu


def _fns():
    from functools import partial

    from approx_topk.experimental.bucketed_argmax import topk_torch, topk_triton
    return [topk_torch, partial(topk_triton, block_size=1, kernel="bk"),
            partial(topk_triton, block_size=8, kernel="bkn")]


@pytest.mark.parametrize("which", [0, 1, 2])
def test_known_answers(which):
    topk = _fns()[which]
    x = torch.stack([100 * torch.arange(0, 20), -100 * torch.arange(0, 20)]).to(torch.float32).cuda()
    v, i = topk(x, k=3, dim=1, interleaved=False)
    assert torch.equal(v.cpu(), torch.tensor([[600.0, 1300, 1900], [0, -700, -1400]]))
    assert torch.equal(i.cpu(), torch.tensor([[6, 13, 19], [0, 7, 14]]))
    vt, it = topk(x.T, k=3, dim=0, interleaved=False)
    assert torch.equal(vt.T, v) and torch.equal(it.T, i)
    v, i = topk(x, k=3, dim=1, interleaved=True)
    assert torch.equal(v.cpu(), torch.tensor([[1800.0, 1900, 1700], [0, -100, -200]]))
    assert torch.equal(i.cpu(), torch.tensor([[18, 19, 17], [0, 1, 2]]))


@pytest.mark.parametrize("interleaved", [False, True])
def test_fuzz_int64_against_torch_level_and_oracle(interleaved):
    from approx_topk.experimental.bucketed_argmax import topk_torch, topk_triton
    for seed in np.random.SeedSequence(123).generate_state(20):
        rng = np.random.RandomState(seed)
        g = torch.Generator().manual_seed(int(rng.randint(100000)))
        b = 2 ** rng.randint(1, 5) if rng.rand() < 0.5 else rng.randint(1, 17)
        n = 2 ** rng.randint(1, 11) if rng.rand() < 0.5 else rng.randint(1, 1025)
        k = -(-n // rng.randint(1, 33))
        x = torch.randint(-(2 ** 15), 2 ** 15, (int(b), int(n)), generator=g)
        ev, ei = oracle.bucketed_argmax(x, int(k), 1, interleaved)
        tv, ti = topk_torch(x.cuda(), k=int(k), dim=1, interleaved=interleaved)
        av, ai = topk_triton(x.cuda(), k=int(k), dim=1, interleaved=interleaved, block_size=4, kernel="bk")
        assert_same(av, ai, ev, ei, f"hip b={b} n={n} k={k}")
        assert_same(tv, ti, ev, ei, f"torch-level b={b} n={n} k={k}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.int32])
def test_config1_shape(dtype):
    from approx_topk.experimental.bucketed_argmax import topk_triton
    g = torch.Generator().manual_seed(1001)
    x = torch.randn(4, 65536, generator=g)
    x = (x * 1000).to(dtype) if not dtype.is_floating_point else x.to(dtype)
    for interleaved in (True, False):
        ev, ei = oracle.bucketed_argmax(x, 1024, 1, interleaved)
        av, ai = topk_triton(x.cuda(), k=1024, dim=1, interleaved=interleaved)
        assert_same(av, ai, ev, ei, f"C1 {dtype} interleaved={interleaved}")


def test_k_larger_than_n_and_neg_inf():
    from approx_topk.experimental.bucketed_argmax import topk_triton
    x = torch.tensor([[1.0, -float("inf"), 3.0, -float("inf"), -float("inf")]])
    for k in (2, 3, 8):
        for interleaved in (True, False):
            ev, ei = oracle.bucketed_argmax(x, k, 1, interleaved)
            av, ai = topk_triton(x.cuda(), k=k, dim=1, interleaved=interleaved)
            assert_same(av, ai, ev, ei, f"k={k} interleaved={interleaved}")


@pytest.mark.parametrize("n,k", [(65536, 64), (50000, 48), (40001, 10), (1 << 20, 1), (4096, 16), (4001, 12)])
def test_few_long_buckets(n, k):
    from approx_topk.experimental.bucketed_argmax import topk_triton
    g = torch.Generator().manual_seed(n + k)
    x = torch.randn(3, n, generator=g)
    ev, ei = oracle.bucketed_argmax(x, k, 1, True)
    av, ai = topk_triton(x.cuda(), k=k, dim=1, interleaved=True)
    assert_same(av, ai, ev, ei, f"n={n} k={k}")


@pytest.mark.parametrize("n,k", [(65536, 64), (50000, 48), (40001, 10), (1 << 20, 1), (4096, 16), (4001, 12), (100, 64), (5000, 4999)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.int64])
def test_contiguous_chunks(n, k, dtype):
    from approx_topk.experimental.bucketed_argmax import topk_triton
    g = torch.Generator().manual_seed(n + k)
    x = torch.randn(3, n, generator=g)
    x = (x * 1000).to(dtype) if not dtype.is_floating_point else x.to(dtype)
    ev, ei = oracle.bucketed_argmax(x, k, 1, False)
    av, ai = topk_triton(x.cuda(), k=k, dim=1, interleaved=False)
    assert_same(av, ai, ev, ei, f"n={n} k={k}")


@pytest.mark.parametrize("layout", ["CEIL_CHUNK", "INTERLEAVED_PADDED"])
@pytest.mark.parametrize("n,k0", [(50000, 48), (4001, 12), (100, 64), (65536, 1024)])
def test_int32_indices_in_the_padded_layouts(layout, n, k0):
    from approx_topk import _native
    g = torch.Generator().manual_seed(n + k0)
    x = torch.randn(3, n, generator=g).cuda()
    code = getattr(_native, layout)
    v64, i64 = _native.stage1(x, k0, 1, code)
    v32, i32 = _native.stage1(x, k0, 1, code, torch.int32)
    assert i32.dtype == torch.int32
    assert torch.equal(i32.long(), i64) and torch.equal(v32, v64)
