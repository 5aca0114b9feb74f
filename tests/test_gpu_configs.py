"""GPU parity on the benchmark configurations' stated workloads (the inputs bench.py times), and
on subnormal inputs through every kernel family.  Values bit-exact, indices identical; recall
against exact torch.topk as the reference defines it (benchmarks/run_recall.py:31-36)."""
import pytest
import torch

import bench
import oracle
from helpers import assert_same, subnormals

pytestmark = pytest.mark.gpu

FLOAT_DTYPES = [torch.float32, torch.float16, torch.bfloat16, torch.float64]


def _topk():
    from approx_topk import topk
    return topk


def _recall(approx_values, x_gpu, k):
    exact = torch.topk(x_gpu.float(), k, dim=-1).values
    return bench.recall_at_k(approx_values.float(), exact, k)


def test_config4_zipf_workload_all_rows():
    # N(0,1) plus Zipf(1.1) boosts (values up to ~1e18, equal boosts tie) on 1 % of the columns
    rows, n, _, k, j, km, _ = bench.CONFIGS["C4"]
    x = bench.make_input("C4")
    assert x.shape == (rows, n) and float(x.max()) > 1e6
    xg = x.cuda()
    v, i = _topk()(xg, k, -1, j=j, k_mult=km)
    ev, ei = oracle.topk(x, k, -1, j=j, k_mult=km)
    assert_same(v, i, ev, ei, "C4 Zipf workload, fused path")
    rec = _recall(v, xg, k)
    assert 0.85 <= rec <= 1.0, rec          # iid closed form 0.9409; the boosts are not iid
    # the same candidates through the streaming kernel alone (k_mult = 1 over the same 512 buckets)
    v1, i1 = _topk()(xg, k * km, -1, j=j, k_mult=1)
    ev1, ei1 = oracle.topk(x, k * km, -1, j=j, k_mult=1)
    assert_same(v1, i1, ev1, ei1, "C4 Zipf workload, stage 1 alone")
    # and through stage 1 + stand-alone select (rows spaced so that the one-kernel path declines)
    wide = torch.empty(rows, n + 3).cuda()
    wide[:, :n] = xg
    v2, i2 = _topk()(wide[:, :n], k, -1, j=j, k_mult=km)
    assert_same(v2, i2, ev, ei, "C4 Zipf workload, two kernels")


def test_config1_recall_against_exact_topk():
    rows, n, _, k, j, km, _ = bench.CONFIGS["C1"]
    x = bench.make_input("C1")
    xg = x.cuda()
    v, i = _topk()(xg, k, -1, j=j, k_mult=km)
    ev, ei = oracle.topk(x, k, -1, j=j, k_mult=km)
    assert_same(v, i, ev, ei, "C1")
    rec = _recall(v, xg, k)
    assert abs(rec - 0.6323) < 0.03, rec    # closed form for iid inputs: 1 - (1 - 1/b)^... = 0.6323
    from approx_topk.experimental import bucketed_argmax
    va, ia = bucketed_argmax.topk_triton(xg, k, -1, interleaved=True)
    assert torch.equal(va, v) and torch.equal(ia, i)
    vt, it = bucketed_argmax.topk_torch(x, k, -1, interleaved=True)     # the host arg-max path
    assert torch.equal(vt, ev) and torch.equal(it, ei)


@pytest.mark.parametrize("name", ["C3", "C5"])
def test_config_recall_on_the_stated_workload(name):
    rows, n, _, k, j, km, _ = bench.CONFIGS[name]
    x = bench.make_input(name)
    xg = x.cuda()
    v, i = _topk()(xg, k, -1, j=j, k_mult=km)
    take = 8 if name == "C3" else 1
    ev, ei = oracle.topk(x[:take], k, -1, j=j, k_mult=km)
    assert_same(v[:take], i[:take], ev, ei, name)
    rec = _recall(v, xg, k)
    expect = {"C3": 0.9957, "C5": 0.9624}[name]
    assert abs(rec - expect) < 0.03, rec


# ---- subnormal inputs ------------------------------------------------------

def _with_subnormals(shape, dtype, seed):
    """Mostly subnormals and zeros of both signs, some ordinary values: a compare that flushed
    subnormals to zero would pick other candidates (and other indices) than the order keys do."""
    g = torch.Generator().manual_seed(seed)
    pool = torch.cat([subnormals(dtype), torch.tensor([1.0, -1.0, 0.5]).to(dtype)])
    weights = torch.tensor([4.0] * 8 + [0.05] * 3)
    pick = torch.multinomial(weights, shape[0] * shape[1], replacement=True, generator=g)
    return pool[pick].reshape(shape)


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
def test_subnormals_streaming_and_contiguous(dtype):
    x = _with_subnormals((6, 8192), dtype, 11)
    xg = x.cuda()
    for j, k in [(1, 512), (2, 512), (4, 1024)]:
        for interleaved in (True, False):
            v, i = _topk()(xg, k, -1, j=j, interleaved=interleaved)
            ev, ei = oracle.topk(x, k, -1, j=j, interleaved=interleaved)
            assert_same(v, i, ev, ei, f"subnormals {dtype} j={j} interleaved={interleaved}")


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
def test_subnormals_few_long_buckets_and_slabs(dtype):
    x = _with_subnormals((2, 1 << 18), dtype, 12)
    xg = x.cuda()
    for j, k in [(1, 16), (4, 64)]:
        v, i = _topk()(xg, k, -1, j=j)
        ev, ei = oracle.topk(x, k, -1, j=j)
        assert_same(v, i, ev, ei, f"subnormals {dtype} folded j={j}")


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
@pytest.mark.parametrize("rows", [3, 140])
def test_subnormals_two_stage(dtype, rows):
    # 140 rows: one kernel for both stages; 3 long rows: stage 1 + stand-alone select
    x = _with_subnormals((rows, 16384 if rows > 100 else 1 << 17), dtype, 13 + rows)
    xg = x.cuda()
    for j, km in [(1, 4), (2, 2), (4, 4)]:
        v, i = _topk()(xg, 256, -1, j=j, k_mult=km)
        ev, ei = oracle.topk(x, 256, -1, j=j, k_mult=km)
        assert_same(v, i, ev, ei, f"subnormals {dtype} rows={rows} j={j} k_mult={km}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_subnormals_argmax_layouts(dtype):
    from approx_topk.experimental import bucketed_argmax
    x = _with_subnormals((5, 5000), dtype, 17)
    for interleaved in (True, False):
        v, i = bucketed_argmax.topk_triton(x.cuda(), 96, -1, interleaved=interleaved)
        ev, ei = oracle.bucketed_argmax(x, 96, -1, interleaved=interleaved)
        assert_same(v, i, ev, ei, f"subnormals arg-max {dtype} interleaved={interleaved}")


# ---- fp32 with two or more entries per bucket: entries are (element bits, sub-row) words ordered as doubles ----

def _few_distinct_fp32(shape, seed):
    """Rows drawn from a handful of values of both signs, zeros of both signs, subnormals, the largest
    finite values and the infinities: every bucket is full of ties, which the lower index must win
    under positive and negative elements alike."""
    tiny = torch.tensor([1], dtype=torch.int32).view(torch.float32).item()          # smallest subnormal
    pool = torch.tensor([float("-inf"), -3.4028234663852886e38, -1.5, -tiny, -0.0, 0.0, tiny, 1.5,
                         3.4028234663852886e38, float("inf"), -1.5, -1.5, 0.0, -0.0], dtype=torch.float32)
    g = torch.Generator().manual_seed(seed)
    return pool[torch.randint(0, pool.numel(), shape, generator=g)]


@pytest.mark.parametrize("j", [2, 3, 4])
def test_fp32_ties_of_both_signs_through_every_path(j):
    topk = _topk()
    k = 64 * 3 * j                                   # 192 buckets
    cases = [
        ((6, 192 * 40), k, 1),                       # streaming kernel alone
        ((6, 192 * 40 + 77), k, 1),                  # with a partial sub-row
        ((300, 192 * 24), k // 2, 2),                # both stages in one kernel
        ((2, 192 * 4096), k // 2, 2),                # slabs, merge, select
        ((3, 48 * j * 200), 12 * j, 4),              # few buckets: folded sub-rows
    ]
    for shape, kk, km in cases:
        x = _few_distinct_fp32(shape, seed=shape[1] + j)
        v, i = topk(x.cuda(), kk, -1, j=j, k_mult=km)
        ev, ei = oracle.topk(x, kk, -1, j=j, k_mult=km)
        assert_same(v, i, ev, ei, f"fp32 ties j={j} shape={shape} k={kk} k_mult={km}")


def test_fp32_negative_rows_keep_the_lower_index():
    # all elements negative and mostly equal: the tie rule under the sign (a larger magnitude is the smaller word)
    topk = _topk()
    g = torch.Generator().manual_seed(11)
    x = -torch.randint(1, 4, (5, 1 << 16), generator=g).float()
    for j, km in [(2, 1), (4, 1), (4, 2)]:
        k = 2048
        v, i = topk(x.cuda(), k, -1, j=j, k_mult=km)
        ev, ei = oracle.topk(x, k, -1, j=j, k_mult=km)
        assert_same(v, i, ev, ei, f"negative rows j={j} k_mult={km}")
