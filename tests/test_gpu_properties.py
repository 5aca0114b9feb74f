"""GPU checks that do not need the oracle at full size: invariants of the result
at the benchmark shapes, random-shape fuzz against the oracle, HIP-graph replay,
side streams, and recall against the closed form."""
import math

import numpy as np
import pytest
import torch

import oracle
from helpers import assert_same, cpu_randn

pytestmark = pytest.mark.gpu


def _topk():
    from approx_topk import topk
    return topk


def _bits(t):
    return t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()])


def _check_stage1_invariants(x, v, i, k, j):
    """x: [rows, n] on the GPU; v, i: stage-1 output with k_mult == 1."""
    rows, n = x.shape
    b = k // j
    assert torch.equal(_bits(x.gather(1, i)), _bits(v)), "values are not x[indices]"
    buckets = torch.arange(b, device=x.device).repeat_interleave(j)
    assert torch.equal(i % b, buckets.expand(rows, -1)), "an index left its bucket"
    if n % b == 0:
        # per-bucket exact top-j with torch on the [L, b] view, compared as sorted value sets
        ref = torch.topk(x.view(rows, n // b, b), j, dim=1).values          # [rows, j, b]
        got = v.view(rows, b, j).transpose(1, 2)                            # [rows, j, b]
        assert torch.equal(got.sort(dim=1).values, ref.sort(dim=1).values)
        # slots ascend within a bucket
        assert bool((got[:, 1:] >= got[:, :-1]).all())
    per_bucket = i.view(rows, b, j).sort(dim=-1).values
    if j > 1:
        assert bool((per_bucket[..., 1:] != per_bucket[..., :-1]).all()), "duplicate index in a bucket"


def test_headline_shape_full_size():
    g = torch.Generator().manual_seed(1002)
    x_cpu = torch.randn(128, 1 << 20, generator=g)
    x = x_cpu.cuda()
    v, i = _topk()(x, 65536, -1, j=2)
    torch.cuda.synchronize()
    _check_stage1_invariants(x, v, i, 65536, 2)
    ev, ei = oracle.topk(x_cpu[:6], 65536, -1, j=2)
    assert_same(v[:6], i[:6], ev, ei, "C2 rows 0..5")
    ev, ei = oracle.topk(x_cpu[125:], 65536, -1, j=2)
    assert_same(v[125:], i[125:], ev, ei, "C2 rows 125..127")


@pytest.mark.parametrize("j", [1, 3, 4])
def test_headline_shape_other_j(j):
    x = torch.randn(32, 1 << 20, device="cuda")
    k = 65536 // 4 * j if j == 3 else 65536
    v, i = _topk()(x, k, -1, j=j)
    _check_stage1_invariants(x, v, i, k, j)


def test_single_long_row_full_size():
    n = 1 << 26
    g = torch.Generator().manual_seed(1005)
    x_cpu = 0.5 * torch.linspace(-1, 1, n) + torch.randn(n, generator=g)
    x = x_cpu.cuda().reshape(1, n)
    v, i = _topk()(x, 16384, -1, j=4, k_mult=2)
    torch.cuda.synchronize()
    assert torch.equal(_bits(x.gather(1, i)), _bits(v))
    ev, ei = oracle.topk(x_cpu.reshape(1, n), 16384, -1, j=4, k_mult=2)
    assert_same(v, i, ev, ei, "C5")
    # stage 1 alone at the same bucketing
    v1, i1 = _topk()(x, 32768, -1, j=4)
    _check_stage1_invariants(x, v1, i1, 32768, 4)


def test_vocab_logits_shape_with_heavy_ties():
    # C4-like: boosts drawn from a tiny set so that equal large values compete
    g = torch.Generator().manual_seed(1004)
    x_cpu = torch.randn(256, 131072, generator=g)
    hot = torch.randint(0, 131072, (256, 1311), generator=g)
    x_cpu.scatter_(1, hot, torch.randint(5, 9, (256, 1311), generator=g).float())
    v, i = _topk()(x_cpu.cuda(), 64, -1, j=1, k_mult=8)
    ev, ei = oracle.topk(x_cpu, 64, -1, j=1, k_mult=8)
    assert_same(v, i, ev, ei, "C4 with ties")


def test_random_shapes_against_oracle():
    rng = np.random.RandomState(2024)
    dtypes = [torch.float32, torch.float16, torch.bfloat16, torch.int32, torch.int16, torch.float64, torch.uint8]
    for case in range(160):
        dtype = dtypes[rng.randint(len(dtypes))]
        j = int(rng.randint(1, 5))
        k_mult = int(rng.choice([1, 1, 2, 4, 8]))
        rows = int(rng.choice([1, 3, 17, 130, 257]))
        b = int(rng.choice([1, 2, 7, 8, 10, 16, 31, 64, 96, 512, 1000, 2048, 20000]))
        length = int(rng.choice([j, j + 1, 4, 8, 9, 16, 33, 100, 128, 700, 9000, 70000]))
        if length < j:
            length = j
        n = b * length + int(rng.randint(0, b))
        if n > 3_000_000:
            continue
        if rows * n > 6_000_000:
            rows = max(1, 6_000_000 // n)
        k0 = b * j
        if k0 % k_mult:
            k_mult = 1
        k = k0 // k_mult
        interleaved = bool(rng.rand() < 0.8)
        g = torch.Generator().manual_seed(case)
        if dtype.is_floating_point:
            x = (torch.randint(-40, 41, (rows, n), generator=g).float() / 8).to(dtype)
        elif dtype == torch.uint8:
            x = torch.randint(0, 60, (rows, n), generator=g).to(dtype)
        else:
            x = torch.randint(-40, 41, (rows, n), generator=g).to(dtype)
        v, i = _topk()(x.cuda(), k, -1, j=j, k_mult=k_mult, interleaved=interleaved)
        ev, ei = oracle.topk(x, k, -1, j=j, k_mult=k_mult, interleaved=interleaved)
        assert_same(v, i, ev, ei, f"case {case}: {dtype} rows={rows} n={n} b={b} j={j} k_mult={k_mult} "
                                  f"interleaved={interleaved}")


def test_hip_graph_replay_matches_eager():
    topk = _topk()
    # (input, k, kwargs): streaming kernel; fused kernel; few long buckets (folded, slabs + merge);
    # contiguous buckets; two kernels with a select that keeps > 48 KiB of keys in LDS; the
    # multi-workgroup select chain
    cases = [
        (torch.randn(64, 1 << 16, device="cuda"), 4096, dict(j=2)),
        (torch.randn(256, 8192, device="cuda", dtype=torch.float16), 256, dict(j=4, k_mult=4)),
        (torch.randn(8, 1 << 18, device="cuda"), 64, dict(j=2)),
        (torch.randn(16, 1 << 16, device="cuda"), 1024, dict(j=2, interleaved=False)),
        (torch.randn(2, 1 << 20, device="cuda"), 8192, dict(j=2, k_mult=2)),
        (torch.randn(1, 1 << 20, device="cuda"), 32768, dict(j=1, k_mult=4)),
        # few short rows through the fused kernel; many rows with a small select; short folded buckets
        (torch.randn(4, 32000, device="cuda", dtype=torch.bfloat16), 64, dict(j=1, k_mult=4)),
        (torch.randn(2048, 4096, device="cuda"), 64, dict(j=2, k_mult=4)),
        (torch.randn(512, 1024, device="cuda"), 16, dict(j=1)),
    ]
    for _ in range(2):   # warm up allocator and library state outside the capture
        for x, k, kw in cases:
            topk(x, k, -1, **kw)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = [topk(x, k, -1, **kw) for x, k, kw in cases]
    for rep in range(4):
        for x, _, _ in cases:
            x.normal_()
        eager = [topk(x, k, -1, **kw) for x, k, kw in cases]   # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for n, (got, want) in enumerate(zip(outs, eager)):
            assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]), f"replay {rep}, case {n}"


def test_side_stream():
    topk = _topk()
    x_cpu = cpu_randn((16, 1 << 15), 77)
    x = x_cpu.cuda()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        v, i = topk(x, 1024, -1, j=2, k_mult=2)
    side.synchronize()
    ev, ei = oracle.topk(x_cpu, 1024, -1, j=2, k_mult=2)
    assert_same(v, i, ev, ei, "side stream")


def _closed_form_recall(k, b, j):
    from scipy.stats import binom
    # expected fraction of the true top-k kept when each lands in a uniform random bucket
    # (formula of notebooks/theoretical_models.py:9-12 in the reference)
    return float((j + binom.cdf(j - 1, np.arange(j, k), 1.0 / b).sum()) / k)


@pytest.mark.parametrize("n,k,j,k_mult", [(65536, 1024, 1, 1), (1 << 18, 4096, 2, 1), (32768, 2048, 4, 4)])
def test_recall_matches_closed_form(n, k, j, k_mult):
    x = torch.randn(64, n, device="cuda")
    v, _ = _topk()(x, k, -1, j=j, k_mult=k_mult)
    kth = torch.topk(x, k, dim=-1).values[:, -1:]
    recall = float(((v >= kth).sum(-1).double() / k).mean())
    expected = _closed_form_recall(k, k * k_mult // j, j)
    assert abs(recall - expected) < 0.02, (recall, expected)


def test_row_longer_than_two_to_the_31():
    """Positions beyond 2^31: index arithmetic must be 64-bit end to end."""
    n = (1 << 31) + 4099
    g = torch.Generator().manual_seed(31)
    x = torch.randint(0, 255, (1, n), generator=g, dtype=torch.uint8)
    x[0, -5:] = 255                      # the only 255s: winners at the very end of the row
    xg = x.cuda()
    for k, j, interleaved in [(64, 2, True), (1 << 16, 1, True), (96, 3, False)]:
        v, i = _topk()(xg, k, -1, j=j, interleaved=interleaved)
        ev, ei = oracle.topk(x, k, -1, j=j, interleaved=interleaved)
        assert_same(v, i, ev, ei, f"k={k} j={j} interleaved={interleaved}")
        assert int(i.max()) >= n - 5
    del xg
    torch.cuda.empty_cache()
