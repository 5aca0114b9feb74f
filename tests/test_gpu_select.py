"""GPU parity of stage 2 alone (atk_select through the C ABI) against the CPU
oracle: exact top-k of given candidates, ties to the lowest original index,
survivors in candidate order.  Covers the one-workgroup kernel (keys in LDS and
keys re-read from global memory) and the multi-workgroup chain of launches that
takes rows with very many candidates."""
import pytest
import torch

import oracle
from helpers import assert_same

pytestmark = pytest.mark.gpu


def _select(cv, ci, k, bound):
    from approx_topk import _native
    v, i = _native.select(cv.cuda(), ci.cuda(), k, bound)
    torch.cuda.synchronize()
    return v, i


def _candidates(rows, k0, dtype, seed, ties, bound):
    g = torch.Generator().manual_seed(seed)
    if ties:      # few distinct values: the cut falls inside a large group of equal keys
        cv = torch.randint(-3, 4, (rows, k0), generator=g).to(dtype)
    elif dtype.is_floating_point:
        cv = torch.randn((rows, k0), generator=g).to(dtype)
    else:
        cv = torch.randint(-30000, 30000, (rows, k0), generator=g).to(dtype)
    # distinct original indices below `bound`, in no particular order
    ci = torch.stack([torch.randperm(bound, generator=g)[:k0] for _ in range(rows)]) if bound <= (1 << 22) else \
        torch.stack([torch.randperm(k0, generator=g) * (bound // k0) + 1 for _ in range(rows)])
    return cv, ci


@pytest.mark.parametrize("rows,k0,k", [
    (5, 64, 10), (300, 512, 64), (7, 1024, 1000), (3, 100, 100), (9, 65, 1), (130, 300, 299),
    (3, 1025, 100), (2, 40000, 777), (2, 70000, 30000),          # one workgroup per row
    (1500, 64, 10), (1100, 256, 100), (1024, 1024, 300), (1030, 2500, 64), (2000, 40, 39),   # many rows: small workgroups
    (2, 65537, 1), (3, 131072, 32768), (1, 300001, 150000), (2, 1 << 20, 1000), (5, 100000, 99999),
])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.int64, torch.uint8])
@pytest.mark.parametrize("ties", [False, True])
def test_select_matches_oracle(rows, k0, k, dtype, ties):
    if dtype == torch.uint8 and not ties:
        pytest.skip("uint8 candidates are always tie-heavy")
    bound = max(k0, 1 << 21) if rows <= 8 else max(k0, 1 << 12)   # (a permutation of `bound` per row)
    cv, ci = _candidates(rows, k0, dtype, k0 + k, ties, bound)
    if dtype == torch.uint8:
        cv = cv.abs().to(dtype)
    v, i = _select(cv, ci, k, bound)
    ev, ei = oracle.stage2(cv, ci, k)
    assert_same(v, i, ev, ei, f"rows={rows} k0={k0} k={k} {dtype} ties={ties}")


def test_select_all_equal_and_wide_indices():
    k0, k = 200000, 12345
    bound = 1 << 40                      # four index digits of 11 bits
    cv = torch.full((2, k0), 1.5)
    cv[1, ::7] = float("nan")            # NaN ranks above everything, ties among NaN by index
    g = torch.Generator().manual_seed(5)
    ci = torch.stack([torch.randperm(k0, generator=g) * (bound // k0) + 3 for _ in range(2)])
    v, i = _select(cv, ci, k, bound)
    ev, ei = oracle.stage2(cv, ci, k)
    assert_same(v, i, ev, ei, "all-equal rows")


@pytest.mark.parametrize("rows,k0", [
    (2, 150000),     # passes over many workgroups
    (2, 70000),      # the chain of launches, ties told apart by index (row state and list counters in the workspace)
    (40, 40000),     # the chain with long segments
    (3, 20000),      # the one-launch form
    (70, 40000),     # one workgroup per row
])
def test_select_under_graph_replay(rows, k0):
    cv, ci = _candidates(rows, k0, torch.float32, 11 + rows, True, 1 << 21)
    from approx_topk import _native
    cvg, cig = cv.cuda(), ci.cuda()
    _native.select(cvg, cig, 5000, 1 << 21)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        v, i = _native.select(cvg, cig, 5000, 1 << 21)
    ev, ei = oracle.stage2(cv, ci, 5000)
    for _ in range(3):
        v.zero_(); i.zero_()
        _native.select(cvg, cig, 77, 1 << 21)    # eager work between the replays
        graph.replay()
        torch.cuda.synchronize()
        assert_same(v, i, ev, ei, f"graph replay rows={rows} k0={k0}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("interleaved", [True, False])
def test_topk_with_many_candidates(dtype, interleaved):
    from approx_topk import topk
    g = torch.Generator().manual_seed(17)
    x = torch.randn((2, 1 << 20), generator=g).to(dtype)
    v, i = topk(x.cuda(), 32768, -1, j=2, k_mult=4, interleaved=interleaved)   # 131072 candidates per row
    ev, ei = oracle.topk(x, 32768, -1, j=2, k_mult=4, interleaved=interleaved)
    assert_same(v, i, ev, ei, f"{dtype} interleaved={interleaved}")


# ---- few rows of thousands of candidates: several workgroups per row in a short chain of launches ----

def _chain_case(rows_spec, k0, k, dtype, bound=1 << 21, seed=0):
    """rows_spec: per row 'spread' (distinct values), 'ties' (seven values), 'equal' (one value),
    'steps' (blocks of equal values: the cut digit is shared by thousands)."""
    g = torch.Generator().manual_seed(seed)
    rows = []
    for kind in rows_spec:
        if kind == "spread":
            r = torch.randn(k0, generator=g) if dtype.is_floating_point else torch.randint(-30000, 30000, (k0,), generator=g)
        elif kind == "ties":
            r = torch.randint(-3, 4, (k0,), generator=g)
        elif kind == "equal":
            r = torch.full((k0,), 2.0)
        elif kind in ("outliers", "tied outliers", "crowded"):
            # two values far from all others stretch the span of the keys: nearly every candidate
            # shares the leading digit of its offset, and the cut is found some digits further down
            if kind == "tied outliers":
                r = torch.randint(-3, 4, (k0,), generator=g).double()
            elif kind == "crowded" and dtype.is_floating_point:
                r = 1.0 + torch.randn(k0, generator=g).double() * 1e-4
            elif dtype.is_floating_point:
                r = torch.randn(k0, generator=g).double()
            else:
                r = torch.randint(-30000, 30000, (k0,), generator=g).double()
            big = float(torch.finfo(dtype).max) / 2 if dtype.is_floating_point else float(torch.iinfo(dtype).max)
            at = torch.randperm(k0, generator=g)[:2]
            r[at[0]], r[at[1]] = big, -big
        else:
            r = (torch.arange(k0) // 3000).float()[torch.randperm(k0, generator=g)]
        rows.append(r.to(dtype))
    cv = torch.stack(rows)
    ci = torch.stack([torch.randperm(bound, generator=g)[:k0] for _ in rows_spec])
    v, i = _select(cv, ci, k, bound)
    ev, ei = oracle.stage2(cv, ci, k)
    assert_same(v, i, ev, ei, f"{rows_spec} k0={k0} k={k} {dtype}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.int32, torch.int16, torch.uint8])
@pytest.mark.parametrize("k0,k", [(8192, 2048), (32768, 16384), (20000, 1), (9001, 9000), (131072, 5000),
                                  (49153, 30000), (65536, 777)])
def test_chain_select_rows_of_every_kind_together(dtype, k0, k):
    # rows that end by prefix, by a ranked list, by a long list and by the whole-row fallback, in one call;
    # up to 32768 candidates in one launch (8, 16 or 32 keys per thread), beyond that as a chain of launches
    kinds = ["spread", "ties", "equal", "steps", "spread"]
    if dtype == torch.uint8:
        kinds = ["ties", "equal", "steps"]
    _chain_case(kinds, k0, k, dtype, seed=k0 + k)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.int32])
@pytest.mark.parametrize("k0,k", [(8192, 4000), (16384, 100), (32768, 16384), (20000, 19000), (65536, 8192),
                                  (131072, 60000), (49153, 3)])
def test_chain_select_narrows_a_crowded_digit(dtype, k0, k):
    # the digit that is cut holds far more candidates than a workgroup ranks: it is narrowed by the
    # next bits, several times over, down to single keys (then the whole-row path takes the row)
    _chain_case(["outliers", "crowded", "tied outliers", "spread"], k0, k, dtype, seed=k0 * 3 + k)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.int32])
@pytest.mark.parametrize("k0,k", [(49153, 30000), (65536, 777), (131072, 5000), (33000, 32999)])
def test_chain_select_with_long_segments(dtype, k0, k):
    # 40 rows of more than 32768 candidates: the chain's workgroups take 4096 candidates each
    kinds = ["spread", "ties", "equal", "steps", "outliers", "crowded", "tied outliers", "spread"] * 5
    _chain_case(kinds, k0, k, dtype, seed=k0 + k + 1)


@pytest.mark.parametrize("k0", [20000, 40000, 70000])
def test_chain_select_of_identical_candidates(k0):
    # only a caller of the stand-alone select can hand over candidates that share key and index:
    # no bit tells them apart, and the row goes to the whole-row path; any k of them are the answer
    cv = torch.full((2, k0), 2.0)
    cv[1, : k0 // 2] = 5.0
    ci = torch.full((2, k0), 7, dtype=torch.int64)
    k = k0 // 2 + 1234
    v, i = _select(cv, ci, k, 1 << 20)
    assert torch.equal(i.cpu(), torch.full((2, k), 7, dtype=torch.int64))
    assert torch.equal(v[0].cpu(), torch.full((k,), 2.0))
    assert torch.equal(v[1].cpu(), torch.cat([torch.full((k0 // 2,), 5.0), torch.full((1234,), 2.0)]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.int32])
@pytest.mark.parametrize("rows,k0,zeros,k", [
    (1, 32768, 16384, 24576),    # a ReLU's zeros: the cut takes half of 16384 equal keys
    (3, 32768, 9000, 27000),     # ... of 9000, several rows
    (2, 20000, 12000, 13000),    # a row that does not fill its last segment
    (1, 32768, 32768, 5),        # nothing but the one key
    (1, 30000, 8192, 21808 + 1), # one zero survives: the lowest index of all
])
def test_one_launch_select_of_rows_with_thousands_of_one_key_at_the_cut(dtype, rows, k0, zeros, k):
    # 16385-32768 candidates of a 2- or 4-byte type: the one-launch form with 32 keys per thread, whose
    # tied rows list the members' indices in LDS; every workgroup of the row must come to the same cut
    g = torch.Generator().manual_seed(k0 + zeros)
    if dtype.is_floating_point:
        cv = torch.rand(rows, k0, generator=g) + 0.5
    else:
        cv = torch.randint(1, 30000, (rows, k0), generator=g)
    for r in range(rows):
        cv[r, torch.randperm(k0, generator=g)[:zeros]] = 0
    cv = cv.to(dtype)
    bound = 1 << 22
    ci = torch.stack([torch.randperm(bound, generator=g)[:k0] for _ in range(rows)])
    v, i = _select(cv, ci, k, bound)
    ev, ei = oracle.stage2(cv, ci, k)
    assert_same(v, i, ev, ei, f"{dtype} rows={rows} k0={k0} zeros={zeros} k={k}")


def test_chain_select_needs_no_cut_when_the_digit_belongs_whole():
    # k falls exactly on a boundary between two values: every member of the cut digit survives
    k0 = 16384
    cv = torch.cat([torch.full((6000,), 3.0), torch.full((k0 - 6000,), 1.0)])[torch.randperm(k0)].reshape(1, k0)
    ci = torch.randperm(1 << 20)[:k0].reshape(1, k0)
    v, i = _select(cv, ci, 6000, 1 << 20)
    ev, ei = oracle.stage2(cv, ci, 6000)
    assert_same(v, i, ev, ei, "whole digit")


def test_chain_select_after_stage1_takes_the_key_ranges_from_the_merge():
    # one long row through the operator: slabs + merge (which leaves the key ranges) + chained select
    from approx_topk import topk
    g = torch.Generator().manual_seed(7)
    x = torch.randint(-2000, 2000, (2, 1 << 22), generator=g).float() / 16        # many ties
    v, i = topk(x.cuda(), 8192, -1, j=4, k_mult=2)
    ev, ei = oracle.topk(x, 8192, -1, j=4, k_mult=2)
    assert_same(v, i, ev, ei, "two long rows")
    x16 = x.half()
    v, i = topk(x16.cuda(), 4096, -1, j=2, k_mult=4)
    ev, ei = oracle.topk(x16, 4096, -1, j=2, k_mult=4)
    assert_same(v, i, ev, ei, "two long fp16 rows")
