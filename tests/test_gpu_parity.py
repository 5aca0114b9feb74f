"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on the
same seeded inputs -- values bit-exact, indices identical, same output order.
Shapes follow the reference's own tests (tests/test_priority_queue.py)."""
import pytest
import torch

import oracle
from helpers import assert_same, cpu_randn, oracle_topk

pytestmark = pytest.mark.gpu

FLOATS = [torch.float32, torch.bfloat16, torch.float16]
ALL_DTYPES = FLOATS + [torch.float64, torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64]


def _topk():
    from approx_topk import topk
    return topk


def _run(x_cpu, k, dim=-1, **kw):
    v, i = _topk()(x_cpu.cuda(), k, dim, **kw)
    torch.cuda.synchronize()
    return v, i


def _check(x_cpu, k, dim=-1, what="", **kw):
    v, i = _run(x_cpu, k, dim, **kw)
    kw.pop("multithread_buckets", None)
    ev, ei = oracle_topk(x_cpu, k, dim, **kw)
    assert_same(v, i, ev, ei, what or f"shape={tuple(x_cpu.shape)} k={k} dim={dim} {kw}")
    if k:
        assert torch.equal(x_cpu.gather(dim, i.cpu()).view(torch.uint8 if x_cpu.element_size() == 1 else
                                                           {2: torch.int16, 4: torch.int32, 8: torch.int64}[x_cpu.element_size()]),
                           v.cpu().view(torch.uint8 if x_cpu.element_size() == 1 else
                                        {2: torch.int16, 4: torch.int32, 8: torch.int64}[x_cpu.element_size()]))


@pytest.mark.parametrize("k", [0, 2, 4])
@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("multithread_buckets", [False, True])
def test_one_bucket_no_batch_equals_exact(k, dtype, interleaved, multithread_buckets):
    x = cpu_randn(1001, 234, dtype)
    v, i = _run(x, k, 0, j=k, interleaved=interleaved, multithread_buckets=multithread_buckets)
    ev, ei = torch.topk(x.float(), k, dim=0)
    assert torch.equal(v.cpu().float().sort().values, ev.sort().values)
    assert torch.equal(x[i.cpu()], v.cpu())
    if k:
        _check(x, k, 0, j=k, interleaved=interleaved)


@pytest.mark.parametrize("k", [0, 2, 4])
@pytest.mark.parametrize("dim", [0, 1, 2])
@pytest.mark.parametrize("interleaved", [False, True])
def test_one_bucket_batched_any_dim(k, dim, interleaved):
    g = torch.Generator().manual_seed(4242)
    x = torch.rand((30, 25, 16), generator=g)
    v, i = _run(x, k, dim, j=k, interleaved=interleaved)
    ev, ei = torch.topk(x, k, dim)
    assert torch.equal(v.cpu().sort(dim).values, ev.sort(dim).values)
    assert torch.equal(i.cpu().sort(dim).values, ei.sort(dim).values)
    assert v.is_contiguous() and list(v.shape) == list(ev.shape)


@pytest.mark.parametrize("dim", [-1, -2])
def test_negative_dim(dim):
    x = cpu_randn((128, 256), 99)
    _check(x, 4, dim, j=4)


def test_call_twice_same_result():
    x = cpu_randn((128,), 56)
    a = _run(x, 4, 0)
    b = _run(x, 4, 0)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


@pytest.mark.parametrize("n", [10, 16])
@pytest.mark.parametrize("interleaved", [False, True])
def test_bucket_size_one_no_batch(n, interleaved):
    x = cpu_randn(n, 856)
    v, i = _run(x, n, 0, j=1, interleaved=interleaved)
    assert torch.equal(i.cpu(), torch.arange(n)) and torch.equal(v.cpu(), x)


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("interleaved", [False, True])
def test_bucket_size_one_batched(dtype, interleaved):
    x = cpu_randn((16, 4, 12), 23, dtype)
    v, i = _run(x, 12, 2, j=1, interleaved=interleaved)
    ev, ei = torch.topk(x.float(), 12, 2)
    assert torch.equal(v.cpu().float().sort(2).values, ev.sort(2).values)
    _check(x, 12, 2, j=1, interleaved=interleaved)


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("interleaved", [False, True])
def test_k_mult_bucket_size_one_equals_exact(dtype, interleaved):
    # 1024 buckets of one element, then an exact top-64 of all of them
    x = cpu_randn((32, 1024), 23, dtype)
    v, i = _run(x, 64, -1, k_mult=16, j=1, interleaved=interleaved)
    ev, ei = torch.topk(x.float(), 64, -1)
    assert torch.equal(v.cpu().float().sort(-1).values, ev.sort(-1).values)
    _check(x, 64, -1, k_mult=16, j=1, interleaved=interleaved)


def _ideal_rows(n, hot):
    xs = torch.zeros(len(hot), n)
    for r, cells in enumerate(hot):
        for pos, val in cells:
            xs[r, pos] = val
    return xs


def test_ideal_contiguous_n17():
    x = _ideal_rows(17, [
        [(0, 11.), (4, 12.), (5, 13.), (8, 14.), (9, 15.), (12, 16.), (13, 17.), (16, 18.)],
        [(2, 21.), (3, 22.), (6, 23.), (7, 24.), (10, 25.), (11, 26.), (14, 27.), (15, 28.)]])
    v, i = _run(x, 8, 1, j=2, interleaved=False)
    ev, ei = torch.topk(x, 8, dim=1)
    assert torch.equal(v.cpu().sort(1).values, ev.sort(1).values)
    assert torch.equal(i.cpu().sort(1).values, ei.sort(1).values)


def test_ideal_interleaved_n17():
    x = _ideal_rows(17, [
        [(0, 11.), (16, 12.), (1, 13.), (13, 14.), (2, 15.), (14, 16.), (3, 17.), (15, 18.)],
        [(4, 21.), (8, 22.), (5, 23.), (9, 24.), (6, 25.), (10, 26.), (7, 27.), (11, 28.)]])
    v, i = _run(x, 8, 1, j=2, interleaved=True)
    ev, ei = torch.topk(x, 8, dim=1)
    assert torch.equal(v.cpu().sort(1).values, ev.sort(1).values)
    assert torch.equal(i.cpu().sort(1).values, ei.sort(1).values)


def test_contiguous_long_sequence_n10000():
    n, k, j, stride = 10_000, 8, 2, 625
    g = torch.Generator().manual_seed(1)
    x = torch.zeros(2, n)
    x[0, list(range(0, n, stride))] = torch.rand(n // stride, generator=g) + 2.0
    x[1, list(range(50, n, stride))] = torch.rand(n // stride, generator=g) + 2.0
    _check(x, k, 1, j=j, interleaved=False)


@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("j", [1, 2, 4])
@pytest.mark.parametrize("k_mult", [1, 2, 4])
def test_reference_parity_shape(interleaved, j, k_mult):
    # randn(5, 32, 512), k=64: the shape of the reference's kernel-vs-torch test
    x = cpu_randn((5, 32, 512), 100)
    _check(x, 64, -1, j=j, k_mult=k_mult, interleaved=interleaved)
    v, i = _run(x, 64, -1, j=j, k_mult=k_mult, interleaved=interleaved)
    tv, ti = oracle.torch_bucketed_topk(x, 64, j, k_mult) if interleaved else (None, None)
    if tv is not None:
        assert torch.equal(v.cpu().sort(-1).values, tv.sort(-1).values)
        assert torch.equal(i.cpu().sort(-1).values, ti.sort(-1).values)


@pytest.mark.parametrize("dtype", ALL_DTYPES)
@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("j,k_mult", [(1, 1), (2, 2), (3, 1), (4, 4)])
def test_all_dtypes_with_ties(dtype, interleaved, j, k_mult):
    g = torch.Generator().manual_seed(7 + j)
    if dtype.is_floating_point:
        x = torch.randint(-6, 7, (3, 7, 333), generator=g).to(dtype) / 2
    elif dtype == torch.uint8:
        x = torch.randint(0, 12, (3, 7, 333), generator=g).to(dtype)
    else:
        x = torch.randint(-6, 7, (3, 7, 333), generator=g).to(dtype)
    _check(x, 12, -1, j=j, k_mult=k_mult, interleaved=interleaved)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.float64])
def test_special_values(dtype):
    g = torch.Generator().manual_seed(3)
    x = torch.randn((4, 4096), generator=g).to(dtype)
    sel = torch.randint(0, 4096, (4, 200), generator=g)
    specials = torch.tensor([float("nan"), float("inf"), -float("inf"), 0.0, -0.0]).to(dtype)
    for r in range(4):
        x[r, sel[r]] = specials[torch.randint(0, 5, (200,), generator=g)]
    for j, km in [(1, 1), (2, 1), (4, 2), (1, 4)]:
        _check(x, 256, -1, j=j, k_mult=km)
        _check(x, 256, -1, j=j, k_mult=km, interleaved=False)


@pytest.mark.parametrize("n,k,j", [(17, 8, 2), (1001, 12, 4), (1000, 16, 1), (65, 64, 1), (4099, 33, 3),
                                   (5000, 1250, 2), (70001, 4096, 4)])
@pytest.mark.parametrize("interleaved", [True, False])
def test_ragged_shapes(n, k, j, interleaved):
    x = cpu_randn((3, n), n + k)
    _check(x, k, -1, j=j, interleaved=interleaved)


def test_all_equal_rows_cut_ties_by_index():
    x = torch.zeros(2, 4096)
    x[1] = 1.5
    for j, km in [(1, 2), (2, 4), (4, 8)]:
        _check(x, 128, -1, j=j, k_mult=km)


def test_row_stride_input():
    big = cpu_randn((6, 3000), 5)
    xg = big.cuda()[:, :2048]
    v, i = _topk()(xg, 64, -1, j=2, k_mult=2)
    ev, ei = oracle_topk(big[:, :2048].contiguous(), 64, -1, j=2, k_mult=2)
    assert_same(v, i, ev, ei, "strided rows")


def test_config_shapes_reduced():
    # C2-like (L=32 interleaved, no stage 2), C3-like fp16, C4-like, C5-like
    _check(cpu_randn((4, 1 << 16), 1002), 4096, -1, j=2)
    _check((cpu_randn((8, 32768), 1003) / 128 ** 0.5).half(), 2048, -1, j=4, k_mult=4)
    _check(cpu_randn((4, 131072), 1004), 64, -1, j=1, k_mult=8)
    n = 1 << 20
    x = 0.5 * torch.linspace(-1, 1, n) + cpu_randn((n,), 1005)
    _check(x.reshape(1, n), 1024, -1, j=4, k_mult=2)


def test_errors_match_reference_types():
    topk = _topk()
    x = torch.randn(8, 64, device="cuda")
    with pytest.raises(NotImplementedError):
        topk(x, 4, 0, j=2)
    with pytest.raises(ValueError):
        topk(x, 4, -1, k_mult=0)
    with pytest.raises(RuntimeError):
        topk(x, 6, -1, j=4)
    with pytest.raises(RuntimeError):
        topk(x, 5, -1, j=5)
    with pytest.raises(RuntimeError):
        topk(x, 128, -1)


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("multithread_buckets", [None, False, True])
def test_opcheck(dtype, interleaved, multithread_buckets):
    x = cpu_randn((32, 128), 0, dtype).cuda()
    torch.library.opcheck(_topk(), args=(x,), kwargs=dict(
        k=12, dim=-1, j=1, interleaved=interleaved, multithread_buckets=multithread_buckets))


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("interleaved", [False, True])
def test_torch_compile_fullgraph(dtype, interleaved):
    topk = _topk()
    compiled = torch.compile(topk, fullgraph=True)
    x = cpu_randn((32, 128), 0, dtype).cuda()
    kw = dict(xs=x, k=12, dim=-1, j=2, interleaved=interleaved, multithread_buckets=None)
    ev, ei = topk(**kw)
    cv, ci = compiled(**kw)
    assert torch.equal(ev, cv) and torch.equal(ei, ci)


# ---- shapes that take the fused one-workgroup-per-row kernel (many rows, k_mult > 1) ----

@pytest.mark.parametrize("dtype", ALL_DTYPES)
@pytest.mark.parametrize("j,k_mult", [(1, 2), (2, 4), (3, 2), (4, 4)])
def test_fused_rows_all_dtypes_with_ties(dtype, j, k_mult):
    g = torch.Generator().manual_seed(11 + j)
    shape = (130, 2048)
    if dtype.is_floating_point:
        x = torch.randint(-9, 10, shape, generator=g).to(dtype) / 4
    elif dtype == torch.uint8:
        x = torch.randint(0, 19, shape, generator=g).to(dtype)
    else:
        x = torch.randint(-9, 10, shape, generator=g).to(dtype)
    _check(x, 48, -1, j=j, k_mult=k_mult)


@pytest.mark.parametrize("n,k,j,k_mult", [
    (4096, 64, 1, 8),      # two tiles, long columns: waves share a tile
    (4100, 64, 2, 4),      # partial last sub-row
    (32768, 2048, 4, 4),   # the sparse-attention shape, fp32
    (16384, 1024, 2, 8),   # 4096 columns: more tiles than waves
    (1000, 100, 4, 2),     # bucket count not a multiple of the vector width -> general path
    (777, 12, 3, 5),
])
def test_fused_rows_shapes(n, k, j, k_mult):
    _check(cpu_randn((136, n), n + k), k, -1, j=j, k_mult=k_mult)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.int16])
@pytest.mark.parametrize("rows,n,k,j", [(9, 49152, 2048, 2), (9, 49252, 4096, 4), (300, 32768, 2048, 4),
                                        (5, 1 << 18, 16384, 4), (3, 33 * 2048 + 7, 4096, 2)])
def test_packed_queues_over_columns_of_33_to_64_sub_rows(dtype, rows, n, k, j):
    # 16-bit types, two or four entries per column, columns of 33-64 sub-rows: the general scan loop
    # with eight loads in flight; ties, and a ragged last sub-row
    g = torch.Generator().manual_seed(n + k + j)
    x = torch.randint(-300, 300, (rows, n), generator=g)
    x = (x / 8).to(dtype) if dtype.is_floating_point else x.to(dtype)
    _check(x, k, -1, j=j)


@pytest.mark.parametrize("dtype,rows,n,k,j,k_mult", [
    (torch.float16, 130, 65536, 4096, 4, 8),     # 32768 candidates: 128 KiB of LDS
    (torch.bfloat16, 9, 65536, 3072, 1, 8),      # 24576 candidates, few rows
    (torch.float32, 130, 65536, 4096, 4, 4),     # 16384 fp32 candidates: 96 KiB
    (torch.float32, 40, 32768, 2048, 2, 8),
    (torch.int16, 130, 65536, 2560, 2, 8),       # 20480 candidates
    (torch.float32, 300, 16384, 1024, 2, 8),     # more rows than CUs: eight waves, the tiles in two rounds
    (torch.float16, 300, 32768, 2048, 1, 8),
    (torch.float16, 256, 32768, 2048, 1, 8),     # no more rows than CUs: sixteen waves
])
def test_fused_rows_with_candidates_beyond_64_kib_of_lds(dtype, rows, n, k, j, k_mult):
    g = torch.Generator().manual_seed(n + k + rows)
    x = torch.randint(-2000, 2000, (rows, n), generator=g)
    x = (x / 16).to(dtype) if dtype.is_floating_point else x.to(dtype)
    _check(x, k, -1, j=j, k_mult=k_mult)


@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.int16, torch.float32, torch.int32])
def test_fused_rows_results_past_the_cache(dtype, interleaved):
    """One round of workgroups whose results are an eighth of the row or more: the kernel whose staged
    results leave in non-temporal stores; with more rows, or misaligned outputs, the usual one.  The
    same results either way, with int64 and int32 indices and with the indices alone."""
    from approx_topk import _native
    from approx_topk.experimental.compact_indices import topk as topk_int32, topk_indices
    layout = _native.INTERLEAVED if interleaved else _native.BALANCED
    n, k, j, k_mult = 8192, 512, 4, 4
    g = torch.Generator().manual_seed(n + int(interleaved))
    for rows, past in [(300, True), (1200, False)]:
        x = torch.randint(-2000, 2000, (rows, n), generator=g)
        x = (x / 16).to(dtype) if dtype.is_floating_point else x.to(dtype)
        xg = x.cuda()
        plan = _native.describe(xg, k * k_mult, j, k, layout)
        assert ("past-cache" in plan) == past and "fused_regs_kernel" in plan, plan
        _check(x, k, -1, j=j, k_mult=k_mult, interleaved=interleaved)
        ev, ei = oracle_topk(x, k, -1, j=j, k_mult=k_mult, interleaved=interleaved)
        v32, i32 = topk_int32(xg, k, -1, j=j, k_mult=k_mult, interleaved=interleaved)
        assert_same(v32, i32.long(), ev, ei, "int32 indices")
        only = topk_indices(xg, k, -1, j=j, k_mult=k_mult, interleaved=interleaved)
        assert torch.equal(only.cpu().long(), ei)
    # outputs that are not 16-byte aligned: single stores, not past the cache
    values = torch.empty(300 * k + 1, dtype=dtype, device="cuda")[1:].view(300, k)
    indices = torch.empty(300 * k + 1, dtype=torch.int64, device="cuda")[1:].view(300, k)
    x = torch.randint(-2000, 2000, (300, n), generator=g)
    x = (x / 16).to(dtype) if dtype.is_floating_point else x.to(dtype)
    xg = x.cuda()
    rc = _native.lib().atk_topk(xg.data_ptr(), 300, n, n, k * k_mult, j, k, layout, _native.dtype_code(dtype),
                                values.data_ptr(), indices.data_ptr(), 0, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0  # (no workspace: both stages run in one kernel)
    torch.cuda.synchronize()
    ev, ei = oracle_topk(x, k, -1, j=j, k_mult=k_mult, interleaved=interleaved)
    assert_same(values, indices, ev, ei, "misaligned outputs")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.float64])
def test_fused_rows_special_values(dtype):
    g = torch.Generator().manual_seed(5)
    x = torch.randn((140, 4096), generator=g).to(dtype)
    specials = torch.tensor([float("nan"), float("inf"), -float("inf"), 0.0, -0.0]).to(dtype)
    for r in range(0, 140, 3):     # every third row holds special values, NaN included
        sel = torch.randint(0, 4096, (300,), generator=g)
        x[r, sel] = specials[torch.randint(0, 5, (300,), generator=g)]
    for j, km in [(1, 4), (2, 2), (4, 2)]:
        _check(x, 256, -1, j=j, k_mult=km)


@pytest.mark.parametrize("dtype", ALL_DTYPES)
@pytest.mark.parametrize("rows,n,k,j,k_mult", [(3, 256, 128, 4, 2), (200, 256, 128, 4, 2), (130, 4096, 1024, 2, 2),
                                               (2, 65536, 8192, 1, 4)])
def test_fused_rows_negative_survivors(dtype, rows, n, k, j, k_mult):
    # half or more of a row survives, so negative values are among the survivors: their
    # values are worked out from their order keys
    g = torch.Generator().manual_seed(rows + n)
    if dtype.is_floating_point:
        x = torch.randn((rows, n), generator=g).to(dtype)
    elif dtype == torch.uint8:
        x = torch.randint(0, 256, (rows, n), generator=g).to(dtype)
    else:
        x = torch.randint(-100, 100, (rows, n), generator=g).to(dtype)
    _check(x, k, -1, j=j, k_mult=k_mult)


def test_fused_rows_all_equal_cut_ties_by_index():
    x = torch.zeros(129, 4096)
    x[1::2] = 1.5
    for j, km in [(1, 2), (2, 4), (4, 8)]:
        _check(x, 128, -1, j=j, k_mult=km)


def test_fused_config3_and_config4_full_shapes():
    x3 = (cpu_randn((1024, 32768), 1003) / 128 ** 0.5).half()
    v, i = _run(x3, 2048, -1, j=4, k_mult=4)
    ev, ei = oracle_topk(x3[:96], 2048, -1, j=4, k_mult=4)
    assert_same(v[:96], i[:96], ev, ei, "C3 first 96 rows")
    assert torch.equal(x3.gather(-1, i.cpu()).view(torch.int16), v.cpu().view(torch.int16))
    x4 = cpu_randn((256, 131072), 1004)
    v, i = _run(x4, 64, -1, j=1, k_mult=8)
    ev, ei = oracle_topk(x4, 64, -1, j=1, k_mult=8)
    assert_same(v, i, ev, ei, "C4")


# ---- few, long buckets: the row is scanned several sub-rows side by side and a merge follows ----

@pytest.mark.parametrize("rows,n,k,j", [
    (32, 65536, 64, 1), (32, 65536, 64, 2), (128, 65536, 64, 4),   # the benchmark sweep's k = 64 shapes
    (5, 40000, 10, 1),       # 10 buckets: fold 24, 60 lanes busy
    (3, 30011, 30, 3),       # ragged row, three entries per bucket
    (2, 70000, 7, 1),        # bucket count not a multiple of the vector width
    (1, 1 << 22, 4, 4),      # one bucket: exact top-4 of a long row, many slabs
    (1, (1 << 20) + 13, 1, 1),
    (3, 20000, 8, 4), (3, 20000, 6, 3),
    # short enough rows that the scanning workgroup merges the folded columns itself
    (6, 4096, 16, 1), (6, 4099, 12, 2), (6, 2048, 12, 3), (130, 8192, 64, 4), (3, 5000, 7, 1), (2, 3000, 1, 1),
])
def test_few_long_buckets(rows, n, k, j):
    _check(cpu_randn((rows, n), n + k + j), k, -1, j=j)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.uint8])
@pytest.mark.parametrize("rows,n,k,j", [
    (200, 256, 16, 1),       # buckets of 16: fold 16 (fp32), one scanned sub-row
    (64, 1024, 64, 4),       # 16 buckets of 64, four entries each: the fold is cut down to leave 4 sub-rows
    (33, 1000, 50, 1), (128, 640, 40, 2), (16, 512, 64, 2), (300, 2048, 32, 1), (5, 4096, 512, 1), (7, 264, 33, 1),
])
def test_few_short_buckets(dtype, rows, n, k, j):
    g = torch.Generator().manual_seed(n + k)
    x = torch.randint(0, 200, (rows, n), generator=g).to(dtype) if dtype == torch.uint8 else \
        torch.randn((rows, n), generator=g).to(dtype)
    _check(x, k, -1, j=j)


@pytest.mark.parametrize("dtype", ALL_DTYPES)
@pytest.mark.parametrize("j,k_mult", [(1, 1), (2, 2), (3, 1), (4, 1)])
@pytest.mark.parametrize("n", [50001, 3001])
def test_few_long_buckets_all_dtypes_with_ties(dtype, j, k_mult, n):
    g = torch.Generator().manual_seed(23 + j)
    shape = (6, n)
    if dtype.is_floating_point:
        x = torch.randint(-9, 10, shape, generator=g).to(dtype) / 4
    elif dtype == torch.uint8:
        x = torch.randint(0, 19, shape, generator=g).to(dtype)
    else:
        x = torch.randint(-9, 10, shape, generator=g).to(dtype)
    _check(x, 12, -1, j=j, k_mult=k_mult)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("rows,n,k,j,k_mult", [
    (4, 32768, 4, 2, 2), (16, 32768, 4, 4, 8), (2, 4096, 2, 1, 2), (64, 1024, 4, 1, 2), (64, 1 << 18, 4, 1, 2),
    (300, 8192, 16, 1, 2), (2100, 2048, 16, 2, 4),
])
def test_few_buckets_with_a_second_stage(dtype, rows, n, k, j, k_mult):
    # aligned rows whose candidates would fit the one-kernel path: narrow sub-rows go to the folding
    # streaming kernel instead, short rows of few sub-rows stay
    g = torch.Generator().manual_seed(rows + n + k)
    x = (torch.randint(-50, 50, (rows, n), generator=g) / 8).to(dtype)
    _check(x, k, -1, j=j, k_mult=k_mult)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.float64])
@pytest.mark.parametrize("n", [40000, 4100])
def test_few_long_buckets_special_values(dtype, n):
    g = torch.Generator().manual_seed(8)
    x = torch.randn((6, n), generator=g).to(dtype)
    specials = torch.tensor([float("nan"), float("inf"), -float("inf"), 0.0, -0.0]).to(dtype)
    for r in range(0, 6, 2):
        sel = torch.randint(0, n, (500,), generator=g)
        x[r, sel] = specials[torch.randint(0, 5, (500,), generator=g)]
    for j, km in [(1, 1), (2, 1), (4, 2)]:
        _check(x, 16, -1, j=j, k_mult=km)


@pytest.mark.parametrize("dtype", [torch.int8, torch.uint8])
@pytest.mark.parametrize("rows,n,k,j", [
    (2, 1 << 20, 4096, 2),      # vector loads, one packed word per entry
    (3, 100003, 64, 4),         # odd row pitch: one column per lane
    (1, 1 << 22, 16, 4),        # folded row cut into slabs
    (130, 8192, 2048, 1), (5, 70001, 999, 3),
])
def test_byte_types_full_range(dtype, rows, n, k, j):
    info = torch.iinfo(dtype)
    g = torch.Generator().manual_seed(n + k)
    x = torch.randint(info.min, info.max + 1, (rows, n), generator=g).to(dtype)   # extremes and many ties
    _check(x, k, -1, j=j)


def test_few_long_buckets_unaligned_rows():
    x = cpu_randn((4, 30001), 77)            # odd row pitch: no 16-byte loads
    _check(x, 16, -1, j=2)
    wide = cpu_randn((4, 30016), 78)
    v, i = _topk()(wide.cuda()[:, 3:30003], 20, -1, j=2)   # misaligned base pointer, pitch > n
    ev, ei = oracle_topk(wide[:, 3:30003].contiguous(), 20, -1, j=2)
    assert_same(v, i, ev, ei, "misaligned view")
    small = cpu_randn((4, 4112), 79)
    v, i = _topk()(small.cuda()[:, 3:4103], 20, -1, j=2)
    ev, ei = oracle_topk(small[:, 3:4103].contiguous(), 20, -1, j=2)
    assert_same(v, i, ev, ei, "misaligned view, short rows")


# ---- contiguous buckets: spans of whole buckets staged in LDS, pieces per thread, long buckets in chunks ----

@pytest.mark.parametrize("rows,n,k,j", [
    (130, 4096, 128, 1),     # 32-element buckets, one thread each
    (7, 4100, 100, 2),       # 82/83-element buckets: four threads per bucket, ragged
    (3, 100003, 4, 2),       # two buckets of 50001/50002: a workgroup per bucket, seven chunks
    (2, 70000, 3, 3),        # one bucket, three entries
    (4, 9000, 1, 1),         # one bucket a little over one chunk
    (5, 2 * 8192 + 5, 2, 1), # buckets of 8194/8195: the last chunk holds two or three elements
    (3, 5000, 1250, 2), (3, 70001, 4096, 4), (2, 333, 333, 1), (2, 1024, 512, 2),
])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.float64, torch.int8])
def test_contiguous_buckets(rows, n, k, j, dtype):
    x = cpu_randn((rows, n), n + k + j)
    x = (x * 40).to(dtype) if not dtype.is_floating_point else x.to(dtype)
    _check(x, k, -1, j=j, interleaved=False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.uint8])
@pytest.mark.parametrize("rows,n,k,j,k_mult", [(2, 3024656, 4, 2, 1), (1, 5000011, 3, 1, 1), (3, 2000003, 2, 4, 4)])
def test_contiguous_buckets_few_and_very_long(dtype, rows, n, k, j, k_mult):
    # a bucket's chunks are shared out over many workgroups, unevenly when they do not divide
    g = torch.Generator().manual_seed(n + k)
    x = torch.randint(0, 200, (rows, n), generator=g).to(dtype) if dtype == torch.uint8 else \
        (torch.randint(-100000, 100000, (rows, n), generator=g) / 64).to(dtype)
    _check(x, k, -1, j=j, k_mult=k_mult, interleaved=False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float64])
@pytest.mark.parametrize("n,k", [(40000, 16), (4100, 64), (100000, 2)])
def test_contiguous_buckets_special_values(dtype, n, k):
    g = torch.Generator().manual_seed(9)
    x = torch.randn((6, n), generator=g).to(dtype)
    specials = torch.tensor([float("nan"), float("inf"), -float("inf"), 0.0, -0.0]).to(dtype)
    for r in range(0, 6, 2):
        sel = torch.randint(0, n, (500,), generator=g)
        x[r, sel] = specials[torch.randint(0, 5, (500,), generator=g)]
    for j, km in [(1, 1), (2, 1), (2, 2)]:
        _check(x, k, -1, j=j, k_mult=km, interleaved=False)


def test_contiguous_buckets_unaligned_rows():
    x = cpu_randn((4, 30001), 81)
    _check(x, 16, -1, j=2, interleaved=False)
    wide = cpu_randn((4, 30016), 82)
    v, i = _topk()(wide.cuda()[:, 3:30003], 20, -1, j=2, interleaved=False)
    ev, ei = oracle_topk(wide[:, 3:30003].contiguous(), 20, -1, j=2, interleaved=False)
    assert_same(v, i, ev, ei, "misaligned view")


# ---- gradient: values are a gather of the input, so their gradient scatters back ----

@pytest.mark.parametrize("k,j,k_mult,dim,interleaved", [(64, 2, 1, -1, True), (32, 4, 4, -1, True), (16, 1, 2, -1, False),
                                                      (4, 4, 1, 0, True)])
def test_gradient_scatters_to_the_selected_positions(k, j, k_mult, dim, interleaved):
    from approx_topk.experimental.differentiable import topk as topk_with_gradient
    x = cpu_randn((6, 512), 3).cuda().requires_grad_(True)
    v, i = topk_with_gradient(x, k, dim, j=j, k_mult=k_mult, interleaved=interleaved)
    pv, pi = _topk()(x.detach(), k, dim, j=j, k_mult=k_mult, interleaved=interleaved)
    assert torch.equal(v.detach(), pv) and torch.equal(i, pi) and not i.requires_grad
    w = torch.randn_like(v)
    (v * w).sum().backward()
    expect = torch.zeros_like(x).scatter(dim, i, w)
    assert torch.equal(x.grad, expect)
    # the same through plain torch ops on the returned indices
    x2 = x.detach().clone().requires_grad_(True)
    (x2.gather(dim, i) * w).sum().backward()
    assert torch.equal(x.grad, x2.grad)



# ---- int32 indices (approx_topk.experimental.compact_indices): same results, narrower ----

@pytest.mark.parametrize("rows,n,k,j,k_mult,interleaved", [
    (6, 32768, 1024, 2, 1, True),       # streaming kernel, 16-byte index stores
    (6, 32768, 1536, 3, 1, True),       # three entries per bucket
    (6, 4096, 16, 1, 1, True),          # few long buckets, merged in the workgroup
    (3, 40000, 10, 1, 1, True),         # folded and cut into slabs: merge kernel
    (1, 1 << 20, 1024, 2, 1, True),     # slabs
    (5, 1001, 12, 4, 1, True),          # no 16-byte loads
    (7, 4100, 100, 2, 1, False),        # contiguous buckets
    (3, 100003, 4, 2, 1, False),        # contiguous, chunks shared over workgroups
    (136, 4096, 64, 1, 8, True),        # fused kernel
    (4, 65536, 512, 2, 2, True),        # two kernels, one workgroup per row in stage 2
    (1, 1 << 20, 32768, 1, 4, True),    # stage 2 over many workgroups
])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.float64, torch.uint8])
def test_int32_indices(rows, n, k, j, k_mult, interleaved, dtype):
    from approx_topk.experimental.compact_indices import topk as topk_i32
    x = cpu_randn((rows, n), n + k + j)
    x = (x * 40).abs().to(dtype) if not dtype.is_floating_point else x.to(dtype)
    xg = x.cuda()
    v32, i32 = topk_i32(xg, k, -1, j=j, k_mult=k_mult, interleaved=interleaved)
    v64, i64 = _topk()(xg, k, -1, j=j, k_mult=k_mult, interleaved=interleaved)
    assert i32.dtype == torch.int32 and i64.dtype == torch.int64
    assert torch.equal(i32.long(), i64)
    assert torch.equal(v32.view(torch.uint8), v64.view(torch.uint8))
    ev, ei = oracle_topk(x, k, -1, j=j, k_mult=k_mult, interleaved=interleaved)
    assert_same(v32, i32.long(), ev, ei, f"{dtype} rows={rows} n={n} k={k} j={j} k_mult={k_mult}")


def test_int32_indices_refuse_rows_beyond_their_range():
    from approx_topk.experimental.compact_indices import topk as topk_i32
    x = torch.zeros((1, (1 << 31) + 8), dtype=torch.uint8, device="cuda")
    with pytest.raises(RuntimeError, match="32-bit"):
        topk_i32(x, 8, -1)
    del x
    torch.cuda.empty_cache()
