"""Short contiguous buckets, loaded whole by the lane that owns them.  With k_mult > 1 and buckets
of 16 to 256 bytes: both stages in one kernel (the `CONTIG` form of fused_regs_kernel).  Without a
second stage and buckets of 16 to 64 bytes: `whole_bucket_kernel`, a lane per bucket.  Bit-exact against the
oracle, which follows the reference's contiguous bucket geometry (priority_queue_approx_topk.cu:47-54)
and its two stages (approx_topk/priority_queue.py:75-88), through every way a row can end there:
by prefix, by a ranked list of tied keys, through LDS (a NaN in the row; more equal keys at the cut
than the list takes), with int32 indices and with the indices alone."""
import pytest
import torch

import oracle
from helpers import assert_same

pytestmark = pytest.mark.gpu

MARK = "short contiguous buckets"

# (rows, n, k, j, k_mult): bucket length n / (k * k_mult / j) elements
SHAPES_2B = [
    (130, 32768, 2048, 4, 4),   # 16 elements, eight waves
    (3, 8192, 512, 2, 2),       # 16 elements, fewer rows than CUs
    (200, 4096, 128, 1, 2),     # j = 1
    (64, 16384, 1024, 4, 2),    # 32 elements: four loads per bucket
    (5, 6144, 128, 2, 4),       # 24 elements: three loads
    (9, 4096, 384, 3, 2),       # j = 3
    (40, 2048, 128, 2, 4),      # 8 elements: one load
    (64, 32768, 1024, 4, 2),    # 64 elements = 128 bytes: two trips of four loads
    (12, 10240, 128, 2, 4),     # 40 elements: four loads, then one
    (20, 65536, 512, 2, 2),     # 128 elements = 256 bytes
]
SHAPES_4B = [
    (130, 32768, 2048, 4, 4),   # 16 elements = 64 bytes
    (3, 8192, 512, 2, 2),
    (200, 4096, 128, 1, 2),
    (64, 8192, 1024, 4, 2),
    (5, 3072, 128, 2, 4),       # 12 elements: three loads
    (9, 4096, 384, 3, 2),
    (40, 1024, 128, 2, 4),      # 4 elements: one load
    (64, 16384, 1024, 4, 2),    # 32 elements = 128 bytes
    (12, 5120, 128, 2, 4),      # 20 elements: four loads, then one
    (20, 32768, 512, 2, 2),     # 64 elements = 256 bytes
]
DTYPES = [torch.float16, torch.bfloat16, torch.int16, torch.float32, torch.int32]


def _shapes(dtype):
    return SHAPES_2B if dtype in (torch.float16, torch.bfloat16, torch.int16) else SHAPES_4B


def _data(kind, rows, n, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    if kind == "spread":
        if dtype.is_floating_point:
            return torch.randn(rows, n, generator=g).to(dtype)
        return torch.randint(-30000, 30000, (rows, n), generator=g, dtype=torch.int32).to(dtype)
    if kind == "ties":          # a dozen distinct values: every cut falls among equal keys
        return (torch.randint(-6, 7, (rows, n), generator=g).float() / 2).to(dtype)
    if kind == "equal":         # all equal: more ties at the cut than the ranked list takes
        return torch.full((rows, n), 3, dtype=torch.float32).to(dtype)
    if kind == "specials":      # NaN rows (stage 1 again with exact keys), infinities, both zeros
        x = torch.randn(rows, n, generator=g)
        x[::3, 5] = float("nan")
        x[1::4, n // 2] = float("inf")
        x[2::4, n // 3] = float("-inf")
        x[:, 7::64] = -0.0
        x[:, 9::64] = 0.0
        return x.to(dtype)
    if kind == "zeros":         # the zeros of a ReLU, negated: results must keep the sign of each zero
        return (torch.relu(torch.randn(rows, n, generator=g)) * -1.0).to(dtype)
    raise ValueError(kind)


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("kind", ["spread", "ties", "equal", "specials", "zeros"])
def test_one_kernel_for_short_contiguous_buckets_matches_the_oracle(dtype, kind):
    from approx_topk import _native, topk
    if not dtype.is_floating_point and kind in ("specials", "zeros"):
        pytest.skip("integers have no NaN and one zero")
    for case, (rows, n, k, j, km) in enumerate(_shapes(dtype)):
        x = _data(kind, rows, n, dtype, 1000 + case)
        xd = x.cuda()
        assert MARK in _native.describe(xd, k * km, j, k, layout=1), (dtype, rows, n, k, j, km)
        v, i = topk(xd, k, -1, j=j, k_mult=km, interleaved=False)
        ov, oi = oracle.topk(x, k, -1, j=j, k_mult=km, interleaved=False)
        assert_same(v, i, ov, oi, f"{dtype} {kind} [{rows}, {n}] k={k} j={j} k_mult={km}")


def test_int32_indices_and_indices_alone():
    from approx_topk import topk
    from approx_topk.experimental.compact_indices import topk_indices
    for dtype in (torch.float16, torch.float32):
        rows, n, k, j, km = _shapes(dtype)[0]
        x = _data("ties", rows, n, dtype, 7).cuda()
        _, want = topk(x, k, -1, j=j, k_mult=km, interleaved=False)
        for index_dtype in (torch.int32, torch.int64):
            got = topk_indices(x, k, -1, j=j, k_mult=km, interleaved=False, index_dtype=index_dtype)
            assert got.dtype == index_dtype and torch.equal(got.long(), want), (dtype, index_dtype)


def test_rows_spaced_apart_and_misaligned_outputs():
    # a row pitch that keeps rows 16-byte aligned but not adjacent; outputs that start off a 16-byte
    # boundary (results then leave one at a time)
    from approx_topk import _native
    L = _native.lib()
    rows, n, k, j, km = 33, 8192, 512, 4, 4
    x = _data("spread", rows, n, torch.float16, 11)
    holder = torch.zeros(rows, n + 24, dtype=torch.float16, device="cuda")
    xd = holder[:, :n]
    xd.copy_(x)
    assert MARK in _native.describe(xd, k * km, j, k, layout=1)
    ov, oi = oracle.topk(x, k, -1, j=j, k_mult=km, interleaved=False)
    for shift in (0, 1):
        vbuf = torch.zeros(rows * k + 8, dtype=torch.float16, device="cuda")
        ibuf = torch.zeros(rows * k + 8, dtype=torch.int64, device="cuda")
        values, indices = vbuf[shift:shift + rows * k].view(rows, k), ibuf[shift:shift + rows * k].view(rows, k)
        rc = L.atk_topk(xd.data_ptr(), rows, n, xd.stride(0), k * km, j, k, 1, _native.dtype_code(xd.dtype),
                        values.data_ptr(), indices.data_ptr(), 0, 0, torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        torch.cuda.synchronize()
        assert_same(values, indices, ov, oi, f"shift {shift}")


def test_shapes_the_kernel_leaves_to_the_two_kernel_path():
    from approx_topk import _native, topk
    # buckets of 512 bytes; a bucket count that does not fill whole tiles; a row with a remainder
    for rows, n, k, j, km in [(6, 65536, 128, 2, 2), (5, 3072, 64, 2, 4), (20, 4100, 128, 2, 2)]:
        x = _data("ties", rows, n, torch.float16, 3)
        xd = x.cuda()
        assert MARK not in _native.describe(xd, k * km, j, k, layout=1)
        v, i = topk(xd, k, -1, j=j, k_mult=km, interleaved=False)
        ov, oi = oracle.topk(x, k, -1, j=j, k_mult=km, interleaved=False)
        assert_same(v, i, ov, oi, f"[{rows}, {n}] k={k} j={j} k_mult={km}")


# ---- stage 1 alone: a lane per bucket ----

WHOLE = "whole_bucket_kernel"

# (rows, buckets, bucket bytes, j)
WHOLE_SHAPES = [
    (300, 256, 64, 2),    # whole workgroups of buckets
    (7, 100, 32, 1),      # a bucket count that leaves the last workgroup's lanes idle
    (1, 37, 48, 3),       # one short row, j = 3
    (16384 // 8, 32, 64, 2),  # many short rows
    (5, 4096, 16, 4),     # one load per bucket; j = 4 needs 16 bytes of 4-byte elements
    (3, 1000, 64, 4),
]


def _whole_cases(dtype):
    es = torch.empty(0, dtype=dtype).element_size()
    for rows, b, bucket_bytes, j in WHOLE_SHAPES:
        m = bucket_bytes // es
        if m >= j:
            yield rows, b * m, b * j, j


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("kind", ["spread", "ties", "specials", "zeros"])
def test_lane_per_bucket_stage1_matches_the_oracle(dtype, kind):
    from approx_topk import _native, topk
    if not dtype.is_floating_point and kind in ("specials", "zeros"):
        pytest.skip("integers have no NaN and one zero")
    for case, (rows, n, k, j) in enumerate(_whole_cases(dtype)):
        x = _data(kind, rows, n, dtype, 2000 + case)
        xd = x.cuda()
        assert WHOLE in _native.describe(xd, k, j, k, layout=1), (dtype, rows, n, k, j)
        v, i = topk(xd, k, -1, j=j, k_mult=1, interleaved=False)
        ov, oi = oracle.topk(x, k, -1, j=j, k_mult=1, interleaved=False)
        assert_same(v, i, ov, oi, f"{dtype} {kind} [{rows}, {n}] k={k} j={j}")


def test_lane_per_bucket_with_spaced_rows_narrow_indices_and_misaligned_outputs():
    from approx_topk import _native
    from approx_topk.experimental.compact_indices import topk_indices
    L = _native.lib()
    rows, n, k, j = 33, 8192, 1024, 2          # buckets of 16 fp16 elements
    x = _data("ties", rows, n, torch.float16, 21)
    holder = torch.zeros(rows, n + 40, dtype=torch.float16, device="cuda")
    xd = holder[:, :n]
    xd.copy_(x)
    assert WHOLE in _native.describe(xd, k, j, k, layout=1)
    ov, oi = oracle.topk(x, k, -1, j=j, k_mult=1, interleaved=False)
    for shift in (0, 1):                      # 1: outputs off a 16-byte boundary, entries leave one at a time
        vbuf = torch.zeros(rows * k + 8, dtype=torch.float16, device="cuda")
        ibuf = torch.zeros(rows * k + 8, dtype=torch.int64, device="cuda")
        values, indices = vbuf[shift:shift + rows * k].view(rows, k), ibuf[shift:shift + rows * k].view(rows, k)
        rc = L.atk_stage1(xd.data_ptr(), rows, n, xd.stride(0), k, j, 1, _native.dtype_code(xd.dtype),
                          values.data_ptr(), indices.data_ptr(), 0, 0, torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        torch.cuda.synchronize()
        assert_same(values, indices, ov, oi, f"shift {shift}")
    for index_dtype in (torch.int32, torch.int64):
        got = topk_indices(xd, k, -1, j=j, k_mult=1, interleaved=False, index_dtype=index_dtype)
        assert got.dtype == index_dtype and torch.equal(got.long().cpu(), oi)


def test_argmax_entry_point_over_whole_chunks():
    # the arg-max entry point's contiguous layout pads a row to k * ceil(n / k): nothing to pad here
    from approx_topk import _native
    from approx_topk.experimental import bucketed_argmax
    x = _data("ties", 50, 512 * 24, torch.bfloat16, 5)
    xd = x.cuda()
    assert WHOLE in _native.describe(xd, 512, 1, 512, layout=_native.CEIL_CHUNK)
    v, i = bucketed_argmax.topk_triton(xd, k=512, dim=1, interleaved=False)
    ov, oi = oracle.bucketed_argmax(x, 512, 1, interleaved=False)
    assert_same(v, i, ov, oi, "arg-max over whole chunks")
