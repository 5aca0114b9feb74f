"""Stage 1 with the results leaving through LDS in whole-wave stores (the `WAVE_STORES` form of
stream_kernel, which the planner takes for launches of 2048 workgroups and more whose workgroups
write at least an eighth of what they read).  Bit-exact against the oracle, which follows the
reference's interleaved bucket geometry and per-bucket queues
(priority_queue_approx_topk.cu:25-35, 58-147): every element type and j that has such a kernel,
exact runs of four and eight sub-rows and the general scan loop, one to eight waves per
workgroup, a partial last sub-row, a last column tile that is not full, heavy ties, NaN rows
(which take the exact path out of the same kernel), int32 indices and the indices alone.  Every
case asserts that the planner really chose these kernels."""
import pytest
import torch

import oracle
from helpers import assert_same

pytestmark = pytest.mark.gpu

# element types and the j that have whole-wave stores: a lane's stretch of output is 128 bytes
# or more of indices, or its elements are shorter than four bytes
KINDS = [
    (torch.float32, 4), (torch.int32, 4),
    (torch.float16, 1), (torch.float16, 2), (torch.float16, 4),
    (torch.bfloat16, 2), (torch.bfloat16, 4), (torch.int16, 1), (torch.int16, 4),
    (torch.uint8, 2), (torch.uint8, 4), (torch.int8, 2), (torch.int8, 4),
]
# sub-rows per bucket: exact runs (4; 8 = two waves of 4), the general loop (6, 12), a partial
# last sub-row (+ rem elements)
LENGTHS = [(4, 0), (6, 0), (8, 0), (12, 5000)]


def _native():
    from approx_topk import _native
    return _native


def _topk():
    from approx_topk import topk
    return topk


def _vec(dtype):
    return min(8, 16 // torch.empty(0, dtype=dtype).element_size())


def _data(kind, rows, n, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    if kind == "ties":  # a dozen distinct values: every queue is full of equal keys
        return torch.randint(0, 12, (rows, n), generator=g).to(dtype)
    if dtype.is_floating_point:
        x = torch.randn(rows, n, generator=g).to(dtype)
        if kind == "specials":  # NaN in every other row, infinities and both zeros in all
            sp = torch.tensor([float("inf"), -float("inf"), 0.0, -0.0, float("nan")]).to(dtype)
            at = torch.randint(0, n, (rows, n // 40), generator=g)
            what = torch.randint(0, 5, (rows, n // 40), generator=g)
            what[1::2] = what[1::2].clamp(max=3)
            for r in range(rows):
                x[r, at[r]] = sp[what[r]]
        return x
    info = torch.iinfo(dtype)
    return torch.randint(info.min, info.max + 1, (rows, n), generator=g, dtype=torch.int64).to(dtype)


def _check(x, k, j, want="wave-stores"):
    native = _native()
    xg = x.cuda()
    plan = native.describe(xg, k, j, k)
    assert want in plan, plan
    v, i = _topk()(xg, k, -1, j=j, k_mult=1)
    ev, ei = oracle.topk(x, k, -1, j=j, k_mult=1)
    assert_same(v, i, ev, ei, plan)
    return xg, ei


@pytest.mark.parametrize("length,rem", LENGTHS)
@pytest.mark.parametrize("dtype,j", KINDS)
def test_wave_stores_match_the_oracle(dtype, j, length, rem):
    b = 64 * _vec(dtype) * 32            # 32 whole column tiles
    rows, n = 64, b * length + rem       # 2048 workgroups
    seed = 1000 * length + 10 * j + KINDS.index((dtype, j))
    _check(_data("spread", rows, n, dtype, seed), b * j, j)


@pytest.mark.parametrize("dtype,j", [(torch.float16, 2), (torch.bfloat16, 4), (torch.float32, 4),
                                     (torch.int16, 4), (torch.uint8, 2), (torch.int8, 4)])
@pytest.mark.parametrize("kind", ["ties", "specials"])
def test_wave_stores_with_ties_and_special_values(dtype, j, kind):
    if kind == "specials" and not dtype.is_floating_point:
        pytest.skip("integer types have no NaN, infinities or signed zeros")
    b = 64 * _vec(dtype) * 32
    _check(_data(kind, 64, b * 6, dtype, 77 + j), b * j, j)


@pytest.mark.parametrize("dtype,j", [(torch.float16, 2), (torch.float32, 4), (torch.uint8, 4)])
def test_wave_stores_last_column_tile_not_full(dtype, j):
    """The row's last column tile has lanes beyond its last column: whole waves still go through
    the hand-over in LDS and only the columns that exist are written."""
    v = _vec(dtype)
    b = 64 * v * 32 - 5 * v               # the last tile lacks five lanes' columns
    _check(_data("spread", 64, b * 8, dtype, 5), b * j, j)


@pytest.mark.parametrize("dtype,j,length", [(torch.float16, 4, 32), (torch.float16, 4, 64),
                                            (torch.float16, 2, 16), (torch.bfloat16, 1, 32)])
def test_wave_stores_with_four_and_eight_waves(dtype, j, length):
    """Longer columns: four and eight waves per workgroup fold their queues before the results
    leave (fp16 [256, 2^20] k=65536, the shape of the reference's recorded rows, scaled down in
    rows; notebooks/data/generic2/measure_speed_approx_finer_multi2.jsonl:1723-1731 there)."""
    b = 64 * _vec(dtype) * 128
    rows = 16
    x = _data("spread", rows, b * length, dtype, 9 + length)
    xg, _ = _check(x, b * j, j)
    plan = _native().describe(xg, b * j, j, b * j)
    assert ("W=8" in plan or "W=4" in plan), plan


@pytest.mark.parametrize("dtype,j", [(torch.float16, 2), (torch.float32, 4), (torch.int8, 2)])
def test_wave_stores_int32_indices_and_indices_alone(dtype, j):
    from approx_topk.experimental.compact_indices import topk as topk_int32, topk_indices
    b = 64 * _vec(dtype) * 32
    x = _data("spread", 64, b * 6, dtype, 21 + j)
    xg, ei = _check(x, b * j, j)
    v32, i32 = topk_int32(xg, b * j, -1, j=j, k_mult=1)
    assert i32.dtype == torch.int32 and torch.equal(i32.cpu().long(), ei)
    ev, _ = oracle.topk(x, b * j, -1, j=j, k_mult=1)
    assert_same(v32, i32.long(), ev, ei, "int32 indices")
    only = topk_indices(xg, b * j, -1, j=j, k_mult=1)
    assert torch.equal(only.cpu().long(), ei)
