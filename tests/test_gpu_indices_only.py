"""`values == NULL` in the C ABI (approx_topk.experimental.compact_indices.topk_indices): the
indices alone, identical to those of the full call, through every kernel family.  The families
the cases reach are read back from the library's own description of each call."""
import pytest
import torch

from helpers import assert_same  # noqa: F401  (keeps the helpers importable from this file's directory)

pytestmark = pytest.mark.gpu

# (dtype, shape, k, j, k_mult, interleaved, nan)
CASES = [
    (torch.float32, (128, 1 << 16), 4096, 2, 1, True, False),    # streaming kernel, 16-byte accesses
    (torch.float32, (7, 30011), 1000, 2, 1, True, False),        # one element per load, partial sub-row
    (torch.float32, (33, 1 << 14), 1024, 4, 1, True, True),      # a NaN: the exact columns
    (torch.bfloat16, (64, 8192), 16, 1, 1, True, False),         # few buckets: folded sub-rows
    (torch.bfloat16, (64, 8192), 16, 1, 1, True, True),          # ... redone with order keys
    (torch.float32, (2, 1 << 22), 2048, 4, 1, True, False),      # slabs and their merge
    (torch.int32, (64, 8192), 256, 2, 1, False, False),          # contiguous buckets through LDS
    (torch.float16, (2, 1 << 20), 64, 2, 1, False, False),       # ... long buckets in chunks, merged
    (torch.float16, (256, 8192), 512, 4, 4, True, False),        # both stages in one kernel, in registers
    (torch.float16, (256, 8192), 512, 4, 4, True, True),         # ... a NaN: through LDS
    (torch.float32, (300, 1 << 16), 64, 1, 8, True, False),      # ... waves sharing tiles
    (torch.float64, (200, 1 << 14), 256, 2, 2, True, False),     # ... 8-byte elements
    (torch.float32, (200, 1 << 16), 4096, 2, 2, True, False),    # ... more column tiles than waves: through LDS
    (torch.float32, (8, 1 << 16), 512, 2, 2, True, False),       # streaming kernel, then one workgroup per row
    (torch.float32, (1, 1 << 22), 8192, 4, 2, True, False),      # ... then the chain over many workgroups
    (torch.int16, (1, 1 << 22), 8192, 4, 2, True, False),        # ... with thousands of equal keys at the cut
    (torch.float32, (1, 1 << 22), 65536, 4, 2, True, False),     # ... too many candidates for one launch: the chain of three
    (torch.uint8, (2, 1 << 23), 1 << 19, 2, 2, True, False),     # ... then passes over many workgroups
    (torch.float32, (2048, 2048), 64, 1, 2, False, False),       # contiguous buckets, then many small selects
]


def _input(dtype, shape, nan, seed):
    g = torch.Generator().manual_seed(seed)
    if dtype.is_floating_point:
        x = torch.randn(shape, generator=g).to(dtype)
        if nan:
            flat = x.view(-1)
            flat[torch.randint(0, flat.numel(), (max(1, flat.numel() // 5000),), generator=g)] = float("nan")
        return x
    if dtype == torch.uint8:
        return torch.randint(0, 256, shape, generator=g, dtype=torch.int32).to(dtype)
    return torch.randint(-30000, 30000, shape, generator=g, dtype=torch.int32).to(dtype)


def test_indices_alone_match_the_full_call_in_every_kernel_family():
    from approx_topk import _native, topk
    from approx_topk.experimental.compact_indices import topk_indices

    seen = ""
    for n, (dtype, shape, k, j, km, interleaved, nan) in enumerate(CASES):
        x = _input(dtype, shape, nan, 100 + n).cuda()
        _, want = topk(x, k, -1, j=j, k_mult=km, interleaved=interleaved)
        label = f"{dtype} {shape} k={k} j={j} k_mult={km} interleaved={interleaved} nan={nan}"
        for index_dtype in (torch.int32, torch.int64):
            got = topk_indices(x, k, -1, j=j, k_mult=km, interleaved=interleaved, index_dtype=index_dtype)
            assert got.dtype == index_dtype and got.shape == want.shape, label
            assert torch.equal(got.long(), want), label
        layout = _native.INTERLEAVED if interleaved else _native.BALANCED
        seen += _native.describe(x, k * km, j, k, layout) + "\n"
    for family in ("stream_kernel", "stream_merge_kernel", "contig_kernel", "contig_merge_kernel",
                   "fused_regs_kernel", "fused_row_kernel", "select_kernel", "chain_solo_kernel", "chain_emit_kernel",
                   "ms_emit_kernel"):
        assert family in seen, (family, seen)


def test_indices_alone_through_the_padded_layouts_and_the_general_kernel():
    # the arg-max layouts (one entry per bucket, rows padded to whole buckets) and the lane-per-bucket kernel
    from approx_topk import _native

    g = torch.Generator().manual_seed(5)
    for shape, k0, layout in [((9, 1000), 48, _native.CEIL_CHUNK), ((9, 1000), 48, _native.INTERLEAVED_PADDED),
                              ((3, 20), 32, _native.INTERLEAVED_PADDED), ((5, 333), 111, _native.BALANCED)]:
        x = torch.randn(shape, generator=g).cuda()
        _, want = _native.stage1(x, k0, 1, layout)
        none, got = _native.stage1(x, k0, 1, layout, torch.int64, False)
        assert none is None and torch.equal(got, want), (shape, k0, layout)


def test_select_alone_without_values():
    import ctypes

    from approx_topk import _native

    g = torch.Generator().manual_seed(9)
    cv = torch.randn(6, 5000, generator=g).cuda()
    ci = torch.stack([torch.randperm(1 << 20, generator=g)[:5000] for _ in range(6)]).cuda()
    _, want = _native.select(cv, ci, 700, 1 << 20)
    got = torch.empty_like(want)
    L = _native.lib()
    need = L.atk_select_workspace_bytes(6, 5000, 700, _native.dtype_code(cv.dtype))
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
    rc = L.atk_select(cv.data_ptr(), ci.data_ptr(), 6, 5000, 700, 1 << 20, _native.dtype_code(cv.dtype), None,
                      got.data_ptr(), ws.data_ptr(), need, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(got, want)
