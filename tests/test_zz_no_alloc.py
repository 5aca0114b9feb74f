"""atk_topk_noalloc (scratch memory inside the library, no allocation) against atk_topk with a
caller workspace: same values and indices, bit for bit, on calls in a row that share the scratch
array -- the second with a smaller input -- and against the oracle."""
import ctypes

import pytest
import torch

import oracle
from helpers import assert_same

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 8 << 20


def _call_noalloc(x, k0, j, k, layout=0):
    from approx_topk import _native
    L = _native.lib()
    rows, n = x.shape
    values = torch.empty(rows, k, dtype=x.dtype, device=x.device)
    indices = torch.empty(rows, k, dtype=torch.int64, device=x.device)
    rc = L.atk_topk_noalloc(x.data_ptr(), rows, n, x.stride(0), k0, j, k, layout, _native.dtype_code(x.dtype),
                            values.data_ptr(), indices.data_ptr(),
                            torch.cuda.current_stream().cuda_stream)
    return rc, values, indices


def _call_with_workspace(x, k0, j, k, layout=0):
    from approx_topk import _native
    L = _native.lib()
    rows, n = x.shape
    code = _native.dtype_code(x.dtype)
    values = torch.empty(rows, k, dtype=x.dtype, device=x.device)
    indices = torch.empty(rows, k, dtype=torch.int64, device=x.device)
    need = L.atk_topk_workspace_bytes_at(x.data_ptr(), rows, n, x.stride(0), k0, j, k, layout, code)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=x.device)
    rc = L.atk_topk(x.data_ptr(), rows, n, x.stride(0), k0, j, k, layout, code, values.data_ptr(),
                    indices.data_ptr(), ws.data_ptr(), need, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    return need, values, indices


def _same(a, b):
    bits = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[a.element_size()]
    return torch.equal(a.view(bits), b.view(bits))


# (rows, n, dtype, k0, j, k): the first of each pair is followed by a smaller call that reuses the scratch
CASES = [
    # one long row: slabs + merge + stand-alone select, then a shorter row of the same kind
    [(1, 1 << 22, torch.float32, 8192, 4, 4096), (1, 1 << 20, torch.float32, 2048, 4, 1024)],
    # stage 1 alone (k == k0) on a row cut into slabs, then a smaller one
    [(2, 1 << 21, torch.float32, 64, 2, 64), (1, 1 << 19, torch.float32, 16, 1, 16)],
    # a batch through stage 1 + select with parked candidates (rows spaced so that one kernel declines), then fewer rows
    [(48, 40000, torch.float16, 1024, 2, 256), (5, 9000, torch.float16, 512, 1, 64)],
    # contiguous buckets shared out over workgroups, then interleaved in one kernel (no scratch at all)
    [(1, 1 << 22, torch.bfloat16, 8, 2, 4), (130, 4096, torch.bfloat16, 256, 4, 64)],
]


@pytest.mark.parametrize("pair", range(len(CASES)))
def test_noalloc_equals_workspace_version_on_consecutive_calls(pair):
    g = torch.Generator().manual_seed(77 + pair)
    for call, (rows, n, dtype, k0, j, k) in enumerate(CASES[pair]):
        layout = 1 if (pair == 3 and call == 0) else 0
        x_cpu = (torch.randint(-60, 61, (rows, n), generator=g).float() / 8).to(dtype)   # many ties
        stride_pad = 7 if pair == 2 else 0   # odd row pitch: the one-kernel path declines
        holder = torch.empty(rows, n + stride_pad, dtype=dtype, device="cuda")
        x = holder[:, :n]
        x.copy_(x_cpu)
        need, ev, ei = _call_with_workspace(x, k0, j, k, layout)
        assert need <= SCRATCH_BYTES
        rc, v, i = _call_noalloc(x, k0, j, k, layout)
        torch.cuda.synchronize()
        assert rc == 0
        assert _same(v, ev) and torch.equal(i, ei), (pair, call)
        # and once more on the same scratch, straight away
        rc, v2, i2 = _call_noalloc(x, k0, j, k, layout)
        torch.cuda.synchronize()
        assert rc == 0 and _same(v2, ev) and torch.equal(i2, ei), (pair, call, "repeat")
        ov, oi = oracle.topk(x_cpu, k, -1, j=j, k_mult=k0 // k, interleaved=layout == 0)
        assert_same(v, i, ov, oi, f"pair {pair} call {call}")
        if pair != 3 or call == 0:
            assert need > 0, "the case was meant to use scratch memory"


def test_noalloc_rejects_what_does_not_fit_and_bad_arguments():
    from approx_topk import _native
    L = _native.lib()
    x = torch.zeros(4096, 16385, dtype=torch.float32, device="cuda")[:, :16384]   # odd row pitch: two kernels
    need = L.atk_topk_workspace_bytes_at(x.data_ptr(), 4096, 16384, x.stride(0), 4096, 1, 1024, 0, 0)
    assert need > SCRATCH_BYTES
    rc, _, _ = _call_noalloc(x, 4096, 1, 1024)
    assert rc == -10
    assert b"scratch" in L.atk_strerror(-10)
    rc, _, _ = _call_noalloc(x, 4096, 3, 1024)      # j does not divide k0
    assert rc == -2
    rc, _, _ = _call_noalloc(x, 1 << 20, 1, 1024)   # k0 > n
    assert rc == -3
    torch.cuda.synchronize()


def test_noalloc_under_graph_capture_and_replay():
    # The entry point is for callers that cannot allocate: captured into a HIP graph (after one
    # eager call, which also looks up the scratch array's address) and replayed, with eager work
    # in between, it gives the workspace version's result every time and allocates nothing.
    g = torch.Generator().manual_seed(5)
    rows, n, k0, j, k = 1, 1 << 22, 8192, 4, 4096                # slabs + merge + select over several workgroups
    xs = [(torch.randint(-60, 61, (rows, n), generator=g).float() / 8).cuda() for _ in range(3)]
    x = torch.empty_like(xs[0])
    x.copy_(xs[0])
    need, ev, ei = _call_with_workspace(x, k0, j, k)
    assert 0 < need <= SCRATCH_BYTES
    rc, v, i = _call_noalloc(x, k0, j, k)
    torch.cuda.synchronize()
    assert rc == 0 and _same(v, ev) and torch.equal(i, ei)

    from approx_topk import _native
    L = _native.lib()
    values = torch.empty(rows, k, dtype=x.dtype, device="cuda")
    indices = torch.empty(rows, k, dtype=torch.int64, device="cuda")
    code = _native.dtype_code(x.dtype)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            before = torch.cuda.memory_stats()["allocation.all.allocated"]
            rc = L.atk_topk_noalloc(x.data_ptr(), rows, n, x.stride(0), k0, j, k, 0, code, values.data_ptr(),
                                    indices.data_ptr(), torch.cuda.current_stream().cuda_stream)
            after = torch.cuda.memory_stats()["allocation.all.allocated"]
        assert rc == 0
        assert after == before                                   # nothing came from torch's allocator either
    torch.cuda.current_stream().wait_stream(side)
    for replay, src in enumerate(xs + xs[:1]):
        x.copy_(src)
        _, ev, ei = _call_with_workspace(x, k0, j, k)             # eager work between the replays
        values.zero_(); indices.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert _same(values, ev) and torch.equal(indices, ei), replay
