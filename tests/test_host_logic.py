"""CPU-side checks: the C-ABI library loads and exports every declared symbol,
argument validation raises the reference's exception types before any GPU work,
and the torch-level entry points agree with the oracle."""
import ctypes
import os
import re

import pytest
import torch

import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from approx_topk import _native
    header = open(os.path.join(ROOT, "include", "approx_topk_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(atk_[a-z0-9_]+)\s*\(", header))
    assert {"atk_version", "atk_strerror", "atk_stage1", "atk_select", "atk_topk"} <= declared
    handle = ctypes.CDLL(_native.library_path())
    for name in declared:
        assert hasattr(handle, name), name
    assert set(_native._SIGNATURES) == declared
    # the clock stamps of the phase timelines (csrc/atk_trace.h) exist only in a library built for them
    assert not hasattr(handle, "atk_trace_fused_row_f16") and not hasattr(handle, "atk_trace_stage1_stream_f32")
    assert _native.lib().atk_version() == _native.ABI_VERSION
    assert _native.lib().atk_strerror(0) == b"ok"
    assert b"j must" in _native.lib().atk_strerror(-2)


def test_workspace_of_one_call_depends_on_the_address():
    from approx_topk import _native
    L = _native.lib()
    # 512 fp16 rows of 32768, 1024 candidates: one kernel, nothing parked
    general = L.atk_topk_workspace_bytes(512, 32768, 1024, 1, 256, 0, 1)
    assert general >= 512 * 1024 * (2 + 8)
    assert L.atk_topk_workspace_bytes_at(4096, 512, 32768, 32768, 1024, 1, 256, 0, 1) == 0
    # a misaligned input or an odd row stride goes through two kernels
    assert L.atk_topk_workspace_bytes_at(4098, 512, 32768, 32768, 1024, 1, 256, 0, 1) == general
    assert L.atk_topk_workspace_bytes_at(4096, 512, 32768, 32769, 1024, 1, 256, 0, 1) == general
    # k == k0: stage 1 alone
    assert L.atk_topk_workspace_bytes_at(4096, 512, 32768, 32768, 1024, 1, 1024, 0, 1) == \
        L.atk_topk_workspace_bytes(512, 32768, 1024, 1, 1024, 0, 1)
    # contiguous buckets: one kernel for buckets of up to 256 bytes (here 32 elements), else two
    assert L.atk_topk_workspace_bytes_at(4096, 512, 32768, 32768, 1024, 1, 256, 1, 1) == 0
    assert L.atk_topk_workspace_bytes_at(4096, 512, 1 << 18, 1 << 18, 1024, 1, 256, 1, 1) == \
        L.atk_topk_workspace_bytes(512, 1 << 18, 1024, 1, 256, 1, 1) > 0


def test_native_argument_checks_need_no_gpu():
    # rejected before any launch, so callable here
    from approx_topk import _native
    L = _native.lib()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    assert L.atk_stage1(p, 1, 8, 8, 6, 4, 0, 0, p, p, None, 0, None) == -2     # j does not divide k0
    assert L.atk_stage1(p, 1, 8, 8, 5, 5, 0, 0, p, p, None, 0, None) == -2     # j out of range
    assert L.atk_stage1(p, 1, 8, 8, 16, 1, 0, 0, p, p, None, 0, None) == -3    # k0 > n
    assert L.atk_stage1(p, 1, 8, 8, 4, 1, 9, 0, p, p, None, 0, None) == -4     # layout
    assert L.atk_stage1(p, 1, 8, 8, 4, 2, 2, 0, p, p, None, 0, None) == -4     # padded layout, j != 1
    assert L.atk_stage1(p, 1, 8, 8, 4, 1, 0, 99, p, p, None, 0, None) == -1    # dtype
    assert L.atk_stage1(None, 1, 8, 8, 4, 1, 0, 0, p, p, None, 0, None) == -7  # null input
    assert L.atk_stage1(p, 1, 8, 4, 4, 1, 0, 0, p, p, None, 0, None) == -7     # row_stride < n
    assert L.atk_stage1(p, 1, 8, 8, 0, 1, 0, 0, p, p, None, 0, None) == 0      # k0 == 0: no-op
    assert L.atk_topk(p, 1, 1 << 20, 1 << 20, 4, 1, 2, 0, 0, p, p, None, 0, None) == -5    # workspace missing (two kernels)
    assert L.atk_topk(p, 1, 8, 8, 4, 1, 5, 0, 0, p, p, None, 0, None) == -3    # k > k0
    assert L.atk_select(p, p, 1, 4, 5, 8, 0, p, p, None, 0, None) == -3
    # misaligned pointers: data to the element size, indices to their width, workspace to 16 bytes
    assert p % 16 == 0
    assert L.atk_stage1(p + 2, 1, 8, 8, 4, 1, 0, 0, p, p, None, 0, None) == -9      # fp32 input at +2
    assert L.atk_stage1(p, 1, 8, 8, 4, 1, 0, 0, p + 1, p, None, 0, None) == -9      # values
    assert L.atk_stage1(p, 1, 8, 8, 4, 1, 0, 0, p, p + 4, None, 0, None) == -9      # int64 indices at +4
    assert L.atk_stage1_i32(p, 1, 8, 8, 4, 1, 0, 0, p, p + 2, None, 0, None) == -9  # int32 indices at +2
    assert L.atk_stage1(p, 1, 8, 8, 4, 1, 0, 0, p, p, p + 8, 64, None) == -9        # workspace at +8
    assert L.atk_topk(p, 1, 1 << 20, 1 << 20, 4, 1, 2, 0, 0, p, p, p + 8, 1 << 30, None) == -9
    assert L.atk_select(p, p + 4, 1, 4, 2, 8, 0, p, p, None, 0, None) == -9         # candidate indices
    assert L.atk_select(p, p, 1, 4, 2, 8, 0, p, p, p + 4, 1 << 20, None) == -9
    assert b"misaligned" in L.atk_strerror(-9)
    assert L.atk_topk_workspace_bytes(3, 100, 8, 1, 8, 0, 0) == 0
    assert L.atk_topk_workspace_bytes(3, 100, 16, 1, 8, 0, 0) >= 3 * 16 * 12


def test_describe_names_the_planned_kernels():
    # the planner's choice for a call, as text (no GPU needed: nothing is enqueued)
    from approx_topk import _native
    L = _native.lib()

    def describe(rows, n, code, k, j, k_mult, x=4096):
        buf = ctypes.create_string_buffer(1024)
        assert L.atk_describe(x, rows, n, n, k * k_mult, j, k, 0, code, 4096, 4096, buf, 1024) == 0
        return buf.value.decode()
    c2 = describe(128, 1 << 20, 0, 65536, 2, 1)
    assert c2.startswith("stream_kernel<f32, J=2, V=4, W=8, U=8, RUN=4, PACKED=0> grid=16384 block=512")
    c3 = describe(1024, 32768, 1, 2048, 4, 4)
    assert c3.startswith("fused_regs_kernel<f16, J=4, V=4, pos16, PACKED=1> grid=1024 block=512")
    c5 = describe(1, 1 << 26, 0, 16384, 4, 2)
    assert c5.startswith("stream_kernel<f32, J=4") and "stream_merge_kernel" in c5 and "chain_solo_kernel" in c5
    # few buckets (narrow sub-rows): the streaming kernel, which folds sub-rows side by side,
    # not the one-kernel path, whose lanes would idle; short rows of few sub-rows stay with it
    assert describe(256, 1 << 22, 1, 4, 1, 2).startswith("stream_kernel<f16, J=1")
    assert describe(4, 32768, 1, 4, 2, 2).startswith("stream_kernel<f16, J=2")
    assert describe(4, 32768, 0, 4, 4, 8).startswith("stream_kernel<f32, J=4")
    assert describe(64, 1024, 1, 8, 1, 2).startswith("fused_regs_kernel<f16, J=1")
    # the select over several workgroups per row: few rows only, one launch up to 32768 candidates
    assert "chain_solo_kernel<f32> grid=16 " in describe(1, 1 << 24, 0, 8192, 2, 2)
    assert "chain_emit_kernel<f32> grid=512 block=256 per_thread=4" in describe(8, 1 << 22, 0, 32768, 2, 2)
    # more rows of more than 32768 candidates: segments of 4096 candidates; beyond 64 rows other selects
    assert "chain_emit_kernel<f32> grid=2048 block=256 per_thread=16" in describe(64, 1 << 18, 0, 16384, 2, 8)
    assert "chain_" not in describe(65, 1 << 18, 0, 16384, 2, 8)
    assert "chain_" not in describe(17, 1 << 20, 0, 16384, 1, 2)
    # a misaligned input: scalar loads, and two kernels instead of the fused one
    odd = describe(1024, 32768, 1, 2048, 4, 4, x=4098)
    assert odd.startswith("stream_kernel<f16, J=4, V=1") and "select_kernel<f16" in odd
    # contiguous buckets of 16-256 bytes with a second stage: one kernel too; longer buckets, a bucket
    # count that does not fill whole column tiles, or a row with a remainder: two kernels
    def contiguous(rows, n, code, k, j, k_mult):
        buf = ctypes.create_string_buffer(1024)
        assert L.atk_describe(4096, rows, n, n, k * k_mult, j, k, 1, code, 4096, 4096, buf, 1024) == 0
        return buf.value.decode()
    short = contiguous(1024, 32768, 1, 2048, 4, 4)
    assert short.startswith("fused_regs_kernel<f16, J=4, V=4, pos16, PACKED=1> grid=1024 block=512")
    assert short.endswith("short contiguous buckets") and "select" not in short
    assert contiguous(1024, 32768, 0, 2048, 4, 4).endswith("short contiguous buckets")   # fp32: 64 bytes
    assert contiguous(1024, 65536, 0, 2048, 4, 4).endswith("short contiguous buckets")   # 128 bytes
    assert contiguous(256, 1 << 18, 0, 2048, 4, 4).startswith("contig_kernel<f32")        # 512 bytes
    # no second stage: a lane per bucket up to 64 bytes, spans of buckets through LDS beyond
    assert contiguous(1024, 32768, 1, 2048, 4, 1).startswith("contig_kernel<f16")         # 128 bytes
    assert contiguous(1024, 32768, 1, 4096, 4, 1).startswith("whole_bucket_kernel<f16, J=4> grid=4096 block=256")
    assert contiguous(16384, 1024, 1, 64, 2, 1).startswith("whole_bucket_kernel<f16, J=2> grid=2048 ")
    assert contiguous(16, 1028, 0, 256, 1, 1).startswith("contig_kernel<f32")             # 1028 = 4 * 256 + 4
    two = contiguous(16, 3072, 1, 64, 2, 4)                                               # 128 buckets: two kernels
    assert two.startswith("whole_bucket_kernel<f16, J=2> grid=8 ") and "select_kernel<f16" in two
    assert contiguous(16, 8200, 1, 512, 2, 2).startswith("contig_kernel<f16")             # 8200 = 16 * 512 + 8
    assert contiguous(1024, 32768, 4, 2048, 4, 4).startswith("contig_kernel<u8")          # 1-byte elements
    # truncation and argument checks
    buf = ctypes.create_string_buffer(8)
    assert L.atk_describe(4096, 128, 1 << 20, 1 << 20, 65536, 2, 65536, 0, 0, 4096, 4096, buf, 8) == 0
    assert buf.value == b"stream_"
    assert L.atk_describe(4096, 1, 8, 8, 6, 4, 6, 0, 0, 4096, 4096, buf, 8) == -2


def test_validation_errors_before_device_check():
    from approx_topk import topk
    x = torch.randn(8, 64)
    with pytest.raises(NotImplementedError):
        topk(x, 4, 0, j=2)
    with pytest.raises(ValueError):
        topk(x, 4, -1, k_mult=0)
    with pytest.raises(RuntimeError, match="j must divide k"):
        topk(x, 6, -1, j=4)
    with pytest.raises(RuntimeError, match="0 < j < 5"):
        topk(x, 5, -1, j=5)
    with pytest.raises(RuntimeError, match="k must not be larger"):
        topk(x, 128, -1)
    with pytest.raises(RuntimeError, match="GPU"):
        topk(x, 4, -1)          # valid arguments, but no CPU path exists
    v, i = topk(x, 0, -1, j=0)  # k == 0 is valid and does no work
    assert v.shape == (8, 0) and i.dtype == torch.int64


def test_fake_impl_shapes():
    from torch._subclasses.fake_tensor import FakeTensorMode
    from approx_topk import topk
    with FakeTensorMode():
        x = torch.empty(5, 32, 512)
        v, i = topk(x, 64, -1, j=2, k_mult=2)
        assert v.shape == (5, 32, 64) and i.shape == (5, 32, 64)
        assert v.dtype == torch.float32 and i.dtype == torch.int64


def test_topk_torch_known_answers_and_oracle():
    from approx_topk.experimental.bucketed_argmax import topk_torch
    x = torch.stack([100 * torch.arange(0, 20), -100 * torch.arange(0, 20)]).float()
    v, i = topk_torch(x, k=3, dim=1, interleaved=False)
    assert v.tolist() == [[600.0, 1300, 1900], [0, -700, -1400]] and i.tolist() == [[6, 13, 19], [0, 7, 14]]
    vt, it = topk_torch(x.T, k=3, dim=0, interleaved=False)
    assert torch.equal(vt.T, v) and torch.equal(it.T, i)
    v, i = topk_torch(x, k=3, dim=1, interleaved=True)
    assert v.tolist() == [[1800.0, 1900, 1700], [0, -100, -200]] and i.tolist() == [[18, 19, 17], [0, 1, 2]]
    g = torch.Generator().manual_seed(1001)
    c1 = torch.randn(4, 65536, generator=g)
    for interleaved in (True, False):
        v, i = topk_torch(c1, 1024, -1, interleaved)
        ev, ei = oracle.bucketed_argmax(c1, 1024, -1, interleaved)
        assert torch.equal(v, ev) and torch.equal(i, ei)


def test_batch_contiguous():
    from approx_topk.experimental.bucketed_argmax import _batch_contiguous
    x = torch.arange(3 * 4 * 5).view(3, 4, 5)
    for t, same in [(x, True), (x[:, :, :-1], True), (x[:, :, ::2], False), (x[:, :-1, :], False),
                    (x.swapdims(0, 1), False)]:
        t2 = _batch_contiguous(t)
        assert (t2 is t) == same
        assert torch.equal(t, t2)
        if not same:
            assert t2.is_contiguous()


def test_rows_view():
    from approx_topk import _native
    x = torch.arange(3 * 4 * 10.0).view(3, 4, 10)
    t, rows, n, step = _native.rows_view(x)
    assert t is x and (rows, n, step) == (12, 10, 10)
    t, rows, n, step = _native.rows_view(x[:, :, :7])
    assert t.data_ptr() == x.data_ptr() and (rows, n, step) == (12, 7, 10)
    t, rows, n, step = _native.rows_view(x[:, :3, :])
    assert t.is_contiguous() and (rows, n, step) == (9, 10, 10)
    t, rows, n, step = _native.rows_view(x.movedim(1, -1))
    assert t.is_contiguous() and (rows, n, step) == (30, 4, 4)



def test_operator_object_offers_register_fake_and_register_autograd():
    # the reference's `topk` is a CustomOpDef with these two methods (priority_queue.py:14,91); in a child
    # process, because both registrations change the operator for everything that runs after them
    import subprocess
    import sys
    import textwrap

    code = textwrap.dedent("""
        import sys
        sys.path.insert(0, %r)
        import torch
        from torch._subclasses.fake_tensor import FakeTensorMode
        from approx_topk import topk

        @topk.register_fake
        def _(xs, k, dim, j=None, k_mult=1, interleaved=True, multithread_buckets=False):
            shape = list(xs.shape)
            shape[dim] = k
            return xs.new_empty(shape), xs.new_empty(shape, dtype=torch.int64)

        with FakeTensorMode():
            v, i = topk(torch.empty(3, 64), 8, -1, 2, 1)
        assert tuple(v.shape) == (3, 8) and i.dtype == torch.int64

        def setup(ctx, inputs, output):
            ctx.save_for_backward(output[1])
            ctx.shape = inputs[0].shape

        def backward(ctx, grad_values, grad_indices):
            (indices,) = ctx.saved_tensors
            return torch.zeros(ctx.shape).scatter(-1, indices, grad_values), None, None, None, None, None, None

        topk.register_autograd(backward, setup_context=setup)
        print("registered")
    """) % os.path.join(ROOT, "pytorch-approx-topk_amd")
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and "registered" in out.stdout, out.stderr[-2000:]
