"""Calls from several host threads at once, each on a stream of its own and through a kernel
family of its own, against the oracle: the library keeps no state that calls share (the launch
numbers it hands out come from one atomic counter), and launches go to the caller's current
stream (as the reference's do, approx_topk/priority_queue_approx_topk.cu:342, 361)."""
import threading

import pytest
import torch

import oracle
from helpers import assert_same

pytestmark = pytest.mark.gpu

# (dtype, shape, k, j, k_mult, interleaved): streaming kernel; both stages in one kernel; slabs and
# their merge, then the select over several workgroups per row; contiguous buckets through LDS
FAMILIES = [
    (torch.float32, (64, 1 << 15), 4096, 2, 1, True),
    (torch.float16, (256, 8192), 512, 4, 4, True),
    (torch.float32, (1, 1 << 22), 8192, 4, 2, True),
    (torch.int32, (64, 8192), 256, 2, 1, False),
]


def test_four_threads_four_streams_four_kernel_families():
    from approx_topk import topk

    g = torch.Generator().manual_seed(3)
    inputs, expected = [], []
    for dtype, shape, k, j, km, interleaved in FAMILIES:
        if dtype.is_floating_point:
            x = (torch.randint(-400, 401, shape, generator=g).float() / 16).to(dtype)     # ties
        else:
            x = torch.randint(-30000, 30000, shape, generator=g, dtype=torch.int32).to(dtype)
        inputs.append(x)
        expected.append(oracle.topk(x, k, -1, j=j, k_mult=km, interleaved=interleaved))
    torch.cuda.synchronize()
    failures: list = []
    start = threading.Barrier(len(FAMILIES))

    def work(t: int):
        try:
            dtype, shape, k, j, km, interleaved = FAMILIES[t]
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                x = inputs[t].cuda(non_blocking=False)
                start.wait(timeout=60)
                for rep in range(25):
                    v, i = topk(x, k, -1, j=j, k_mult=km, interleaved=interleaved)
                    if rep % 6 == 0:
                        stream.synchronize()
                        assert_same(v, i, expected[t][0], expected[t][1], f"thread {t} rep {rep}")
                stream.synchronize()
                assert_same(v, i, expected[t][0], expected[t][1], f"thread {t} last")
        except BaseException as e:  # noqa: BLE001  (reported by the main thread)
            failures.append((t, repr(e)))

    threads = [threading.Thread(target=work, args=(t,)) for t in range(len(FAMILIES))]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=110)
    assert not any(th.is_alive() for th in threads), "a thread did not finish"
    assert not failures, failures
