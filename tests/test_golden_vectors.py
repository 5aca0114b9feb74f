"""The known answers of the reference's own tests (tests/golden/known_answers.json):
checked against the CPU oracle without a GPU, and against the HIP path on one."""
import json
import os

import pytest
import torch

import oracle

with open(os.path.join(os.path.dirname(__file__), "golden", "known_answers.json")) as f:
    VECTORS = json.load(f)["vectors"]
IDS = [v["name"] for v in VECTORS]


def _input(vec):
    dtype = getattr(torch, vec["dtype"])
    if "x" in vec:
        return torch.tensor(vec["x"], dtype=dtype)
    x = torch.zeros((len(vec["hot"]), vec["n"]), dtype=dtype)
    for r, cells in enumerate(vec["hot"]):
        for pos, val in cells:
            x[r, pos] = val
    return x


def _check(vec, values, indices):
    dtype = getattr(torch, vec["dtype"])
    ev, ei = torch.tensor(vec["values"], dtype=dtype), torch.tensor(vec["indices"])
    values, indices = values.cpu(), indices.cpu()
    if vec["compare"] == "sorted":
        values, indices = values.sort(-1).values, indices.sort(-1).values
        ev, ei = ev.sort(-1).values, ei.sort(-1).values
    assert torch.equal(values, ev), vec["name"]
    assert torch.equal(indices, ei), vec["name"]


@pytest.mark.parametrize("vec", VECTORS, ids=IDS)
def test_oracle_matches_golden(vec):
    x = _input(vec)
    if vec["op"] == "topk":
        v, i = oracle.topk(x, vec["k"], -1, j=vec["j"], k_mult=vec["k_mult"], interleaved=vec["interleaved"])
    else:
        v, i = oracle.bucketed_argmax(x, vec["k"], 1, vec["interleaved"])
    _check(vec, v, i)


@pytest.mark.gpu
@pytest.mark.parametrize("vec", VECTORS, ids=IDS)
def test_hip_matches_golden(vec):
    from approx_topk import topk
    from approx_topk.experimental.bucketed_argmax import topk_triton
    x = _input(vec).cuda()
    if vec["op"] == "topk":
        v, i = topk(x, vec["k"], -1, j=vec["j"], k_mult=vec["k_mult"], interleaved=vec["interleaved"])
    else:
        v, i = topk_triton(x, k=vec["k"], dim=1, interleaved=vec["interleaved"])
    _check(vec, v, i)
