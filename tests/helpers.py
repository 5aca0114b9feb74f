"""Shared helpers for the parity tests."""
import torch

import oracle


def cpu_randn(shape, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g).to(dtype)


def assert_same(got_v, got_i, exp_v, exp_i, what=""):
    """Bit-exact values (compared as raw integers so NaN and -0.0 count) and
    identical indices, element for element."""
    got_v, got_i = got_v.cpu(), got_i.cpu()
    assert got_v.shape == exp_v.shape and got_i.shape == exp_i.shape, (what, got_v.shape, exp_v.shape)
    assert got_v.dtype == exp_v.dtype and got_i.dtype == torch.int64, what
    bits = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[got_v.element_size()]
    same_v = torch.equal(got_v.contiguous().view(bits), exp_v.contiguous().view(bits))
    same_i = torch.equal(got_i, exp_i)
    if not (same_v and same_i):
        bad = (got_i != exp_i).nonzero()
        raise AssertionError(f"{what}: values equal={same_v} indices equal={same_i}; "
                             f"first differing index entries {bad[:5].tolist()} "
                             f"got {got_i[tuple(bad[0])] if len(bad) else None} "
                             f"expected {exp_i[tuple(bad[0])] if len(bad) else None}")


def oracle_topk(x_cpu, k, dim=-1, j=1, k_mult=1, interleaved=True):
    return oracle.topk(x_cpu, k, dim, j=j, k_mult=k_mult, interleaved=interleaved)


def subnormals(dtype):
    """The smallest and largest subnormal of a float dtype and one in between, both signs,
    next to +0.0 and -0.0: values a flush-to-zero compare would all call equal."""
    tiny = torch.finfo(dtype).smallest_normal
    eps = torch.finfo(dtype).eps
    least = tiny * eps                      # smallest subnormal
    vals = [least, 3 * least, tiny - least, 0.0]
    t = torch.tensor(vals + [-v for v in vals], dtype=torch.float64).to(dtype)
    assert bool(((t != 0) == torch.tensor([True] * 3 + [False] + [True] * 3 + [False])).all())
    return t
