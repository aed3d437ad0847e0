"""Shared helpers for the test-suite: seeded inputs and the tolerance of the bar."""

import math

import torch

# fp32 bar against the oracle: rtol 1e-4, atol 1e-5.
RTOL = 1e-4
ATOL = 1e-5


def make_params(shape, seed=0, dtype=torch.float32, all_randn=False):
    """Per-cell parameters.  ``all_randn`` mirrors the reference's own tests, which draw
    weights, biases and scales from N(0, 1) (gridnet/backend_cuda_test.py:26-29)."""
    g = torch.Generator().manual_seed(seed)
    if all_randn:
        w = torch.randn(27, *shape, generator=g, dtype=dtype)
        b = torch.randn(*shape, generator=g, dtype=dtype)
        r = torch.randn(*shape, generator=g, dtype=dtype)
    else:
        w = torch.randn(27, *shape, generator=g, dtype=dtype) / math.sqrt(27)
        b = 0.1 * torch.randn(*shape, generator=g, dtype=dtype)
        r = 0.5 + torch.rand(*shape, generator=g, dtype=dtype)
    return w, b, r


def make_acts(batch, shape, seed=1, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(batch, *shape, generator=g, dtype=dtype)


def assert_close(actual, expected, rtol=RTOL, atol=ATOL, what=""):
    actual = actual.detach().cpu().double()
    expected = expected.detach().cpu().double()
    err = (actual - expected).abs()
    bound = atol + rtol * expected.abs()
    bad = err > bound
    if bad.any():
        idx = torch.nonzero(bad)[0].tolist()
        worst = (err - bound).max().item()
        raise AssertionError(
            f"{what}: {int(bad.sum())} of {bad.numel()} entries outside rtol={rtol} atol={atol}; "
            f"first at {idx}: got {actual[tuple(idx)].item()} want {expected[tuple(idx)].item()}; "
            f"max excess {worst:.3e}, max abs err {err.max().item():.3e}"
        )
