"""Pins the gated oracle: closed-form recurrences, brute force, finite differences."""

import numpy as np
import pytest
import torch

from oracle.gated import gated_step_brute, gated_step_fast, gated_step_ref

STEPS = [gated_step_ref, gated_step_fast]
ids = ["ref_style", "fast"]


def params(shape, seed=0, dtype=torch.float32, scale=0.3):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(27, 2, *shape, generator=g, dtype=dtype) * scale
    b = torch.randn(2, *shape, generator=g, dtype=dtype)
    x = torch.randn(2, *shape, generator=g, dtype=dtype)
    return w, b, x


@pytest.mark.parametrize("step", STEPS, ids=ids)
def test_zero_weights_scalar_recurrence(step):
    """w = 0: every cell follows x <- s x + (1 - s) tanh(b0) with s = sigmoid(b1)."""
    shape = (8, 8, 4)
    w, b, x = params(shape)
    y = step(torch.zeros_like(w), b, x, 3, 4, "tanh")
    s = torch.sigmoid(b[1])
    want = x
    for _ in range(3):
        want = s * want + (1 - s) * torch.tanh(b[0])
    assert torch.allclose(y, want, atol=1e-6)


@pytest.mark.parametrize("step", STEPS, ids=ids)
def test_centre_tap_recurrence_and_channel_order(step):
    """Only tap 13; channel 0 feeds the activation, channel 1 the gate (swapping them changes
    the answer because relu and sigmoid differ)."""
    shape = (4, 8, 8)
    w, b, x = params(shape, seed=3)
    wc = torch.zeros_like(w)
    wc[13] = w[13]
    y = step(wc, b, x, 2, 4, "relu")
    want = x
    for _ in range(2):
        gate = torch.sigmoid(wc[13, 1] * want + b[1])
        want = gate * want + (1 - gate) * torch.relu(wc[13, 0] * want + b[0])
    assert torch.allclose(y, want, atol=1e-6)


@pytest.mark.parametrize("step", STEPS, ids=ids)
def test_zero_iterations_identity(step):
    w, b, x = params((8, 8, 8))
    assert torch.equal(step(w, b, x, 0, 8), x)


def test_brute_force_agrees():
    shape = (8, 4, 4)
    w, b, x = params(shape, seed=5, dtype=torch.float64)
    want = gated_step_brute(w.numpy(), b.numpy(), x[:1].numpy(), 2, 4, "tanh")
    for step in STEPS:
        assert np.allclose(step(w, b, x[:1], 2, 4, "tanh").numpy(), want, atol=1e-12)


def test_ref_style_and_fast_agree_with_gradients():
    shape = (8, 8, 16)
    w, b, x = params(shape, seed=7, dtype=torch.float64)
    gy = torch.randn(2, *shape, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    outs = []
    for step in STEPS:
        leaves = [t.clone().requires_grad_(True) for t in (w, b, x)]
        y = step(*leaves, 2, 4, "silu")
        outs.append((y, *torch.autograd.grad(y, leaves, gy)))
    for a, e in zip(*outs):
        assert torch.allclose(a, e, rtol=1e-10, atol=1e-10)


def test_finite_differences():
    shape = (4, 4, 4)
    w, b, x = params(shape, seed=9, dtype=torch.float64)
    leaves = [t.requires_grad_(True) for t in (w, b, x[:1])]
    assert torch.autograd.gradcheck(lambda *p: gated_step_fast(*p, 2, 2, "tanh"), leaves,
                                    eps=1e-6, atol=1e-6, rtol=1e-5)
