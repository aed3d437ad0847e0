"""Pins the CPU oracle's forward pass with closed forms and library routines.

The reference holds no golden vectors for this path; these cases are chosen so that a
wrong tap order, a transposed axis, a dropped halo, a refreshed (non-stale) halo, a
normalisation over the wrong set, or a residual on the normalised value each fail.
"""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle.brute import gridnet_step_brute
from oracle.fast import gridnet_step_fast
from oracle.ref_style import gridnet_step_ref, neighbour_gather_index

from helpers import make_acts, make_params

STEPS = [gridnet_step_ref, gridnet_step_fast]
ids = ["ref_style", "fast"]


def shift_zero_fill(x, di, dj, dk):
    """y[i, j, k] = x[i + di, j + dj, k + dk], zero outside the grid."""
    out = torch.zeros_like(x)
    _, m, n, k = x.shape
    src = x[:, max(di, 0): m + min(di, 0), max(dj, 0): n + min(dj, 0), max(dk, 0): k + min(dk, 0)]
    out[:, max(-di, 0): m + min(-di, 0), max(-dj, 0): n + min(-dj, 0),
        max(-dk, 0): k + min(-dk, 0)] = src
    return out


def test_gather_index_matches_definition():
    # gridnet/backend_torch.py:283-298, cell (1, 2, 3) tap (a, b, c) = (2, 0, 1), bs = 4
    bs, side = 4, 6
    idx = neighbour_gather_index(bs).reshape(bs, bs, bs, 3, 3, 3)
    assert idx[1, 2, 3, 2, 0, 1].item() == (3 + 1) + side * ((2 + 0) + side * (1 + 2))
    assert idx[0, 0, 0, 1, 1, 1].item() == 1 + side * (1 + side * 1)  # tap 13 is the cell itself


@pytest.mark.parametrize("step", STEPS, ids=ids)
@pytest.mark.parametrize("tap", range(27))
def test_single_tap_is_a_shift(step, tap):
    """One tap set to 1, one iteration, relu on positive data: y = x + shift_t(x).

    Non-cubic grid so that swapping any two axes changes the answer.
    """
    shape = (8, 12, 4)
    a, b, c = tap // 9, (tap // 3) % 3, tap % 3
    x = make_acts(2, shape).abs() + 0.1
    w = torch.zeros(27, *shape)
    w[tap] = 1.0
    y = step(w, torch.zeros(shape), torch.ones(shape), x, 1, 4, 1e-5, False, "relu")
    want = x + shift_zero_fill(x, a - 1, b - 1, c - 1)
    assert torch.allclose(y, want, atol=1e-6)


@pytest.mark.parametrize("step", STEPS, ids=ids)
@pytest.mark.parametrize("activation", ["silu", "relu", "leaky_relu", "tanh"])
def test_centre_tap_scalar_recurrence(step, activation):
    """Only tap 13: each cell follows x <- x + r*act(w*x + b), whatever the blocking."""
    shape = (8, 8, 16)
    w13, b, r = make_params(shape, seed=3)
    w = torch.zeros(27, *shape)
    w[13] = w13[13] * 3
    x = make_acts(2, shape)
    y = step(w, b, r, x, 3, 4, 1e-5, False, activation)
    want = x.double()
    for _ in range(3):
        u = w[13].double() * want + b.double()
        if activation == "silu":
            f = u / (1 + torch.exp(-u))
        elif activation == "relu":
            f = u.clamp_min(0)
        elif activation == "leaky_relu":
            f = torch.where(u > 0, u, 0.01 * u)
        else:
            f = torch.tanh(u)
        want = want + r.double() * f
    assert torch.allclose(y.double(), want, atol=2e-5)


@pytest.mark.parametrize("step", STEPS, ids=ids)
@pytest.mark.parametrize("shape,bs", [((16, 16, 16), 8), ((32, 64, 128), 8)])
def test_zero_iterations_is_identity(step, shape, bs):
    # restates gridnet/backend_torch_test.py:10-25
    if step is gridnet_step_ref and shape[2] == 128:
        shape = (16, 32, 64)  # keep the Python block loop short
    x = make_acts(2, shape)
    w, b, _ = make_params(shape, all_randn=True)
    y = step(w, b, torch.ones(shape), x, 0, bs)
    assert torch.equal(y, x)


@pytest.mark.parametrize("step", STEPS, ids=ids)
@pytest.mark.parametrize("normalize", [True, False])
def test_zero_weights_closed_form(step, normalize):
    """w = 0: y = x + T * r * act(b); generalises gridnet/backend_torch_test.py:28-60."""
    shape = (16, 16, 16)
    x = make_acts(2, shape)
    _, b, _ = make_params(shape)
    r = torch.full(shape, 0.31)
    y = step(torch.zeros(27, *shape), b, r, x, 10, 8, 1e-5, normalize, "silu")
    assert torch.allclose(y, x + 10 * 0.31 * F.silu(b), atol=1e-5)


@pytest.mark.parametrize("step", STEPS, ids=ids)
def test_one_iteration_uniform_weights_is_conv3d(step):
    """T = 1 with the same 27 weights at every cell is a zero-padded cross-correlation."""
    shape = (8, 16, 12)
    g = torch.Generator().manual_seed(5)
    kern = torch.randn(27, generator=g)
    w = kern.reshape(27, 1, 1, 1).expand(27, *shape).contiguous()
    _, b, r = make_params(shape)
    x = make_acts(3, shape)
    conv = F.conv3d(x[:, None], kern.reshape(1, 1, 3, 3, 3), padding=1)[:, 0]
    want = x + r * torch.tanh(conv + b)
    for bs in (4,):
        y = step(w, b, r, x, 1, bs, 1e-5, False, "tanh")
        assert torch.allclose(y, want, atol=1e-5)


@pytest.mark.parametrize("step", STEPS, ids=ids)
def test_one_iteration_is_block_size_invariant(step):
    shape = (8, 8, 8)
    w, b, r = make_params(shape, all_randn=True)
    x = make_acts(2, shape)
    y4 = step(w, b, r, x, 1, 4, 1e-5, False, "silu")
    y8 = step(w, b, r, x, 1, 8, 1e-5, False, "silu")
    y2 = step(w, b, r, x, 1, 2, 1e-5, False, "silu")
    assert torch.allclose(y4, y8, atol=1e-5) and torch.allclose(y2, y8, atol=1e-5)


@pytest.mark.parametrize("step", STEPS, ids=ids)
def test_halo_is_stale_across_blocks_and_fresh_within(step):
    """Tap 12 (neighbour k-1), two iterations, 1-D chain along K, relu on positive data.

    Inside a block the second iteration sees the first one's update of its left
    neighbour: y[k] = x[k] + 2 x[k-1] + x[k-2].  The first cell of a block reads the
    frozen copy of the previous block's last cell: y[k] = x[k] + 2 x[k-1].
    """
    shape = (4, 4, 8)
    x = make_acts(1, shape).abs() + 0.1
    w = torch.zeros(27, *shape)
    w[12] = 1.0
    y = step(w, torch.zeros(shape), torch.ones(shape), x, 2, 4, 1e-5, False, "relu")
    xm1 = shift_zero_fill(x, 0, 0, -1)
    xm2 = shift_zero_fill(x, 0, 0, -2)
    want = x + 2 * xm1 + xm2
    first = torch.zeros(shape, dtype=torch.bool)
    first[:, :, 0::4] = True
    want = torch.where(first, x + 2 * xm1, want)
    assert torch.allclose(y, want, atol=1e-5)


@pytest.mark.parametrize("step", STEPS, ids=ids)
def test_single_block_equals_repeated_global_update(step):
    """bs = grid side: T inner iterations are T applications of the global op."""
    shape = (4, 4, 4)
    w, b, r = make_params(shape, all_randn=True)
    x = make_acts(2, shape)
    y = step(w, b, r, x, 3, 4, 1e-5, False, "tanh")
    h = x
    for _ in range(3):
        h = step(w, b, r, h, 1, 4, 1e-5, False, "tanh")
    assert torch.allclose(y, h, atol=1e-5)


@pytest.mark.parametrize("step", STEPS, ids=ids)
def test_normalize_hand_computed_window(step):
    """normalize=True on one 2^3 block: stats run over the 4^3 window including the 56
    zero halo entries, population std, eps added to the std, residual on the raw value."""
    shape = (2, 2, 2)
    x = torch.arange(1.0, 9.0).reshape(1, 2, 2, 2)
    w = torch.zeros(27, *shape)
    w[13] = 2.0
    b = torch.full(shape, 0.5)
    r = torch.full(shape, 0.25)
    eps = 0.1
    vals = np.zeros(64)
    vals[:8] = np.arange(1.0, 9.0)
    mu = vals.sum() / 64
    sd = math.sqrt(((vals - mu) ** 2).sum() / 64)
    z = (np.arange(1.0, 9.0) - mu) / (sd + eps)
    want = np.arange(1.0, 9.0) + 0.25 * np.tanh(2.0 * z + 0.5)
    y = step(w, b, r, x, 1, 2, eps, True, "tanh")
    assert np.allclose(y.reshape(-1).double().numpy(), want, atol=1e-6)


@pytest.mark.parametrize("normalize", [True, False])
@pytest.mark.parametrize("activation", ["silu", "leaky_relu"])
def test_brute_force_agrees(normalize, activation):
    shape = (8, 4, 8)
    w, b, r = make_params(shape, all_randn=True, dtype=torch.float64)
    x = make_acts(1, shape, dtype=torch.float64)
    want = gridnet_step_brute(w.numpy(), b.numpy(), r.numpy(), x.numpy(), 2, 4, 1e-5,
                              normalize, activation)
    for step in STEPS:
        y = step(w, b, r, x, 2, 4, 1e-5, normalize, activation)
        assert np.allclose(y.numpy(), want, atol=1e-10)


@pytest.mark.parametrize("shape,bs,normalize", [
    ((16, 16, 16), 8, True), ((16, 32, 8), 8, False), ((16, 8, 8), 4, True), ((32, 16, 8), 4, False)])
def test_ref_style_and_fast_agree(shape, bs, normalize):
    # the reference's own shape matrix (gridnet/backend_cuda_test.py:11-17), trimmed for CPU time
    w, b, r = make_params(shape, all_randn=True)
    x = make_acts(2, shape)
    y1 = gridnet_step_ref(w, b, r, x, 2, bs, 1e-5, normalize, "silu")
    y2 = gridnet_step_fast(w, b, r, x, 2, bs, 1e-5, normalize, "silu")
    assert torch.allclose(y1, y2, rtol=1e-4, atol=2e-5)


def test_unknown_activation_raises():
    shape = (4, 4, 4)
    w, b, r = make_params(shape)
    with pytest.raises(ValueError, match="unknown activation"):
        gridnet_step_ref(w, b, r, make_acts(1, shape), 1, 4, activation="gelu")


def test_indivisible_block_size_asserts():
    shape = (6, 4, 4)
    w, b, r = make_params(shape)
    with pytest.raises(AssertionError):
        gridnet_step_fast(w, b, r, make_acts(1, shape), 1, 4)
