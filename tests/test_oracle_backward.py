"""Pins the oracle's gradients: autograd of the forward (already pinned) is the judge,
the hand-derived formulas in ``oracle.manual`` (the ones the HIP kernels implement)
must agree with it, and closed forms / finite differences pin autograd's inputs."""

import pytest
import torch
import torch.nn.functional as F

from oracle.fast import gridnet_step_fast
from oracle.manual import gridnet_step_backward_manual, layer_norm_backward_manual
from oracle.network import layer_norm_oracle, layer_norm_plain, network_forward
from oracle.ref_style import gridnet_step_ref

from helpers import make_acts, make_params


def autograd_grads(step, w, b, r, x, gy, *args):
    leaves = [t.detach().clone().requires_grad_(True) for t in (w, b, r, x)]
    y = step(*leaves, *args)
    return torch.autograd.grad(y, leaves, gy)


@pytest.mark.parametrize("activation", ["silu", "relu", "leaky_relu", "tanh"])
@pytest.mark.parametrize("normalize", [False, True])
@pytest.mark.parametrize("shape,bs,inner", [((8, 8, 8), 4, 2), ((8, 16, 8), 8, 3), ((4, 4, 4), 4, 1)])
def test_manual_backward_matches_autograd(activation, normalize, shape, bs, inner):
    w, b, r = make_params(shape, all_randn=True, dtype=torch.float64)
    w = w * 0.3
    x = make_acts(2, shape, dtype=torch.float64)
    gy = make_acts(2, shape, seed=7, dtype=torch.float64)
    want = autograd_grads(gridnet_step_fast, w, b, r, x, gy, inner, bs, 1e-5, normalize, activation)
    got = gridnet_step_backward_manual(w, b, r, x, gy, inner, bs, 1e-5, normalize, activation)
    for name, g, e in zip(("dweight", "dbias", "dscale", "dx"), got, want):
        assert torch.allclose(g, e, rtol=1e-9, atol=1e-9), name


def test_ref_style_autograd_matches_fast_autograd():
    shape, bs = (8, 8, 16), 4
    w, b, r = make_params(shape, all_randn=True, dtype=torch.float64)
    x = make_acts(2, shape, dtype=torch.float64)
    gy = make_acts(2, shape, seed=7, dtype=torch.float64)
    for normalize in (False, True):
        g1 = autograd_grads(gridnet_step_ref, w, b, r, x, gy, 2, bs, 1e-5, normalize, "silu")
        g2 = autograd_grads(gridnet_step_fast, w, b, r, x, gy, 2, bs, 1e-5, normalize, "silu")
        for a, e in zip(g1, g2):
            assert torch.allclose(a, e, rtol=1e-9, atol=1e-9)


@pytest.mark.parametrize("normalize", [False, True])
def test_finite_differences(normalize):
    shape, bs = (4, 4, 4), 2
    w, b, r = make_params(shape, all_randn=True, dtype=torch.float64)
    x = make_acts(1, shape, dtype=torch.float64)
    leaves = [t.requires_grad_(True) for t in (w * 0.3, b, r, x)]
    assert torch.autograd.gradcheck(
        lambda *p: gridnet_step_fast(*p, 2, bs, 1e-3, normalize, "tanh"), leaves,
        eps=1e-6, atol=1e-6, rtol=1e-5)


def test_centre_tap_closed_form_gradients():
    """Only tap 13, T = 1, tanh: y = x + r tanh(w x + b), so with upstream g:
    dr = g tanh(u), db = g r (1 - tanh^2 u), dw13 = db * x, dx = g + db * w (per sample)."""
    shape, bs = (4, 8, 4), 4
    w13, b, r = make_params(shape, all_randn=True, dtype=torch.float64)
    w = torch.zeros(27, *shape, dtype=torch.float64)
    w[13] = w13[13]
    x = make_acts(3, shape, dtype=torch.float64)
    gy = make_acts(3, shape, seed=9, dtype=torch.float64)
    dw, db, dr, dx = gridnet_step_backward_manual(w, b, r, x, gy, 1, bs, 1e-5, False, "tanh")
    u = w[13] * x + b
    t = torch.tanh(u)
    d = gy * r * (1 - t * t)
    assert torch.allclose(dr, (gy * t).sum(0))
    assert torch.allclose(db, d.sum(0))
    assert torch.allclose(dw[13], (d * x).sum(0))
    assert torch.allclose(dx, gy + d * w[13])
    off = torch.ones(27, dtype=torch.bool)
    off[13] = False
    # the other 26 taps see the neighbours' values: dw[t] = sum_b delta * shift_t(x)
    assert torch.allclose(dw[14][:, :, :-1], (d[..., :-1] * x[..., 1:]).sum(0))
    assert torch.allclose(dw[4][1:], (d[:, 1:] * x[:, :-1]).sum(0))


def test_parameter_gradients_sum_over_the_batch():
    shape, bs = (8, 8, 8), 4
    w, b, r = make_params(shape, dtype=torch.float64)
    x = make_acts(2, shape, dtype=torch.float64)
    gy = make_acts(2, shape, seed=7, dtype=torch.float64)
    both = gridnet_step_backward_manual(w, b, r, x, gy, 2, bs, 1e-5, False, "leaky_relu")
    one = gridnet_step_backward_manual(w, b, r, x[:1], gy[:1], 2, bs, 1e-5, False, "leaky_relu")
    two = gridnet_step_backward_manual(w, b, r, x[1:], gy[1:], 2, bs, 1e-5, False, "leaky_relu")
    for k in range(3):
        assert torch.allclose(both[k], one[k] + two[k])
    assert torch.allclose(both[3], torch.cat([one[3], two[3]]))


def test_layer_norm_conventions_match_library():
    shape = (8, 4, 16)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(3, *shape, generator=g, dtype=torch.float64) * 3 + 1
    gamma = torch.randn(shape, generator=g, dtype=torch.float64)
    beta = torch.randn(shape, generator=g, dtype=torch.float64)
    assert torch.allclose(layer_norm_oracle(x, gamma, beta), layer_norm_plain(x, gamma, beta))
    # eps sits inside the square root: a constant sample normalises to beta exactly
    const = torch.full((1, *shape), 2.5, dtype=torch.float64)
    assert torch.allclose(layer_norm_oracle(const, gamma, beta), beta[None])


def test_layer_norm_backward_manual_matches_autograd():
    shape = (8, 4, 16)
    g = torch.Generator().manual_seed(4)
    x = (torch.randn(3, *shape, generator=g, dtype=torch.float64) * 2 + 0.5).requires_grad_(True)
    gamma = torch.randn(shape, generator=g, dtype=torch.float64).requires_grad_(True)
    beta = torch.randn(shape, generator=g, dtype=torch.float64).requires_grad_(True)
    dy = torch.randn(3, *shape, generator=g, dtype=torch.float64)
    y = F.layer_norm(x, shape, gamma, beta, 1e-5)
    ex, eg, eb = torch.autograd.grad(y, (x, gamma, beta), dy)
    dx, dgamma, dbeta, _, _ = layer_norm_backward_manual(dy, x.detach(), gamma.detach())
    assert torch.allclose(dx, ex) and torch.allclose(dgamma, eg) and torch.allclose(dbeta, eb)


def test_network_is_step_then_norm():
    shape, bs = (8, 8, 8), 4
    w, b, r = make_params(shape)
    x = make_acts(2, shape)
    gamma, beta = torch.ones(shape) * 1.5, torch.full(shape, 0.25)
    y = network_forward(w, b, r, gamma, beta, x, 2, 2, bs, "leaky_relu")
    h = x
    for _ in range(2):
        h = gridnet_step_ref(w, b, r, h, 2, bs, 1e-5, False, "leaky_relu")
        h = F.layer_norm(h, shape, gamma, beta, 1e-5)
    assert torch.allclose(y, h, atol=1e-5)
    # every sample leaves a LayerNorm with mean beta-ish and unit-ish spread
    flat = ((y - beta) / gamma).flatten(1)
    assert flat.mean(1).abs().max() < 1e-5 and (flat.var(1, correction=0) - 1).abs().max() < 1e-3


@pytest.mark.parametrize("activation,normalize", [("silu", False), ("leaky_relu", False), ("tanh", True)])
def test_manual_chain_matches_autograd_chain(activation, normalize):
    """The loop without autograd (what the full-size GPU checks are held to) against autograd of
    the same loop."""
    from oracle.network import network_forward_backward, network_forward_backward_manual

    shape, bs, batch, inner, outer = (8, 16, 8), 4, 3, 2, 3
    w, b, r = make_params(shape, seed=31, dtype=torch.float64)
    g = torch.Generator().manual_seed(32)
    gamma = 1 + 0.2 * torch.randn(shape, generator=g, dtype=torch.float64)
    beta = 0.2 * torch.randn(shape, generator=g, dtype=torch.float64)
    x0 = make_acts(batch, shape, seed=33, dtype=torch.float64)
    gy = make_acts(batch, shape, seed=34, dtype=torch.float64)
    kw = dict(inner_iterations=inner, outer_iterations=outer, block_size=bs, activation=activation,
              normalize=normalize)
    want = network_forward_backward([w, b, r, gamma, beta], x0, gy, **kw)
    got = network_forward_backward_manual([w, b, r, gamma, beta], x0, gy, **kw)
    for name, a, e in zip(("y", "dweight", "dbias", "dscale", "dgamma", "dbeta", "dx0"), got, want):
        assert torch.allclose(a, e, rtol=1e-9, atol=1e-11), name
