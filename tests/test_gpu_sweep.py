"""Seeded random sweep over shapes the hand-picked cases leave out.

The tuned fp32 kernels choose their launch plan from the shape (batch chunks per workgroup,
slots per workgroup, whether a workgroup owns the whole batch of its block or the gradient arrays
get a copy per batch chunk), so a fixed list of cases exercises a fixed set of plans.
Here grid, block size, batch, inner iterations, activation and the accumulate/overwrite flags are
drawn at random (fixed seeds) and every draw is held to the generic kernels run in fp64 on the
same fp32 inputs -- the two share no device code, and each is held to the CPU oracle elsewhere
(test_gpu_step.py); likewise with normalize=True and for the gated variant of the step.  A second sweep holds the chain with the LayerNorm folded into the step
kernels to the op-by-op chain of the same library, in both shapes of the loop."""

import math
import random

import pytest
import torch

from helpers import assert_close, make_acts, make_params

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SMOOTH = ("silu", "tanh")  # gradients under relu/leaky_relu flip at the kink in fp32 vs fp64


def draw_step(seed):
    rng = random.Random(seed)
    bs = rng.choice((4, 8))
    dims = tuple(bs * rng.randint(1, 5 if bs == 4 else 3) for _ in range(3))
    batch = rng.choice((1, 2, 3, 5, 8, 13, 31, 32, 33, 47, 64, 70))
    inner = rng.choice((0, 1, 1, 2, 3, 4, 5, 7))
    return dims, bs, batch, inner, rng.choice(SMOOTH), rng.random() < 0.5


@pytest.mark.parametrize("seed", range(24))
def test_random_step_tuned_fp32_against_generic_fp64(seed):
    import gridnet_cuda

    shape, bs, batch, inner, activation, preset = draw_step(seed)
    print(f"sweep step seed={seed} shape={shape} bs={bs} B={batch} inner={inner} act={activation} "
          f"preset={preset}", flush=True)
    w, b, r = make_params(shape, seed=1000 + seed)
    if inner >= 5:
        w, r = w * 0.5, r * 0.5
    x, gy = make_acts(batch, shape, seed=2000 + seed), make_acts(batch, shape, seed=3000 + seed)
    # gradient buffers arrive holding something (the entry point accumulates), or zero-filled
    start = [make_acts(1, t.shape, seed=4000 + seed + i)[0] if preset else torch.zeros_like(t)
             for i, t in enumerate((w, b, r, x))]

    def call(dtype):
        tw, tb, tr, tx, tgy = (t.to(device=DEV, dtype=dtype) for t in (w, b, r, x, gy))
        y = torch.full_like(tx, float("nan"))
        gridnet_cuda.forward(tw, tb, tr, tx, y, inner, bs, 1e-5, False, activation)
        outs = [t.to(device=DEV, dtype=dtype) for t in start]
        gridnet_cuda.backward(tw, tb, tr, tx, tgy, *outs, inner, bs, 1e-5, False, activation)
        return [y] + outs

    fast, slow = call(torch.float32), call(torch.float64)
    summed = 1e-5 * max(1.0, math.sqrt(batch * max(inner, 1) / 2))
    for name, got, want in zip(("y", "dweight", "dbias", "dscale", "dx"), fast, slow):
        assert torch.isfinite(got).all(), name
        assert_close(got, want, atol=summed if name in ("dweight", "dbias", "dscale") else 1e-5,
                     what=name)


def draw_kinked(seed):
    """Draws under relu / leaky_relu, sized so that inputs exist which keep every pre-activation
    of the fp64 run clear of the kink (cells x batch x iterations below ~2e5)."""
    rng = random.Random(9000 + seed)
    bs = rng.choice((4, 8))
    dims = tuple(bs * rng.randint(1, 3) for _ in range(3))
    inner = rng.choice((1, 1, 2, 3, 4, 5))
    cells = dims[0] * dims[1] * dims[2]
    fits = [b for b in (1, 2, 3, 5, 7, 9, 13, 17, 31, 33) if b * cells * inner <= 200_000]
    return dims, bs, rng.choice(fits[-4:]), inner, rng.choice(("relu", "leaky_relu")), rng.random() < 0.5


@pytest.mark.parametrize("seed", range(16))
def test_random_step_kinked_activations(seed):
    """relu and leaky_relu (the training default) through the same launch plans: batches that
    the slots do not divide, batches split over workgroups, preset gradient buffers.  The
    derivative jumps at 0, so the inputs are chosen with every fp64 pre-activation at least
    2e-6 away from it (ten times what fp32 rounding moves one by)."""
    import gridnet_cuda
    from helpers import acts_clear_of_kink

    shape, bs, batch, inner, activation, preset = draw_kinked(seed)
    print(f"sweep kinked seed={seed} shape={shape} bs={bs} B={batch} inner={inner} act={activation} "
          f"preset={preset}", flush=True)
    w, b, r = make_params(shape, seed=9100 + seed)
    if inner >= 5:
        w, r = w * 0.5, r * 0.5
    x = acts_clear_of_kink(w, b, r, batch, shape, inner, bs, 1e-5, False, activation, seed=9200 + seed)
    gy = make_acts(batch, shape, seed=9300 + seed)
    start = [make_acts(1, t.shape, seed=9400 + seed + i)[0] if preset else torch.zeros_like(t)
             for i, t in enumerate((w, b, r, x))]

    def call(dtype):
        tw, tb, tr, tx, tgy = (t.to(device=DEV, dtype=dtype) for t in (w, b, r, x, gy))
        y = torch.full_like(tx, float("nan"))
        gridnet_cuda.forward(tw, tb, tr, tx, y, inner, bs, 1e-5, False, activation)
        outs = [t.to(device=DEV, dtype=dtype) for t in start]
        gridnet_cuda.backward(tw, tb, tr, tx, tgy, *outs, inner, bs, 1e-5, False, activation)
        return [y] + outs

    fast, slow = call(torch.float32), call(torch.float64)
    summed = 1e-5 * max(1.0, math.sqrt(batch * inner / 2))
    for name, got, want in zip(("y", "dweight", "dbias", "dscale", "dx"), fast, slow):
        assert torch.isfinite(got).all(), name
        assert_close(got, want, atol=summed if name in ("dweight", "dbias", "dscale") else 1e-5,
                     what=name)


def draw_normalized(seed):
    if seed == 0:  # the draw that once showed a missing barrier in the tuned backward
        return (24, 24, 24), 8, 40, 1, "tanh"
    rng = random.Random(7000 + seed)
    bs = rng.choice((4, 8))
    shape = tuple(bs * rng.randint(1, 3) for _ in range(3))
    return shape, bs, rng.choice((1, 2, 5, 17, 40)), rng.choice((0, 1, 2, 3, 5)), rng.choice(SMOOTH)


@pytest.mark.parametrize("seed", range(16))
def test_random_normalized_step_tuned_fp32_against_generic_fp64(seed):
    """normalize=True: the tuned kernels keep running sums for the window statistics and hand
    two numbers per (element, block) to the cross-block kernel; the generic kernels (the only
    implementation in fp64) reduce over the window twice per iteration."""
    import gridnet_cuda

    shape, bs, batch, inner, activation = draw_normalized(seed)
    print(f"sweep normalized seed={seed} shape={shape} bs={bs} B={batch} inner={inner} "
          f"act={activation}", flush=True)
    w, b, r = make_params(shape, seed=7100 + seed)
    x, gy = make_acts(batch, shape, seed=7200 + seed), make_acts(batch, shape, seed=7300 + seed)

    def call(dtype):
        tw, tb, tr, tx, tgy = (t.to(device=DEV, dtype=dtype) for t in (w, b, r, x, gy))
        y = torch.full_like(tx, float("nan"))
        gridnet_cuda.forward(tw, tb, tr, tx, y, inner, bs, 1e-5, True, activation)
        outs = [torch.zeros_like(t) for t in (tw, tb, tr, tx)]
        gridnet_cuda.backward(tw, tb, tr, tx, tgy, *outs, inner, bs, 1e-5, True, activation)
        return [y] + outs

    fast, slow = call(torch.float32), call(torch.float64)
    # the division by (std + eps) and the two window sums of the backward double the rounding
    # of a plain step: twice the bar's tolerances here, the bar itself against the oracle on
    # the reference's own matrix (test_gpu_step.py)
    summed = 2e-5 * max(1.0, math.sqrt(batch * max(inner, 1) / 2))
    for name, got, want in zip(("y", "dweight", "dbias", "dscale", "dx"), fast, slow):
        assert torch.isfinite(got).all(), name
        assert_close(got, want, rtol=2e-4, atol=summed if name != "y" else 2e-5, what=name)


@pytest.mark.parametrize("offset", [30.0, -100.0])
@pytest.mark.parametrize("bs", [8, 4])
def test_normalized_step_on_inputs_far_from_zero(bs, offset):
    """Windows whose mean dwarfs their spread (blocks away from the grid's border, whose windows
    hold no zeros from outside the grid): the tuned kernels take the window statistics from
    running sums, variance = E[x^2] - mean^2 as in the reference's kernel
    (src/gridnet_cuda_kernels.cu:164-170), but of a window that is kept minus one of its own
    values, so the subtraction does not eat the digits (without that shift the forward result
    was 7e-3 off at an offset of 100 with 4^3 blocks)."""
    import gridnet_cuda

    shape, batch, inner = (32, 16, 16), 3, 3
    print(f"normalized far from zero bs={bs} offset={offset}", flush=True)
    w, b, r = make_params(shape, seed=7500)
    x, gy = make_acts(batch, shape, seed=7501) + offset, make_acts(batch, shape, seed=7502)

    def call(dtype):
        tw, tb, tr, tx, tgy = (t.to(device=DEV, dtype=dtype) for t in (w, b, r, x, gy))
        y = torch.full_like(tx, float("nan"))
        gridnet_cuda.forward(tw, tb, tr, tx, y, inner, bs, 1e-5, True, "silu")
        outs = [torch.zeros_like(t) for t in (tw, tb, tr, tx)]
        gridnet_cuda.backward(tw, tb, tr, tx, tgy, *outs, inner, bs, 1e-5, True, "silu")
        return [y] + outs

    fast, slow = call(torch.float32), call(torch.float64)
    for name, got, want in zip(("y", "dweight", "dbias", "dscale", "dx"), fast, slow):
        # y carries the offset itself: its fp32 representation alone is 4e-6 off at 100
        assert_close(got, want, rtol=2e-4, atol=5e-5, what=name)


def draw_gated(seed):
    rng = random.Random(8000 + seed)
    bs = rng.choice((4, 8))
    shape = tuple(bs * rng.randint(1, 3) for _ in range(3))
    return (shape, bs, rng.choice((1, 2, 5, 17, 40, 64)), rng.choice((0, 1, 2, 3, 5)),
            rng.choice(SMOOTH), rng.random() < 0.5)


@pytest.mark.parametrize("seed", range(16))
def test_random_gated_step_tuned_fp32_against_generic_fp64(seed):
    import gridnet_cuda

    shape, bs, batch, inner, activation, preset = draw_gated(seed)
    print(f"sweep gated seed={seed} shape={shape} bs={bs} B={batch} inner={inner} act={activation} "
          f"preset={preset}", flush=True)
    gen = torch.Generator().manual_seed(8100 + seed)
    w = torch.randn(27, 2, *shape, generator=gen) / 27 ** 0.5
    b = 0.1 * torch.randn(2, *shape, generator=gen)
    x, gy = make_acts(batch, shape, seed=8200 + seed), make_acts(batch, shape, seed=8300 + seed)
    start = [make_acts(1, t.shape, seed=8400 + seed + i)[0] if preset else torch.zeros_like(t)
             for i, t in enumerate((w, b, x))]

    def call(dtype):
        tw, tb, tx, tgy = (t.to(device=DEV, dtype=dtype) for t in (w, b, x, gy))
        y = torch.full_like(tx, float("nan"))
        gridnet_cuda.forward_gated(tw, tb, tx, y, inner, bs, activation)
        outs = [t.to(device=DEV, dtype=dtype) for t in start]
        gridnet_cuda.backward_gated(tw, tb, tx, tgy, *outs, inner, bs, activation)
        return [y] + outs

    fast, slow = call(torch.float32), call(torch.float64)
    summed = 1e-5 * max(1.0, math.sqrt(batch * max(inner, 1) / 2))
    for name, got, want in zip(("y", "dweight", "dbias", "dx"), fast, slow):
        assert torch.isfinite(got).all(), name
        assert_close(got, want, atol=summed if name in ("dweight", "dbias") else 1e-5, what=name)


def draw_chain(seed):
    rng = random.Random(100 + seed)
    bs = rng.choice((4, 8))
    dims = tuple(bs * rng.randint(1, 4 if bs == 4 else 2) for _ in range(3))
    batch = rng.choice((1, 2, 5, 9, 32, 40))
    inner = rng.choice((1, 2, 3, 4))
    outer = rng.choice((1, 2, 3, 5))
    return dims, bs, batch, inner, outer, rng.choice(SMOOTH + ("leaky_relu",)), rng.random() < 0.4


@pytest.mark.parametrize("seed", range(16))
def test_random_chain_fused_against_op_by_op(seed):
    from gridnet_amd.network import GridnetBody
    from gridnet_amd.runner import BodyRunner

    shape, bs, batch, inner, outer, activation, residual = draw_chain(seed)
    print(f"sweep chain seed={seed} shape={shape} bs={bs} B={batch} inner={inner} outer={outer} "
          f"act={activation} residual={residual}", flush=True)
    w, b, r = make_params(shape, seed=5000 + seed)
    w = w * 0.5
    gamma = 1 + 0.2 * make_acts(1, shape, seed=5100 + seed)[0]
    beta = 0.2 * make_acts(1, shape, seed=5200 + seed)[0]
    x, gy = make_acts(batch, shape, seed=5300 + seed), make_acts(batch, shape, seed=5400 + seed)
    params = [t.to(DEV) for t in (w, b, r, gamma, beta)]

    run = BodyRunner(*params, batch, inner, outer, bs, activation, backward=True, fused=True,
                     outer_residual=residual)
    y = run.forward(x.to(DEV)).clone()
    fused = [y] + [g.clone() for g in run.backward(gy.to(DEV))]

    # the same chain op by op through the autograd wrappers (one call per step and LayerNorm)
    body = GridnetBody(shape, inner, outer, bs, activation=activation, outer_residual=residual,
                       device=DEV)
    with torch.no_grad():
        for p, t in zip((body.network.weight, body.network.bias, body.network.residual_scale, body.norm.weight,
                         body.norm.bias), params):
            p.copy_(t)
    x0 = x.to(DEV).requires_grad_(True)
    out = body(x0)
    leaves = [body.network.weight, body.network.bias, body.network.residual_scale, body.norm.weight,
              body.norm.bias, x0]
    grads = torch.autograd.grad(out, leaves, gy.to(DEV))
    steps = [out.detach()] + list(grads)

    terms = batch * inner * outer
    summed = 1e-5 * max(1.0, math.sqrt(terms / 2))
    names = ("y", "dweight", "dbias", "dscale", "dgamma", "dbeta", "dx0")
    if activation == "leaky_relu":
        # both chains are fp32, but they round differently: a pre-activation within rounding
        # distance of the kink can take different branches.  The forward result is continuous.
        names, fused, steps = names[:1], fused[:1], steps[:1]
    for name, got, want in zip(names, fused, steps):
        assert torch.isfinite(got).all(), name
        assert_close(got, want, atol=summed if name.startswith("d") and name != "dx0" else 1e-5,
                     what=name)
