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


# ---- inputs that keep clear of the kink of relu / leaky_relu --------------------------------
# The derivative of these activations jumps at 0.  A pre-activation that the fp64 oracle puts
# within rounding distance of 0 can come out on the other side in fp32, and then the gradient of
# that cell (and of everything upstream of it) differs grossly although nothing is wrong.  In a
# chain of outer steps the fp32 pre-activations are off by up to ~1e-5, so a comparison of
# GRADIENTS against the oracle is only meaningful on inputs whose smallest |pre-activation| is
# well above that; such inputs exist with fair odds only while cells x iterations stays below
# ~1e5 (the smallest of N standard normal draws is ~1/N).  Larger cases use a smooth activation.
KINKED = ("relu", "leaky_relu")


def chain_kink_margin(t, wl):
    """Smallest |pre-activation| over all cells, inner iterations and outer steps of the fp64
    oracle chain on inputs ``t`` (dict as gridnet_amd.configs.make_inputs returns)."""
    from oracle.fast import gridnet_step_fast
    from oracle.network import network_forward

    smallest = [math.inf]

    def note(u):
        smallest[0] = min(smallest[0], u.abs().min().item())

    def step(*args):
        return gridnet_step_fast(*args, watch=note)

    with torch.no_grad():
        network_forward(*[t[k].double() for k in ("weight", "bias", "scale", "gamma", "beta")],
                        t["x0"].double(), wl.inner, wl.outer, wl.block_size, wl.activation,
                        wl.normalize, step_fn=step)
    return smallest[0]


def inputs_clear_of_kink(wl, make, margin=2e-5, tries=200):
    """``make(seed)`` for the first seed whose oracle chain keeps every pre-activation at least
    ``margin`` away from 0; any seed for smooth activations."""
    if wl.activation not in KINKED:
        return make(0)
    for seed in range(tries):
        t = make(seed)
        if chain_kink_margin(t, wl) >= margin:
            return t
    raise AssertionError(f"no seed below {tries} keeps {wl.name} {margin} clear of the kink: "
                         "the case has too many cells x iterations for a kinked activation")


def step_kink_margin(w, b, r, x, inner, bs, eps, normalize, activation):
    """Smallest |pre-activation| of one fp64 oracle step."""
    from oracle.fast import gridnet_step_fast

    smallest = [math.inf]

    def note(u):
        smallest[0] = min(smallest[0], u.abs().min().item())

    with torch.no_grad():
        gridnet_step_fast(w.double(), b.double(), r.double(), x.double(), inner, bs, eps, normalize,
                          activation, watch=note)
    return smallest[0]


def acts_clear_of_kink(w, b, r, batch, shape, inner, bs, eps, normalize, activation, seed,
                       dtype=torch.float32, margin=2e-6, tries=200):
    """Input activations (make_acts with seed, seed + 1000, ...) for which one step keeps every
    pre-activation ``margin`` away from 0: ten times what fp32 rounding moves it by."""
    if activation not in KINKED or inner == 0:
        return make_acts(batch, shape, seed=seed, dtype=dtype)
    for k in range(tries):
        x = make_acts(batch, shape, seed=seed + 1000 * k, dtype=dtype)
        if step_kink_margin(w, b, r, x, inner, bs, eps, normalize, activation) >= margin:
            return x
    raise AssertionError(f"no input among {tries} keeps shape {shape} {margin} clear of the kink")
