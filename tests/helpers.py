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


def assert_chain_close(names, got, want, t, wl, params=("weight", "bias", "scale", "gamma", "beta")):
    """Outputs of a chain of outer steps against the fp64 oracle chain, at the bar.  Where an entry
    lies outside it the question is whether the kernels did that or what fp32 does to this
    problem, and the same chain evaluated on the CPU in fp32 (torch's own operators: the
    reference's arithmetic) arbitrates.  Worst entries of two fp32 evaluations are extreme values
    of different rounding patterns, so the comparison is one of distributions: beyond every
    threshold k = 1, 2, 4, ... bar units the device has at most twice as many entries as the CPU
    evaluation has beyond k / 2, plus three, and none beyond max(1, twice the CPU's worst).
    (At 32^3 with silu, three outer steps of four inner iterations, one weight-gradient entry in
    884 736 sits at the bar for either evaluation: 0.8-2.0 bar units on the CPU depending on
    gamma and beta, 0.75-1.3 on the device depending on the rounding of its sigmoid.)"""
    from oracle.network import network_forward_backward

    arbiter = None
    for i, (name, g, w) in enumerate(zip(names, got, want)):
        try:
            assert_close(g, w, what=name)
        except AssertionError:
            if arbiter is None:
                arbiter = network_forward_backward(
                    [t[k].float() for k in params], t["x0"].float(), t["grad_out"].float(),
                    inner_iterations=wl.inner, outer_iterations=wl.outer, block_size=wl.block_size,
                    activation=wl.activation, normalize=wl.normalize)
            bound = ATOL + RTOL * w.abs()
            dev = (g.detach().cpu().double() - w).abs() / bound
            cpu = (arbiter[i].double() - w).abs() / bound
            worst_dev, worst_cpu = dev.max().item(), cpu.max().item()
            print(f"  {name}: device worst {worst_dev:.3f} bar units, CPU fp32 worst {worst_cpu:.3f}", flush=True)
            assert worst_dev <= max(1.0, 2 * worst_cpu), (
                f"{name}: {worst_dev:.3f} bar units from the fp64 chain where the CPU's fp32 "
                f"evaluation is at {worst_cpu:.3f}")
            k = 1.0
            while k < worst_dev:
                n_dev, n_cpu = int((dev > k).sum()), int((cpu > k / 2).sum())
                assert n_dev <= 2 * n_cpu + 3, (
                    f"{name}: {n_dev} entries beyond {k:g} bar units, the CPU's fp32 evaluation has "
                    f"{n_cpu} beyond {k / 2:g}")
                k *= 2


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
