"""GPU parity of the chain backward that takes every outer step in ONE launch
(gridnet_hip_chain_backward_all: the loop of gridnet/scripts/train_imagenet.py:76-86 taken
backward by resident workgroups that hand their results to each other through memory while the
kernel runs): against the CPU oracle at sizes it finishes in seconds, against the
launch-per-step chain of the same library at the benchmark's full shape, run-to-run
reproducibility, accumulation into the gradient buffers, and the give-up path of its bounded
waits (forced from the host; every kernel still ends normally).
Bar: rtol 1e-4 / atol 1e-5."""

import dataclasses

import pytest
import torch

from helpers import assert_close

from test_gpu_fused import NAMES, oracle, randomise_affine

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def runner(wl, t, chain_all):
    from gridnet_amd.runner import BodyRunner

    d = {k: v.to(DEV) for k, v in t.items() if k != "readout"}
    run = BodyRunner(d["weight"], d["bias"], d["scale"], d["gamma"], d["beta"], t["x0"].shape[0],
                     wl.inner, wl.outer, wl.block_size, wl.activation, wl.normalize,
                     backward=True, fused=True, chain=True, chain_all=chain_all)
    assert run.chain_all == bool(chain_all)
    return run, d


def run_chain(wl, t, chain_all):
    run, d = runner(wl, t, chain_all)
    y = run.forward(d["x0"]).clone()
    grads = [g.clone() for g in run.backward(d["grad_out"])]
    assert run.chain_all_status() == 0
    return (y, *grads)


def workload(grid, batch, inner, outer, activation):
    from gridnet_amd.configs import WORKLOADS

    return dataclasses.replace(WORKLOADS["C3"], grid=grid, batch=batch, inner=inner, outer=outer,
                               activation=activation, backward=True)


# smooth activations: the comparison of gradients is entry by entry (tests/helpers.py on kinks)
@pytest.mark.parametrize("grid,batch,inner,outer,activation", [
    (16, 6, 2, 2, "silu"), (16, 7, 4, 3, "tanh"), (32, 6, 2, 3, "silu"), (32, 9, 1, 4, "tanh"),
    (16, 33, 3, 2, "silu"), (16, 6, 8, 3, "tanh"), (32, 7, 5, 2, "silu")])
def test_one_launch_chain_matches_oracle(grid, batch, inner, outer, activation):
    from gridnet_amd.configs import make_inputs

    wl = workload(grid, batch, inner, outer, activation)
    print(f"one-launch chain grid={grid} batch={batch} inner={inner} outer={outer} act={activation}", flush=True)
    t = randomise_affine(make_inputs(wl, seed=3))
    if inner >= 5:  # keep that many residual updates contractive (fp32 rounding otherwise grows)
        t["weight"], t["scale"] = t["weight"] * 0.5, t["scale"] * 0.5
    got = run_chain(wl, t, True)
    again = run_chain(wl, t, True)
    for name, g, e in zip(NAMES, got, again):
        assert torch.equal(g, e), f"{name}: two runs differ"
    for name, g, e in zip(NAMES, got, run_chain(wl, t, False)):
        assert_close(g, e.double(), what=name + " vs launch per step")
    # parameter gradients are fp32 sums over batch, inner and outer iterations: as in
    # tests/test_gpu_cross_check.py their atol grows with the square root of the number of terms
    terms = batch * inner * outer
    for name, g, e in zip(NAMES, got, oracle(wl, t, True)):
        summed = name in ("dweight", "dbias", "dscale", "dgamma", "dbeta") and terms > 64
        assert_close(g, e, what=name, atol=1e-5 * (terms / 64) ** 0.5 if summed else 1e-5)


@pytest.mark.parametrize("shape,batch,inner,outer", [((16, 24, 8), 6, 2, 3), ((8, 16, 40), 7, 3, 2), ((8, 8, 8), 6, 1, 2)])
def test_one_launch_chain_on_grids_that_are_not_cubes(shape, batch, inner, outer):
    """M, N and K differ (and a single block along an axis has no neighbour there): the records'
    addressing and the row-wise completion of dx at the end must not depend on a cubic grid."""
    from gridnet_amd.runner import BodyRunner
    from helpers import make_acts, make_params
    from oracle.network import network_forward_backward

    print(f"one-launch chain shape={shape} B={batch} inner={inner} outer={outer}", flush=True)
    w, b, r = make_params(shape, seed=71)
    g = torch.Generator().manual_seed(72)
    gamma = 1 + 0.2 * torch.randn(shape, generator=g)
    beta = 0.2 * torch.randn(shape, generator=g)
    x0, gy = make_acts(batch, shape, seed=73), make_acts(batch, shape, seed=74)
    results = []
    for one_launch in (False, True):
        run = BodyRunner(*(v.to(DEV) for v in (w, b, r, gamma, beta)), batch, inner, outer, 8, "silu", False,
                         backward=True, fused=True, chain=True, chain_all=one_launch)
        assert run.chain_all == one_launch
        y = run.forward(x0.to(DEV)).clone()
        results.append((y, *[v.clone() for v in run.backward(gy.to(DEV))]))
        assert run.chain_all_status() == 0
    exp = network_forward_backward([v.double() for v in (w, b, r, gamma, beta)], x0.double(), gy.double(),
                                   inner_iterations=inner, outer_iterations=outer, block_size=8,
                                   activation="silu", normalize=False)
    for name, a, e, o in zip(NAMES, results[1], results[0], exp):
        assert_close(a, e.double(), what=name + " vs launch per step")
        assert_close(a, o, what=name)


def test_one_launch_chain_accumulates_into_the_gradient_buffers():
    """Without GRIDNET_OVERWRITE_PARAMS the parameter gradients are added to what the buffers hold."""
    from gridnet_amd import native as n
    from gridnet_amd.configs import make_inputs

    wl = workload(16, 8, 2, 3, "silu")
    t = randomise_affine(make_inputs(wl, seed=5))
    run, d = runner(wl, t, True)
    run.forward(d["x0"])
    fresh = [g.clone() for g in run.backward(d["grad_out"])]
    grads = [torch.full_like(g, 0.5) for g in fresh[:5]]
    dx = torch.empty_like(fresh[5])
    n.check(n.lib.gridnet_hip_chain_backward_all(
        run.dt, run.w.data_ptr(), run.b.data_ptr(), run.r.data_ptr(), run.gamma.data_ptr(),
        run.beta.data_ptr(), run.x0.data_ptr(), run.s_all.data_ptr(), run.stats.data_ptr(),
        d["grad_out"].data_ptr(), *[g.data_ptr() for g in grads], dx.data_ptr(), run.B, run.M, run.N,
        run.K, run.inner, run.outer, run.bs, run.act, 0, run.ca_ws.data_ptr(), run.ca_ws_bytes,
        n.current_stream(run.w)))
    assert run.chain_all_status() == 0
    for name, g, f in zip(NAMES[1:6], grads, fresh[:5]):
        assert_close(g, f.double() + 0.5, what=name + " accumulated")
    assert torch.equal(dx, fresh[5])


@pytest.mark.parametrize("activation", ["silu", "leaky_relu"])
def test_one_launch_chain_at_the_benchmark_shape(activation):
    """C3 (64^3 grid, batch 32, inner 4, outer 12): every block a resident workgroup.  Against the
    launch-per-step chain; under leaky_relu a pre-activation within rounding of the kink can land
    on either side in the two evaluations of the sums, so the fraction outside the bar is bounded
    there (tests/test_gpu_full_configs.py) and every entry is held under silu."""
    from gridnet_amd.configs import WORKLOADS, make_inputs

    wl = dataclasses.replace(WORKLOADS["C3"], activation=activation)
    print(f"one-launch chain at C3 under {activation}", flush=True)
    t = make_inputs(wl)
    got = run_chain(wl, t, True)
    again = run_chain(wl, t, True)
    for name, g, e in zip(NAMES, got, again):
        assert torch.equal(g, e), f"{name}: two runs differ"
    steps = run_chain(wl, t, False)
    assert torch.equal(got[0], steps[0])  # the forward is the same code
    for name, g, e in list(zip(NAMES, got, steps))[1:]:
        if activation == "silu":
            assert_close(g, e.double(), what=name + " vs launch per step")
        else:
            err = (g.double() - e.double()).abs()
            outside = (err > 1e-5 + 1e-4 * e.double().abs()).double().mean().item()
            print(f"  {name}: {outside:.2e} of the entries outside the bar of the launch-per-step chain", flush=True)
            assert outside < 1e-2, name


def test_one_launch_chain_gives_up_cleanly_and_the_runner_falls_back():
    """With signalling switched off from the host every wait inside the kernel runs out: the
    kernel ends, the status word says so, and the checked backward repeats launch by launch."""
    from gridnet_amd import native as n
    from gridnet_amd.configs import make_inputs

    wl = workload(16, 8, 2, 3, "silu")
    t = randomise_affine(make_inputs(wl, seed=4))
    want = run_chain(wl, t, False)
    run, d = runner(wl, t, True)
    run.forward(d["x0"])
    old = n.lib.gridnet_hip_chain_set_spin_limit(-20)
    try:
        run.backward(d["grad_out"])
        assert run.chain_all_status() != 0
        got = [g.clone() for g in run.backward_checked(d["grad_out"])]
        assert not run.chain_all
    finally:
        n.lib.gridnet_hip_chain_set_spin_limit(old)
    for name, g, e in zip(NAMES[1:], got, want[1:]):
        assert torch.equal(g, e), name


def test_unsupported_problems_are_refused():
    from gridnet_amd import native as n

    sup = n.lib.gridnet_hip_chain_all_supported
    assert sup(n.F32, 32, 64, 64, 64, 4, 12, 8, 0) == 1
    assert sup(n.F32, 32, 128, 128, 128, 4, 12, 8, 0) == 0   # 4096 blocks are not resident at once
    assert sup(n.F32, 5, 64, 64, 64, 4, 12, 8, 0) == 0       # batch below the minimum
    assert sup(n.F32, 32, 64, 64, 64, 8, 12, 8, 0) == 1      # the reference's ImageNet default shape
    assert sup(n.F32, 32, 64, 64, 64, 9, 12, 8, 0) == 0      # inner iterations
    assert sup(n.F32, 32, 64, 64, 64, 4, 1, 8, 0) == 0       # a chain has at least two steps
    assert sup(n.F64, 32, 64, 64, 64, 4, 12, 8, 0) == 0
    assert sup(n.F32, 32, 64, 64, 64, 4, 12, 4, 0) == 0
    assert sup(n.F32, 32, 64, 64, 64, 4, 12, 8, 1) == 0
    rc = n.lib.gridnet_hip_chain_backward_all(n.F32, *([1] * 15), 5, 64, 64, 64, 4, 12, 8, 1, 0, None, 0, None)
    assert rc != 0 and "one-launch chain" in n.last_error()
