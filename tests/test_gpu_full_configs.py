"""Every benchmark configuration at its FULL size, on the path ``bench.py`` times (the chain
with the LayerNorm folded into the step kernels, fp32).

The CPU oracle takes minutes for a whole workload at these sizes (the last C3 test below runs it
for three outer steps).  The arbiter here is the op-by-op chain of
the same library run in fp64 on the same fp32 inputs: the generic kernels (one thread per cell,
scatter with atomics) and the separate LayerNorm kernels, which share no device code with the
tuned fp32 kernels and are themselves held to the oracle on the shapes it does reach
(test_gpu_step.py, test_gpu_layernorm.py, test_gpu_network.py).  Beside it runs the op-by-op
chain in fp32: a second fp32 evaluation of the same function in a different order.

Forward results: every entry inside the bar (rtol 1e-4 / atol 1e-5) of the fp64 chain; measured
worst entries 0.08 to 0.16 of the bar's bound at all four shapes.

Gradients of a chain of 12 to 16 outer steps: parameter gradients are sums of up to 10^4 fp32
terms per entry and a few entries in a million leave the bar in ANY fp32 evaluation (under
silu at C3: 44 of 7 million dweight entries for the fused chain, 40 for the op-by-op chain).
Asserted under a smooth activation: the errors of the fused chain are distributed like those of
the op-by-op fp32 chain -- at every threshold k = 1, 2, 4, ... bar units, no more entries beyond
k than twice the number the op-by-op chain has beyond k / 2 (give or take three entries), and no
entry beyond four times its worst.  (The worst single entry of seven million is a noisy yardstick:
two valid fp32 evaluations differ by a factor of two to three in it, and it moves whenever a
kernel of either chain changes its summation order.)
Under leaky_relu (the workloads' own activation) some of the 10^8 pre-activations lie within
fp32 rounding of the kink, where fp32 and fp64 take different branches of the derivative; the
LayerNorm couples all cells of a sample, so every such flip moves every upstream gradient a
little.  The activation is kept and the FRACTION of entries outside the bar is bounded: below
1 % and no more than twice the op-by-op fp32 chain's fraction (measured at C3: 0.24 % of the
dweight entries for the fused chain, 0.60 % for the op-by-op chain).  All counts are printed.
"""

import dataclasses

import pytest
import torch

from helpers import ATOL, RTOL

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PARAMS = ("weight", "bias", "scale", "gamma", "beta")
NAMES = ("y", "dweight", "dbias", "dscale", "dgamma", "dbeta", "dx0")


def chain(wl, t, dtype, fused):
    """(y, grads...) of the chain on device copies of ``t`` in ``dtype``; buffers are released."""
    from gridnet_amd.runner import BodyRunner

    d = {k: v.to(device=DEV, dtype=dtype) for k, v in t.items() if k != "readout"}
    run = BodyRunner(*(d[k] for k in PARAMS), d["x0"].shape[0], wl.inner, wl.outer, wl.block_size,
                     wl.activation, wl.normalize, backward=wl.backward, fused=fused)
    out = [run.forward(d["x0"]).clone()]
    if wl.backward:
        out += [g.clone() for g in run.backward(d["grad_out"])]
    torch.cuda.synchronize()
    del run
    return out


def excess(got, want):
    """Per entry: |got - want| in units of the bar's bound atol + rtol |want| (<= 1 is inside)."""
    want = want.double()
    return (got.double() - want).abs() / (ATOL + RTOL * want.abs())


def hold_to_fp64(name, fused, steps, ref, kinked=False):
    """The fused result against the fp64 chain, with the op-by-op fp32 chain as the yardstick of
    what fp32 does to this problem.  Smooth activations: beyond every threshold k = 1, 2, 4, ...
    bar units lie at most twice as many entries as the yardstick has beyond k / 2, plus three, and
    none lies beyond max(1, 4 x the yardstick's worst).  ``kinked``: the fraction of entries outside
    the bar stays below 1 % and below twice the yardstick's fraction (plus one entry in 10^4)."""
    ef, es = excess(fused, ref), excess(steps, ref)
    worst_f, worst_s = ef.max().item(), es.max().item()
    out_f, out_s = (ef > 1).double().mean().item(), (es > 1).double().mean().item()
    print(f"  {name:8s} fused: worst {worst_f:9.3f} bar units, {int((ef > 1).sum())} of {ef.numel()} "
          f"outside the bar ({out_f:.2e}) | op-by-op fp32: worst {worst_s:9.3f}, "
          f"{int((es > 1).sum())} outside ({out_s:.2e})", flush=True)
    assert torch.isfinite(fused).all(), name
    if kinked:
        assert out_f <= 1e-2 and out_f <= 2 * out_s + 1e-4, (
            f"{name}: {out_f:.3e} of the entries are outside the bar (op-by-op fp32 chain: {out_s:.3e})")
    else:
        limit = max(1.0, 4.0 * worst_s)
        assert worst_f <= limit, (
            f"{name}: worst entry {worst_f:.3f} bar units from the fp64 chain, limit {limit:.3f} "
            f"(op-by-op fp32 worst {worst_s:.3f})")
        k = 1.0
        while k < worst_f:
            n_f, n_s = int((ef > k).sum()), int((es > k / 2).sum())
            assert n_f <= 2 * n_s + 3, (
                f"{name}: {n_f} entries beyond {k:g} bar units, the op-by-op fp32 chain has {n_s} beyond {k / 2:g}")
            k *= 2


def layernorm_invariants(y, gamma_is_one=True):
    flat = y.flatten(1).double()
    assert flat.mean(1).abs().max().item() < 1e-4
    assert (flat.var(1, unbiased=False) - 1).abs().max().item() < 1e-3


def test_c3_full_fused_training_step():
    """C3: 64^3, 8^3 blocks, batch 32, inner 4, outer 12, forward + backward."""
    from gridnet_amd.configs import WORKLOADS, make_inputs

    wl = WORKLOADS["C3"]
    t = make_inputs(wl)
    print(f"full config {wl.name}", flush=True)
    fused = chain(wl, t, torch.float32, True)
    again = chain(wl, t, torch.float32, True)
    for name, a, b in zip(NAMES, fused, again):
        assert torch.equal(a, b), f"{name}: the fused chain is not bitwise reproducible"
    layernorm_invariants(fused[0])
    steps = chain(wl, t, torch.float32, False)
    ref = chain(wl, t, torch.float64, False)
    hold_to_fp64("y", fused[0], steps[0], ref[0])
    # gradients under the workload's own leaky_relu: kink flips allowed in a bounded fraction
    for name, f, s, r in list(zip(NAMES, fused, steps, ref))[1:]:
        hold_to_fp64(name, f, s, r, kinked=True)
    # samples do not interact: the first 4 alone give the same y (bit for bit) and the same dx
    small = dataclasses.replace(wl, batch=4)
    ts = {k: (v[:4] if k in ("x0", "grad_out") else v) for k, v in t.items()}
    sub = chain(small, ts, torch.float32, True)
    assert torch.equal(sub[0], fused[0][:4])
    assert (excess(sub[6], fused[6][:4]) > 2).double().mean().item() < 1e-5


def test_c3_full_fused_gradients_smooth_activation():
    """The same chain under silu (no kink): every gradient entry is held, none excused."""
    from gridnet_amd.configs import WORKLOADS, make_inputs

    wl = dataclasses.replace(WORKLOADS["C3"], activation="silu")
    t = make_inputs(wl)
    print(f"full config {wl.name} under silu", flush=True)
    fused = chain(wl, t, torch.float32, True)
    steps = chain(wl, t, torch.float32, False)
    ref = chain(wl, t, torch.float64, False)
    for name, f, s, r in zip(NAMES, fused, steps, ref):
        hold_to_fp64(name, f, s, r)


@pytest.mark.parametrize("name,cut", [("C3", dict(outer=3)), ("C5", dict(batch=32, outer=2))])
def test_full_size_arbiter_is_held_to_the_cpu_oracle(name, cut):
    """The arbiter of this file at the full C3 shape (64^3 grid, 8^3 blocks, batch 32, inner 4) and on
    C5's grid (64^3, 4^3 blocks, inner 8) against the CPU oracle itself: the loop without autograd
    (oracle.network, pinned against autograd in tests/test_oracle_backward.py), fp64, the workloads'
    own leaky_relu.  The oracle takes 5 to 10 seconds per outer step at these sizes, so the suite
    runs three outer steps of C3 and two of C5 with a quarter of its batch.  The fp64 chain on the
    GPU must agree with it to 1e-9; at C3 the fused fp32 chain is then held to the ORACLE the way
    the tests above hold it to the fp64 chain."""
    from gridnet_amd.configs import WORKLOADS, make_inputs
    from oracle.network import network_forward_backward_manual

    import os

    # GRIDNET_FULL_ORACLE=1: the workloads uncut (C3: about a minute of CPU time, C5: ten)
    wl = WORKLOADS[name] if os.environ.get("GRIDNET_FULL_ORACLE") else dataclasses.replace(WORKLOADS[name], **cut)
    t = make_inputs(wl)
    print(f"full size against the CPU oracle: {wl.name} with batch={wl.batch} outer={wl.outer}", flush=True)
    want = network_forward_backward_manual(
        [t[k].double() for k in PARAMS], t["x0"].double(), t["grad_out"].double(), wl.inner, wl.outer,
        wl.block_size, wl.activation, wl.normalize)
    ref = chain(wl, t, torch.float64, False)
    for gname, a, e in zip(NAMES, ref, want):
        e = e.to(DEV)
        err = ((a - e).abs() / (1 + e.abs())).max().item()
        print(f"  {gname:8s} fp64 chain against the oracle: worst {err:.2e} (relative to 1 + |value|)", flush=True)
        assert err < 1e-9, gname
    if name != "C3":
        return  # (the cut C5 run is about the arbiter; the fused chain is held to it at C5's full size above)
    fused = chain(wl, t, torch.float32, True)
    steps = chain(wl, t, torch.float32, False)
    hold_to_fp64("y", fused[0], steps[0], want[0].to(DEV))
    for gname, f, s_, e in list(zip(NAMES, fused, steps, want))[1:]:
        hold_to_fp64(gname, f, s_, e.to(DEV), kinked=True)


def test_c4_full_fused_forward():
    """C4: 128^3, 8^3 blocks, batch 8, inner 4, outer 16, forward only; input built from
    224x224x3 images patch-embedded into the [..., 0] face, 1000-way readout from [..., -1]."""
    from gridnet_amd.configs import WORKLOADS, make_inputs, read_out

    wl = WORKLOADS["C4"]
    t = make_inputs(wl)
    print(f"full config {wl.name}", flush=True)
    assert t["x0"][..., 1:].abs().max().item() == 0 and t["bias"].abs().max().item() == 0
    (fused,), (again,) = chain(wl, t, torch.float32, True), chain(wl, t, torch.float32, True)
    assert torch.equal(fused, again)
    layernorm_invariants(fused)
    (steps,), (ref,) = chain(wl, t, torch.float32, False), chain(wl, t, torch.float64, False)
    hold_to_fp64("y", fused, steps, ref)
    logits = read_out(fused.cpu(), t["readout"])
    want = read_out(ref.cpu().double(), t["readout"].double())
    assert logits.shape == (wl.batch, 1000)
    assert torch.allclose(logits.double(), want, rtol=1e-3, atol=1e-3)


def test_c2_full_fused_forward():
    """C2: 32^3, 8^3 blocks, batch 64, inner 4, outer 8, forward only, zero bias; input built
    from 28x28 images projected onto the [..., 0] face, 10-way readout from [..., -1]."""
    from gridnet_amd.configs import WORKLOADS, make_inputs, read_out

    wl = WORKLOADS["C2"]
    t = make_inputs(wl)
    print(f"full config {wl.name}", flush=True)
    assert t["x0"][..., 1:].abs().max().item() == 0 and t["bias"].abs().max().item() == 0
    (fused,), (again,) = chain(wl, t, torch.float32, True), chain(wl, t, torch.float32, True)
    assert torch.equal(fused, again)
    layernorm_invariants(fused)
    (steps,), (ref,) = chain(wl, t, torch.float32, False), chain(wl, t, torch.float64, False)
    hold_to_fp64("y", fused, steps, ref)
    logits = read_out(fused.cpu(), t["readout"])
    want = read_out(ref.cpu().double(), t["readout"].double())
    assert logits.shape == (wl.batch, 10)
    assert torch.allclose(logits.double(), want, rtol=1e-3, atol=1e-3)


def test_c5_full_fused_training_step():
    """C5: 64^3, 4^3 blocks, batch 128, inner 8, outer 16, forward + backward, with its own
    weights (N(0, 1/27), residual scale 1: nothing made contractive)."""
    from gridnet_amd.configs import WORKLOADS, make_inputs

    wl = WORKLOADS["C5"]
    t = make_inputs(wl)
    print(f"full config {wl.name}", flush=True)
    fused = chain(wl, t, torch.float32, True)
    again = chain(wl, t, torch.float32, True)
    for name, a, b in zip(NAMES, fused, again):
        assert torch.equal(a, b), f"{name}: the fused chain is not bitwise reproducible"
    layernorm_invariants(fused[0])
    steps = chain(wl, t, torch.float32, False)
    ref = chain(wl, t, torch.float64, False)
    hold_to_fp64("y", fused[0], steps[0], ref[0])
    for name, f, s, r in list(zip(NAMES, fused, steps, ref))[1:]:
        hold_to_fp64(name, f, s, r, kinked=True)
