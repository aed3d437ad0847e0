"""Where the HIP path is compared at a tolerance looser than the bar, show that the slack is
fp32 conditioning of the problem and not the kernels.

The bar is rtol 1e-4 / atol 1e-5 against the oracle evaluated in fp64.  Two groups of cases
elsewhere in this suite were given more room: deep recurrences (8 inner iterations, the C5
depth) had their weights made contractive, and the ``normalize=True`` fixture is held at twice
the bar.  Here the same cases run WITHOUT that help, three ways on the same fp32 inputs:

  (i)   the oracle in fp64                                   -- the truth;
  (ii)  the op-for-op restatement of the reference's torch path (oracle.ref_style) in fp32 on
        the CPU                                              -- what fp32 does to this problem
        in the reference's own evaluation order (gridnet/backend_torch.py:118-140);
  (iii) the HIP path in fp32 on the GPU.

Asserted, entry errors taken in units of the bar's bound (atol + rtol |truth|): the worst entry
of (iii) is within the bar; or the RMS error of (iii) is at most twice that of (ii) and its
worst entry at most four times the worst of (ii) (the maximum over 10^5 entries of a rounding
error is a noisy figure, the RMS is not).  All figures are printed.  Measured: with C5's own
weights the HIP path is inside the bar where the fp32 CPU evaluation is not (dweight 0.94
against 1.20 bar units); on the single deep steps with scales up to 1.5 both leave the bar
together (16 iterations: dweight ~97 bar units for both), the HIP path's RMS error being
1.0 to 1.6 times the CPU's (a serial chain of 27 FMAs per cell against torch's blocked sums).
"""

import dataclasses
import os

import numpy as np
import pytest
import torch

from helpers import ATOL, RTOL, inputs_clear_of_kink

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PARAMS = ("weight", "bias", "scale", "gamma", "beta")
NAMES = ("y", "dweight", "dbias", "dscale", "dgamma", "dbeta", "dx0")


def bar_units(got, want):
    """(worst, rms) of the entry errors in units of the bar's bound."""
    want = want.double()
    e = (got.detach().cpu().double() - want).abs() / (ATOL + RTOL * want.abs())
    return e.max().item(), e.square().mean().sqrt().item()


def arbitrate(names, truth, cpu32, hip32):
    for name, ref, c, h in zip(names, truth, cpu32, hip32):
        (uc, rc), (uh, rh) = bar_units(c, ref), bar_units(h, ref)
        print(f"  {name:8s} fp32 reference-order CPU: worst {uc:7.3f} rms {rc:7.4f} bar units | "
              f"HIP fp32: worst {uh:7.3f} rms {rh:7.4f}", flush=True)
        ok = uh <= 1.0 or (rh <= 2.0 * rc and uh <= 4.0 * uc)
        assert ok, (f"{name}: HIP is {uh:.3f} (rms {rh:.4f}) bar units from the fp64 oracle, the "
                    f"fp32 CPU evaluation {uc:.3f} (rms {rc:.4f})")


@pytest.mark.parametrize("fused", [False, True], ids=["op-by-op", "fused"])
def test_c5_depth_with_its_own_weights(fused):
    """C5 reduced (16^3 grid, batch 2, 2 outer steps) with ITS OWN parameter distribution:
    4^3 blocks, 8 inner iterations, weights N(0, 1/27), residual scale 1."""
    from gridnet_amd.configs import WORKLOADS, make_inputs
    from gridnet_amd.runner import BodyRunner
    from oracle.network import network_forward_backward
    from oracle.ref_style import gridnet_step_ref

    wl = dataclasses.replace(WORKLOADS["C5"], grid=16, batch=2, outer=2)
    print(f"arbitration {wl.name} grid=16 batch=2 outer=2 fused={fused}", flush=True)
    t = inputs_clear_of_kink(wl, lambda seed: make_inputs(wl, seed=seed))
    kw = dict(inner_iterations=wl.inner, outer_iterations=wl.outer, block_size=wl.block_size,
              activation=wl.activation, normalize=False)
    truth = network_forward_backward([t[k].double() for k in PARAMS], t["x0"].double(),
                                     t["grad_out"].double(), **kw)
    cpu32 = network_forward_backward([t[k] for k in PARAMS], t["x0"], t["grad_out"],
                                     step_fn=gridnet_step_ref, **kw)
    d = {k: v.to(DEV) for k, v in t.items()}
    run = BodyRunner(*(d[k] for k in PARAMS), wl.batch, wl.inner, wl.outer, wl.block_size,
                     wl.activation, False, backward=True, fused=fused)
    hip32 = [run.forward(d["x0"]).clone()] + [g.clone() for g in run.backward(d["grad_out"])]
    arbitrate(NAMES, truth, cpu32, hip32)


@pytest.mark.parametrize("inner,bs,activation", [(8, 4, "tanh"), (8, 8, "silu"), (16, 8, "silu"), (32, 4, "silu")])
def test_deep_single_step_with_uncontracted_weights(inner, bs, activation):
    """One step, many inner iterations, weights N(0, 1/27) and scales in [0.5, 1.5) as they come."""
    from gridnet_amd.backend_cuda import GridnetCudaOp
    from helpers import make_acts, make_params
    from oracle.fast import gridnet_step_fast
    from oracle.ref_style import gridnet_step_ref

    shape, batch = (16, 8, 24), 2
    print(f"arbitration deep step inner={inner} bs={bs} act={activation}", flush=True)
    w, b, r = make_params(shape, seed=11)
    x, gy = make_acts(batch, shape, seed=12), make_acts(batch, shape, seed=13)

    def autograd(fn, dtype, dev="cpu"):
        leaves = [v.to(device=dev, dtype=dtype).requires_grad_(True) for v in (w, b, r, x)]
        y = fn(*leaves)
        return [y.detach()] + list(torch.autograd.grad(y, leaves, gy.to(device=dev, dtype=dtype)))

    truth = autograd(lambda *a: gridnet_step_fast(*a, inner, bs, 1e-5, False, activation), torch.float64)
    cpu32 = autograd(lambda *a: gridnet_step_ref(*a, inner, bs, 1e-5, False, activation), torch.float32)
    hip32 = autograd(lambda *a: GridnetCudaOp.apply(*a, inner, bs, 1e-5, False, activation),
                     torch.float32, DEV)
    arbitrate(("y", "dweight", "dbias", "dscale", "dx"), truth, cpu32, hip32)


def test_normalize_fixture():
    """The committed normalize=True step (tests/golden/step_normalize.npz, written by the oracle in
    fp64): the division by (std + eps) and the window sums of its backward amplify rounding."""
    from gridnet_amd.backend_cuda import GridnetCudaOp
    from oracle.ref_style import gridnet_step_ref

    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "step_normalize.npz"))
    inputs, outputs = ("weight", "bias", "scale", "x"), ("y", "dweight", "dbias", "dscale", "dx")
    print("arbitration normalize=True fixture", flush=True)
    truth = [torch.from_numpy(gold[k]) for k in outputs]
    both = []
    for dev in ("cpu", DEV):
        leaves = [torch.from_numpy(gold[k]).to(dev).requires_grad_(True) for k in inputs]
        fn = gridnet_step_ref if dev == "cpu" else GridnetCudaOp.apply
        y = fn(*leaves, 3, 4, 1e-5, True, "silu")
        both.append([y.detach()] + list(torch.autograd.grad(y, leaves, torch.from_numpy(gold["grad_out"]).to(dev))))
    # the fixture itself is stored in fp32: half an ulp of slack on top of the comparison
    arbitrate(outputs, truth, *both)
