"""The committed C1 fixture (tests/golden/c1_network.npz, written by make_c1_fixture.py from the
CPU oracle) against the oracle on the CPU and against the HIP path on the GPU."""

import dataclasses
import os

import numpy as np
import pytest
import torch

from helpers import assert_close

FIXTURE = os.path.join(os.path.dirname(__file__), "golden", "c1_network.npz")
NAMES = ("y", "dweight", "dbias", "dscale", "dgamma", "dbeta", "dx0")


def c1():
    from gridnet_amd.configs import WORKLOADS, make_inputs

    wl = dataclasses.replace(WORKLOADS["C1"], backward=True)
    return wl, make_inputs(wl, seed=0)


def test_fixture_inputs_are_the_seeded_ones():
    _, t = c1()
    gold = np.load(FIXTURE)
    assert abs(float(gold["x0_checksum"]) - t["x0"].double().sum().item()) < 1e-9


def test_oracle_reproduces_fixture_in_fp32():
    """ref-style (the reference's op sequence) in fp32 lands on the fp64 fixture within the bar."""
    from oracle.network import network_forward_backward
    from oracle.ref_style import gridnet_step_ref

    wl, t = c1()
    gold = np.load(FIXTURE)
    out = network_forward_backward(
        [t[k] for k in ("weight", "bias", "scale", "gamma", "beta")], t["x0"], t["grad_out"],
        inner_iterations=wl.inner, outer_iterations=wl.outer, block_size=wl.block_size,
        activation=wl.activation, normalize=wl.normalize, step_fn=gridnet_step_ref)
    for name, got in zip(NAMES, out):
        assert_close(got, torch.from_numpy(gold[name]), what=name)


@pytest.mark.gpu
@pytest.mark.parametrize("fused", [False, True], ids=["op-by-op", "fused"])
def test_hip_path_reproduces_fixture(fused):
    from gridnet_amd.runner import BodyRunner

    wl, t = c1()
    gold = np.load(FIXTURE)
    d = {k: v.to("cuda:0") for k, v in t.items()}
    run = BodyRunner(d["weight"], d["bias"], d["scale"], d["gamma"], d["beta"], wl.batch, wl.inner,
                     wl.outer, wl.block_size, wl.activation, wl.normalize, fused=fused)
    y = run.forward(d["x0"]).clone()
    grads = run.backward(d["grad_out"])
    for name, got in zip(NAMES, (y, *grads)):
        assert_close(got, torch.from_numpy(gold[name]), what=name)


# ---- one outer step with normalize=True and one gated step (tests/golden/make_step_fixtures.py)
STEP_FIXTURES = {
    "normalize": ("step_normalize.npz", ("weight", "bias", "scale", "x"), ("y", "dweight", "dbias", "dscale", "dx")),
    "gated": ("step_gated.npz", ("weight", "bias", "x"), ("y", "dweight", "dbias", "dx")),
}


def load_step(kind):
    name, inputs, outputs = STEP_FIXTURES[kind]
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", name))
    return gold, inputs, outputs


@pytest.mark.parametrize("kind", sorted(STEP_FIXTURES))
def test_ref_style_oracle_reproduces_step_fixture_in_fp32(kind):
    """The op-for-op restatement of the reference's torch path, run in fp32 on the CPU, lands on
    the fixture (which the vectorised oracle wrote in fp64) within the bar."""
    from oracle.gated import gated_step_ref
    from oracle.ref_style import gridnet_step_ref

    gold, inputs, outputs = load_step(kind)
    leaves = [torch.from_numpy(gold[k]).requires_grad_(True) for k in inputs]
    if kind == "normalize":
        y = gridnet_step_ref(*leaves, 3, 4, 1e-5, True, "silu")
    else:
        y = gated_step_ref(*leaves, 3, 4, "tanh")
    grads = torch.autograd.grad(y, leaves, torch.from_numpy(gold["grad_out"]))
    for name, got in zip(outputs, (y, *grads)):
        assert_close(got, torch.from_numpy(gold[name]), rtol=2e-4, atol=2e-5, what=f"{kind} {name}")


@pytest.mark.gpu
@pytest.mark.parametrize("kind", sorted(STEP_FIXTURES))
def test_hip_path_reproduces_step_fixture(kind):
    from gridnet_amd.backend_cuda import GatedGridnetCudaOp, GridnetCudaOp

    gold, inputs, outputs = load_step(kind)
    leaves = [torch.from_numpy(gold[k]).to("cuda:0").requires_grad_(True) for k in inputs]
    if kind == "normalize":
        y = GridnetCudaOp.apply(*leaves, 3, 4, 1e-5, True, "silu")
    else:
        y = GatedGridnetCudaOp.apply(*leaves, 3, 4, "tanh")
    grads = torch.autograd.grad(y, leaves, torch.from_numpy(gold["grad_out"]).to("cuda:0"))
    for name, got in zip(outputs, (y, *grads)):
        assert_close(got, torch.from_numpy(gold[name]), rtol=2e-4 if kind == "normalize" else 1e-4,
                     atol=2e-5 if kind == "normalize" else 1e-5, what=f"{kind} {name}")
