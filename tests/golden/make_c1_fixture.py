"""Writes tests/golden/c1_network.npz: the C1 workload (16^3 grid, 8^3 blocks, batch 2, inner 2,
outer 2, leaky_relu) evaluated by the CPU oracle in fp64 from the seeded fp32 inputs of
gridnet_amd.configs -- result and all gradients, stored as fp32.

This is a REGRESSION fixture produced by this repository's own oracle (which the closed-form
tests pin); it is not an output of the reference, whose Python was not run.
Usage: python tests/golden/make_c1_fixture.py
"""

import dataclasses
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from gridnet_amd.configs import WORKLOADS, make_inputs  # noqa: E402
from oracle.network import network_forward_backward  # noqa: E402

wl = dataclasses.replace(WORKLOADS["C1"], backward=True)
t = make_inputs(wl, seed=0)
out = network_forward_backward(
    [t[k].double() for k in ("weight", "bias", "scale", "gamma", "beta")], t["x0"].double(),
    t["grad_out"].double(), inner_iterations=wl.inner, outer_iterations=wl.outer,
    block_size=wl.block_size, activation=wl.activation, normalize=wl.normalize)
names = ("y", "dweight", "dbias", "dscale", "dgamma", "dbeta", "dx0")
np.savez_compressed(os.path.join(os.path.dirname(__file__), "c1_network.npz"),
                    x0_checksum=np.float64(t["x0"].double().sum().item()),
                    **{n: v.float().numpy() for n, v in zip(names, out)})
print("written", {n: tuple(v.shape) for n, v in zip(names, out)})
