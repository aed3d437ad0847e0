"""Writes tests/golden/step_normalize.npz and tests/golden/step_gated.npz: one outer step with
per-window normalisation (the reference's default mode) and one gated step, on a (8, 16, 8) grid
with 4^3 blocks, batch 3, evaluated by the CPU oracle in fp64 from seeded fp32 inputs -- inputs,
result and all gradients (autograd of the oracle), stored as fp32.

REGRESSION fixtures produced by this repository's own oracle (pinned by tests/test_oracle_*.py);
they are not outputs of the reference, whose Python was not run.
Usage: python tests/golden/make_step_fixtures.py
"""

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle.fast import gridnet_step_fast  # noqa: E402
from oracle.gated import gated_step_fast  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
SHAPE, BS, BATCH = (8, 16, 8), 4, 3


def save(name, inputs, fn):
    leaves = {k: v.double().requires_grad_(True) for k, v in inputs.items() if k != "grad_out"}
    y = fn(**leaves)
    grads = torch.autograd.grad(y, list(leaves.values()), inputs["grad_out"].double())
    out = {k: v.numpy() for k, v in inputs.items()}
    out["y"] = y.detach().float().numpy()
    for k, g in zip(leaves, grads):
        out["d" + k] = g.float().numpy()
    np.savez_compressed(os.path.join(HERE, name), **out)
    print("written", name, {k: v.shape for k, v in out.items()})


g = torch.Generator().manual_seed(2024)
save("step_normalize.npz",
     {"weight": torch.randn(27, *SHAPE, generator=g) / 27 ** 0.5,
      "bias": 0.1 * torch.randn(*SHAPE, generator=g),
      "scale": 0.5 + torch.rand(*SHAPE, generator=g),
      "x": 2.0 + torch.randn(BATCH, *SHAPE, generator=g),
      "grad_out": torch.randn(BATCH, *SHAPE, generator=g)},
     lambda weight, bias, scale, x: gridnet_step_fast(weight, bias, scale, x, 3, BS, 1e-5, True, "silu"))
save("step_gated.npz",
     {"weight": torch.randn(27, 2, *SHAPE, generator=g) / 27 ** 0.5,
      "bias": 0.5 * torch.randn(2, *SHAPE, generator=g),
      "x": torch.randn(BATCH, *SHAPE, generator=g),
      "grad_out": torch.randn(BATCH, *SHAPE, generator=g)},
     lambda weight, bias, x: gated_step_fast(weight, bias, x, 3, BS, "tanh"))
