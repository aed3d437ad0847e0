"""The five benchmark/parity workloads and their seeded synthetic inputs.

Inputs are drawn on the CPU from ``torch.Generator().manual_seed(seed)`` in a fixed order, so
a checker and the device path can be fed identical bits.  Parameter scales follow the
reference's initialisation (gridnet/__init__.py:42-49): weight [27, g, g, g] ~ N(0, 1/27);
bias ~ N(0, 0.01) (std 0.1) or zero; residual_scale = 1; LayerNorm weight 1, bias 0.
"""

import math
from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    grid: int
    block_size: int
    batch: int
    inner: int
    outer: int
    backward: bool
    zero_bias: bool = False
    activation: str = "leaky_relu"
    normalize: bool = False

    @property
    def cells(self) -> int:
        return self.grid ** 3

    @property
    def cell_updates(self) -> int:
        """One cell-update = one inner-iteration update of one cell of one batch element."""
        return self.batch * self.cells * self.inner * self.outer

    def algorithmic_bytes(self) -> dict:
        """fp32 bytes with every logical tensor of every logical op touched once.

        Per outer step, A = B*G*4 (one activation tensor), P = G*4 (one parameter plane):
        stencil fwd = R x, W y, R 29P; LayerNorm fwd = R, W, R 2P; LayerNorm bwd = R dy, R x,
        W dx, R P, W 2P; stencil bwd = R x, R dy, W dx, R 29P, W 29P.
        """
        a, p = self.batch * self.cells * 4, self.cells * 4
        per = {
            "step_fwd": 2 * a + 29 * p,
            "ln_fwd": 2 * a + 2 * p,
            "ln_bwd": 3 * a + 3 * p,
            "step_bwd": 3 * a + 58 * p,
        }
        fwd = per["step_fwd"] + per["ln_fwd"]
        bwd = per["ln_bwd"] + per["step_bwd"]
        per["total"] = self.outer * (fwd + (bwd if self.backward else 0))
        return per


WORKLOADS = {
    "C1": Workload("C1 16^3 bs8 B2 inner2 outer2 fwd", 16, 8, 2, 2, 2, False),
    "C2": Workload("C2 32^3 bs8 B64 inner4 outer8 fwd", 32, 8, 64, 4, 8, False, zero_bias=True),
    "C3": Workload("C3 64^3 bs8 B32 inner4 outer12 fwd+bwd", 64, 8, 32, 4, 12, True),
    "C4": Workload("C4 128^3 bs8 B8 inner4 outer16 fwd", 128, 8, 8, 4, 16, False, zero_bias=True),
    "C5": Workload("C5 64^3 bs4 B128 inner8 outer16 fwd+bwd", 64, 4, 128, 8, 16, True),
}


def make_inputs(wl: Workload, seed: int = 0, batch: int = None, grid: int = None,
                dtype=torch.float32):
    """CPU tensors: dict(weight, bias, scale, gamma, beta, x0, grad_out)."""
    g = grid or wl.grid
    b = batch if batch is not None else wl.batch
    gen = torch.Generator().manual_seed(seed)
    shape = (g, g, g)
    weight = torch.randn(27, *shape, generator=gen, dtype=dtype) / math.sqrt(27)
    bias = 0.1 * torch.randn(*shape, generator=gen, dtype=dtype)
    if wl.zero_bias:
        bias = torch.zeros_like(bias)
    x0 = torch.randn(b, *shape, generator=gen, dtype=dtype)
    grad_out = torch.randn(b, *shape, generator=gen, dtype=dtype)
    return {
        "weight": weight,
        "bias": bias,
        "scale": torch.ones(*shape, dtype=dtype),
        "gamma": torch.ones(*shape, dtype=dtype),
        "beta": torch.zeros(*shape, dtype=dtype),
        "x0": x0,
        "grad_out": grad_out,
    }
