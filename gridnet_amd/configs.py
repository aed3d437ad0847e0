"""The five benchmark/parity workloads and their seeded synthetic inputs.

Inputs are drawn on the CPU from ``torch.Generator().manual_seed(seed)`` in a fixed order, so
a checker and the device path can be fed identical bits.  Parameter scales follow the
reference's initialisation (gridnet/__init__.py:42-49): weight [27, g, g, g] ~ N(0, 1/27);
bias ~ N(0, 0.01) (std 0.1) or zero; residual_scale = 1; LayerNorm weight 1, bias 0.

The initial grid is N(0, 1) everywhere for the training workloads.  The two image-shaped
workloads build it the way the reference's models do, from a synthetic image written into the
``[..., 0]`` face (gridnet/scripts/train_mnist.py:57-60, train_imagenet.py:70-74) of a grid that is
zero elsewhere, and are read out from the ``[..., -1]`` face by a linear layer (``readout``;
outside the timed region, as embedding is):
  ``mnist``    28x28 single-channel images, uniform [0, 1), flattened and sent through a random
               784 x g^2 projection ~ N(0, 1/784) onto the whole face;
  ``patches``  224x224x3 images ~ N(0, 1) cut into 14x14 patches of 16x16 pixels; every patch
               (768 values) goes through one shared random 768 x t^2 projection ~ N(0, 1/768)
               and fills a t x t tile, t = (g - 2) // 14 (9 at g = 128): 14t x 14t values
               centred in the face.
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
    embed: str = "randn"      # how the initial grid is built: "randn", "mnist" or "patches"
    classes: int = 0          # width of the linear readout from the [..., -1] face (0: none)

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
    "C2": Workload("C2 32^3 bs8 B64 inner4 outer8 fwd", 32, 8, 64, 4, 8, False, zero_bias=True,
                   embed="mnist", classes=10),
    "C3": Workload("C3 64^3 bs8 B32 inner4 outer12 fwd+bwd", 64, 8, 32, 4, 12, True),
    "C4": Workload("C4 128^3 bs8 B8 inner4 outer16 fwd", 128, 8, 8, 4, 16, False, zero_bias=True,
                   embed="patches", classes=1000),
    "C5": Workload("C5 64^3 bs4 B128 inner8 outer16 fwd+bwd", 64, 4, 128, 8, 16, True),
    # C3 with the inner iteration count of the reference's own ImageNet script
    # (gridnet/scripts/train_imagenet.py:101-104: inner 8, outer 12, grid 64, batch 32)
    "C3i8": Workload("C3i8 64^3 bs8 B32 inner8 outer12 fwd+bwd", 64, 8, 32, 8, 12, True),
    # the defaults of the reference's MNIST script (gridnet/scripts/train_mnist.py:45-53, 74-78):
    # 32^3 grid, 8^3 blocks, batch 256, one inner iteration, 64 outer steps, silu, training
    "M": Workload("M 32^3 bs8 B256 inner1 outer64 fwd+bwd silu", 32, 8, 256, 1, 64, True, activation="silu"),
}


def embed_images(wl: Workload, batch: int, g: int, gen, dtype=torch.float32):
    """(x0, image, projection) for the image-shaped workloads: x0 [batch, g, g, g] is zero but
    for its ``[..., 0]`` face."""
    x0 = torch.zeros(batch, g, g, g, dtype=dtype)
    if wl.embed == "mnist":
        image = torch.rand(batch, 28, 28, generator=gen, dtype=dtype)
        proj = torch.randn(784, g * g, generator=gen, dtype=dtype) / math.sqrt(784)
        x0[..., 0] = (image.flatten(1) @ proj).reshape(batch, g, g)
    elif wl.embed == "patches":
        t = max(1, (g - 2) // 14)
        image = torch.randn(batch, 3, 224, 224, generator=gen, dtype=dtype)
        proj = torch.randn(768, t * t, generator=gen, dtype=dtype) / math.sqrt(768)
        # [B, 3, 14, 16, 14, 16] -> [B, 14, 14, 3*16*16]
        patches = image.reshape(batch, 3, 14, 16, 14, 16).permute(0, 2, 4, 1, 3, 5).reshape(batch, 14, 14, 768)
        tiles = (patches @ proj).reshape(batch, 14, 14, t, t).permute(0, 1, 3, 2, 4).reshape(batch, 14 * t, 14 * t)
        o = (g - 14 * t) // 2
        x0[:, o:o + 14 * t, o:o + 14 * t, 0] = tiles
    else:
        raise ValueError(f"unknown embedding {wl.embed!r}")
    return x0, image, proj


def make_inputs(wl: Workload, seed: int = 0, batch: int = None, grid: int = None,
                dtype=torch.float32):
    """CPU tensors: dict(weight, bias, scale, gamma, beta, x0, grad_out), plus ``readout``
    [g*g, classes] for the workloads that have one."""
    g = grid or wl.grid
    b = batch if batch is not None else wl.batch
    gen = torch.Generator().manual_seed(seed)
    shape = (g, g, g)
    weight = torch.randn(27, *shape, generator=gen, dtype=dtype) / math.sqrt(27)
    bias = 0.1 * torch.randn(*shape, generator=gen, dtype=dtype)
    if wl.zero_bias:
        bias = torch.zeros_like(bias)
    if wl.embed == "randn":
        x0 = torch.randn(b, *shape, generator=gen, dtype=dtype)
    else:
        x0, _, _ = embed_images(wl, b, g, gen, dtype)
    grad_out = torch.randn(b, *shape, generator=gen, dtype=dtype)
    out = {
        "weight": weight,
        "bias": bias,
        "scale": torch.ones(*shape, dtype=dtype),
        "gamma": torch.ones(*shape, dtype=dtype),
        "beta": torch.zeros(*shape, dtype=dtype),
        "x0": x0,
        "grad_out": grad_out,
    }
    if wl.classes:
        out["readout"] = torch.randn(g * g, wl.classes, generator=gen, dtype=dtype) / g
    return out


def read_out(y: torch.Tensor, readout: torch.Tensor) -> torch.Tensor:
    """The linear readout from the ``[..., -1]`` face: [B, g, g, g] -> [B, classes]."""
    return y[..., -1].flatten(1) @ readout
