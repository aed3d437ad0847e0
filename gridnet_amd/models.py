"""The step either side of the grid update: embedding an input into the first layers of the
grid, and reading a prediction out of its last layers.

Mirrors of the reference's model classes around the hot path, with the same constructor
arguments, the same forward and the same state-dict keys (so a checkpoint written by the
reference's training scripts loads with ``load_state_dict``):

  ``Readout``            gridnet/__init__.py:102-121
  ``MnistGridModel``     gridnet/scripts/train_mnist.py:14-65   (class ``Model`` there)
  ``ImageNetGridModel``  gridnet/scripts/train_imagenet.py:17-87 (class ``Model`` there)

The grid update and the LayerNorm between outer steps run on the HIP kernels
(``gridnet_amd.Gridnet`` / ``GatedGridnet`` / ``GridLayerNorm``); embedding and readout are
ordinary torch modules, as in the reference.
"""

from typing import Tuple

import torch
import torch.nn as nn

from . import GatedGridnet, Gridnet
from .layernorm import GridLayerNorm
from .network import fused_body


class Readout(nn.Module):
    """LayerNorm + Linear over the last ``output_layers`` K-layers of the grid."""

    def __init__(self, grid_shape: Tuple[int, int, int], out_channels: int, device,
                 dtype=torch.float32, output_layers: int = 1):
        super().__init__()
        size = grid_shape[0] * grid_shape[1] * output_layers
        self.output_layers = output_layers
        self.norm = nn.LayerNorm(size, device=device, dtype=dtype)
        self.proj = nn.Linear(size, out_channels, device=device, dtype=dtype)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        h = x[:, :, :, -self.output_layers:].flatten(1)
        return self.proj(self.norm(h))


class MnistGridModel(nn.Module):
    """28x28 images written into the ``[..., 0]`` face of a learned 32^3 initial grid."""

    def __init__(self, inner_iters: int, outer_iters: int, init_scale: float,
                 residual_scale: float, activation: str, gated: bool, remember_bias: float,
                 device, fused_body: bool = False):
        super().__init__()
        # not in the reference: run the loop as one autograd node on the fused entry points
        if fused_body and gated:
            raise ValueError("the fused body covers the plain (not gated) network only")
        self.fused_body = fused_body
        self.outer_iters = outer_iters
        self.device = device
        self.init_in = nn.Parameter(torch.randn(32, 32, 32, device=device))
        if gated:
            self.network = GatedGridnet((32, 32, 32), inner_iters, 8, init_scale=init_scale,
                                        device=device, activation=activation)
            with torch.no_grad():
                self.network.bias[1].fill_(remember_bias)
        else:
            self.network = Gridnet((32, 32, 32), inner_iters, 8, init_scale=init_scale,
                                   residual_scale=residual_scale, device=device, normalize=False,
                                   activation=activation)
        self.norm = GridLayerNorm((32,) * 3, device=device)
        self.readout = Readout((32, 32, 32), out_channels=10, device=device)

    def embed(self, batch: torch.Tensor) -> torch.Tensor:
        batch = batch.reshape(-1, 28, 28)
        init_acts = self.init_in[None].repeat(batch.shape[0], 1, 1, 1)
        init_acts[:, 2:-2, 2:-2, 0] = batch
        return init_acts

    def forward(self, batch: torch.Tensor) -> torch.Tensor:
        h = self.embed(batch)
        if self.fused_body:
            return self.readout(fused_body(h, self.network, self.norm, self.outer_iters))
        for _ in range(self.outer_iters):
            h = self.norm(self.network(h))
        return self.readout(h)


class ImageNetGridModel(nn.Module):
    """256x256 images patch-embedded into the first ``emb_channels`` K-layers of the grid."""

    def __init__(self, *, inner_iters: int, outer_iters: int, outer_residual: bool,
                 init_scale: float, residual_scale: float, emb_channels: int, grid_size: int,
                 activation: str, separate_params: bool, device, fused_body: bool = False):
        super().__init__()
        assert 256 % grid_size == 0
        # not in the reference: run the loop as one autograd node on the fused entry points
        self.fused_body = fused_body
        self.outer_iters = outer_iters
        self.outer_residual = outer_residual
        self.emb_channels = emb_channels
        self.device = device
        self.init_in = nn.Parameter(torch.randn(grid_size, grid_size, grid_size, device=device))

        def make_model():
            return Gridnet((grid_size,) * 3, inner_iters, 8, init_scale=init_scale,
                           residual_scale=residual_scale, device=device, normalize=False,
                           activation=activation)

        self.separate_params = separate_params
        if separate_params:
            self.networks = nn.ModuleList([make_model() for _ in range(outer_iters)])
        else:
            self.network = make_model()
        self.patch_emb = nn.Conv2d(3, emb_channels, kernel_size=256 // grid_size,
                                   stride=256 // grid_size, device=device)
        self.norm = GridLayerNorm((grid_size,) * 3, device=device)
        self.readout = Readout((grid_size,) * 3, out_channels=1000, device=device)

    def embed(self, images: torch.Tensor) -> torch.Tensor:
        init_acts = self.init_in[None].repeat(images.shape[0], 1, 1, 1)
        init_acts[:, :, :, : self.emb_channels] = self.patch_emb(images).permute(0, 2, 3, 1)
        return init_acts

    def forward(self, images: torch.Tensor) -> torch.Tensor:
        h = self.embed(images)
        if self.fused_body:
            return self.readout(fused_body(h, self.networks if self.separate_params else self.network,
                                           self.norm, self.outer_iters, self.outer_residual))
        for i in range(self.outer_iters):
            net = self.networks[i] if self.separate_params else self.network
            if self.outer_residual:
                norm_h = self.norm(h)
                h = h + (net(norm_h) - norm_h)
            else:
                h = self.norm(net(h))
        return self.readout(h)
