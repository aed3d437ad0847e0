"""The body the reference's models repeat: outer step, then LayerNorm, ``outer`` times.

gridnet/scripts/train_mnist.py:62-64 and gridnet/scripts/train_imagenet.py:76-86 (including
the ``outer_residual`` variant ``n = norm(h); h = h + (net(n) - n)``); parameters are shared
across the outer iterations.  Embedding and readout are the callers' business.
"""

import torch.nn as nn


class GridnetBody(nn.Module):
    def __init__(self, shape, inner_iterations: int, outer_iterations: int, block_size: int,
                 device, activation: str = "leaky_relu", normalize: bool = False,
                 init_scale: float = 1.0, residual_scale: float = 1.0,
                 outer_residual: bool = False, dtype=None):
        super().__init__()
        import torch

        from . import Gridnet
        from .layernorm import GridLayerNorm

        dtype = dtype or torch.float32
        self.outer_iterations = outer_iterations
        self.outer_residual = outer_residual
        self.network = Gridnet(shape, inner_iterations, block_size, device=device, dtype=dtype,
                               init_scale=init_scale, residual_scale=residual_scale,
                               normalize=normalize, activation=activation)
        self.norm = GridLayerNorm(shape, device=device, dtype=dtype)

    def forward(self, h):
        for _ in range(self.outer_iterations):
            if self.outer_residual:
                nh = self.norm(h)
                h = h + (self.network(nh) - nh)
            else:
                h = self.norm(self.network(h))
        return h
