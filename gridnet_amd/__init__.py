"""gridnet_amd: the block-local grid update of gridnet on MI355X (gfx950).

Host-side mirror of the part of the reference's Python API that sits on this path
(gridnet/__init__.py:21-64 ``Gridnet``, :124-194 ``gridnet_step``), on top of hand-written
HIP kernels in ``libgridnet_hip.so``.  There is deliberately no CPU implementation and no
fallback in this package: an op that cannot run on the HIP library raises.
"""

import math
from typing import Tuple

import torch
import torch.nn as nn

try:
    from .backend_cuda import GatedGridnetCudaOp, GridnetCudaOp
    from .layernorm import GridLayerNorm, grid_layer_norm
    _IMPORT_ERROR = None
except ImportError as exc:  # library not built yet (``python -m gridnet_amd.build``) or stale
    GridnetCudaOp = GatedGridnetCudaOp = GridLayerNorm = grid_layer_norm = None
    _IMPORT_ERROR = exc

SUPPORTED_BLOCK_SIZES = (4, 8)


def gridnet_step(weight, bias, residual_scale, init_activations, inner_iterations: int,
                 block_size: int, eps: float = 1e-5, normalize: bool = True,
                 activation: str = "silu"):
    """One outer step of the grid update; signature of gridnet/__init__.py:124-134.

    The reference dispatches HIP/CUDA tensors with block_size 4 or 8 to its extension and
    everything else to its pure-torch path.  Only the first branch exists here; the second
    raises, so nothing can silently run off the HIP kernels.
    """
    if GridnetCudaOp is None:
        raise RuntimeError(f"gridnet HIP library is not available: {_IMPORT_ERROR}")
    if weight.device.type != "cuda":
        raise NotImplementedError(
            f"gridnet_amd runs on HIP devices only, got tensors on {weight.device}")
    if block_size not in SUPPORTED_BLOCK_SIZES:
        raise NotImplementedError(
            f"gridnet block_size {block_size} not supported by the HIP kernels (4 or 8)")
    return GridnetCudaOp.apply(weight, bias, residual_scale, init_activations, inner_iterations,
                               block_size, eps, normalize, activation)


def gated_gridnet_step(weight, bias, init_activations, inner_iterations: int, block_size: int,
                       activation: str = "tanh"):
    """Gated outer step; signature of gridnet/__init__.py:197-204.  HIP tensors only."""
    if GatedGridnetCudaOp is None:
        raise RuntimeError(f"gridnet HIP library is not available: {_IMPORT_ERROR}")
    if weight.device.type != "cuda":
        raise NotImplementedError(
            f"gridnet_amd runs on HIP devices only, got tensors on {weight.device}")
    if block_size not in SUPPORTED_BLOCK_SIZES:
        raise NotImplementedError(
            f"gridnet block_size {block_size} not supported by the HIP kernels (4 or 8)")
    return GatedGridnetCudaOp.apply(weight, bias, init_activations, inner_iterations, block_size,
                                    activation)


class GatedGridnet(nn.Module):
    """Parameters and defaults of gridnet/__init__.py:67-99 (same state-dict keys)."""

    def __init__(self, shape: Tuple[int, int, int], inner_iterations: int, block_size: int,
                 device, dtype=torch.float32, init_scale: float = 1.0, activation: str = "tanh"):
        super().__init__()
        self.shape = tuple(shape)
        self.inner_iterations = inner_iterations
        self.block_size = block_size
        self.activation = activation
        self.weight = nn.Parameter(
            torch.randn(27, 2, *shape, device=device, dtype=dtype) * (init_scale / math.sqrt(27)))
        self.bias = nn.Parameter(torch.zeros(2, *shape, device=device, dtype=dtype))
        self.device = device
        self.dtype = dtype

    def forward(self, x):
        return gated_gridnet_step(self.weight, self.bias, x, self.inner_iterations,
                                  self.block_size, self.activation)


class Gridnet(nn.Module):
    """Parameters and defaults of gridnet/__init__.py:21-64 (same state-dict keys)."""

    def __init__(self, shape: Tuple[int, int, int], inner_iterations: int, block_size: int,
                 device, dtype=torch.float32, eps: float = 1e-5, init_scale: float = 1.0,
                 residual_scale: float = 1.0, normalize: bool = True, activation: str = "silu"):
        super().__init__()
        self.shape = tuple(shape)
        self.inner_iterations = inner_iterations
        self.block_size = block_size
        self.eps = eps
        self.normalize = normalize
        self.activation = activation
        self.weight = nn.Parameter(
            torch.randn(27, *shape, device=device, dtype=dtype) * (init_scale / math.sqrt(27)))
        self.bias = nn.Parameter(torch.zeros(*shape, device=device, dtype=dtype))
        self.residual_scale = nn.Parameter(
            torch.ones(*shape, device=device, dtype=dtype) * residual_scale)
        self.device = device
        self.dtype = dtype

    def forward(self, x):
        return gridnet_step(self.weight, self.bias, self.residual_scale, x,
                            self.inner_iterations, self.block_size, self.eps, self.normalize,
                            self.activation)


from .network import FusedBodyOp, GridnetBody, fused_body  # noqa: E402

__all__ = ["gridnet_step", "gated_gridnet_step", "Gridnet", "GatedGridnet", "GridnetCudaOp",
           "GatedGridnetCudaOp", "GridLayerNorm", "grid_layer_norm", "GridnetBody", "FusedBodyOp",
           "fused_body"]
