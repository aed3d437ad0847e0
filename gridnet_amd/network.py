"""The body the reference's models repeat: outer step, then LayerNorm, ``outer`` times.

gridnet/scripts/train_mnist.py:62-64 and gridnet/scripts/train_imagenet.py:76-86 (including
the ``outer_residual`` variant ``n = norm(h); h = h + (net(n) - n)``); parameters are shared
across the outer iterations.  Embedding and readout are the callers' business.
"""

import torch
import torch.nn as nn
from torch.autograd.function import once_differentiable


class FusedBodyOp(torch.autograd.Function):
    """The whole loop as ONE autograd node on the entry points that fold the LayerNorm into the
    step kernels (``gridnet_hip_fused_*``): what ``BodyRunner(fused=True)`` does on buffers of
    its own, with torch's autograd around it.  float32, ``normalize=False``, at least one inner
    iteration, shared parameters; other set-ups keep to the op-by-op loop.  Every call owns its
    buffers (the raw outputs of all outer steps are what the backward needs), so several
    forwards may be outstanding before their backwards run."""

    @staticmethod
    def forward(ctx, x0, weight, bias, scale, gamma, beta, inner_iterations, outer_iterations,
                block_size, activation, outer_residual):
        from .runner import BodyRunner

        need_grad = any(ctx.needs_input_grad[:6])
        for name, t in (("weight", weight), ("bias", bias), ("residual_scale", scale),
                        ("norm.weight", gamma), ("norm.bias", beta)):
            if not t.is_contiguous():
                raise RuntimeError(f"{name} must be contiguous")
        run = BodyRunner(weight.detach(), bias.detach(), scale.detach(), gamma.detach(),
                         beta.detach(), x0.shape[0], inner_iterations, outer_iterations, block_size,
                         activation, backward=need_grad, fused=True, outer_residual=outer_residual)
        y = run.forward(x0.detach().contiguous())
        ctx.run = run if need_grad else None
        if need_grad:
            # the runner reads these tensors again in the backward (it recomputes from them):
            # registering them lets autograd refuse a backward after an in-place change, such as
            # an optimizer step taken while this forward was still outstanding
            ctx.save_for_backward(x0, weight, bias, scale, gamma, beta)
        return y

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_out):
        run, ctx.run = ctx.run, None
        if run is None:
            raise RuntimeError("FusedBodyOp: the buffers of this forward were released by its first "
                               "backward; a second backward (retain_graph=True) is not supported")
        ctx.saved_tensors  # raises if an input was modified in place since the forward
        dw, db, dr, dgamma, dbeta, dx0 = run.backward(grad_out.contiguous())
        return dx0, dw, db, dr, dgamma, dbeta, None, None, None, None, None


def fused_body(h, network, norm, outer_iterations: int, outer_residual: bool = False):
    """``outer_iterations`` x (``network``, ``norm``) on ``h`` through :class:`FusedBodyOp`;
    ``network`` a :class:`gridnet_amd.Gridnet` with ``normalize=False``, ``norm`` a
    :class:`gridnet_amd.GridLayerNorm` (their parameters are shared by all iterations)."""
    if network.normalize:
        raise RuntimeError("the fused body covers normalize=False only")
    return FusedBodyOp.apply(h, network.weight, network.bias, network.residual_scale, norm.weight,
                             norm.bias, network.inner_iterations, outer_iterations,
                             network.block_size, network.activation, outer_residual)


class GridnetBody(nn.Module):
    def __init__(self, shape, inner_iterations: int, outer_iterations: int, block_size: int,
                 device, activation: str = "leaky_relu", normalize: bool = False,
                 init_scale: float = 1.0, residual_scale: float = 1.0,
                 outer_residual: bool = False, dtype=None, fused: bool = False):
        super().__init__()

        from . import Gridnet
        from .layernorm import GridLayerNorm

        dtype = dtype or torch.float32
        self.outer_iterations = outer_iterations
        self.outer_residual = outer_residual
        self.fused = fused  # one autograd node over the whole loop, see FusedBodyOp
        self.network = Gridnet(shape, inner_iterations, block_size, device=device, dtype=dtype,
                               init_scale=init_scale, residual_scale=residual_scale,
                               normalize=normalize, activation=activation)
        self.norm = GridLayerNorm(shape, device=device, dtype=dtype)

    def forward(self, h):
        if self.fused:
            return fused_body(h, self.network, self.norm, self.outer_iterations, self.outer_residual)
        for _ in range(self.outer_iterations):
            if self.outer_residual:
                nh = self.norm(h)
                h = h + (self.network(nh) - nh)
            else:
                h = self.norm(self.network(h))
        return h
