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
    step kernels (``gridnet_hip_fused_*`` / ``gridnet_hip_chain_backward``): what
    ``BodyRunner(fused=True)`` does on buffers of its own, with torch's autograd around it.
    float32, ``normalize=False``, at least one inner iteration; other set-ups keep to the
    op-by-op loop.  ``params`` is one (weight, bias, residual_scale) triple shared by all outer
    steps, or ``outer_iterations`` triples in a row (the reference's ``--separate_params``).
    Every call owns its buffers (the raw outputs of all outer steps are what the backward needs),
    so several forwards may be outstanding before their backwards run."""

    @staticmethod
    def forward(ctx, x0, gamma, beta, inner_iterations, outer_iterations, block_size, activation,
                outer_residual, *params):
        from .runner import BodyRunner

        if len(params) not in (3, 3 * outer_iterations):
            raise ValueError("one (weight, bias, residual_scale) triple, or one per outer step")
        need_grad = any(ctx.needs_input_grad)
        for name, t in [("norm.weight", gamma), ("norm.bias", beta)] + \
                [(("weight", "bias", "residual_scale")[k % 3], t) for k, t in enumerate(params)]:
            if not t.is_contiguous():
                raise RuntimeError(f"{name} must be contiguous")
        detached = [t.detach() for t in params]
        separate = len(params) > 3
        sets = [detached[k::3] for k in range(3)] if separate else detached
        run = BodyRunner(*sets, gamma.detach(), beta.detach(), x0.shape[0], inner_iterations,
                         outer_iterations, block_size, activation, backward=need_grad, fused=True,
                         outer_residual=outer_residual)
        y = run.forward(x0.detach().contiguous())
        ctx.run = run if need_grad else None
        ctx.separate = separate
        if need_grad:
            # the runner reads these tensors again in the backward (it recomputes from them):
            # registering them lets autograd refuse a backward after an in-place change, such as
            # an optimizer step taken while this forward was still outstanding
            ctx.save_for_backward(x0, gamma, beta, *params)
        return y

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_out):
        run, ctx.run = ctx.run, None
        if run is None:
            raise RuntimeError("FusedBodyOp: the buffers of this forward were released by its first "
                               "backward; a second backward (retain_graph=True) is not supported")
        ctx.saved_tensors  # raises if an input was modified in place since the forward
        # checked: the one-launch chain backward reports through a status word whether its bounded
        # waits held (read after a synchronisation; a failed launch is repeated step by step)
        dw, db, dr, dgamma, dbeta, dx0 = run.backward_checked(grad_out.contiguous())
        if ctx.separate:
            grads = [g for triple in zip(dw, db, dr) for g in triple]
        else:
            grads = [dw, db, dr]
        return (dx0, dgamma, dbeta, None, None, None, None, None, *grads)


def fused_body(h, network, norm, outer_iterations: int, outer_residual: bool = False):
    """``outer_iterations`` x (``network``, ``norm``) on ``h`` through :class:`FusedBodyOp`.
    ``network``: a :class:`gridnet_amd.Gridnet` with ``normalize=False`` whose parameters all
    iterations share, or a sequence of ``outer_iterations`` of them (one per iteration, alike
    but for their parameter values); ``norm`` a :class:`gridnet_amd.GridLayerNorm`."""
    nets = list(network) if isinstance(network, (list, tuple, nn.ModuleList)) else [network]
    if len(nets) not in (1, outer_iterations):
        raise ValueError("one network, or one per outer iteration")
    first = nets[0]
    for net in nets:
        if net.normalize:
            raise RuntimeError("the fused body covers normalize=False only")
        if (net.inner_iterations, net.block_size, net.activation) != \
                (first.inner_iterations, first.block_size, first.activation):
            raise ValueError("the networks of a fused body differ only in their parameter values")
    params = [p for net in nets for p in (net.weight, net.bias, net.residual_scale)]
    return FusedBodyOp.apply(h, norm.weight, norm.bias, first.inner_iterations, outer_iterations,
                             first.block_size, first.activation, outer_residual, *params)


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
