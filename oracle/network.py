"""The callers' outer loop around the block-local update (CPU oracle).

Test infrastructure (see ``oracle/__init__.py``).  Order of operations from
gridnet/scripts/train_mnist.py:62-64 and gridnet/scripts/train_imagenet.py:76-86:
``h = net(h); h = LayerNorm((M, N, K))(h)`` repeated ``outer`` times with shared
parameters, or with ``outer_residual``: ``n = norm(h); h = h + (net(n) - n)``.
LayerNorm is torch's (biased variance, eps inside the square root, elementwise
affine), gridnet/scripts/train_mnist.py:54.
"""

import torch
import torch.nn.functional as F

from .fast import gridnet_step_fast


def layer_norm_oracle(x, gamma, beta, eps=1e-5):
    """Library routine: per-sample LayerNorm over all grid cells."""
    return F.layer_norm(x, tuple(x.shape[1:]), gamma, beta, eps)


def layer_norm_plain(x, gamma, beta, eps=1e-5):
    """The same from its definition, for pinning conventions (biased var, eps in sqrt)."""
    flat = x.flatten(1)
    mu = flat.mean(1, keepdim=True)
    var = ((flat - mu) ** 2).mean(1, keepdim=True)
    xhat = ((flat - mu) / torch.sqrt(var + eps)).reshape(x.shape)
    return xhat * gamma + beta


def network_forward(
    weight,
    bias,
    residual_scale,
    gamma,
    beta,
    x0,
    inner_iterations: int,
    outer_iterations: int,
    block_size: int,
    activation: str = "leaky_relu",
    normalize: bool = False,
    eps: float = 1e-5,
    ln_eps: float = 1e-5,
    outer_residual: bool = False,
    step_fn=gridnet_step_fast,
):
    h = x0
    for _ in range(outer_iterations):
        if outer_residual:
            nh = layer_norm_oracle(h, gamma, beta, ln_eps)
            h = h + (
                step_fn(weight, bias, residual_scale, nh, inner_iterations, block_size,
                        eps, normalize, activation)
                - nh
            )
        else:
            h = step_fn(weight, bias, residual_scale, h, inner_iterations, block_size,
                        eps, normalize, activation)
            h = layer_norm_oracle(h, gamma, beta, ln_eps)
    return h


def network_forward_backward(params, x0, grad_out, **kw):
    """Forward and autograd backward; ``params`` = (weight, bias, scale, gamma, beta).

    Returns (y, dweight, dbias, dscale, dgamma, dbeta, dx0).
    """
    leaves = [p.detach().clone().requires_grad_(True) for p in params]
    xin = x0.detach().clone().requires_grad_(True)
    y = network_forward(*leaves, xin, **kw)
    grads = torch.autograd.grad(y, leaves + [xin], grad_out)
    return (y.detach(), *grads)


def network_forward_backward_manual(params, x0, grad_out, inner_iterations, outer_iterations,
                                    block_size, activation="leaky_relu", normalize=False, eps=1e-5,
                                    ln_eps=1e-5):
    """The plain loop (``h = norm(net(h))``) forward and backward WITHOUT autograd: the step's
    hand-derived backward and the LayerNorm backward of ``oracle.manual``, step by step in
    reverse.  Same return value as ``network_forward_backward``; it keeps one tensor per outer
    step instead of autograd's graph, which is what lets it run at the benchmark's full sizes."""
    from .manual import gridnet_step_backward_manual, layer_norm_backward_manual

    weight, bias, scale, gamma, beta = params
    inputs, raws = [], []
    h = x0
    with torch.no_grad():
        for _ in range(outer_iterations):
            inputs.append(h)
            raw = gridnet_step_fast(weight, bias, scale, h, inner_iterations, block_size, eps, normalize,
                                    activation)
            raws.append(raw)
            h = layer_norm_plain(raw, gamma, beta, ln_eps)
        y = h
        dw, db, dr = torch.zeros_like(weight), torch.zeros_like(bias), torch.zeros_like(scale)
        dgamma, dbeta = torch.zeros_like(gamma), torch.zeros_like(beta)
        g = grad_out
        for j in reversed(range(outer_iterations)):
            g, dg, dbt, _, _ = layer_norm_backward_manual(g, raws[j], gamma, ln_eps)
            dgamma += dg
            dbeta += dbt
            sw, sb, sr, g = gridnet_step_backward_manual(weight, bias, scale, inputs[j], g, inner_iterations,
                                                         block_size, eps, normalize, activation)
            dw += sw
            db += sb
            dr += sr
            raws[j] = inputs[j] = None
    return y, dw, db, dr, dgamma, dbeta, g
