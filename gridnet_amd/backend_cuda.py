"""The autograd boundary of the block-local grid update on HIP devices.

Mirror of the reference's wrapper (gridnet/backend_cuda.py:5-108): same class name, the same
nine positional ``apply`` arguments, the same assertions, the same early ``clone()`` for an
empty batch, the same tensors saved for backward, zero-filled gradient buffers, and the same
nine-tuple returned from ``backward``.  It calls the top-level ``gridnet_cuda`` module exactly
as the reference's file does, so either file works on top of libgridnet_hip.so.
"""

import gridnet_cuda
import torch


class GridnetCudaOp(torch.autograd.Function):
    @staticmethod
    def forward(ctx, weight, bias, residual_scale, init_activations, inner_iters: int,
                block_size: int, eps: float, normalize: bool, activation: str):
        x = init_activations
        batch_size, m, n, k = x.shape
        assert m % block_size == 0 and n % block_size == 0 and k % block_size == 0, (
            f"{block_size=} incompatible with {x.shape=}")
        assert weight.shape == (27, m, n, k), f"{weight.shape=} invalid for {x.shape=}"
        assert bias.shape == weight.shape[1:], f"{bias.shape=} invalid for {weight.shape=}"
        assert bias.shape == residual_scale.shape, (
            f"{bias.shape=} invalid for {residual_scale.shape=}")
        for other, label in ((bias, "bias"), (residual_scale, "residual_scale"),
                             (x, "init_activations")):
            assert weight.dtype == other.dtype, (
                f"mismatching dtypes: {weight.dtype=} {label}.dtype={other.dtype}")
        for other, label in ((bias, "bias"), (residual_scale, "residual_scale"),
                             (x, "init_activations")):
            assert weight.device == other.device, (
                f"mismatching devices: {weight.device=} {label}.device={other.device}")
        if not batch_size:
            return x.clone()
        ctx.save_for_backward(weight, bias, residual_scale, x)
        ctx.inner_iters = inner_iters
        ctx.block_size = block_size
        ctx.eps = eps
        ctx.normalize = normalize
        ctx.activation = activation
        outputs = torch.empty_like(x)
        gridnet_cuda.forward(weight, bias, residual_scale, x, outputs, inner_iters, block_size,
                             eps, normalize, activation)
        return outputs

    @staticmethod
    def backward(ctx, grad_output):
        weight, bias, residual_scale, x = ctx.saved_tensors
        weight_grad = torch.zeros_like(weight)
        bias_grad = torch.zeros_like(bias)
        residual_scale_grad = torch.zeros_like(bias)
        x_grad = torch.zeros_like(x)
        gridnet_cuda.backward(weight, bias, residual_scale, x, grad_output, weight_grad,
                              bias_grad, residual_scale_grad, x_grad, ctx.inner_iters,
                              ctx.block_size, ctx.eps, ctx.normalize, ctx.activation)
        return (weight_grad, bias_grad, residual_scale_grad, x_grad, None, None, None, None, None)


class GatedGridnetCudaOp(torch.autograd.Function):
    """Mirror of gridnet/backend_cuda.py:111-190: six positional ``apply`` arguments."""

    @staticmethod
    def forward(ctx, weight, bias, init_activations, inner_iters: int, block_size: int,
                activation: str):
        x = init_activations
        batch_size, m, n, k = x.shape
        assert m % block_size == 0 and n % block_size == 0 and k % block_size == 0, (
            f"{block_size=} incompatible with {x.shape=}")
        assert weight.shape == (27, 2, m, n, k), f"{weight.shape=} invalid for {x.shape=}"
        assert bias.shape == weight.shape[1:], f"{bias.shape=} invalid for {weight.shape=}"
        assert weight.dtype == bias.dtype, f"mismatching dtypes: {weight.dtype=} {bias.dtype=}"
        assert weight.dtype == x.dtype, f"mismatching dtypes: {weight.dtype=} {x.dtype=}"
        assert weight.device == bias.device, f"mismatching devices: {weight.device=} {bias.device=}"
        assert weight.device == x.device, f"mismatching devices: {weight.device=} {x.device=}"
        if not batch_size:
            return x.clone()
        ctx.save_for_backward(weight, bias, x)
        ctx.inner_iters = inner_iters
        ctx.block_size = block_size
        ctx.activation = activation
        outputs = torch.empty_like(x)
        gridnet_cuda.forward_gated(weight, bias, x, outputs, inner_iters, block_size, activation)
        return outputs

    @staticmethod
    def backward(ctx, grad_output):
        weight, bias, x = ctx.saved_tensors
        weight_grad = torch.zeros_like(weight)
        bias_grad = torch.zeros_like(bias)
        x_grad = torch.zeros_like(x)
        gridnet_cuda.backward_gated(weight, bias, x, grad_output, weight_grad, bias_grad, x_grad,
                                    ctx.inner_iters, ctx.block_size, ctx.activation)
        return (weight_grad, bias_grad, x_grad, None, None, None)
