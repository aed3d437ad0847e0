"""Per-sample LayerNorm over the whole grid on the HIP kernels, as an autograd op.

Stands where the reference's callers use ``torch.nn.LayerNorm((M, N, K))`` between outer
steps (gridnet/scripts/train_mnist.py:54,64; gridnet/scripts/train_imagenet.py:67,86):
biased variance, eps inside the square root, elementwise affine [M, N, K] weight and bias.
"""

import torch
import torch.nn as nn

from . import native as _n


def _launch_forward(x, gamma, beta, eps):
    B = x.shape[0]
    n = x[0].numel() if B else gamma.numel()
    y = torch.empty_like(x)
    mean = torch.empty(B, dtype=x.dtype, device=x.device)
    rstd = torch.empty(B, dtype=x.dtype, device=x.device)
    if B == 0:
        return y, mean, rstd
    dt = _n.dtype_id(x)
    with torch.cuda.device(x.device):
        nbytes = _n.lib.gridnet_hip_layernorm_workspace_bytes(dt, B, n)
        ws = _n.workspace(nbytes, x.device)
        _n.check(_n.lib.gridnet_hip_layernorm_forward(
            dt, x.data_ptr(), gamma.data_ptr(), beta.data_ptr(), y.data_ptr(), mean.data_ptr(),
            rstd.data_ptr(), B, n, float(eps), ws.data_ptr(), nbytes, _n.current_stream(x)))
    return y, mean, rstd


class GridLayerNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, gamma, beta, eps: float):
        for t, name in ((x, "input"), (gamma, "weight"), (beta, "bias")):
            _n.check_input(t, name)
        assert gamma.shape == x.shape[1:] and beta.shape == x.shape[1:], (
            f"affine parameters {tuple(gamma.shape)} do not match sample shape {tuple(x.shape[1:])}")
        assert x.dtype == gamma.dtype == beta.dtype, "mismatching dtypes"
        y, mean, rstd = _launch_forward(x, gamma, beta, eps)
        ctx.save_for_backward(x, gamma, mean, rstd)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, gamma, mean, rstd = ctx.saved_tensors
        dy = dy.contiguous()
        B = x.shape[0]
        n = gamma.numel()
        dx = torch.empty_like(x)
        dgamma = torch.empty_like(gamma)
        dbeta = torch.empty_like(gamma)
        if B == 0:
            return dx, dgamma.zero_(), dbeta.zero_(), None
        dt = _n.dtype_id(x)
        with torch.cuda.device(x.device):
            nbytes = _n.lib.gridnet_hip_layernorm_workspace_bytes(dt, B, n)
            ws = _n.workspace(nbytes, x.device)
            _n.check(_n.lib.gridnet_hip_layernorm_backward(
                dt, dy.data_ptr(), x.data_ptr(), gamma.data_ptr(), mean.data_ptr(),
                rstd.data_ptr(), dx.data_ptr(), dgamma.data_ptr(), dbeta.data_ptr(), B, n,
                _n.OVERWRITE_PARAMS, ws.data_ptr(), nbytes, _n.current_stream(x)))
        return dx, dgamma, dbeta, None


def grid_layer_norm(x, weight, bias, eps: float = 1e-5):
    return GridLayerNormFn.apply(x, weight, bias, eps)


class GridLayerNorm(nn.Module):
    """Same parameters and state-dict keys as ``nn.LayerNorm(shape)``: ``weight``, ``bias``."""

    def __init__(self, shape, eps: float = 1e-5, device=None, dtype=torch.float32):
        super().__init__()
        self.normalized_shape = tuple(shape)
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(*shape, device=device, dtype=dtype))
        self.bias = nn.Parameter(torch.zeros(*shape, device=device, dtype=dtype))

    def forward(self, x):
        return grid_layer_norm(x.contiguous(), self.weight, self.bias, self.eps)
