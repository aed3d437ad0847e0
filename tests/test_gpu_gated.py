"""GPU parity of the gated op (forward and gradients) against the CPU oracle, through
GatedGridnetCudaOp.apply -> gridnet_cuda.forward_gated/backward_gated -> C ABI.
Matrix of the reference's own gated tests (gridnet/backend_cuda_test.py:39-58, 113-152)."""

import pytest
import torch

from oracle.gated import gated_step_fast

from helpers import assert_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def make(shape, dtype, seed=0, scale=0.25):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(27, 2, *shape, generator=g, dtype=dtype) * scale
    b = torch.randn(2, *shape, generator=g, dtype=dtype)
    x = torch.randn(2, *shape, generator=g, dtype=dtype)
    gy = torch.randn(2, *shape, generator=g, dtype=dtype)
    return w, b, x, gy


@pytest.mark.parametrize("dtype,rtol,atol", [(torch.float32, 1e-4, 1e-5), (torch.float64, 1e-9, 1e-9)])
@pytest.mark.parametrize("shape,bs,inner,activation", [
    ((16, 16, 16), 8, 1, "tanh"), ((16, 16, 16), 8, 2, "tanh"), ((32, 64, 128), 8, 2, "tanh"),
    ((32, 64, 128), 4, 2, "tanh"), ((8, 16, 8), 4, 3, "leaky_relu"), ((8, 8, 16), 8, 4, "silu"),
    ((8, 8, 8), 4, 0, "relu")])
def test_gated_parity(dtype, rtol, atol, shape, bs, inner, activation):
    from gridnet_amd.backend_cuda import GatedGridnetCudaOp

    print(f"gated shape={shape} bs={bs} inner={inner} act={activation} {dtype}", flush=True)
    w, b, x, gy = make(shape, dtype)
    leaves = [t.to(DEV).requires_grad_(True) for t in (w, b, x)]
    y = GatedGridnetCudaOp.apply(*leaves, inner, bs, activation)
    grads = torch.autograd.grad(y, leaves, gy.to(DEV))
    ref = [t.double().requires_grad_(True) for t in (w, b, x)]
    ey = gated_step_fast(*ref, inner, bs, activation)
    egrads = torch.autograd.grad(ey, ref, gy.double(), allow_unused=True)
    egrads = [torch.zeros_like(r) if e is None else e for e, r in zip(egrads, ref)]
    assert_close(y, ey, rtol, atol, "y")
    for name, g, e in zip(("dweight", "dbias", "dx"), grads, egrads):
        assert torch.isfinite(g).all()
        assert_close(g, e, rtol, atol, name)


@pytest.mark.parametrize("inner", [16, 21, 22, 32])
@pytest.mark.parametrize("bs", [8, 4])
def test_gated_deep_inner_iterations(bs, inner):
    """Up to the reference's limit of 32 (src/gridnet_cuda_kernels.cu:925).  With 8^3 blocks the
    tuned backward keeps the history of 21 iterations in LDS; beyond that the generic kernels
    take over, and the results must not show where."""
    from gridnet_amd.backend_cuda import GatedGridnetCudaOp

    print(f"gated deep bs={bs} inner={inner}", flush=True)
    w, b, x, gy = make((8, 8, 16), torch.float32, seed=3, scale=0.1)
    leaves = [t.to(DEV).requires_grad_(True) for t in (w, b, x)]
    y = GatedGridnetCudaOp.apply(*leaves, inner, bs, "tanh")
    grads = torch.autograd.grad(y, leaves, gy.to(DEV))
    ref = [t.double().requires_grad_(True) for t in (w, b, x)]
    ey = gated_step_fast(*ref, inner, bs, "tanh")
    egrads = torch.autograd.grad(ey, ref, gy.double())
    assert_close(y, ey, what="y")
    for name, g, e in zip(("dweight", "dbias", "dx"), grads, egrads):
        assert_close(g, e, atol=1e-5 * max(1.0, (inner / 2) ** 0.5) if name != "dx" else 1e-5, what=name)


def test_gated_dispatcher_and_errors():
    import gridnet_amd
    from gridnet_amd.backend_cuda import GatedGridnetCudaOp

    w, b, x, _ = make((8, 8, 8), torch.float32)
    w, b, x = w.to(DEV), b.to(DEV), x.to(DEV)
    y = gridnet_amd.gated_gridnet_step(w, b, x, 2, 8, "tanh")
    assert_close(y, gated_step_fast(w.cpu().double(), b.cpu().double(), x.cpu().double(), 2, 8, "tanh"))
    with pytest.raises(RuntimeError, match="unknown activation function: gelu"):
        GatedGridnetCudaOp.apply(w, b, x, 1, 8, "gelu")
    with pytest.raises(AssertionError, match="invalid"):
        GatedGridnetCudaOp.apply(w[:, :1], b, x, 1, 8, "tanh")
    xg = x.clone().requires_grad_(True)
    out = GatedGridnetCudaOp.apply(w, b, xg, 33, 8, "tanh")
    with pytest.raises(RuntimeError, match="cannot backprop through more than 32 inner iterations"):
        out.backward(torch.ones_like(out))
