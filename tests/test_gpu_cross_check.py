"""Full-size differential check of the two native implementations against each other.

The tuned fp32 kernels (step_fast.hip) and the generic kernels (step_generic.hip, run here in
fp64) share no device code: different thread mapping, scatter with atomics against gather,
one kernel against two.  Each is held to the CPU oracle on shapes the oracle finishes in seconds
(test_gpu_step.py); here they are compared with each other on the SAME fp32 inputs at the
benchmark's full shapes, where the oracle is out of reach.  Bar as everywhere: rtol 1e-4,
atol 1e-5 against the fp64 result for y and dx.  Parameter gradients are sums over
batch x inner iterations terms, accumulated in fp32 by every implementation (the reference's
kernels included); the rounding of such a sum grows like the square root of the number of terms,
so their atol is scaled from the bar's own cases (batch 2, one or two iterations) by
sqrt(terms / 2): 8e-5 at the graded shape, where 243 of 7 million dweight entries sit between
1e-5 and 4e-5 off."""

import math

import pytest
import torch

from helpers import KINKED, assert_close, make_acts, make_params

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def run(dtype, w, b, r, x, gy, inner, bs, activation, normalize=False):
    from gridnet_amd.backend_cuda import GridnetCudaOp

    leaves = [t.to(device=DEV, dtype=dtype).requires_grad_(True) for t in (w, b, r, x)]
    y = GridnetCudaOp.apply(*leaves, inner, bs, 1e-5, normalize, activation)
    grads = torch.autograd.grad(y, leaves, gy.to(device=DEV, dtype=dtype))
    return (y.detach(), *grads)


CASES = [
    # the graded shape, whole batch: 512 blocks, one workgroup per block owns all 32 samples
    ((64, 64, 64), 8, 4, 32, "leaky_relu", 1.0),
    # bs=4 at the C5 grid (4096 blocks), batch trimmed, its 8 inner iterations (contractive weights)
    ((64, 64, 64), 4, 8, 6, "leaky_relu", 0.5),
    # fewer blocks than CUs: the batch is split over workgroups, one copy of the gradient arrays each
    ((32, 16, 24), 8, 3, 37, "silu", 1.0),
    ((16, 16, 16), 4, 2, 129, "tanh", 1.0),
    # a single sample, and a long thin grid
    ((8, 8, 256), 8, 5, 1, "relu", 1.0),
]


@pytest.mark.parametrize("shape,bs,inner,batch,activation,scale", CASES)
def test_tuned_fp32_against_generic_fp64(shape, bs, inner, batch, activation, scale):
    print(f"cross-check shape={shape} bs={bs} inner={inner} B={batch} act={activation}", flush=True)
    # the benchmark's parameter scales (weights N(0, 1/27)): with N(0, 1) weights four chained
    # updates reach magnitudes where fp32 rounding of near-cancelling sums alone passes atol
    w, b, r = make_params(shape, seed=31)
    w, r = w * scale, r * scale
    x, gy = make_acts(batch, shape, seed=32), make_acts(batch, shape, seed=33)
    fast = run(torch.float32, w, b, r, x, gy, inner, bs, activation)
    slow = run(torch.float64, w, b, r, x, gy, inner, bs, activation)
    assert_close(fast[0], slow[0], what="y")
    for got in fast:
        assert torch.isfinite(got).all()
    if activation in KINKED:
        # Among millions of pre-activations some lie within fp32 rounding distance of the kink,
        # where the two precisions may take different branches of the derivative: the gradients
        # then differ grossly around such a cell without either being wrong.  The forward result
        # is continuous there and was compared above; the gradients are compared under silu.
        activation = "silu"
        fast = run(torch.float32, w, b, r, x, gy, inner, bs, activation)
        slow = run(torch.float64, w, b, r, x, gy, inner, bs, activation)
    summed = 1e-5 * max(1.0, math.sqrt(batch * inner / 2))
    for name, got, want in zip(("y", "dweight", "dbias", "dscale", "dx"), fast, slow):
        assert_close(got, want, atol=summed if name in ("dweight", "dbias", "dscale") else 1e-5,
                     what=name)


@pytest.mark.parametrize("shape,bs,inner,batch", [
    ((64, 64, 64), 8, 4, 32),   # the graded shape with the reference's default normalize=True
    ((64, 64, 64), 4, 3, 5),    # 4096 blocks of 4^3
    ((24, 40, 16), 8, 2, 70),   # fewer blocks than CUs: batch split over workgroups
])
def test_tuned_fp32_against_generic_fp64_normalized(shape, bs, inner, batch):
    """normalize=True at full size (silu, the reference's default activation).  Twice the bar's
    tolerances, as in the sweep of small shapes: the division by (std + eps) and the two window
    sums of the backward double the rounding of a plain step."""
    print(f"cross-check normalized shape={shape} bs={bs} inner={inner} B={batch}", flush=True)
    w, b, r = make_params(shape, seed=41)
    x, gy = make_acts(batch, shape, seed=42), make_acts(batch, shape, seed=43)
    fast = run(torch.float32, w, b, r, x, gy, inner, bs, "silu", True)
    slow = run(torch.float64, w, b, r, x, gy, inner, bs, "silu", True)
    summed = 2e-5 * max(1.0, math.sqrt(batch * inner / 2))
    for name, got, want in zip(("y", "dweight", "dbias", "dscale", "dx"), fast, slow):
        assert torch.isfinite(got).all(), name
        assert_close(got, want, rtol=2e-4, atol=2e-5 if name in ("y", "dx") else summed, what=name)


@pytest.mark.parametrize("shape,bs,inner,batch", [
    ((64, 64, 64), 8, 4, 32),   # one workgroup of 512 threads per block owns the whole batch
    ((64, 64, 64), 4, 3, 5),    # 4096 blocks, two 64-thread slots per workgroup
    ((24, 40, 16), 8, 2, 70),   # fewer blocks than CUs: batch split, one copy of the gradient arrays per chunk
])
def test_gated_tuned_fp32_against_generic_fp64(shape, bs, inner, batch):
    """The gated variant at full size (tanh, the activation the reference's scripts pair it with)."""
    from gridnet_amd.backend_cuda import GatedGridnetCudaOp

    print(f"cross-check gated shape={shape} bs={bs} inner={inner} B={batch}", flush=True)
    gen = torch.Generator().manual_seed(51)
    w = torch.randn(27, 2, *shape, generator=gen) / 27 ** 0.5
    b = 0.1 * torch.randn(2, *shape, generator=gen)
    x, gy = make_acts(batch, shape, seed=52), make_acts(batch, shape, seed=53)

    def call(dtype):
        leaves = [t.to(device=DEV, dtype=dtype).requires_grad_(True) for t in (w, b, x)]
        y = GatedGridnetCudaOp.apply(*leaves, inner, bs, "tanh")
        return (y.detach(), *torch.autograd.grad(y, leaves, gy.to(device=DEV, dtype=dtype)))

    fast, slow = call(torch.float32), call(torch.float64)
    summed = 1e-5 * max(1.0, math.sqrt(batch * inner / 2))
    for name, got, want in zip(("y", "dweight", "dbias", "dx"), fast, slow):
        assert torch.isfinite(got).all(), name
        assert_close(got, want, atol=summed if name in ("dweight", "dbias") else 1e-5, what=name)
