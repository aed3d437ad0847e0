"""GPU parity of the per-sample LayerNorm kernels against torch.nn.functional.layer_norm
evaluated on the CPU in fp64 (the library routine the reference's callers use)."""

import pytest
import torch
import torch.nn.functional as F

from helpers import assert_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def case(batch, shape, dtype, seed=0, offset=0.0, spread=1.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(batch, *shape, generator=g, dtype=dtype) * spread + offset
    gamma = 1 + 0.3 * torch.randn(shape, generator=g, dtype=dtype)
    beta = 0.2 * torch.randn(shape, generator=g, dtype=dtype)
    dy = torch.randn(batch, *shape, generator=g, dtype=dtype)
    return x, gamma, beta, dy


def reference(x, gamma, beta, dy):
    x, gamma, beta = (t.double().requires_grad_(True) for t in (x, gamma, beta))
    y = F.layer_norm(x, tuple(x.shape[1:]), gamma, beta, 1e-5)
    return (y.detach(), *torch.autograd.grad(y, (x, gamma, beta), dy.double()))


def ours(x, gamma, beta, dy):
    from gridnet_amd import grid_layer_norm

    x, gamma, beta = (t.to(DEV).requires_grad_(True) for t in (x, gamma, beta))
    y = grid_layer_norm(x, gamma, beta, 1e-5)
    return (y.detach().cpu(), *[g.cpu() for g in torch.autograd.grad(y, (x, gamma, beta), dy.to(DEV))])


@pytest.mark.parametrize("batch,shape", [(2, (16, 16, 16)), (3, (32, 32, 32)), (5, (8, 8, 8)),
                                         (32, (64, 64, 64)), (1, (8, 16, 24)), (2, (5, 7, 3))])
def test_layernorm_parity_fp32(batch, shape):
    print(f"layernorm batch={batch} shape={shape}", flush=True)
    args = case(batch, shape, torch.float32)
    for name, a, e in zip(("y", "dx", "dgamma", "dbeta"), ours(*args), reference(*args)):
        assert_close(a, e, what=name)


def test_layernorm_parity_fp64():
    args = case(3, (16, 8, 24), torch.float64)
    for name, a, e in zip(("y", "dx", "dgamma", "dbeta"), ours(*args), reference(*args)):
        assert_close(a, e, 1e-10, 1e-10, name)


def test_layernorm_large_offset_needs_centred_variance():
    """mean 100, spread 0.1: E[x^2]-mean^2 in fp32 would lose every digit of the variance."""
    args = case(2, (32, 32, 32), torch.float32, offset=100.0, spread=0.1)
    got, want = ours(*args), reference(*args)
    assert_close(got[0], want[0], 2e-3, 2e-3, "y")  # x itself carries only ~1e-5 relative


def test_layernorm_is_bitwise_reproducible():
    args = case(4, (16, 16, 16), torch.float32)
    first, second = ours(*args), ours(*args)
    for a, b in zip(first, second):
        assert torch.equal(a, b)


def test_module_matches_torch_module_keys():
    from gridnet_amd import GridLayerNorm

    ours_mod = GridLayerNorm((8, 8, 8), device=DEV)
    theirs = torch.nn.LayerNorm((8, 8, 8))
    assert set(ours_mod.state_dict()) == set(theirs.state_dict())
    assert ours_mod.eps == theirs.eps
