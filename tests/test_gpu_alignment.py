"""Tensors that start at addresses which are multiples of 4 bytes only.

The reference's kernels read and write element by element (packed accessors,
src/gridnet_cuda_kernels.cu:103-107), so any contiguous tensor is acceptable to them, for
example a view that starts one element into a larger buffer.  The kernels here move 64- and
128-bit vectors; these tests hand every entry point such views for ALL of its tensors and
expect what the same call returns for tensors at the allocator's own (256-byte) alignment."""

import pytest
import torch

from helpers import assert_close, make_acts, make_params

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def odd(t):
    """A contiguous copy of `t` that starts one element into its buffer."""
    buf = torch.empty(t.numel() + 1, dtype=t.dtype, device=DEV)
    view = buf[1:].view(t.shape)
    view.copy_(t)
    assert view.is_contiguous() and view.data_ptr() % 8 == t.element_size() % 8
    return view


def even(t):
    return t.to(DEV).clone()


def step_call(place, w, b, r, x, gy, inner, bs, normalize, activation):
    import gridnet_cuda

    w, b, r, x, gy = (place(t.to(DEV)) for t in (w, b, r, x, gy))
    y = place(torch.full_like(x, float("nan")))
    gridnet_cuda.forward(w, b, r, x, y, inner, bs, 1e-5, normalize, activation)
    outs = [place(torch.zeros_like(t)) for t in (w, b, r, x)]
    gridnet_cuda.backward(w, b, r, x, gy, *outs, inner, bs, 1e-5, normalize, activation)
    torch.cuda.synchronize()
    return [y] + outs


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("normalize", [False, True], ids=["plain", "normalize"])
@pytest.mark.parametrize("bs", [8, 4])
def test_step_with_tensors_at_odd_addresses(bs, normalize, dtype):
    shape, inner, batch = (16, 8, 24), 3, 5
    print(f"odd addresses: step bs={bs} normalize={normalize} {dtype}", flush=True)
    w, b, r = make_params(shape, seed=61, dtype=dtype)
    x, gy = make_acts(batch, shape, seed=62, dtype=dtype), make_acts(batch, shape, seed=63, dtype=dtype)
    want = step_call(even, w, b, r, x, gy, inner, bs, normalize, "silu")
    got = step_call(odd, w, b, r, x, gy, inner, bs, normalize, "silu")
    for name, g, e in zip(("y", "dweight", "dbias", "dscale", "dx"), got, want):
        assert torch.isfinite(g).all(), name
        if dtype == torch.float32:  # same kernels, same order of operations: same bits
            assert torch.equal(g.cpu(), e.cpu()), name
        else:  # the fp64 kernels scatter with atomics
            assert_close(g.cpu(), e.cpu(), what=name)


@pytest.mark.parametrize("bs", [8, 4])
def test_gated_step_with_tensors_at_odd_addresses(bs):
    import gridnet_cuda

    shape, inner, batch = (8, 16, 8), 2, 3
    print(f"odd addresses: gated bs={bs}", flush=True)
    gen = torch.Generator().manual_seed(64)
    w = torch.randn(27, 2, *shape, generator=gen) / 27 ** 0.5
    b = 0.1 * torch.randn(2, *shape, generator=gen)
    x, gy = make_acts(batch, shape, seed=65), make_acts(batch, shape, seed=66)

    def call(place):
        pw, pb, px, pgy = (place(t.to(DEV)) for t in (w, b, x, gy))
        y = place(torch.full_like(px, float("nan")))
        gridnet_cuda.forward_gated(pw, pb, px, y, inner, bs, "tanh")
        outs = [place(torch.zeros_like(t)) for t in (pw, pb, px)]
        gridnet_cuda.backward_gated(pw, pb, px, pgy, *outs, inner, bs, "tanh")
        torch.cuda.synchronize()
        return [y] + outs

    for name, g, e in zip(("y", "dweight", "dbias", "dx"), call(odd), call(even)):
        assert torch.isfinite(g).all(), name
        assert_close(g.cpu(), e.cpu(), what=name)


def test_layernorm_with_tensors_at_odd_addresses():
    from gridnet_amd.layernorm import grid_layer_norm

    shape, batch = (16, 8, 24), 5
    print("odd addresses: layernorm", flush=True)
    x, gy = make_acts(batch, shape, seed=67), make_acts(batch, shape, seed=68)
    gamma, beta = 1 + 0.1 * make_acts(1, shape, seed=69)[0], 0.1 * make_acts(1, shape, seed=70)[0]

    def call(place):
        leaves = [place(t.to(DEV)).requires_grad_(True) for t in (x, gamma, beta)]
        y = grid_layer_norm(*leaves)
        grads = torch.autograd.grad(y, leaves, place(gy.to(DEV)))
        return [y.detach(), *grads]

    for name, g, e in zip(("y", "dx", "dgamma", "dbeta"), call(odd), call(even)):
        assert_close(g.cpu(), e.cpu(), what=name)


def test_fused_chain_with_tensors_at_odd_addresses():
    """The chain with the LayerNorm folded into the step kernels, all buffers one element off."""
    from gridnet_amd.runner import BodyRunner

    shape, bs, inner, outer, batch = (16, 16, 16), 8, 2, 3, 4
    print("odd addresses: fused chain", flush=True)
    w, b, r = make_params(shape, seed=71)
    gamma, beta = 1 + 0.1 * make_acts(1, shape, seed=72)[0], 0.1 * make_acts(1, shape, seed=73)[0]
    x, gy = make_acts(batch, shape, seed=74), make_acts(batch, shape, seed=75)

    def call(place):
        run = BodyRunner(*(place(t.to(DEV)) for t in (w, b, r, gamma, beta)), batch, inner, outer, bs,
                         "silu", backward=True, fused=True)
        if place is odd:  # the workspaces too: four bytes past the allocator's alignment
            for name in ("fw_ws", "fb_ws", "ln_ws", "bw_ws"):
                nbytes = getattr(run, name).numel()
                setattr(run, name, torch.empty(nbytes + 4, dtype=torch.uint8, device=DEV)[4:])
                assert getattr(run, name).data_ptr() % 8 == 4
        y = run.forward(place(x.to(DEV)))
        grads = run.backward(place(gy.to(DEV)))
        torch.cuda.synchronize()
        return [y.clone()] + [g.clone() for g in grads]

    for i, (g, e) in enumerate(zip(call(odd), call(even))):
        assert_close(g.cpu(), e.cpu(), what=f"output {i}")
