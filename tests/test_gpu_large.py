"""Batches whose tensors hold more than 2^31 elements.

The reference indexes with 32 bits (PackedTensorAccessor32, src/gridnet_cuda_kernels.cu:103-107)
and so stops below 2^31 elements per tensor; the library here indexes cells within a sample with
32 bits and samples with 64.  An oracle run of this size is out of reach, so the checks are
properties that hold at any size: a sample's output and input gradient do not depend on the
rest of the batch (the samples past the 2^31st element must come out as they do in a batch of
their own), and parameter gradients are sums over the batch (the whole batch at once = its two
halves accumulated one after the other)."""

import pytest
import torch

from helpers import assert_close, make_params

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SHAPE = (64, 64, 64)
CELLS = 64 ** 3
BATCH = 2 ** 31 // CELLS + 8  # the last 8 samples start past element 2^31
TAIL = slice(BATCH - 8, BATCH)


def need_memory(gib):
    torch.cuda.empty_cache()  # what earlier tests left in torch's cache counts as used
    free, _ = torch.cuda.mem_get_info()
    if free < gib * 2 ** 30:
        pytest.skip(f"needs {gib} GiB of free device memory, {free / 2 ** 30:.0f} GiB are free")


def big_randn(seed, dtype=torch.float32):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return torch.randn(BATCH, *SHAPE, generator=g, device=DEV, dtype=dtype)


def sum_scale(reference):
    """Tolerance for a sum of BATCH terms taken in two different orders."""
    return 2e-5 * reference.abs().max().item() + 1e-6


@pytest.mark.parametrize("bs,normalize,dtype", [
    (8, False, torch.float32), (8, True, torch.float32), (4, False, torch.float32), (4, True, torch.float32),
    (8, False, torch.float64),  # the kernels that serve every dtype and shape
], ids=["bs8", "bs8-normalize", "bs4", "bs4-normalize", "bs8-f64"])
def test_step_past_2_31_elements(bs, normalize, dtype):
    import gridnet_cuda

    need_memory(64 if dtype == torch.float32 else 128)
    inner, act = 2, "silu"
    print(f"large batch: step B={BATCH} bs={bs} normalize={normalize} {dtype}", flush=True)
    w, b, r = (t.to(DEV) for t in make_params(SHAPE, seed=71, dtype=dtype))
    x, gy = big_randn(72, dtype), big_randn(73, dtype)
    assert x.numel() > 2 ** 31
    close = dict(rtol=1e-10, atol=1e-11) if dtype == torch.float64 else {}

    def run(xs, gs, grads=None):
        y = torch.empty_like(xs)
        gridnet_cuda.forward(w, b, r, xs, y, inner, bs, 1e-5, normalize, act)
        dx = torch.zeros_like(xs)
        if grads is None:
            grads = [torch.zeros_like(t) for t in (w, b, r)]
        gridnet_cuda.backward(w, b, r, xs, gs, *grads, dx, inner, bs, 1e-5, normalize, act)
        return y, dx, grads

    y, dx, grads = run(x, gy)
    y_tail, dx_tail, _ = run(x[TAIL].clone(), gy[TAIL].clone())
    assert_close(y[TAIL], y_tail, what="y of the samples past 2^31", **close)
    assert_close(dx[TAIL], dx_tail, what="dx of the samples past 2^31", **close)
    y_head, dx_head, _ = run(x[:8].clone(), gy[:8].clone())
    assert_close(y[:8], y_head, what="y of the first samples", **close)
    assert_close(dx[:8], dx_head, what="dx of the first samples", **close)
    del y, dx, y_tail, dx_tail, y_head, dx_head

    half = BATCH // 2
    _, _, halves = run(x[:half], gy[:half])
    run(x[half:], gy[half:], halves)  # accumulates into what the first half left
    torch.cuda.synchronize()
    for name, whole, parts in zip(("dweight", "dbias", "dscale"), grads, halves):
        assert torch.isfinite(whole).all(), name
        assert_close(whole, parts, rtol=1e-4, atol=sum_scale(parts), what=name)  # two orders of summation


def test_gated_step_past_2_31_elements():
    import gridnet_cuda

    need_memory(64)
    inner, bs, act = 2, 8, "tanh"
    print(f"large batch: gated step B={BATCH}", flush=True)
    g = torch.Generator().manual_seed(74)
    w = (torch.randn(27, 2, *SHAPE, generator=g) / 27 ** 0.5).to(DEV)
    b = (0.1 * torch.randn(2, *SHAPE, generator=g)).to(DEV)
    x, gy = big_randn(75), big_randn(76)

    def run(xs, gs):
        y = torch.empty_like(xs)
        gridnet_cuda.forward_gated(w, b, xs, y, inner, bs, act)
        dw, db, dx = torch.zeros_like(w), torch.zeros_like(b), torch.zeros_like(xs)
        gridnet_cuda.backward_gated(w, b, xs, gs, dw, db, dx, inner, bs, act)
        return y, dx, dw, db

    y, dx, dw, db = run(x, gy)
    y_tail, dx_tail, _, _ = run(x[TAIL].clone(), gy[TAIL].clone())
    torch.cuda.synchronize()
    assert_close(y[TAIL], y_tail, what="y of the samples past 2^31")
    assert_close(dx[TAIL], dx_tail, what="dx of the samples past 2^31")
    assert torch.isfinite(dw).all() and torch.isfinite(db).all()


@pytest.mark.parametrize("fused", [False, True], ids=["steps", "fused"])
def test_chain_past_2_31_elements(fused):
    from gridnet_amd.runner import BodyRunner

    need_memory(140)
    inner, outer, bs = 2, 2, 8
    print(f"large batch: chain B={BATCH} fused={fused}", flush=True)
    w, b, r = (t.to(DEV) for t in make_params(SHAPE, seed=77))
    g = torch.Generator().manual_seed(78)
    gamma = (1 + 0.1 * torch.randn(*SHAPE, generator=g)).to(DEV)
    beta = (0.1 * torch.randn(*SHAPE, generator=g)).to(DEV)
    x, gy = big_randn(79), big_randn(80)

    def run(xs, gs):
        body = BodyRunner(w, b, r, gamma, beta, xs.shape[0], inner, outer, bs, activation="silu", fused=fused)
        y = body.forward(xs).clone()
        grads = body.backward(gs)
        torch.cuda.synchronize()
        return y, grads[-1].clone(), [t.clone() for t in grads[:-1]]

    y, dx, grads = run(x, gy)
    y_tail, dx_tail, _ = run(x[TAIL].clone(), gy[TAIL].clone())
    assert_close(y[TAIL], y_tail, what="result for the samples past 2^31")
    assert_close(dx[TAIL], dx_tail, what="dx0 of the samples past 2^31")
    for name, t in zip(("dweight", "dbias", "dscale", "dgamma", "dbeta"), grads):
        assert torch.isfinite(t).all(), name
