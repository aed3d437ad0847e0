"""Parameter gradients on SMALL grids (fewer blocks than the chip has CUs), where the batch of a
block is split over several workgroups: every chunk leaves its share in a copy of the gradient
arrays of its own and one kernel adds the copies in chunk order, so the tuned fp32 kernels use no
atomics anywhere and two runs give the same bits.  (The reference scatters with global atomics,
src/gridnet_cuda_kernels.cu:439-449.)

Covered: the plain backward, the gated backward, the fused chain (two-kernel and one-kernel
backward); accumulate against overwrite; a caller that hands over only the required part of the
workspace (the batch is then split less: same result to rounding, still reproducible).
"""

import pytest
import torch

from helpers import ATOL, RTOL, assert_close, make_acts, make_params

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NAMES = ("dweight", "dbias", "dscale", "dx")


def plain_backward(shape, batch, bs, inner, normalize, activation, seed, preset=None, ws_bytes=None):
    from gridnet_amd import native as n

    w, b, r = (t.to(DEV) for t in make_params(shape, seed=seed))
    x = make_acts(batch, shape, seed=seed + 1).to(DEV)
    gy = make_acts(batch, shape, seed=seed + 2).to(DEV)
    M, N, K = shape
    outs = [torch.full_like(t, preset) if preset is not None else torch.empty_like(t) for t in (w, b, r, x)]
    flags = 0 if preset is not None else (n.OVERWRITE_PARAMS | n.OVERWRITE_DX)
    nbytes = ws_bytes or n.lib.gridnet_hip_backward_workspace_bytes(0, batch, M, N, K, inner, bs, int(normalize))
    ws = n.workspace(nbytes, w.device)
    ws.fill_(0x7f)  # scratch contents must not matter
    n.check(n.lib.gridnet_hip_backward(0, w.data_ptr(), b.data_ptr(), r.data_ptr(), x.data_ptr(), gy.data_ptr(),
                                       *[o.data_ptr() for o in outs], batch, M, N, K, inner, bs, 1e-5,
                                       int(normalize), n.activation_id(activation), flags, ws.data_ptr(), nbytes,
                                       n.current_stream(w)))
    torch.cuda.synchronize()
    return [o.cpu() for o in outs]


@pytest.mark.parametrize("shape,batch,bs,inner,normalize,activation", [
    ((16, 16, 16), 8, 8, 3, False, "silu"),        # 8 blocks, 8 chunks of one element
    ((16, 16, 16), 9, 4, 2, False, "leaky_relu"),  # 64 blocks of 4^3, two slots per workgroup
    ((32, 32, 32), 13, 8, 4, False, "tanh"),       # 64 blocks, ragged chunks
    ((16, 8, 24), 6, 8, 2, True, "silu"),          # per-window normalisation
    ((8, 8, 8), 5, 8, 1, False, "relu"),           # a single block
])
def test_plain_backward_is_reproducible_on_small_grids(shape, batch, bs, inner, normalize, activation):
    print(f"reproducible plain backward shape={shape} B={batch} bs={bs} inner={inner} norm={normalize} "
          f"act={activation}", flush=True)
    first = plain_backward(shape, batch, bs, inner, normalize, activation, seed=5)
    again = plain_backward(shape, batch, bs, inner, normalize, activation, seed=5)
    for name, a, b in zip(NAMES, first, again):
        assert torch.isfinite(a).all(), name
        assert torch.equal(a, b), f"{name}: two runs differ"
    # accumulating into preset buffers = the preset plus what an overwriting call gives, bit for bit
    # (the copies are added up first, the old contents last)
    acc = plain_backward(shape, batch, bs, inner, normalize, activation, seed=5, preset=0.25)
    for name, a, b in zip(NAMES, first, acc):
        if name == "dx":  # added to by two kernels in turn: the same sum in another order
            assert_close(b, (a + 0.25).double(), RTOL, ATOL, name)
        else:
            assert torch.equal(a + 0.25, b), f"{name}: accumulate differs from preset + overwrite"


def test_required_part_of_the_workspace_is_enough():
    """With only the D tensor's worth of scratch there is no room for gradient copies: the batch is
    not split, the result is the same to rounding and still reproducible."""
    shape, batch, bs, inner = (16, 16, 16), 8, 8, 3
    full = plain_backward(shape, batch, bs, inner, False, "silu", seed=5)
    need = batch * shape[0] * shape[1] * shape[2] * 4
    small = plain_backward(shape, batch, bs, inner, False, "silu", seed=5, ws_bytes=need)
    again = plain_backward(shape, batch, bs, inner, False, "silu", seed=5, ws_bytes=need)
    for name, a, b, c in zip(NAMES, full, small, again):
        assert torch.equal(b, c), f"{name}: two runs differ"
        assert_close(b, a.double(), RTOL, ATOL, name)
    # room for some copies but not for all the chunks the chip could take: split less
    some = plain_backward(shape, batch, bs, inner, False, "silu", seed=5,
                          ws_bytes=(need + 255) // 256 * 256 + 3 * 31 * 16 ** 3 * 4)
    for name, a, b in zip(NAMES, full, some):
        assert_close(b, a.double(), RTOL, ATOL, name)


@pytest.mark.parametrize("shape,batch,bs,inner", [((16, 16, 16), 7, 8, 2), ((16, 16, 8), 6, 4, 3)])
def test_gated_backward_is_reproducible_on_small_grids(shape, batch, bs, inner):
    import gridnet_cuda

    print(f"reproducible gated backward shape={shape} B={batch} bs={bs} inner={inner}", flush=True)
    g = torch.Generator().manual_seed(11)
    w = (torch.randn(27, 2, *shape, generator=g) / 27 ** 0.5).to(DEV)
    b = (0.1 * torch.randn(2, *shape, generator=g)).to(DEV)
    x = make_acts(batch, shape, seed=12).to(DEV)
    gy = make_acts(batch, shape, seed=13).to(DEV)
    runs = []
    for _ in range(2):
        dw, db, dx = torch.zeros_like(w), torch.zeros_like(b), torch.zeros_like(x)
        gridnet_cuda.backward_gated(w, b, x, gy, dw, db, dx, inner, bs, "tanh")
        torch.cuda.synchronize()
        runs.append((dw.cpu(), db.cpu(), dx.cpu()))
    for name, a, c in zip(("dweight", "dbias", "dx"), *runs):
        assert torch.isfinite(a).all(), name
        assert torch.equal(a, c), f"{name}: two runs differ"


@pytest.mark.parametrize("chain", [False, True])
@pytest.mark.parametrize("shape,batch,bs,inner,outer", [((16, 16, 16), 6, 8, 2, 3), ((32, 32, 32), 5, 8, 4, 2),
                                                        ((16, 16, 16), 10, 4, 3, 2)])
def test_fused_chain_is_reproducible_on_small_grids(shape, batch, bs, inner, outer, chain):
    from gridnet_amd.runner import BodyRunner

    if chain and bs != 8:
        pytest.skip("the one-kernel backward is built for 8^3 blocks")
    print(f"reproducible fused chain shape={shape} B={batch} bs={bs} inner={inner} outer={outer} chain={chain}",
          flush=True)
    w, b, r = make_params(shape, seed=21)
    g = torch.Generator().manual_seed(22)
    gamma, beta = 1 + 0.2 * torch.randn(shape, generator=g), 0.2 * torch.randn(shape, generator=g)
    x0, gy = make_acts(batch, shape, seed=23), make_acts(batch, shape, seed=24)
    runs = []
    for _ in range(2):
        run = BodyRunner(*(v.to(DEV) for v in (w, b, r, gamma, beta)), batch, inner, outer, bs, "silu", False,
                         backward=True, fused=True, chain=chain)
        assert run.chain == chain
        y = run.forward(x0.to(DEV)).clone()
        runs.append([y.cpu()] + [v.clone().cpu() for v in run.backward(gy.to(DEV))])
        del run
    for name, a, c in zip(("y", "dweight", "dbias", "dscale", "dgamma", "dbeta", "dx0"), *runs):
        assert torch.isfinite(a).all(), name
        assert torch.equal(a, c), f"{name}: two runs differ"
