"""GPU parity of one outer step (forward and all four gradients) against the CPU oracle,
called through the reference's own op interface (GridnetCudaOp.apply -> gridnet_cuda ->
C ABI).  Bar: rtol 1e-4 / atol 1e-5 in fp32 against the oracle evaluated in fp64 on the same
fp32 inputs; fp64 runs are held to 1e-9."""

import pytest
import torch

from oracle.fast import gridnet_step_fast
from oracle.manual import gridnet_step_backward_manual

from helpers import ATOL, RTOL, acts_clear_of_kink, assert_close, make_acts, make_params

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def run_op(w, b, r, x, gy, inner, bs, eps, normalize, activation):
    from gridnet_amd.backend_cuda import GridnetCudaOp

    leaves = [t.to(DEV).requires_grad_(True) for t in (w, b, r, x)]
    y = GridnetCudaOp.apply(*leaves, inner, bs, eps, normalize, activation)
    if gy is None:
        return y.detach().cpu(), None
    grads = torch.autograd.grad(y, leaves, gy.to(DEV))
    return y.detach().cpu(), [g.cpu() for g in grads]


def oracle(w, b, r, x, gy, inner, bs, eps, normalize, activation):
    w, b, r, x = (t.double() for t in (w, b, r, x))
    y = gridnet_step_fast(w, b, r, x, inner, bs, eps, normalize, activation)
    if gy is None:
        return y, None
    grads = gridnet_step_backward_manual(w, b, r, x, gy.double(), inner, bs, eps, normalize,
                                         activation)
    return y, list(grads)


def compare(case, dtype=torch.float32, all_randn=False, rtol=RTOL, atol=ATOL, batch=2):
    shape, bs, inner, normalize, activation = case
    print(f"case shape={shape} bs={bs} inner={inner} normalize={normalize} act={activation} "
          f"dtype={dtype} B={batch}", flush=True)
    w, b, r = make_params(shape, seed=11, dtype=dtype, all_randn=all_randn)
    if inner >= 8:  # keep deep recurrences contractive: fp32 rounding otherwise grows past the bar
        w, r = w * 0.5, r * 0.5
    x = acts_clear_of_kink(w, b, r, batch, shape, inner, bs, 1e-5, normalize, activation, seed=12,
                           dtype=dtype)
    gy = make_acts(batch, shape, seed=13, dtype=dtype)
    y, grads = run_op(w, b, r, x, gy, inner, bs, 1e-5, normalize, activation)
    ey, egrads = oracle(w, b, r, x, gy, inner, bs, 1e-5, normalize, activation)
    assert_close(y, ey, rtol, atol, "y")
    for name, g, e in zip(("dweight", "dbias", "dscale", "dx"), grads, egrads):
        assert_close(g, e, rtol, atol, name)


# the reference's own matrix (gridnet/backend_cuda_test.py:11-17, 64-71), plus more depths
MATRIX = [
    ((16, 16, 16), 8, 2, True, "silu"),
    ((16, 16, 16), 8, 1, True, "silu"),
    ((32, 64, 128), 8, 2, True, "silu"),
    ((32, 64, 128), 4, 2, True, "silu"),
    ((32, 16, 8), 4, 2, False, "silu"),
    ((32, 16, 8), 8, 2, False, "silu"),
    ((16, 16, 16), 8, 2, False, "leaky_relu"),
    ((32, 64, 128), 8, 2, False, "leaky_relu"),
    ((32, 64, 128), 4, 2, False, "leaky_relu"),
    ((16, 8, 24), 8, 4, False, "leaky_relu"),
    ((16, 8, 24), 4, 8, False, "tanh"),
    ((8, 8, 8), 8, 0, False, "relu"),
    ((8, 16, 8), 4, 3, False, "relu"),
    ((8, 16, 8), 8, 5, True, "tanh"),
    ((8, 16, 8), 4, 3, True, "relu"),
    # 4^3 blocks with rows of 16, 32 and 64 cells (the cross-block part is dealt by whole rows there)
    ((4, 4, 16), 4, 2, False, "relu"),
    ((12, 8, 32), 4, 2, False, "silu"),
    ((8, 12, 64), 4, 3, False, "tanh"),
    ((8, 12, 64), 4, 3, True, "tanh"),
    ((16, 8, 32), 8, 2, True, "silu"),
    ((8, 4, 16), 4, 2, True, "relu"),
    # one inner iteration with rows of 16, 32, 64 and 128 cells: the forward is a plain stencil there
    # and goes by whole rows (csrc/fwd_rows.hip), whatever the block size
    ((8, 12, 16), 4, 1, False, "silu"),
    ((16, 8, 32), 8, 1, False, "tanh"),
    ((8, 16, 64), 8, 1, False, "leaky_relu"),
    ((4, 8, 128), 4, 1, False, "relu"),
    # no inner iteration on a grid of several blocks: the gradient passes through unchanged
    ((16, 24, 16), 8, 0, True, "silu"),
    ((8, 16, 8), 4, 0, False, "tanh"),
]


@pytest.mark.parametrize("case", MATRIX, ids=lambda c: "-".join(map(str, c)).replace(" ", ""))
def test_step_parity_fp32(case):
    compare(case)


@pytest.mark.parametrize("case", MATRIX[:6] + MATRIX[9:11] + MATRIX[-2:],
                         ids=lambda c: "-".join(map(str, c)).replace(" ", ""))
def test_step_parity_fp64(case):
    compare(case, dtype=torch.float64, rtol=1e-9, atol=1e-9)


@pytest.mark.parametrize("case", MATRIX[:6], ids=lambda c: "-".join(map(str, c)).replace(" ", ""))
def test_reference_matrix_at_reference_bounds(case):
    """All-N(0,1) parameters as in gridnet/backend_cuda_test.py:25-36: values reach the
    hundreds, so the reference's own absolute bound (2e-4) is applied relative to scale."""
    shape, bs, inner, normalize, activation = case
    w, b, r = make_params(shape, seed=21, all_randn=True)
    x = make_acts(2, shape, seed=22)
    y, _ = run_op(w, b, r, x, None, inner, bs, 1e-5, normalize, activation)
    ey, _ = oracle(w, b, r, x, None, inner, bs, 1e-5, normalize, activation)
    scale = max(1.0, ey.abs().max().item())
    assert (y.double() - ey).abs().max().item() < 2e-4 * scale


@pytest.mark.parametrize("batch", [1, 3, 33])
@pytest.mark.parametrize("bs", [4, 8])
def test_batch_sizes(batch, bs):
    compare(((16, 8, 8), bs, 2, False, "leaky_relu"), batch=batch)


@pytest.mark.parametrize("normalize", [False, True], ids=["plain", "normalize"])
@pytest.mark.parametrize("bs", [8, 4])
@pytest.mark.parametrize("inner", [16, 32])
def test_deep_inner_iterations(inner, bs, normalize):
    # small weights keep 32 residual updates tame: with larger ones the 27-term fp32 sums of 32
    # chained iterations leave single entries of dweight a few 1e-6 past the bar
    shape = (8, 8, 16)
    w, b, r = make_params(shape, seed=3)
    w, r = w * 0.25, r * 0.2
    x, gy = make_acts(2, shape, seed=4), make_acts(2, shape, seed=5)
    y, grads = run_op(w, b, r, x, gy, inner, bs, 1e-5, normalize, "tanh")
    ey, eg = oracle(w, b, r, x, gy, inner, bs, 1e-5, normalize, "tanh")
    # with normalize every iteration divides by (std + eps) and takes two window sums more
    rtol, atol = (2e-4, 2e-5) if normalize else (RTOL, ATOL)
    assert_close(y, ey, rtol, atol, what="y")
    for name, g, e in zip(("dweight", "dbias", "dscale", "dx"), grads, eg):
        assert_close(g, e, rtol, atol, what=name)


def test_empty_batch_returns_a_clone():
    from gridnet_amd.backend_cuda import GridnetCudaOp

    shape = (8, 8, 8)
    w, b, r = (t.to(DEV) for t in make_params(shape))
    x = torch.zeros(0, *shape, device=DEV)
    y = GridnetCudaOp.apply(w, b, r, x, 2, 8, 1e-5, False, "silu")
    assert y.shape == x.shape


def test_error_paths_raise_like_the_reference():
    import gridnet_cuda
    from gridnet_amd.backend_cuda import GridnetCudaOp

    shape = (8, 8, 8)
    w, b, r = (t.to(DEV) for t in make_params(shape))
    x = make_acts(2, shape).to(DEV)
    with pytest.raises(RuntimeError, match="unknown activation function: gelu"):
        GridnetCudaOp.apply(w, b, r, x, 1, 8, 1e-5, False, "gelu")
    with pytest.raises(RuntimeError, match="initActivations must be contiguous"):
        gridnet_cuda.forward(w, b, r, x.transpose(1, 2), torch.empty_like(x), 1, 8, 1e-5, False,
                             "silu")
    with pytest.raises(RuntimeError, match="bias must be a CUDA tensor"):
        gridnet_cuda.forward(w, b.cpu(), r, x, torch.empty_like(x), 1, 8, 1e-5, False, "silu")
    xg = x.clone().requires_grad_(True)
    y = GridnetCudaOp.apply(w, b, r, xg, 33, 8, 1e-5, False, "tanh")  # forward allows it
    with pytest.raises(RuntimeError, match="cannot backprop through more than 32 inner iterations"):
        y.backward(torch.ones_like(y))


def test_gradient_outputs_are_accumulated_into():
    """The reference adds into the buffers its wrapper zero-fills (gridnet/backend_cuda.py:78-81,
    src/gridnet_cuda_kernels.cu:424-449); prior contents must survive."""
    import gridnet_cuda

    shape, bs = (8, 8, 16), 8
    w, b, r = (t.to(DEV) for t in make_params(shape))
    x, gy = make_acts(2, shape).to(DEV), make_acts(2, shape, seed=9).to(DEV)
    outs = [torch.zeros_like(w), torch.zeros_like(b), torch.zeros_like(b), torch.zeros_like(x)]
    gridnet_cuda.backward(w, b, r, x, gy, *outs, 2, bs, 1e-5, False, "leaky_relu")
    again = [torch.full_like(t, 0.5) for t in outs]
    gridnet_cuda.backward(w, b, r, x, gy, *again, 2, bs, 1e-5, False, "leaky_relu")
    for first, second in zip(outs, again):
        assert torch.allclose(second, first + 0.5, rtol=1e-5, atol=1e-6)


def test_dispatcher_takes_the_hip_path():
    import warnings

    import gridnet_amd

    shape = (8, 8, 8)
    w, b, r = (t.to(DEV) for t in make_params(shape))
    x = make_acts(2, shape).to(DEV)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        y = gridnet_amd.gridnet_step(w, b, r, x, 2, 8, 1e-5, False, "leaky_relu")
    ey = gridnet_step_fast(w.cpu().double(), b.cpu().double(), r.cpu().double(), x.cpu().double(),
                           2, 8, 1e-5, False, "leaky_relu")
    assert_close(y, ey, what="y")


@pytest.mark.parametrize("bs", [8, 4])
def test_largest_grid_the_index_range_allows(bs):
    """424^3 cells: 27 * M * N * K is 4 % below 2^31 (the bound of the 32-bit cell indexing
    inside a sample), and 53^3 = 148 877 blocks (106^3 of side 4) is more than the reference's launch
    geometry can address (gridDim.y <= 65 535, src/gridnet_cuda_kernels.cu:751).  Too large for
    the CPU oracle, so the result is held to the closed form that the oracle tests pin on small
    grids: with positive data relu is the identity with derivative 1, and one inner iteration
    does not depend on the blocks, so with w = 0 except tap 26 = 1
        y = x + r (b + S26 x),   dx = dy + S26^T (r dy),   dW[t] = r dy St x,   db = r dy,
        dr = dy (b + S26 x)
    where St x is x shifted by tap t's offset with zeros outside the grid."""
    import gc

    from gridnet_amd.backend_cuda import GridnetCudaOp

    g = 424
    shape = (g, g, g)
    print(f"largest grid {shape} bs={bs}", flush=True)
    gen = torch.Generator(device=DEV).manual_seed(5)
    w = torch.zeros(27, *shape, device=DEV)
    w[26] = 1.0
    b = torch.rand(shape, device=DEV, generator=gen) + 0.1
    r = torch.rand(shape, device=DEV, generator=gen) + 0.5
    x = torch.rand(1, *shape, device=DEV, generator=gen) + 0.1
    dy = torch.randn(1, *shape, device=DEV, generator=gen)

    def shifted(v, t):  # v[c + off_t], zero outside the grid
        da, db_, dc = t // 9 - 1, (t // 3) % 3 - 1, t % 3 - 1
        out = torch.zeros_like(v)
        src = [slice(max(d, 0), g + min(d, 0)) for d in (da, db_, dc)]
        dst = [slice(max(-d, 0), g + min(-d, 0)) for d in (da, db_, dc)]
        out[(..., *dst)] = v[(..., *src)]
        return out

    leaves = [t.requires_grad_(True) for t in (w, b, r, x)]
    y = GridnetCudaOp.apply(*leaves, 1, bs, 1e-5, False, "relu")
    dw, db, dr, dx = torch.autograd.grad(y, leaves, dy)
    u = b + shifted(x, 26)[0]
    assert_close(y[0, ::7, ::5, ::3], (x[0] + r * u)[::7, ::5, ::3], what="y")
    assert_close(y[0, -1, -1, :], (x[0] + r * u)[-1, -1, :], what="y, last row")  # S26 x = 0 there
    delta = (r * dy[0]).detach()
    assert_close(db[::7, ::5, ::3], delta[::7, ::5, ::3], what="dbias")
    assert_close(dr[::7, ::5, ::3], (dy[0] * u).detach()[::7, ::5, ::3], what="dscale")
    back = torch.zeros_like(delta)
    back[1:, 1:, 1:] = delta[:-1, :-1, :-1]  # S26^T
    assert_close(dx[0, ::7, ::5, ::3], (dy[0] + back)[::7, ::5, ::3], what="dx")
    del back, u
    for t in (0, 1, 13, 25, 26):  # both ends of the plane range, the centre, two more
        want = delta * shifted(x.detach(), t)[0]
        assert_close(dw[t, ::7, ::5, ::3], want[::7, ::5, ::3], what=f"dweight[{t}]")
        # whole planes at the far corner, where the linear index is largest
        assert_close(dw[t, -16:, -16:, -16:], want[-16:, -16:, -16:], what=f"dweight[{t}] corner")
        del want
    del w, dw, leaves, y
    gc.collect()
    torch.cuda.empty_cache()


def test_machine_ceiling_probes_report_sane_figures():
    """libgridnet_probe.so (the figures bench.py quotes beside the vendor peaks; a library of its
    own, not part of the update path): every quantity comes back positive and below what the part
    can do; an unknown quantity is refused."""
    from gridnet_amd import probe as p

    fma, lds, clock, copy = (p.probe(k) for k in ("fma_tfma_per_s", "lds_gb_per_s", "clock_ghz", "copy_gb_per_s"))
    print(f"probes: {fma:.1f} TFMA/s, LDS {lds:.0f} GB/s, {clock:.2f} GHz, copy {copy:.0f} GB/s", flush=True)
    assert 5.0 < fma < 80.0         # 39.3 TFMA/s is the unpacked fp32 peak of 256 CUs at 2.4 GHz
    assert 1.0e4 < lds < 4.0e5
    assert 0.5 < clock < 3.5
    assert 500.0 < copy < 8000.0    # read + write against 8 TB/s
    read = p.probe("read_gb_per_s")
    print(f"        reads alone {read:.0f} GB/s", flush=True)
    assert 500.0 < read < 8000.0
    widths = {k: p.probe(k) for k in p.LDS_WIDTH_PROBES}
    print("LDS pipe cycles per wave-level read:", {k: round(v, 2) for k, v in widths.items()}, flush=True)
    assert all(1.0 < v < 64.0 for v in widths.values())
    assert widths["ds_read_b32"] < widths["ds_read_b128"]
    with pytest.raises(RuntimeError, match="unknown"):
        p.probe_id(99)


@pytest.mark.parametrize("activation", ["silu", "tanh"])
@pytest.mark.parametrize("shape,bs,inner", [((8, 8, 32), 4, 1), ((8, 8, 8), 8, 2), ((8, 8, 8), 4, 3)])
def test_smooth_activations_to_a_few_ulp(activation, shape, bs, inner):
    """The activation and its derivative on their own: with all weights zero every inner iteration
    sees the pre-activation u = bias, so y = x + inner*act(bias) and dbias = inner*act'(bias) for
    residual_scale = 1 and an incoming gradient of ones.  Pre-activations from -100 to 100, dense
    around 0: the kernels' fp32 silu (exp2 and reciprocal instructions with a compensated
    argument) and tanh must stay within a few units in the last place of the fp64 value, where
    the bar of the parity tests (1e-4 relative) would hide a sloppy exponential."""
    n = shape[0] * shape[1] * shape[2]
    g = torch.Generator().manual_seed(5)
    u = torch.cat([torch.linspace(-100, 100, n // 2), 8 * torch.randn(n - n // 2, generator=g)]).float()
    u[:8] = torch.tensor([0.0, -0.0, 1e-30, -1e-30, 87.5, -87.5, 103.9, -103.9])
    b = u.reshape(shape)
    w, r, x = torch.zeros(27, *shape), torch.ones(shape), torch.zeros(1, *shape)
    y, grads = run_op(w, b, r, x, torch.ones(1, *shape), inner, bs, 1e-5, False, activation)
    ud = b.double()
    if activation == "silu":
        s = torch.sigmoid(ud)
        f, d = ud * s, s * (1 + ud * (1 - s))
    else:
        f = torch.tanh(ud)
        d = 1 - f * f
    ulp = 2.0 ** -23
    # 4 ulp of the value.  silu' = s (1 + u (1 - s)) takes 1 - s from an s that is rounded to
    # fp32: 2^-24 |u| s of absolute error comes with the formula, whatever exponential is behind it
    # tanh is formed as (1 - e) / (1 + e), a difference of numbers near 1 when u is near 0 (the
    # reference's 2 sigmoid(2u) - 1, src/activations.h:130, is one too): absolute there
    floor = 2 * ulp if activation == "tanh" else 1e-30
    assert_close(y[0].double() / inner, f, rtol=4 * ulp, atol=floor, what=f"{activation}(u)")
    err = (grads[1].double() / inner - d).abs()
    bound = 4 * ulp * d.abs() + floor
    if activation == "silu":
        bound = bound + 2 * ulp * ud.abs() * s
    assert bool((err <= bound).all()), f"{activation}'(u): worst excess {(err - bound).max().item():.3e}"
