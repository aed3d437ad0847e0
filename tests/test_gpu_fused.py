"""GPU parity of the entry points that fold the LayerNorm into the step kernels
(gridnet_hip_fused_forward / _backward and the LayerNorm pieces beside them): the whole chain
outer x (step, LayerNorm), forward and backward, against the CPU oracle (fp64 evaluation of the
reference's op sequence, gridnet/scripts/train_imagenet.py:76-86) and against the op-by-op
chain of the same library.  Bar: rtol 1e-4 / atol 1e-5."""

import dataclasses

import pytest
import torch

from oracle.network import network_forward, network_forward_backward

from helpers import assert_chain_close, assert_close, inputs_clear_of_kink

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PARAMS = ("weight", "bias", "scale", "gamma", "beta")
NAMES = ("y", "dweight", "dbias", "dscale", "dgamma", "dbeta", "dx0")


def runner_for(wl, t, backward, fused):
    from gridnet_amd.runner import BodyRunner

    d = {k: v.to(DEV) for k, v in t.items()}
    run = BodyRunner(d["weight"], d["bias"], d["scale"], d["gamma"], d["beta"], t["x0"].shape[0],
                     wl.inner, wl.outer, wl.block_size, wl.activation, wl.normalize,
                     backward=backward, fused=fused)
    return run, d


def randomise_affine(t, seed=7):
    """gamma = 1, beta = 0 would hide a mix-up of the two, or of which cell's pair is used."""
    g = torch.Generator().manual_seed(seed)
    t["gamma"] = 1 + 0.2 * torch.randn(t["gamma"].shape, generator=g)
    t["beta"] = 0.2 * torch.randn(t["beta"].shape, generator=g)
    return t


def run_fused(wl, t, backward):
    run, d = runner_for(wl, t, backward, True)
    y = run.forward(d["x0"]).clone()
    if not backward:
        return (y,)
    return (y, *[g.clone() for g in run.backward(d["grad_out"])])


def oracle(wl, t, backward):
    if not backward:
        return (network_forward(*[t[k].double() for k in PARAMS], t["x0"].double(), wl.inner,
                                wl.outer, wl.block_size, wl.activation, wl.normalize),)
    return network_forward_backward(
        [t[k].double() for k in PARAMS], t["x0"].double(), t["grad_out"].double(),
        inner_iterations=wl.inner, outer_iterations=wl.outer, block_size=wl.block_size,
        activation=wl.activation, normalize=wl.normalize)


# leaky_relu (the workloads' own activation) where inputs can be found that keep every
# pre-activation of the chain clear of its kink, silu at the sizes where they cannot
@pytest.mark.parametrize("name,grid,batch,outer,activation", [
    ("C1", 16, 2, 2, None), ("C3", 16, 2, 2, None), ("C5", 16, 1, 2, None), ("C3", 16, 1, 1, None),
    ("C3", 32, 3, 3, "silu"), ("C5", 16, 5, 3, "silu")])
def test_fused_chain_matches_oracle(name, grid, batch, outer, activation):
    from gridnet_amd.configs import WORKLOADS, make_inputs

    wl = dataclasses.replace(WORKLOADS[name], grid=grid, batch=batch, outer=outer, backward=True)
    if activation:
        wl = dataclasses.replace(wl, activation=activation)
    print(f"fused {wl.name} grid={grid} batch={batch} outer={outer} act={wl.activation}", flush=True)

    def make(seed):
        t = randomise_affine(make_inputs(wl, seed=seed))
        if wl.inner >= 8:  # keep 8 residual updates contractive (fp32 rounding otherwise grows)
            t["weight"], t["scale"] = t["weight"] * 0.5, t["scale"] * 0.5
        return t

    t = inputs_clear_of_kink(wl, make)
    assert_chain_close(NAMES, run_fused(wl, t, True), oracle(wl, t, True), t, wl)


@pytest.mark.parametrize("name,grid,batch,outer", [("C2", 32, 4, 3), ("C4", 32, 2, 2)])
def test_fused_forward_only_matches_oracle(name, grid, batch, outer):
    from gridnet_amd.configs import WORKLOADS, make_inputs

    wl = dataclasses.replace(WORKLOADS[name], grid=grid, batch=batch, outer=outer)
    print(f"fused forward {wl.name} grid={grid} batch={batch} outer={outer}", flush=True)
    t = randomise_affine(make_inputs(wl))
    (got,), (exp,) = run_fused(wl, t, False), oracle(wl, t, False)
    assert_close(got, exp, what="y")


@pytest.mark.parametrize("name,grid,batch,outer", [("C3", 32, 3, 3), ("C5", 16, 5, 3), ("C2", 16, 2, 1)])
def test_fused_residual_forward_matches_oracle(name, grid, batch, outer):
    """The outer_residual shape of the loop, n = norm(h); h = h + (net(n) - n)
    (gridnet/scripts/train_imagenet.py:81-83), through gridnet_hip_fused_forward_residual."""
    from gridnet_amd.configs import WORKLOADS, make_inputs
    from gridnet_amd.runner import BodyRunner

    wl = dataclasses.replace(WORKLOADS[name], grid=grid, batch=batch, outer=outer, backward=False)
    print(f"fused residual forward {wl.name} grid={grid} batch={batch} outer={outer}", flush=True)
    t = randomise_affine(make_inputs(wl))
    if wl.inner >= 8:
        t["weight"], t["scale"] = t["weight"] * 0.5, t["scale"] * 0.5
    d = {k: v.to(DEV) for k, v in t.items()}
    run = BodyRunner(d["weight"], d["bias"], d["scale"], d["gamma"], d["beta"], batch, wl.inner,
                     wl.outer, wl.block_size, wl.activation, wl.normalize, backward=False,
                     fused=True, outer_residual=True)
    got = run.forward(d["x0"]).clone()
    exp = network_forward(*[t[k].double() for k in PARAMS], t["x0"].double(), wl.inner, wl.outer,
                          wl.block_size, wl.activation, wl.normalize, outer_residual=True)
    # the result is not normalised: values grow with the number of outer steps
    assert_close(got, exp, what="h")
    assert torch.equal(d["x0"].cpu(), t["x0"]), "the input was modified"


@pytest.mark.parametrize("name,grid,batch,outer,activation", [
    ("C3", 16, 2, 2, None), ("C3", 16, 1, 1, None), ("C5", 16, 1, 2, None),
    ("C3", 32, 3, 3, "silu"), ("C5", 16, 5, 3, "silu"), ("C3", 16, 2, 4, "tanh")])
def test_fused_residual_chain_matches_oracle(name, grid, batch, outer, activation):
    """Forward and backward of the outer_residual shape of the loop through
    gridnet_hip_fused_forward_residual / _backward_residual against autograd of the oracle."""
    from gridnet_amd.configs import WORKLOADS, make_inputs
    from gridnet_amd.runner import BodyRunner

    wl = dataclasses.replace(WORKLOADS[name], grid=grid, batch=batch, outer=outer, backward=True)
    if activation:
        wl = dataclasses.replace(wl, activation=activation)
    print(f"fused residual {wl.name} grid={grid} batch={batch} outer={outer} act={wl.activation}", flush=True)

    def make(seed):
        t = randomise_affine(make_inputs(wl, seed=seed))
        # the result is not normalised: smaller updates keep h (and the gradients) O(1); 8 inner
        # iterations need them smaller still, or fp32 rounding grows past the bar
        f = 0.25 if wl.inner >= 8 else 0.5
        t["weight"], t["scale"] = t["weight"] * f, t["scale"] * f
        return t

    def margin(t):  # smallest |pre-activation| of the oracle chain in this shape of the loop
        from oracle.fast import gridnet_step_fast
        smallest = [float("inf")]

        def step(*args):
            return gridnet_step_fast(*args, watch=lambda u: smallest.__setitem__(
                0, min(smallest[0], u.abs().min().item())))

        with torch.no_grad():
            network_forward(*[t[k].double() for k in PARAMS], t["x0"].double(), wl.inner, wl.outer,
                            wl.block_size, wl.activation, wl.normalize, outer_residual=True, step_fn=step)
        return smallest[0]

    t = make(0)
    if wl.activation in ("relu", "leaky_relu"):
        t = next(c for c in (make(seed) for seed in range(200)) if margin(c) >= 2e-5)
    d = {k: v.to(DEV) for k, v in t.items()}
    run = BodyRunner(d["weight"], d["bias"], d["scale"], d["gamma"], d["beta"], batch, wl.inner,
                     wl.outer, wl.block_size, wl.activation, wl.normalize, backward=True,
                     fused=True, outer_residual=True)
    got = (run.forward(d["x0"]).clone(), *[g.clone() for g in run.backward(d["grad_out"])])
    exp = network_forward_backward(
        [t[k].double() for k in PARAMS], t["x0"].double(), t["grad_out"].double(),
        inner_iterations=wl.inner, outer_iterations=wl.outer, block_size=wl.block_size,
        activation=wl.activation, normalize=wl.normalize, outer_residual=True)
    # Parameter gradients are sums over batch x inner x outer terms, accumulated in fp32 (by the
    # reference's kernels too), and in this shape of the loop the terms do not shrink from step
    # to step: their atol is scaled from the bar's own cases (two terms) by sqrt(terms / 2).
    summed = 1e-5 * max(1.0, (batch * wl.inner * wl.outer / 2) ** 0.5)
    for name_, a, e in zip(NAMES, got, exp):
        assert_close(a, e, atol=1e-5 if name_ in ("y", "dx0") else summed, what=name_)
    assert torch.equal(d["grad_out"].cpu(), t["grad_out"]), "the upstream gradient was modified"
    # twice the same result: nothing is left over from one call to the next
    again = (run.forward(d["x0"]).clone(), *[g.clone() for g in run.backward(d["grad_out"])])
    for name_, a, e in zip(NAMES, again, got):
        assert torch.equal(a, e), f"{name_}: second run differs"


# 4^3 blocks: every row length the row-wise cross-block kernel (csrc/cross_rows.hip) takes: 16, 32,
# 64 and 128 cells, one to eight waves per workgroup; a grid one block wide; (8, 4, 24): a row length
# it leaves to the kernel dealt by block face
@pytest.mark.parametrize("shape,bs,residual", [
    ((8, 16, 24), 8, False), ((24, 8, 16), 8, False),
    ((8, 12, 16), 4, False), ((12, 4, 32), 4, False), ((4, 8, 64), 4, False), ((8, 4, 128), 4, False),
    ((8, 4, 24), 4, False),
    ((4, 12, 32), 4, True), ((8, 8, 64), 4, True), ((12, 8, 16), 4, True), ((8, 16, 24), 8, True)])
def test_fused_chain_non_cubic_grid(shape, bs, residual):
    """Axes of different lengths: catches a swapped stride in the window, face or row indexing."""
    from gridnet_amd.runner import BodyRunner
    from helpers import make_acts, make_params

    inner, outer, batch = 2, 2, 3
    print(f"fused non-cubic shape={shape} bs={bs} residual={residual}", flush=True)
    w, b, r = make_params(shape, seed=21)
    if residual:  # the result is not normalised in this shape of the loop: keep it O(1)
        w, r = w * 0.5, r * 0.5
    g = torch.Generator().manual_seed(3)
    gamma = 1 + 0.2 * torch.randn(shape, generator=g)
    beta = 0.2 * torch.randn(shape, generator=g)
    x0, gy = make_acts(batch, shape, seed=22), make_acts(batch, shape, seed=23)
    run = BodyRunner(*(v.to(DEV) for v in (w, b, r, gamma, beta)), batch, inner, outer, bs,
                     "silu", False, backward=True, fused=True, outer_residual=residual)
    y = run.forward(x0.to(DEV)).clone()
    got = (y, *[v.clone() for v in run.backward(gy.to(DEV))])
    exp = network_forward_backward([v.double() for v in (w, b, r, gamma, beta)], x0.double(),
                                   gy.double(), inner_iterations=inner, outer_iterations=outer,
                                   block_size=bs, activation="silu", normalize=False,
                                   outer_residual=residual)
    summed = 1e-5 * max(1.0, (batch * inner * outer / 2) ** 0.5)
    for name_, a, e in zip(NAMES, got, exp):
        assert_close(a, e, atol=1e-5 if name_ in ("y", "dx0") or not residual else summed, what=name_)


def test_fused_full_size_agrees_with_op_by_op_chain():
    """The graded shape (64^3 grid, 8^3 blocks, inner 4) at full size, where the oracle is too
    slow: the fused chain against the op-by-op chain of the same library (itself checked against
    the oracle on smaller shapes; twice the bar, see below), and bitwise reproducibility of the
    fused chain."""
    from gridnet_amd.configs import WORKLOADS, make_inputs

    # silu: with 12 million pre-activations some land within rounding distance of the kink of
    # leaky_relu, where two fp32 evaluation orders may take different branches and then differ
    # grossly in the gradients without either being wrong
    wl = dataclasses.replace(WORKLOADS["C3"], batch=4, outer=3, activation="silu")
    t = randomise_affine(make_inputs(wl))
    print(f"fused vs op-by-op {wl.name} batch=4 outer=3 silu", flush=True)
    run_s, d = runner_for(wl, t, True, False)
    ys = run_s.forward(d["x0"]).clone()
    gs = [g.clone() for g in run_s.backward(d["grad_out"])]
    first = run_fused(wl, t, True)
    # two fp32 evaluations in different orders, each within the bar of the exact result:
    # twice the bar between them
    for name_, a, e in zip(NAMES, first, (ys, *gs)):
        assert_close(a, e.double().cpu(), rtol=2e-4, atol=2e-5, what=name_)
    again = run_fused(wl, t, True)
    for name_, a, e in zip(NAMES, again, first):
        assert torch.equal(a, e), f"{name_}: fused chain is not bitwise reproducible"


@pytest.mark.parametrize("shape,batch,inner,outer,activation", [
    ((16, 16, 16), 3, 1, 3, "silu"),       # 8 blocks: batch split over workgroups, gradient copies
    ((8, 24, 16), 5, 2, 2, "tanh"),        # non-cubic, a single block along M (no neighbour there)
    ((24, 8, 8), 1, 3, 4, "silu"),         # one sample, blocks in a row
    ((16, 32, 24), 7, 4, 3, "silu"),
    ((64, 64, 64), 2, 4, 3, "silu"),       # 512 blocks: one workgroup per block, no gradient copies:
                                           # plain stores on the last step, read-add-write on the others
    ((64, 64, 64), 2, 4, 2, "leaky_relu"), # the same plan under the workloads' own activation (forward only)
    ((8, 8, 8), 4, 2, 3, "relu"),          # a single block: nothing crosses a boundary
    ((16, 16, 16), 3, 5, 2, "tanh"),       # 5 to 8 inner iterations: the kernels' wide variant (the
    ((16, 24, 8), 2, 8, 3, "silu"),        # history of pre-activations takes the room of table rows)
    ((32, 32, 32), 2, 7, 2, "silu"),
    ((16, 16, 16), 2, 8, 1, "tanh"),
    ((16, 16, 16), 2, 4, 1, "silu"),       # one outer step: the call that finishes dx itself
])
def test_chain_backward_matches_fused_backward(shape, batch, inner, outer, activation):
    """gridnet_hip_chain_backward (what crosses a block boundary travels from step to step, dx of
    every step but the first stays unfinished) against gridnet_hip_fused_backward (every dx
    finished by the cross-block kernel): the same chain both ways, and against the oracle where it
    finishes in seconds."""
    from gridnet_amd.runner import BodyRunner
    from helpers import KINKED, make_acts, make_params

    print(f"chain vs fused backward shape={shape} B={batch} inner={inner} outer={outer} act={activation}",
          flush=True)
    w, b, r = make_params(shape, seed=61)
    if inner >= 7:  # keep that many residual updates contractive (fp32 rounding otherwise grows)
        w, r = w * 0.5, r * 0.5
    g = torch.Generator().manual_seed(62)
    gamma = 1 + 0.2 * torch.randn(shape, generator=g)
    beta = 0.2 * torch.randn(shape, generator=g)
    x0, gy = make_acts(batch, shape, seed=63), make_acts(batch, shape, seed=64)
    results = []
    for chain in (False, True):
        run = BodyRunner(*(v.to(DEV) for v in (w, b, r, gamma, beta)), batch, inner, outer, 8, activation,
                         False, backward=True, fused=True, chain=chain, chain_all=False)
        assert run.chain == chain
        y = run.forward(x0.to(DEV)).clone()
        results.append((y, *[v.clone() for v in run.backward(gy.to(DEV))]))
    big = shape[0] * shape[1] * shape[2] * batch * inner * outer > 300_000
    # two fp32 evaluations in different orders: twice the bar between them; under relu /
    # leaky_relu on millions of cells a few pre-activations sit on the kink, where the order of
    # evaluation decides the branch: the forward result (continuous) is compared there
    kinked_and_big = activation in KINKED and big
    for name_, a, e in zip(NAMES, results[1], results[0]):
        if name_ == "y":
            assert torch.equal(a, e), "the forward is the same kernel"
        elif not kinked_and_big:
            assert_close(a, e.double().cpu(), rtol=2e-4, atol=2e-5, what=name_)
    if not big:
        exp = network_forward_backward([v.double() for v in (w, b, r, gamma, beta)], x0.double(), gy.double(),
                                       inner_iterations=inner, outer_iterations=outer, block_size=8,
                                       activation=activation, normalize=False)
        if activation not in KINKED:
            # parameter gradients are fp32 sums of batch x inner x outer terms: as elsewhere in this
            # file their atol is scaled from the bar's own cases (two terms) by sqrt(terms / 2)
            summed = 1e-5 * max(1.0, (batch * inner * outer / 2) ** 0.5)
            for name_, a, e in zip(NAMES, results[1], exp):
                assert_close(a, e, what=name_, atol=summed if name_ in ("dweight", "dbias", "dscale", "dgamma", "dbeta") else 1e-5)


def test_chain_entry_point_rejects_what_it_does_not_cover():
    from gridnet_amd import native as n

    assert n.lib.gridnet_hip_chain_supported(n.F32, 4, 8, 0) == 1
    assert n.lib.gridnet_hip_chain_supported(n.F32, 8, 8, 0) == 1   # the reference's ImageNet default
    assert n.lib.gridnet_hip_chain_supported(n.F32, 9, 8, 0) == 0   # the LDS holds the history of 8
    assert n.lib.gridnet_hip_chain_supported(n.F32, 4, 4, 0) == 0   # 8^3 blocks only
    assert n.lib.gridnet_hip_chain_supported(n.F64, 4, 8, 0) == 0
    assert n.lib.gridnet_hip_chain_supported(n.F32, 4, 8, 1) == 0
    assert n.lib.gridnet_hip_chain_halo_floats(32, 64, 64, 64, 8) == 32 * 512 * 488
    x = torch.zeros(1, 8, 8, 8, device=DEV)
    p = x.data_ptr()
    args = [p] * 11
    # halo_out without x_stats: an unfinished dx is for a step whose input passes a LayerNorm
    rc = n.lib.gridnet_hip_chain_backward(n.F32, p, p, p, p, p, p, None, p, p, p, p, None, p, p, p, p, p, p,
                                          p, None, 1, 8, 8, 8, 2, 8, 2, 0, p, 1 << 20, n.current_stream(x))
    assert rc != 0 and "halo_out" in n.last_error()
    rc = n.lib.gridnet_hip_chain_backward(n.F32, p, p, p, p, p, p, None, p, p, p, p, None, None, p, p, p, p, p,
                                          p, None, 1, 8, 8, 8, 9, 8, 2, 0, p, 1 << 20, n.current_stream(x))
    assert rc != 0 and "inner" in n.last_error()
    rc = n.lib.gridnet_hip_chain_backward(n.F32, p, p, p, p, p, p, None, p, p, p, p, None, None, p, p, p, p, p,
                                          p, None, 1, 8, 8, 8, 2, 8, 2, 0, p, 0, n.current_stream(x))
    assert rc != 0 and "workspace" in n.last_error()


def test_fused_rejects_what_it_does_not_cover():
    from gridnet_amd import native as n

    x = torch.zeros(1, 8, 8, 8, device=DEV, dtype=torch.float64)
    p = x.data_ptr()
    rc = n.lib.gridnet_hip_fused_forward(n.F64, p, p, p, p, p, p, None, p, p, 1, 8, 8, 8, 1, 8, 1e-5,
                                         0, p, 1 << 20, n.current_stream(x))
    assert rc != 0 and "float32" in n.last_error()
    rc = n.lib.gridnet_hip_fused_forward(n.F32, p, p, p, p, p, p, None, p, p, 1, 8, 8, 8, 0, 8, 1e-5,
                                         0, p, 1 << 20, n.current_stream(x))
    assert rc != 0 and "inner" in n.last_error()
    rc = n.lib.gridnet_hip_fused_forward(n.F32, p, p, p, p, p, p, None, p, p, 1, 8, 8, 8, 1, 8, 1e-5,
                                         0, p, 0, n.current_stream(x))
    assert rc != 0 and "workspace" in n.last_error()


@pytest.mark.parametrize("bs,shape,batch", [(8, (16, 32, 16), 5), (4, (8, 8, 16), 3), (8, (16, 16, 16), 20)])
def test_fused_forward_flags_match_the_plain_entry_points(bs, shape, batch):
    """gridnet_hip_fused_forward_flags: with no flag and with GRIDNET_FUSED_RESIDUAL it is the two
    forward entry points beside it, and the order in which the workgroups take the blocks
    (GRIDNET_FUSED_WALK_REVERSE) changes no bit of the results; unknown flag bits are refused."""
    from gridnet_amd import native as n
    from helpers import make_acts, make_params

    print(f"fused forward flags bs={bs} shape={shape} batch={batch}", flush=True)
    w, b, r = (v.to(DEV) for v in make_params(shape, seed=41))
    g = torch.Generator().manual_seed(42)
    gamma = (1 + 0.2 * torch.randn(shape, generator=g)).to(DEV)
    beta = (0.2 * torch.randn(shape, generator=g)).to(DEV)
    x = make_acts(batch, shape, seed=43).to(DEV)
    flat = x.flatten(1)
    stats = torch.stack([flat.mean(1), 1 / torch.sqrt(flat.var(1, unbiased=False) + 1e-5)], 1).contiguous()
    M, N, K = shape
    ws_bytes = n.lib.gridnet_hip_fused_workspace_bytes(batch, M, N, K, 3, bs, 0)
    ws = n.workspace(ws_bytes, x.device)
    stream = n.current_stream(x)
    act = n.activation_id("silu")

    def call(fn, *flags):
        y, ys = torch.full_like(x, float("nan")), torch.empty(batch, 2, device=DEV)
        n.check(fn(n.dtype_id(x), w.data_ptr(), b.data_ptr(), r.data_ptr(), gamma.data_ptr(), beta.data_ptr(),
                   x.data_ptr(), stats.data_ptr(), y.data_ptr(), ys.data_ptr(), batch, M, N, K, 3, bs, 1e-5, act,
                   *flags, ws.data_ptr(), ws_bytes, stream))
        return y, ys

    for base, flag in ((n.lib.gridnet_hip_fused_forward, 0), (n.lib.gridnet_hip_fused_forward_residual, n.FUSED_RESIDUAL)):
        want = call(base)
        for extra in (0, n.FUSED_WALK_REVERSE):
            got = call(n.lib.gridnet_hip_fused_forward_flags, flag | extra)
            assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]), (flag, extra)
    with pytest.raises(RuntimeError, match="flag"):
        call(n.lib.gridnet_hip_fused_forward_flags, 4)


@pytest.mark.parametrize("shape,bs,batch,residual,activation", [
    ((8, 12, 16), 4, 3, False, "silu"), ((16, 8, 32), 8, 9, False, "silu"), ((8, 16, 64), 8, 5, True, "silu"),
    ((4, 8, 128), 4, 2, True, "silu"), ((16, 16, 32), 8, 20, False, "silu"),
    ((16, 16, 32), 8, 17, False, "tanh"), ((8, 12, 16), 4, 3, False, "leaky_relu"), ((8, 8, 64), 8, 16, True, "tanh")])
def test_fused_chain_with_one_inner_iteration(shape, bs, batch, residual, activation):
    """inner_iterations = 1 (the default of the reference's MNIST script,
    gridnet/scripts/train_mnist.py:77): the forward is a plain stencil over the whole grid and goes by
    whole K-rows (csrc/fwd_rows.hip), with the LayerNorm folded in and in both shapes of the loop;
    rows of 16 to 128 cells, one to eight waves per workgroup, a batch that is split into chunks."""
    from gridnet_amd.runner import BodyRunner
    from helpers import make_acts, make_params

    inner, outer = 1, 3
    print(f"fused chain, one inner iteration: shape={shape} bs={bs} batch={batch} residual={residual} act={activation}", flush=True)
    w, b, r = make_params(shape, seed=51)
    if residual:
        w, r = w * 0.5, r * 0.5
    g = torch.Generator().manual_seed(52)
    gamma = 1 + 0.2 * torch.randn(shape, generator=g)
    beta = 0.2 * torch.randn(shape, generator=g)
    x0, gy = make_acts(batch, shape, seed=53), make_acts(batch, shape, seed=54)
    run = BodyRunner(*(v.to(DEV) for v in (w, b, r, gamma, beta)), batch, inner, outer, bs,
                     activation, False, backward=True, fused=True, outer_residual=residual)
    y = run.forward(x0.to(DEV)).clone()
    got = (y, *[v.clone() for v in run.backward(gy.to(DEV))])
    exp = network_forward_backward([v.double() for v in (w, b, r, gamma, beta)], x0.double(),
                                   gy.double(), inner_iterations=inner, outer_iterations=outer,
                                   block_size=bs, activation=activation, normalize=False,
                                   outer_residual=residual)
    summed = 1e-5 * max(1.0, (batch * inner * outer / 2) ** 0.5)
    for name_, a, e in zip(NAMES, got, exp):
        assert_close(a, e, atol=1e-5 if name_ in ("y", "dx0") else summed, what=name_)
    # forward only, with the walk alternating: the same bits
    fwd = BodyRunner(*(v.to(DEV) for v in (w, b, r, gamma, beta)), batch, inner, outer, bs,
                     activation, False, backward=False, fused=True, outer_residual=residual)
    assert torch.equal(fwd.forward(x0.to(DEV)), y)
