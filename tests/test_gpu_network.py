"""GPU parity of the whole path (outer x (step, LayerNorm), forward and backward) on the
benchmark workloads, plus size-independent properties at the full training shape."""

import dataclasses

import pytest
import torch

from oracle.network import network_forward_backward, network_forward

from helpers import assert_chain_close, assert_close, inputs_clear_of_kink

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PARAMS = ("weight", "bias", "scale", "gamma", "beta")


def runner_for(wl, t, backward=True):
    from gridnet_amd.runner import BodyRunner

    d = {k: v.to(DEV) for k, v in t.items()}
    run = BodyRunner(d["weight"], d["bias"], d["scale"], d["gamma"], d["beta"], t["x0"].shape[0],
                     wl.inner, wl.outer, wl.block_size, wl.activation, wl.normalize,
                     backward=backward)
    return run, d


def check_against_oracle(wl, t, backward):
    print(f"workload {wl.name} batch={t['x0'].shape[0]} grid={t['x0'].shape[1]}", flush=True)
    run, d = runner_for(wl, t, backward)
    y = run.forward(d["x0"]).clone()
    kw = dict(inner_iterations=wl.inner, outer_iterations=wl.outer, block_size=wl.block_size,
              activation=wl.activation, normalize=wl.normalize)
    if not backward:
        want = network_forward(*[t[k].double() for k in PARAMS], t["x0"].double(), wl.inner,
                               wl.outer, wl.block_size, wl.activation, wl.normalize)
        assert_close(y, want, what="y")
        return
    grads = [g.clone() for g in run.backward(d["grad_out"])]
    want = network_forward_backward([t[k].double() for k in PARAMS], t["x0"].double(),
                                    t["grad_out"].double(), **kw)
    names = ("y", "dweight", "dbias", "dscale", "dgamma", "dbeta", "dx0")
    assert_chain_close(names, (y, *grads), want, t, wl)


def test_c1_exact_config_forward_and_backward():
    from gridnet_amd.configs import WORKLOADS, make_inputs

    wl = dataclasses.replace(WORKLOADS["C1"], backward=True)
    check_against_oracle(wl, inputs_clear_of_kink(wl, lambda seed: make_inputs(wl, seed=seed)), True)


# Gradients are compared under leaky_relu (the workloads' own activation) where inputs can be
# found that keep every pre-activation of the chain clear of its kink, and under silu at the
# sizes where they cannot; forward-only workloads need neither (the function is continuous).
@pytest.mark.parametrize("name,grid,batch,outer,activation", [
    ("C2", 32, 4, 3, None), ("C4", 32, 2, 2, None),
    ("C3", 16, 2, 3, None), ("C5", 16, 1, 2, None),
    ("C3", 32, 3, 3, "silu"), ("C5", 16, 5, 2, "silu")])
def test_workload_shapes_reduced(name, grid, batch, outer, activation):
    """The benchmark workloads with their own block size, inner depth and bias, on a
    grid/batch/outer count the CPU oracle finishes in seconds."""
    from gridnet_amd.configs import WORKLOADS, make_inputs

    wl = dataclasses.replace(WORKLOADS[name], grid=grid, batch=batch, outer=outer)
    if activation:
        wl = dataclasses.replace(wl, activation=activation)

    def make(seed):
        t = make_inputs(wl, seed=seed)
        if wl.inner >= 8:  # keep 8 residual updates contractive (fp32 rounding otherwise grows)
            t["weight"] = t["weight"] * 0.5
            t["scale"] = t["scale"] * 0.5
        return t

    t = inputs_clear_of_kink(wl, make) if wl.backward else make(0)
    check_against_oracle(wl, t, wl.backward)


def test_c3_full_grid_one_outer_step():
    """The graded shape at its full 64^3 grid and 8^3 blocks (512 blocks: one workgroup owns
    the whole batch of a block), batch trimmed so that the fp64 oracle stays in seconds."""
    from gridnet_amd.configs import WORKLOADS, make_inputs

    wl = dataclasses.replace(WORKLOADS["C3"], batch=2, outer=1)
    # one step: fp32 rounding moves a pre-activation by ~2e-7, and 2 million of them leave no
    # room for more than ten times that
    t = inputs_clear_of_kink(wl, lambda seed: make_inputs(wl, seed=seed), margin=2e-6)
    check_against_oracle(wl, t, True)


def test_c3_full_size_properties():
    """Full C3 (batch 32, 12 outer steps): bitwise reproducibility of every output, finiteness,
    LayerNorm invariants of the result, and batch independence of y and dx."""
    from gridnet_amd.configs import WORKLOADS, make_inputs

    wl = WORKLOADS["C3"]
    t = make_inputs(wl)
    run, d = runner_for(wl, t)
    y1 = run.forward(d["x0"]).clone()
    g1 = [g.clone() for g in run.backward(d["grad_out"])]
    y2 = run.forward(d["x0"]).clone()
    g2 = [g.clone() for g in run.backward(d["grad_out"])]
    assert torch.equal(y1, y2)
    for a, b in zip(g1, g2):
        assert torch.equal(a, b), "backward is not bitwise reproducible"
        assert torch.isfinite(a).all()
    flat = y1.flatten(1)
    assert flat.mean(1).abs().max().item() < 1e-4          # gamma = 1, beta = 0
    assert (flat.var(1, unbiased=False) - 1).abs().max().item() < 1e-3
    # samples do not interact: the first 4 samples alone give the same y and dx for them
    small = dataclasses.replace(wl, batch=4)
    ts = {k: (v[:4] if k in ("x0", "grad_out") else v) for k, v in t.items()}
    run_s, ds = runner_for(small, ts)
    ys = run_s.forward(ds["x0"]).clone()
    gs = run_s.backward(ds["grad_out"])
    assert torch.equal(ys, y1[:4])
    assert_close(gs[5], g1[5][:4], what="dx0 of a sub-batch")
    # parameter gradients are sums over the batch: zero upstream gradient on all but 4 samples
    masked = d["grad_out"].clone()
    masked[4:] = 0
    run.forward(d["x0"])
    gm = run.backward(masked)
    assert_close(gm[0], gs[0], rtol=1e-4, atol=2e-5, what="dweight restricted to a sub-batch")


def test_zero_weights_closed_form_full_size():
    """w = 0, full C3 step: y = x + T r act(b), whatever the blocking (closed form restated from
    gridnet/backend_torch_test.py:28-60)."""
    import gridnet_amd
    from gridnet_amd.configs import WORKLOADS, make_inputs

    wl = WORKLOADS["C3"]
    t = make_inputs(wl)
    x = t["x0"].to(DEV)
    b, r = t["bias"].to(DEV), torch.full_like(t["bias"], 0.31).to(DEV)
    y = gridnet_amd.gridnet_step(torch.zeros_like(t["weight"]).to(DEV), b, r, x, wl.inner,
                                 wl.block_size, 1e-5, False, "silu")
    want = x + wl.inner * 0.31 * torch.nn.functional.silu(b)
    assert torch.allclose(y, want, rtol=1e-5, atol=1e-5)


def test_graph_replay_matches_eager():
    """The C-ABI calls only enqueue kernels (no allocation, no synchronisation, fill kernels
    instead of memsets), so a captured step replays to the eager result every time."""
    from gridnet_amd.configs import WORKLOADS, make_inputs

    # results are bitwise reproducible (every sum has a fixed order)
    wl = dataclasses.replace(WORKLOADS["C3"], batch=4, outer=2)
    t = make_inputs(wl)
    run, d = runner_for(wl, t)
    y_ref = run.forward(d["x0"]).clone()
    g_ref = [g.clone() for g in run.backward(d["grad_out"])]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        run.forward(d["x0"])
        run.backward(d["grad_out"])
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            y_buf = run.forward(d["x0"])
            g_buf = run.backward(d["grad_out"])
    for _ in range(3):
        for g in g_buf:
            g.fill_(7.0)            # eager work between replays
        y_buf.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_buf, y_ref)
        for a, b in zip(g_buf, g_ref):
            assert torch.equal(a, b)


def test_autograd_body_matches_runner():
    """GridnetBody (autograd ops, torch-managed memory) and BodyRunner (preallocated) agree."""
    from gridnet_amd import GridnetBody
    from gridnet_amd.configs import WORKLOADS, make_inputs

    wl = dataclasses.replace(WORKLOADS["C3"], grid=16, batch=3, outer=2)
    t = make_inputs(wl)
    run, d = runner_for(wl, t)
    y = run.forward(d["x0"]).clone()
    grads = [g.clone() for g in run.backward(d["grad_out"])]
    body = GridnetBody((16, 16, 16), wl.inner, wl.outer, wl.block_size, DEV, wl.activation)
    with torch.no_grad():
        body.network.weight.copy_(d["weight"])
        body.network.bias.copy_(d["bias"])
        body.network.residual_scale.copy_(d["scale"])
    x = d["x0"].clone().requires_grad_(True)
    out = body(x)
    out.backward(d["grad_out"])
    assert_close(out, y, what="y")
    assert_close(body.network.weight.grad, grads[0], what="dweight")
    assert_close(body.norm.weight.grad, grads[3], what="dgamma")
    assert_close(x.grad, grads[5], what="dx0")


@pytest.mark.parametrize("outer_residual", [False, True], ids=["plain", "outer_residual"])
@pytest.mark.parametrize("bs", [8, 4])
def test_fused_autograd_body_matches_op_by_op_body(bs, outer_residual):
    """GridnetBody(fused=True): the loop as one autograd node on the fused entry points, against
    the same module looping over the step and LayerNorm ops; two forwards are outstanding before
    the first backward runs (every call owns its buffers)."""
    from gridnet_amd import GridnetBody

    shape, inner, outer, batch = (16, 16, 8), 2, 3, 5
    print(f"fused autograd body bs={bs} outer_residual={outer_residual}", flush=True)
    torch.manual_seed(5)
    bodies = [GridnetBody(shape, inner, outer, bs, DEV, "silu", outer_residual=outer_residual, fused=f)
              for f in (False, True)]
    with torch.no_grad():
        for p in bodies[0].parameters():
            p.add_(0.1 * torch.randn_like(p))
    bodies[1].load_state_dict(bodies[0].state_dict())
    xs = [torch.randn(batch, *shape, device=DEV) for _ in range(2)]
    gys = [torch.randn(batch, *shape, device=DEV) for _ in range(2)]
    results = []
    for body in bodies:
        leaves = [x.clone().requires_grad_(True) for x in xs]
        outs = [body(leaf) for leaf in leaves]          # both forwards first
        for out, gy in zip(outs, gys):
            out.backward(gy)                            # gradients of the parameters add up
        results.append([o.detach() for o in outs] + [leaf.grad for leaf in leaves] +
                       [p.grad for p in body.parameters()])
    names = ["y0", "y1", "dx0", "dx1"] + [n for n, _ in bodies[0].named_parameters()]
    for name, want, got in zip(names, *results):
        assert_close(got, want, atol=1e-5 if name[0] in "yd" and "." not in name else 4e-5, what=name)
    with torch.no_grad():                               # no graph: nothing is kept for a backward
        assert_close(bodies[1](xs[0]), results[0][0], what="y without grad")


def test_models_with_the_fused_body_match_the_reference_loop():
    from gridnet_amd.models import ImageNetGridModel, MnistGridModel

    torch.manual_seed(6)
    dev = torch.device(DEV)
    print("models with fused_body", flush=True)
    pairs = []
    a = MnistGridModel(2, 2, 1.0, 1.0, "leaky_relu", False, 0.0, dev)
    b = MnistGridModel(2, 2, 1.0, 1.0, "leaky_relu", False, 0.0, dev, fused_body=True)
    pairs.append((a, b, torch.rand(3, 1, 28, 28, device=dev)))
    kw = dict(inner_iters=2, outer_iters=2, outer_residual=True, init_scale=1.0, residual_scale=0.5,
              emb_channels=4, grid_size=16, activation="silu", separate_params=False, device=dev)
    pairs.append((ImageNetGridModel(**kw), ImageNetGridModel(fused_body=True, **kw),
                  torch.randn(2, 3, 256, 256, device=dev)))
    for plain, fused, batch in pairs:
        fused.load_state_dict(plain.state_dict())
        for m in (plain, fused):
            m(batch).square().mean().backward()
        torch.testing.assert_close(fused(batch), plain(batch), rtol=1e-4, atol=1e-5)
        for (name, p), q in zip(plain.named_parameters(), fused.parameters()):
            torch.testing.assert_close(q.grad, p.grad, rtol=1e-3, atol=1e-5, msg=lambda m, n=name: f"{n}: {m}")
    with pytest.raises(ValueError):
        MnistGridModel(2, 2, 1.0, 1.0, "tanh", True, 0.0, dev, fused_body=True)


@pytest.mark.parametrize("outer_residual", [False, True], ids=["plain", "outer_residual"])
def test_fused_body_with_separate_parameters_per_outer_step(outer_residual):
    """The reference's --separate_params (gridnet/scripts/train_imagenet.py:54-58, 76-80): one
    Gridnet per outer iteration.  The fused body takes the list and returns every network's own
    gradients; held to the op-by-op loop of the same model."""
    from gridnet_amd.models import ImageNetGridModel

    torch.manual_seed(8)
    dev = torch.device(DEV)
    print(f"separate_params outer_residual={outer_residual}", flush=True)
    kw = dict(inner_iters=2, outer_iters=3, outer_residual=outer_residual, init_scale=1.0,
              residual_scale=0.5, emb_channels=4, grid_size=16, activation="silu", separate_params=True,
              device=dev)
    plain, fused = ImageNetGridModel(**kw), ImageNetGridModel(fused_body=True, **kw)
    fused.load_state_dict(plain.state_dict())
    weights = [net.weight for net in plain.networks]
    assert not torch.equal(weights[0], weights[1]), "the networks must differ for this to test anything"
    batch = torch.randn(2, 3, 256, 256, device=dev)
    for m in (plain, fused):
        m(batch).square().mean().backward()
    torch.testing.assert_close(fused(batch), plain(batch), rtol=1e-4, atol=1e-5)
    for (name, p), q in zip(plain.named_parameters(), fused.parameters()):
        assert q.grad is not None, name
        torch.testing.assert_close(q.grad, p.grad, rtol=1e-3, atol=1e-5, msg=lambda m, n=name: f"{n}: {m}")


def test_two_streams_in_flight_do_not_disturb_each_other():
    """The library keeps no state between calls and launches on the stream it is given: two
    chains enqueued alternately on two streams (their kernels free to overlap on the device)
    give what each gives alone."""
    from gridnet_amd.configs import WORKLOADS, make_inputs
    from gridnet_amd.runner import BodyRunner

    wl = dataclasses.replace(WORKLOADS["C3"], grid=32, batch=6, outer=3)
    print("two streams", flush=True)
    inputs = [make_inputs(wl, seed=s) for s in (0, 1)]
    dev = torch.device(DEV)

    def build(t, fused):
        d = {k: v.to(dev) for k, v in t.items()}
        return BodyRunner(d["weight"], d["bias"], d["scale"], d["gamma"], d["beta"], wl.batch, wl.inner,
                          wl.outer, wl.block_size, "silu", backward=True, fused=fused), d

    alone = []
    for t, fused in zip(inputs, (True, False)):
        run, d = build(t, fused)
        y = run.forward(d["x0"]).clone()
        alone.append([y] + [g.clone() for g in run.backward(d["grad_out"])])
    torch.cuda.synchronize()

    runs = [build(t, fused) for t, fused in zip(inputs, (True, False))]
    streams = [torch.cuda.Stream(device=dev) for _ in runs]
    for st in streams:
        st.wait_stream(torch.cuda.current_stream(dev))
    outs = [None, None]
    for rep in range(3):  # several rounds, so that the two really are in flight together
        for i, ((run, d), st) in enumerate(zip(runs, streams)):
            with torch.cuda.stream(st):
                y = run.forward(d["x0"])
                outs[i] = [y] + list(run.backward(d["grad_out"]))
    torch.cuda.synchronize()
    for i in range(2):
        for j, (got, want) in enumerate(zip(outs[i], alone[i])):
            # no atomics anywhere (64 blocks < CUs: the batch is split over workgroups, each chunk
            # has its own copy of the gradient arrays): bit for bit the same
            assert torch.equal(got, want), f"stream {i} output {j}"
