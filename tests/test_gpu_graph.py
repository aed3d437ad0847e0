"""The network body captured as one HIP graph: every replay must give what the eager calls give.

The C ABI never allocates or synchronises and clears memory with kernels, so a caller may capture
it.  Replays are separated by eager work and synchronisations of the program's own, and the
input changes between them (in place: a graph replays addresses, not values)."""

import pytest
import torch


pytestmark = pytest.mark.gpu
DEV = "cuda:0"


# one_launch: the chain backward as ONE cooperative launch of resident workgroups that signal each
# other through counters in the workspace (cleared by a kernel in front of every launch)
@pytest.mark.parametrize("fused,one_launch", [(False, False), (True, False), (True, True)])
def test_graph_replays_match_eager(fused, one_launch):
    from gridnet_amd.configs import WORKLOADS, make_inputs
    from gridnet_amd.runner import BodyRunner
    import dataclasses

    wl = dataclasses.replace(WORKLOADS["C3"], batch=8 if one_launch else 4, outer=3)
    print(f"graph replay: {wl.name} with batch {wl.batch} outer 3 fused={fused} one_launch={one_launch}", flush=True)
    t = {k: v.to(DEV) for k, v in make_inputs(wl, seed=0).items()}
    run = BodyRunner(t["weight"], t["bias"], t["scale"], t["gamma"], t["beta"], wl.batch, wl.inner,
                     wl.outer, wl.block_size, wl.activation, wl.normalize, backward=True, fused=fused,
                     chain_all=one_launch)
    assert run.chain_all == one_launch
    x0, gy = t["x0"].clone(), t["grad_out"].clone()

    def one_step():
        y = run.forward(x0)
        return (y,) + tuple(run.backward(gy))

    def snapshot(outs):
        return [o.clone() for o in outs]

    one_step()  # set-up done by the first call (kernel attributes, occupancy queries)
    torch.cuda.synchronize()
    side = torch.cuda.Stream(device=DEV)
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        one_step()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            outs = one_step()
    torch.cuda.synchronize()

    gen = torch.Generator().manual_seed(1)
    for rep in range(4):
        x0.copy_(torch.randn(x0.shape, generator=gen).to(DEV))
        gy.copy_(torch.randn(gy.shape, generator=gen).to(DEV))
        torch.cuda.synchronize()
        want = snapshot(one_step())  # eager, on the current stream
        torch.cuda.synchronize()
        for o in outs:
            o.fill_(float("nan"))  # the replay has to produce every output again
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, got, exp in zip(("y", "dweight", "dbias", "dscale", "dgamma", "dbeta", "dx"),
                                  outs, want):
            # every sum has a fixed order (also where the batch is split over workgroups): same bits
            assert torch.equal(got, exp), f"replay {rep}: {name} differs from the eager result"
        assert run.chain_all_status() == 0
