"""gridnet_hip_backward_static -- the backward entry point that takes no workspace and
allocates nothing -- against gridnet_hip_backward, both called through the C ABI.

Two calls in a row on the same GPU, the second on a smaller problem (the static array keeps the
first call's contents).  The kernels sum in a fixed order on every grid (on grids with fewer
blocks than the chip has CUs each chunk of the batch leaves its gradients in a copy of its own,
in the scratch behind the D tensor, and the copies are added in chunk order), so the two entry
points must agree bit for bit as long as both have room for the same number of copies, which the
cases here do.  A problem whose scratch does not fit the array is refused before anything is
enqueued.
"""

import pytest
import torch

from helpers import make_acts, make_params

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def call_pair(shape, batch, bs, inner, normalize, activation, seed):
    """dweight, dbias, dscale, dx from (gridnet_hip_backward, gridnet_hip_backward_static)."""
    from gridnet_amd import native as n

    print(f"no-alloc case shape={shape} B={batch} bs={bs} inner={inner} normalize={normalize} "
          f"act={activation}", flush=True)
    w, b, r = (t.to(DEV) for t in make_params(shape, seed=seed))
    x = make_acts(batch, shape, seed=seed + 1).to(DEV)
    gy = make_acts(batch, shape, seed=seed + 2).to(DEV)
    M, N, K = shape
    act = n.activation_id(activation)
    stream = n.current_stream(w)
    results = []
    for static in (False, True):
        # accumulate mode on preset buffers: the reference's semantics, and a run that ignored
        # its outputs would show
        outs = [torch.full_like(t, 0.25) for t in (w, b, r, x)]
        args = [0, w.data_ptr(), b.data_ptr(), r.data_ptr(), x.data_ptr(), gy.data_ptr(),
                *[o.data_ptr() for o in outs], batch, M, N, K, inner, bs, 1e-5, int(normalize), act, 0]
        if static:
            n.check(n.lib.gridnet_hip_backward_static(*args, stream))
        else:
            nbytes = n.lib.gridnet_hip_backward_workspace_bytes(0, batch, M, N, K, inner, bs,
                                                                int(normalize))
            assert 0 < nbytes <= n.STATIC_SCRATCH_BYTES
            ws = n.workspace(nbytes, w.device)
            n.check(n.lib.gridnet_hip_backward(*args, ws.data_ptr(), nbytes, stream))
        torch.cuda.synchronize()
        results.append([o.cpu() for o in outs])
    return results


def test_static_scratch_matches_workspace_entry_point_twice():
    from gridnet_amd import native as n

    n.check(n.lib.gridnet_hip_static_init())
    names = ("dweight", "dbias", "dscale", "dx")
    # first call: 512 blocks (every workgroup owns its block's whole batch): bit for bit
    want, got = call_pair((64, 64, 64), 3, 8, 4, False, "leaky_relu", seed=21)
    for name, a, b in zip(names, want, got):
        assert torch.equal(a, b), f"{name}: static-scratch call differs from the workspace call"
    # second call, smaller, into the array the first call left its D tensor in; with
    # normalize=True the scratch also carries the two numbers per (element, block)
    want, got = call_pair((32, 32, 16), 2, 4, 3, True, "silu", seed=31)
    for name, a, b in zip(names, want, got):
        assert torch.equal(a, b), f"{name}: static-scratch call differs from the workspace call"
    # and once more at 8^3 blocks on a grid of few blocks (batch split over workgroups: the copies
    # of the gradient arrays share the static array with the D tensor)
    want, got = call_pair((16, 16, 32), 5, 8, 2, False, "tanh", seed=41)
    for name, a, b in zip(names, want, got):
        assert torch.equal(a, b), f"{name}: static-scratch call differs from the workspace call"


def test_static_scratch_call_matches_the_oracle():
    """The same kernels run behind both entry points, so the comparison above checks the scratch
    plumbing; this one holds a static-scratch call to the hand-derived backward of the oracle
    (oracle/manual.py: the formulas of src/gridnet_cuda_kernels.cu:321-449 in fp64) at the bar."""
    from gridnet_amd import native as n
    from helpers import assert_close
    from oracle.manual import gridnet_step_backward_manual

    shape, batch, inner = (16, 16, 16), 3, 2
    w, b, r = make_params(shape, seed=51)
    x, gy = make_acts(batch, shape, seed=52), make_acts(batch, shape, seed=53)
    d = [t.to(DEV) for t in (w, b, r, x, gy)]
    outs = [torch.empty_like(t) for t in (d[0], d[1], d[2], d[3])]
    n.check(n.lib.gridnet_hip_backward_static(
        0, *[t.data_ptr() for t in d], *[o.data_ptr() for o in outs], batch, *shape, inner, 8, 1e-5, 0,
        n.activation_id("silu"), n.OVERWRITE, n.current_stream(d[0])))
    torch.cuda.synchronize()
    dw, db, dr, dx = gridnet_step_backward_manual(w.double(), b.double(), r.double(), x.double(), gy.double(),
                                                  inner, 8, 1e-5, False, "silu")
    for name, got, exp in zip(("dweight", "dbias", "dscale", "dx"), outs, (dw, db, dr, dx)):
        assert_close(got, exp, what=name)


def test_static_scratch_rejects_what_does_not_fit():
    from gridnet_amd import native as n

    p = torch.zeros(8, device=DEV).data_ptr()  # never dereferenced: the call is refused first
    need = n.lib.gridnet_hip_backward_workspace_bytes(0, 64, 64, 64, 64, 4, 8, 0)
    assert need > n.STATIC_SCRATCH_BYTES
    rc = n.lib.gridnet_hip_backward_static(0, p, p, p, p, p, p, p, p, p, 64, 64, 64, 64, 4, 8, 1e-5,
                                           0, 1, 0, None)
    assert rc == 4 and "static array holds" in n.last_error()
