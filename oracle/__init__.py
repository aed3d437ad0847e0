"""CPU oracle for the gridnet block-local grid update.

TEST INFRASTRUCTURE ONLY.  Nothing under this package is part of the product:
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import it, and only as the checker.  The shipped op lives in
``gridnet_amd`` and fails loudly when its HIP library is missing; it never
falls back to anything in here.

Modules
-------
ref_style   op-for-op restatement of the reference's pure-torch path
            (gridnet/backend_torch.py:9-142, 270-298): Python loop over blocks,
            gather-built 27-neighbour patches.  This is what the CPU baseline
            times.
fast        block-vectorised equivalent (all blocks at once), fp32/fp64,
            differentiable through torch autograd; used for larger parity cases.
brute       numpy triple loops in fp64, forward only, for tiny grids.
manual      explicit backward formulas (the ones the HIP kernels implement),
            in torch, checked against autograd of ``fast``.
network     the callers' outer loop: step then LayerNorm, ``outer`` times
            (gridnet/scripts/train_mnist.py:62-64, train_imagenet.py:76-86).

Parity pinning: the reference holds no golden vectors for this path (its tests
are differential on unseeded random tensors), and its Python was not imported
or run.  Each function is pinned by closed forms and library routines in
``tests/test_oracle_*.py``: 27 single-tap shift cases, the centre-tap scalar
recurrence, the zero-weight closed form and the zero-iteration identity (both
restated from gridnet/backend_torch_test.py:10-60), conv3d equivalence for
spatially uniform weights, staleness across a block boundary, brute force in
fp64, gradcheck, and ``torch.nn.functional.layer_norm`` for the LayerNorm.
"""
