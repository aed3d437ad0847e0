"""Drop-in for the reference's compiled extension module of the same name.

The reference's autograd wrapper does ``import gridnet_cuda`` and calls four positional
functions (gridnet/backend_cuda.py:1,61,82,154,171; bound in src/gridnet_cuda.cpp:188-194).
This module provides them on top of libgridnet_hip.so (hand-written gfx950 kernels) through
ctypes: same argument order, same None return, same RuntimeError texts for the host-checkable
failures.  Launches go to torch's current stream and never synchronise.
"""

import torch

from gridnet_amd import native as _n

__all__ = ["forward", "backward", "forward_gated", "backward_gated"]


def _check_call(named, activations):
    """Host-side checks that the native side relies on.  The reference's binding gets them from
    its typed, sized accessors (``packed_accessor32<scalar_t, N>`` raises on a dtype or rank
    mismatch and bounds every index, src/gridnet_cuda.cpp:103-107); raw pointers do not, and an
    out-of-bounds access on the device is a fault, not an exception.  ``named``: (tensor, name,
    expected shape) triples; every tensor must be a contiguous HIP tensor of the first one's
    dtype and device."""
    ref = named[0][0]
    for t, name, _ in named:
        _n.check_input(t, name)
    if activations.dim() != 4:
        raise RuntimeError(f"initActivations must be [B, M, N, K], got {tuple(activations.shape)}")
    for t, name, shape in named:
        if t.dtype != ref.dtype:
            raise RuntimeError(f"{name} has dtype {t.dtype}, expected {ref.dtype} like {named[0][1]}")
        if t.device != ref.device:
            raise RuntimeError(f"{name} is on {t.device}, expected {ref.device} like {named[0][1]}")
        if tuple(t.shape) != tuple(shape):
            raise RuntimeError(f"{name} has shape {tuple(t.shape)}, expected {tuple(shape)}")


def forward(weight, bias, scale, initActivations, outActivations, innerIterations, blockSize,
            eps, normalize, activation):
    """One outer step; replaces gridnet_forward, src/gridnet_cuda.cpp:61-89."""
    grid, x = tuple(initActivations.shape[1:]), tuple(initActivations.shape)
    _check_call(((weight, "weight", (27, *grid)), (bias, "bias", grid), (scale, "scale", grid),
                 (initActivations, "initActivations", x), (outActivations, "outActivations", x)),
                initActivations)
    act = _n.activation_id(activation)
    B, M, N, K = initActivations.shape
    with torch.cuda.device(weight.device):
        _n.check(_n.lib.gridnet_hip_forward(
            _n.dtype_id(weight), weight.data_ptr(), bias.data_ptr(), scale.data_ptr(),
            initActivations.data_ptr(), outActivations.data_ptr(), B, M, N, K,
            int(innerIterations), int(blockSize), float(eps), int(bool(normalize)), act,
            _n.current_stream(weight)))


def backward(weight, bias, scale, initActivations, outGrads, weightGradOut, biasGradOut,
             scaleGradOut, activationsGradOut, innerIterations, blockSize, eps, normalize,
             activation):
    """Backward of one outer step; replaces gridnet_backward, src/gridnet_cuda.cpp:91-131.

    As in the reference the four gradient outputs are accumulated into (its wrapper hands
    them over zero-filled, gridnet/backend_cuda.py:78-81).
    """
    grid, x = tuple(initActivations.shape[1:]), tuple(initActivations.shape)
    _check_call(((weight, "weight", (27, *grid)), (bias, "bias", grid), (scale, "scale", grid),
                 (initActivations, "initActivations", x), (outGrads, "outGrads", x),
                 (weightGradOut, "weightGradOut", (27, *grid)), (biasGradOut, "biasGradOut", grid),
                 (scaleGradOut, "scaleGradOut", grid), (activationsGradOut, "activationsGradOut", x)),
                initActivations)
    act = _n.activation_id(activation)
    B, M, N, K = initActivations.shape
    dt = _n.dtype_id(weight)
    with torch.cuda.device(weight.device):
        nbytes = _n.lib.gridnet_hip_backward_workspace_bytes(
            dt, B, M, N, K, int(innerIterations), int(blockSize), int(bool(normalize)))
        ws = _n.workspace(nbytes, weight.device)
        _n.check(_n.lib.gridnet_hip_backward(
            dt, weight.data_ptr(), bias.data_ptr(), scale.data_ptr(), initActivations.data_ptr(),
            outGrads.data_ptr(), weightGradOut.data_ptr(), biasGradOut.data_ptr(),
            scaleGradOut.data_ptr(), activationsGradOut.data_ptr(), B, M, N, K,
            int(innerIterations), int(blockSize), float(eps), int(bool(normalize)), act, 0,
            ws.data_ptr(), nbytes, _n.current_stream(weight)))


def forward_gated(weight, bias, initActivations, outActivations, innerIterations, blockSize,
                  activation):
    """Gated outer step; replaces gated_gridnet_forward, src/gridnet_cuda.cpp:133-158."""
    grid, x = tuple(initActivations.shape[1:]), tuple(initActivations.shape)
    _check_call(((weight, "weight", (27, 2, *grid)), (bias, "bias", (2, *grid)),
                 (initActivations, "initActivations", x), (outActivations, "outActivations", x)),
                initActivations)
    act = _n.activation_id(activation)
    B, M, N, K = initActivations.shape
    with torch.cuda.device(weight.device):
        _n.check(_n.lib.gridnet_hip_forward_gated(
            _n.dtype_id(weight), weight.data_ptr(), bias.data_ptr(), initActivations.data_ptr(),
            outActivations.data_ptr(), B, M, N, K, int(innerIterations), int(blockSize), act,
            _n.current_stream(weight)))


def backward_gated(weight, bias, initActivations, outGrads, weightGradOut, biasGradOut,
                   activationsGradOut, innerIterations, blockSize, activation):
    """Backward of the gated step; replaces gated_gridnet_backward, src/gridnet_cuda.cpp:160-186.
    Gradient outputs are accumulated into, as in the reference."""
    grid, x = tuple(initActivations.shape[1:]), tuple(initActivations.shape)
    _check_call(((weight, "weight", (27, 2, *grid)), (bias, "bias", (2, *grid)),
                 (initActivations, "initActivations", x), (outGrads, "outGrads", x),
                 (weightGradOut, "weightGradOut", (27, 2, *grid)),
                 (biasGradOut, "biasGradOut", (2, *grid)),
                 (activationsGradOut, "activationsGradOut", x)),
                initActivations)
    act = _n.activation_id(activation)
    B, M, N, K = initActivations.shape
    dt = _n.dtype_id(weight)
    with torch.cuda.device(weight.device):
        nbytes = _n.lib.gridnet_hip_backward_gated_workspace_bytes(
            dt, B, M, N, K, int(innerIterations), int(blockSize))
        ws = _n.workspace(nbytes, weight.device)
        _n.check(_n.lib.gridnet_hip_backward_gated(
            dt, weight.data_ptr(), bias.data_ptr(), initActivations.data_ptr(),
            outGrads.data_ptr(), weightGradOut.data_ptr(), biasGradOut.data_ptr(),
            activationsGradOut.data_ptr(), B, M, N, K, int(innerIterations), int(blockSize), act, 0,
            ws.data_ptr(), nbytes, _n.current_stream(weight)))
