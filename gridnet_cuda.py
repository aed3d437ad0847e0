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


def forward(weight, bias, scale, initActivations, outActivations, innerIterations, blockSize,
            eps, normalize, activation):
    """One outer step; replaces gridnet_forward, src/gridnet_cuda.cpp:61-89."""
    for t, name in ((weight, "weight"), (bias, "bias"), (scale, "scale"),
                    (initActivations, "initActivations"), (outActivations, "outActivations")):
        _n.check_input(t, name)
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
    for t, name in ((weight, "weight"), (bias, "bias"), (scale, "scale"),
                    (initActivations, "initActivations"), (outGrads, "outGrads"),
                    (weightGradOut, "weightGradOut"), (biasGradOut, "biasGradOut"),
                    (scaleGradOut, "scaleGradOut"), (activationsGradOut, "activationsGradOut")):
        _n.check_input(t, name)
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
    for t, name in ((weight, "weight"), (bias, "bias"), (initActivations, "initActivations"),
                    (outActivations, "outActivations")):
        _n.check_input(t, name)
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
    for t, name in ((weight, "weight"), (bias, "bias"), (initActivations, "initActivations"),
                    (outGrads, "outGrads"), (weightGradOut, "weightGradOut"),
                    (biasGradOut, "biasGradOut"), (activationsGradOut, "activationsGradOut")):
        _n.check_input(t, name)
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
