"""CPU checks of the drop-in boundary: the library loads, exports what the header declares,
answers its host-only entry points, and the Python shim has the reference's call surface."""

import ctypes
import inspect
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "gridnet_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gridnet_hip_\w+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    for want in ("gridnet_hip_forward", "gridnet_hip_backward", "gridnet_hip_layernorm_forward",
                 "gridnet_hip_layernorm_backward", "gridnet_hip_last_error"):
        assert want in names


def test_library_exports_every_declared_symbol():
    from gridnet_amd import native

    lib = ctypes.CDLL(native.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} declared in include/gridnet_hip.h but not exported"
    assert set(native.EXPORTS) == set(declared_symbols())


def test_host_only_entry_points():
    from gridnet_amd import native

    assert native.lib.gridnet_hip_version() >= 1
    assert [native.activation_id(n) for n in ("relu", "leaky_relu", "silu", "tanh")] == [0, 1, 2, 3]
    with pytest.raises(RuntimeError, match="unknown activation function: gelu"):
        native.activation_id("gelu")
    # argument validation happens before anything touches a device
    rc = native.lib.gridnet_hip_forward(0, 8, 8, 8, 8, 8, 2, 12, 8, 8, 1, 8, 1e-5, 0, 0, None)
    assert rc == 1 and "incompatible" in native.last_error()
    rc = native.lib.gridnet_hip_forward(0, 8, 8, 8, 8, 8, 2, 8, 8, 8, 1, 2, 1e-5, 0, 0, None)
    assert rc == 1 and "block_size" in native.last_error()
    rc = native.lib.gridnet_hip_backward(0, 8, 8, 8, 8, 8, 8, 8, 8, 8, 2, 8, 8, 8, 33, 8, 1e-5, 0,
                                         0, 0, None, 0, None)
    assert rc == 3
    assert native.last_error() == "cannot backprop through more than 32 inner iterations"
    rc = native.lib.gridnet_hip_forward(0, 8, 8, 8, 8, 8, 2, 8, 8, 8, 1, 8, 1e-5, 0, 7, None)
    assert rc == 2 and "unknown activation function" in native.last_error()
    # 32-bit cell indexing inside a sample: 27 * 432^3 is past 2^31, 27 * 424^3 is not
    rc = native.lib.gridnet_hip_forward(0, 8, 8, 8, 8, 8, 1, 432, 432, 432, 1, 8, 1e-5, 0, 0, None)
    assert rc == 1 and "grid too large" in native.last_error()
    rc = native.lib.gridnet_hip_forward(0, None, 8, 8, 8, 8, 1, 424, 424, 424, 1, 8, 1e-5, 0, 0, None)
    assert rc == 1 and "null input pointer" in native.last_error()
    # backward workspaces: one activation tensor (D) for the plain step, two floats per block and
    # batch element more with normalize, two tensors (D0, D1) for the gated step; none in fp64
    act = 32 * 64 ** 3 * 4
    assert native.lib.gridnet_hip_backward_workspace_bytes(0, 32, 64, 64, 64, 4, 8, 0) == act
    assert native.lib.gridnet_hip_backward_workspace_bytes(0, 32, 64, 64, 64, 4, 8, 1) == act + 32 * 512 * 8
    assert native.lib.gridnet_hip_backward_workspace_bytes(1, 32, 64, 64, 64, 4, 8, 0) == 0
    assert native.lib.gridnet_hip_backward_gated_workspace_bytes(0, 32, 64, 64, 64, 4, 8) == 2 * act
    assert native.lib.gridnet_hip_backward_gated_workspace_bytes(1, 32, 64, 64, 64, 4, 8) == 0
    # the history of more than 21 inner iterations does not fit the LDS at 8^3 blocks: generic kernels
    assert native.lib.gridnet_hip_backward_gated_workspace_bytes(0, 32, 64, 64, 64, 22, 8) == 0
    rc = native.lib.gridnet_hip_backward_gated(0, 8, 8, 8, 8, 8, 8, 8, 2, 8, 8, 8, 2, 8, 0, 0, None, 0, None)
    assert rc == 4 and "workspace" in native.last_error()
    rc = native.lib.gridnet_hip_backward(0, 8, 8, 8, 8, 8, 8, 8, 8, 8, 2, 8, 8, 8, 2, 8, 1e-5, 1, 0, 0,
                                         None, 0, None)
    assert rc == 4 and "workspace" in native.last_error()
    # the entry point on static scratch refuses, before touching a device, what its array cannot hold
    assert native.lib.gridnet_hip_backward_workspace_bytes(0, 64, 64, 64, 64, 4, 8, 0) > native.STATIC_SCRATCH_BYTES
    rc = native.lib.gridnet_hip_backward_static(0, 8, 8, 8, 8, 8, 8, 8, 8, 8, 64, 64, 64, 64, 4, 8, 1e-5,
                                                0, 0, 0, None)
    assert rc == 4 and "static array holds" in native.last_error()
    assert native.lib.gridnet_hip_layernorm_workspace_bytes(0, 32, 64 ** 3) == (32 * 64 * 2 + 64) * 4
    rc = native.lib.gridnet_hip_layernorm_forward(0, 8, 8, 8, 8, 8, 8, 4, 4096, 1e-5, None, 0, None)
    assert rc == 4 and "workspace" in native.last_error()


def test_shim_has_the_reference_call_surface():
    """Positional signatures of src/gridnet_cuda.cpp:61-72, 91-106, 133-141, 160-171."""
    import gridnet_cuda

    assert list(inspect.signature(gridnet_cuda.forward).parameters) == [
        "weight", "bias", "scale", "initActivations", "outActivations", "innerIterations",
        "blockSize", "eps", "normalize", "activation"]
    assert list(inspect.signature(gridnet_cuda.backward).parameters) == [
        "weight", "bias", "scale", "initActivations", "outGrads", "weightGradOut", "biasGradOut",
        "scaleGradOut", "activationsGradOut", "innerIterations", "blockSize", "eps", "normalize",
        "activation"]
    assert len(inspect.signature(gridnet_cuda.forward_gated).parameters) == 7
    assert len(inspect.signature(gridnet_cuda.backward_gated).parameters) == 10


def test_shim_rejects_host_tensors_like_the_reference_binding():
    import torch

    import gridnet_cuda

    t = torch.zeros(1, 8, 8, 8)
    w = torch.zeros(27, 8, 8, 8)
    p = torch.zeros(8, 8, 8)
    with pytest.raises(RuntimeError, match="weight must be a CUDA tensor"):
        gridnet_cuda.forward(w, p, p, t, t.clone(), 1, 8, 1e-5, False, "silu")


def test_shim_validates_dtypes_and_shapes_on_the_host(monkeypatch):
    """Raw pointers carry no dtype or size: what the reference's typed accessors would refuse
    (src/gridnet_cuda.cpp:103-107) is refused here before any native call.  The device check is
    patched out so that host tensors reach the checks behind it."""
    import torch

    import gridnet_cuda
    from gridnet_amd import native

    monkeypatch.setattr(native, "check_input", lambda t, name: None)

    def forbid(*a, **k):
        raise AssertionError("a native entry point was reached")

    for name in ("gridnet_hip_forward", "gridnet_hip_backward", "gridnet_hip_forward_gated",
                 "gridnet_hip_backward_gated"):
        monkeypatch.setattr(native.lib, name, forbid)
    w, p, x = torch.zeros(27, 8, 8, 16), torch.zeros(8, 8, 16), torch.zeros(2, 8, 8, 16)
    ok = (w, p, p, x, x.clone())
    cases = {
        "bias has dtype": (w, p.double(), p, x, x.clone()),
        "initActivations has dtype": (w, p, p, x.double(), x.clone()),
        "outActivations has shape": (w, p, p, x, x[:1].clone()),
        "weight has shape": (w[:, :, :, :8].contiguous(), p, p, x, x.clone()),
        "scale has shape": (w, p, p[:4].contiguous(), x, x.clone()),
    }
    for message, args in cases.items():
        with pytest.raises(RuntimeError, match=message):
            gridnet_cuda.forward(*args, 1, 8, 1e-5, False, "silu")
    grads = (torch.zeros_like(w), torch.zeros_like(p), torch.zeros_like(p), torch.zeros_like(x))
    with pytest.raises(RuntimeError, match="weightGradOut has shape"):
        gridnet_cuda.backward(w, p, p, x, x.clone(), grads[0][:26].contiguous(), *grads[1:], 1, 8, 1e-5,
                              False, "silu")
    with pytest.raises(RuntimeError, match="activationsGradOut has dtype"):
        gridnet_cuda.backward(w, p, p, x, x.clone(), *grads[:3], grads[3].double(), 1, 8, 1e-5, False,
                              "silu")
    with pytest.raises(RuntimeError, match="outGrads has shape"):
        gridnet_cuda.backward(w, p, p, x, x[:1].clone(), *grads, 1, 8, 1e-5, False, "silu")
    wg, pg = torch.zeros(27, 2, 8, 8, 16), torch.zeros(2, 8, 8, 16)
    with pytest.raises(RuntimeError, match="weight has shape"):
        gridnet_cuda.forward_gated(w, pg, x, x.clone(), 1, 8, "tanh")
    with pytest.raises(RuntimeError, match="biasGradOut has shape"):
        gridnet_cuda.backward_gated(wg, pg, x, x.clone(), torch.zeros_like(wg), torch.zeros_like(p),
                                    torch.zeros_like(x), 1, 8, "tanh")
    with pytest.raises(RuntimeError, match=r"must be \[B, M, N, K\]"):
        gridnet_cuda.forward(w, p, p, x[0], x[0].clone(), 1, 8, 1e-5, False, "silu")
    # and a well-formed call passes every check
    gridnet_cuda._check_call(tuple(zip(ok, "abcde", [(27, 8, 8, 16), (8, 8, 16), (8, 8, 16), x.shape, x.shape])), x)


def test_dispatcher_never_falls_back():
    import torch

    import gridnet_amd

    w, p, t = torch.zeros(27, 8, 8, 8), torch.zeros(8, 8, 8), torch.zeros(1, 8, 8, 8)
    with pytest.raises(NotImplementedError, match="HIP devices only"):
        gridnet_amd.gridnet_step(w, p, p, t, 1, 8)


def test_autograd_op_keeps_the_reference_contract():
    import torch

    from gridnet_amd.backend_cuda import GridnetCudaOp

    params = list(inspect.signature(GridnetCudaOp.forward).parameters)
    assert params == ["ctx", "weight", "bias", "residual_scale", "init_activations", "inner_iters",
                      "block_size", "eps", "normalize", "activation"]
    w, p = torch.zeros(27, 8, 8, 8), torch.zeros(8, 8, 8)
    # gridnet/backend_cuda.py:20-22 and :51-52
    with pytest.raises(AssertionError, match="incompatible"):
        GridnetCudaOp.apply(w, p, p, torch.zeros(1, 8, 8, 8), 1, 3, 1e-5, False, "silu")
    with pytest.raises(AssertionError, match="invalid"):
        GridnetCudaOp.apply(w[:26], p, p, torch.zeros(1, 8, 8, 8), 1, 8, 1e-5, False, "silu")
    with pytest.raises(AssertionError, match="mismatching dtypes"):
        GridnetCudaOp.apply(w, p.double(), p, torch.zeros(1, 8, 8, 8), 1, 8, 1e-5, False, "silu")
    empty = torch.zeros(0, 8, 8, 8)
    out = GridnetCudaOp.apply(w, p, p, empty, 1, 8, 1e-5, False, "silu")
    assert out.shape == empty.shape and out.data_ptr() != empty.data_ptr() or out.numel() == 0


def test_shim_matches_the_call_sites_in_the_reference_tree():
    """Where the reference is on disk (this container, not the GPU box): every call of the
    extension module in gridnet/backend_cuda.py, read as text and parsed, must fit the shim's
    function of that name -- same number of positional arguments, no keywords."""
    import ast
    import os

    import gridnet_cuda

    path = "/root/reference/gridnet/backend_cuda.py"
    if not os.path.exists(path):
        pytest.skip("the reference tree is not on this machine")
    with open(path) as fh:
        tree = ast.parse(fh.read())
    calls = [n for n in ast.walk(tree)
             if isinstance(n, ast.Call) and isinstance(n.func, ast.Attribute)
             and isinstance(n.func.value, ast.Name) and n.func.value.id == "gridnet_cuda"]
    assert {c.func.attr for c in calls} == {"forward", "backward", "forward_gated", "backward_gated"}
    for call in calls:
        params = inspect.signature(getattr(gridnet_cuda, call.func.attr)).parameters
        assert not call.keywords, call.func.attr
        assert len(call.args) == len(params), (call.func.attr, len(call.args), len(params))
