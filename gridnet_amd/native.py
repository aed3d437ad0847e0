"""ctypes binding of libgridnet_hip.so (the C ABI declared in include/gridnet_hip.h).

The library is the product; there is no fallback.  If it has not been built this module
raises ImportError on import, which the dispatcher in ``gridnet_amd/__init__.py`` treats the
way the reference treats a missing extension (gridnet/__init__.py:14-18) -- and calling an op
on a HIP tensor without it raises instead of silently running something else.
"""

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# GRIDNET_HIP_LIBRARY lets a caller point at another build of the same ABI
LIB_PATH = os.environ.get("GRIDNET_HIP_LIBRARY") or os.path.join(_HERE, "libgridnet_hip.so")

F32, F64 = 0, 1
FUSED_RESIDUAL, FUSED_WALK_REVERSE = 1, 2  # gridnet_hip_fused_forward_flags
OVERWRITE_PARAMS = 1
OVERWRITE_DX = 2
OVERWRITE = 3
STATIC_SCRATCH_BYTES = 40 << 20  # GRIDNET_STATIC_SCRATCH_BYTES

EXPORTS = (
    "gridnet_hip_version",
    "gridnet_hip_last_error",
    "gridnet_hip_activation_id",
    "gridnet_hip_forward",
    "gridnet_hip_backward_workspace_bytes",
    "gridnet_hip_backward",
    "gridnet_hip_static_init",
    "gridnet_hip_backward_static",
    "gridnet_hip_forward_gated",
    "gridnet_hip_backward_gated_workspace_bytes",
    "gridnet_hip_backward_gated",
    "gridnet_hip_layernorm_workspace_bytes",
    "gridnet_hip_layernorm_forward",
    "gridnet_hip_layernorm_backward",
    "gridnet_hip_fused_workspace_bytes",
    "gridnet_hip_fused_forward",
    "gridnet_hip_fused_forward_residual",
    "gridnet_hip_fused_forward_flags",
    "gridnet_hip_layernorm_apply",
    "gridnet_hip_layernorm_backward_sums",
    "gridnet_hip_fused_backward",
    "gridnet_hip_fused_backward_residual",
    "gridnet_hip_chain_supported",
    "gridnet_hip_chain_halo_floats",
    "gridnet_hip_chain_backward",
    "gridnet_hip_chain_all_supported",
    "gridnet_hip_chain_all_workspace_bytes",
    "gridnet_hip_chain_backward_all",
    "gridnet_hip_chain_set_spin_limit",
)


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m gridnet_amd.build` "
            "(hipcc --offload-arch=gfx950)"
        )
    try:
        lib = ctypes.CDLL(LIB_PATH)
    except OSError as exc:  # unresolved HIP runtime, wrong arch, ...
        raise ImportError(f"cannot load {LIB_PATH}: {exc}") from exc
    p, i, d, l, z = ctypes.c_void_p, ctypes.c_int, ctypes.c_double, ctypes.c_long, ctypes.c_size_t
    lib.gridnet_hip_version.restype = i
    lib.gridnet_hip_version.argtypes = []
    lib.gridnet_hip_last_error.restype = ctypes.c_char_p
    lib.gridnet_hip_last_error.argtypes = []
    lib.gridnet_hip_activation_id.restype = i
    lib.gridnet_hip_activation_id.argtypes = [ctypes.c_char_p]
    lib.gridnet_hip_forward.restype = i
    lib.gridnet_hip_forward.argtypes = [i, p, p, p, p, p, i, i, i, i, i, i, d, i, i, p]
    lib.gridnet_hip_backward_workspace_bytes.restype = z
    lib.gridnet_hip_backward_workspace_bytes.argtypes = [i, i, i, i, i, i, i, i]
    lib.gridnet_hip_backward.restype = i
    lib.gridnet_hip_backward.argtypes = [i, p, p, p, p, p, p, p, p, p, i, i, i, i, i, i, d, i, i, i,
                                         p, z, p]
    lib.gridnet_hip_static_init.restype = i
    lib.gridnet_hip_static_init.argtypes = []
    lib.gridnet_hip_backward_static.restype = i
    lib.gridnet_hip_backward_static.argtypes = [i, p, p, p, p, p, p, p, p, p, i, i, i, i, i, i, d, i, i, i, p]
    lib.gridnet_hip_forward_gated.restype = i
    lib.gridnet_hip_forward_gated.argtypes = [i, p, p, p, p, i, i, i, i, i, i, i, p]
    lib.gridnet_hip_backward_gated_workspace_bytes.restype = z
    lib.gridnet_hip_backward_gated_workspace_bytes.argtypes = [i, i, i, i, i, i, i]
    lib.gridnet_hip_backward_gated.restype = i
    lib.gridnet_hip_backward_gated.argtypes = [i, p, p, p, p, p, p, p, i, i, i, i, i, i, i, i, p, z, p]
    lib.gridnet_hip_layernorm_workspace_bytes.restype = z
    lib.gridnet_hip_layernorm_workspace_bytes.argtypes = [i, i, l]
    lib.gridnet_hip_layernorm_forward.restype = i
    lib.gridnet_hip_layernorm_forward.argtypes = [i, p, p, p, p, p, p, i, l, d, p, z, p]
    lib.gridnet_hip_layernorm_backward.restype = i
    lib.gridnet_hip_layernorm_backward.argtypes = [i, p, p, p, p, p, p, p, p, i, l, i, p, z, p]
    lib.gridnet_hip_fused_workspace_bytes.restype = z
    lib.gridnet_hip_fused_workspace_bytes.argtypes = [i, i, i, i, i, i, i]
    lib.gridnet_hip_fused_forward.restype = i
    lib.gridnet_hip_fused_forward.argtypes = [i, p, p, p, p, p, p, p, p, p, i, i, i, i, i, i, d, i,
                                              p, z, p]
    lib.gridnet_hip_fused_forward_flags.restype = i
    lib.gridnet_hip_fused_forward_flags.argtypes = [i, p, p, p, p, p, p, p, p, p, i, i, i, i, i, i, d, i, i,
                                                    p, z, p]
    lib.gridnet_hip_fused_forward_residual.restype = i
    lib.gridnet_hip_fused_forward_residual.argtypes = lib.gridnet_hip_fused_forward.argtypes
    lib.gridnet_hip_layernorm_apply.restype = i
    lib.gridnet_hip_layernorm_apply.argtypes = [i, p, p, p, p, p, i, l, p]
    lib.gridnet_hip_layernorm_backward_sums.restype = i
    lib.gridnet_hip_layernorm_backward_sums.argtypes = [i, p, p, p, p, p, i, l, p, z, p]
    lib.gridnet_hip_fused_backward.restype = i
    lib.gridnet_hip_fused_backward.argtypes = [i] + [p] * 18 + [i] * 8 + [p, z, p]
    lib.gridnet_hip_fused_backward_residual.restype = i
    lib.gridnet_hip_fused_backward_residual.argtypes = [i] + [p] * 20 + [i] * 8 + [p, z, p]
    lib.gridnet_hip_chain_supported.restype = i
    lib.gridnet_hip_chain_supported.argtypes = [i, i, i, i]
    lib.gridnet_hip_chain_halo_floats.restype = z
    lib.gridnet_hip_chain_halo_floats.argtypes = [i, i, i, i, i]
    lib.gridnet_hip_chain_backward.restype = i
    lib.gridnet_hip_chain_backward.argtypes = [i] + [p] * 20 + [i] * 8 + [p, z, p]
    lib.gridnet_hip_chain_all_supported.restype = i
    lib.gridnet_hip_chain_all_supported.argtypes = [i] * 9
    lib.gridnet_hip_chain_all_workspace_bytes.restype = z
    lib.gridnet_hip_chain_all_workspace_bytes.argtypes = [i] * 7
    lib.gridnet_hip_chain_backward_all.restype = i
    lib.gridnet_hip_chain_backward_all.argtypes = [i] + [p] * 15 + [i] * 9 + [p, z, p]
    lib.gridnet_hip_chain_set_spin_limit.restype = i
    lib.gridnet_hip_chain_set_spin_limit.argtypes = [i]
    return lib


try:
    lib = _load()
except AttributeError as exc:  # an older build of the library without some entry point
    raise ImportError(f"{LIB_PATH} is stale ({exc}): rebuild with `python -m gridnet_amd.build`") from exc


def last_error() -> str:
    return lib.gridnet_hip_last_error().decode()


def check(status: int) -> None:
    if status != 0:
        raise RuntimeError(last_error())


def activation_id(name: str) -> int:
    act = lib.gridnet_hip_activation_id(str(name).encode())
    if act < 0:
        raise RuntimeError(last_error())  # "unknown activation function: X"
    return act


def dtype_id(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.float64:
        return F64
    raise RuntimeError(f"gridnet_hip supports float32 and float64 tensors, got {t.dtype}")


def check_input(t: torch.Tensor, name: str) -> None:
    """The reference binding's CHECK_INPUT (src/gridnet_cuda.cpp:6-10), same messages."""
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def current_stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def workspace(nbytes: int, device) -> torch.Tensor:
    """Scratch from torch's caching allocator (stream-ordered reuse, no hipMalloc per call)."""
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)
