"""ctypes binding of libgridnet_probe.so: machine ceilings that bench.py quotes beside the vendor
peaks (sustained fp32 FMA rate, LDS read rate, core clock under load, an HBM copy and HBM reads alone, LDS-pipe cycles
per read width), measured with the kernels' own compiler flags.  Not part of the update path and
not part of libgridnet_hip.so: it allocates its own buffers, runs on the null stream and
synchronises."""

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libgridnet_probe.so")

PROBES = {"fma_tfma_per_s": 0, "lds_gb_per_s": 1, "clock_ghz": 2, "copy_gb_per_s": 3, "read_gb_per_s": 8}
# LDS-pipe cycles per wave-level read instruction, by width
LDS_WIDTH_PROBES = {"ds_read_b32": 4, "ds_read_b64": 5, "ds_read_b128": 6, "ds_read2_b64": 7}

_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: build it with `python -m gridnet_amd.build`")
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.gridnet_probe.restype = ctypes.c_int
        _lib.gridnet_probe.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
        _lib.gridnet_probe_last_error.restype = ctypes.c_char_p
        _lib.gridnet_probe_last_error.argtypes = []
    return _lib


def probe_id(kind: int) -> float:
    lib = _load()
    out = ctypes.c_double(0.0)
    if lib.gridnet_probe(kind, ctypes.byref(out)) != 0:
        raise RuntimeError(lib.gridnet_probe_last_error().decode())
    return out.value


def probe(what: str) -> float:
    """One of the machine ceilings on the current device."""
    return probe_id(PROBES[what] if what in PROBES else LDS_WIDTH_PROBES[what])
