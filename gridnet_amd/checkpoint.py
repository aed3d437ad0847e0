"""The checkpoint blob the reference's web front end loads.

Written by gridnet/scripts/convert_to_web.py:33-71 and read by web/ts/checkpoint.ts:28-99:

    <u32 little-endian: length of the metadata> <metadata: JSON, utf-8> <parameter data>

metadata = {"params": [[name, shape], ...], "precision": 16 | 32,
            "config": {"activation", "innerIters", "outerIters", "outerResidual"}}
and the data are the parameters in that order, flattened, little-endian float32 or -- for
precision 16 -- the reference's own 16-bit packing, which is NOT IEEE rounding: sign, exponent
clamped from below at -15, mantissa truncated to 10 bits; the reader rebuilds
sign | (exp + 127) << 23 | frac << 13.  Zero and everything below 2^-15 therefore come back as
(+-)2^-15 * (1 + frac): the quirk is part of the format and is kept bit for bit.
"""

import json
import struct
from collections import OrderedDict

import numpy as np
import torch


def pack_float16(values: np.ndarray) -> np.ndarray:
    """float32 -> the 16-bit words of convert_to_web.py:53-68."""
    words = np.ascontiguousarray(values, dtype="<f4").view("<u4").astype(np.int64)
    sign = (words >> 31) & 1
    exp = ((words >> 23) & 0xFF) - 127
    frac = words & ((1 << 23) - 1)
    exp = np.maximum(exp, -15)  # the converter clamps small exponents; large ones wrap as there
    return ((sign << 15) | (((exp + 15) & 0b11111) << 10) | (frac >> 13)).astype("<u2")


def unpack_float16(halves: np.ndarray) -> np.ndarray:
    """The inverse as web/ts/checkpoint.ts:79-92 computes it."""
    half = np.ascontiguousarray(halves, dtype="<u2").astype(np.int64)
    sign = (half >> 15) & 1
    exp = ((half >> 10) & 0b11111) - 15
    frac = half & ((1 << 10) - 1)
    words = ((sign << 31) | ((exp + 127) << 23) | (frac << 13)) & 0xFFFFFFFF
    return words.astype("<u4").view("<f4")


def write_web_checkpoint(path, state, *, activation="leaky_relu", inner_iters=8, outer_iters=12,
                         outer_residual=False, precision=32):
    """``state``: ordered mapping name -> tensor (a model's ``state_dict()``)."""
    assert precision in (16, 32)
    metadata = dict(
        params=[(k, list(v.shape)) for k, v in state.items()],
        precision=precision,
        config={"activation": activation, "innerIters": inner_iters, "outerIters": outer_iters,
                "outerResidual": outer_residual},
    )
    metadata_bytes = json.dumps(metadata).encode("utf-8")
    with open(path, "wb") as f:
        f.write(struct.pack("<I", len(metadata_bytes)))
        f.write(metadata_bytes)
        for v in state.values():
            data = v.detach().reshape(-1).float().cpu().numpy()
            if precision == 32:
                f.write(np.ascontiguousarray(data, dtype="<f4").tobytes())
            else:
                f.write(pack_float16(data).tobytes())


def read_web_checkpoint(path):
    """Returns (state: OrderedDict name -> float32 tensor, config: dict, precision: int)."""
    with open(path, "rb") as f:
        blob = f.read()
    (size,) = struct.unpack("<I", blob[:4])
    metadata = json.loads(blob[4:4 + size].decode("utf-8"))
    precision = metadata.get("precision") or 32
    raw = blob[4 + size:]
    if precision == 32:
        flat = np.frombuffer(raw, dtype="<f4")
    else:
        flat = unpack_float16(np.frombuffer(raw, dtype="<u2"))
    state, at = OrderedDict(), 0
    for name, shape in metadata["params"]:
        n = int(np.prod(shape)) if len(shape) else 1
        state[name] = torch.from_numpy(np.array(flat[at:at + n], dtype=np.float32)).reshape(shape)
        at += n
    if at != flat.size:
        raise ValueError(f"checkpoint holds {flat.size} values, its metadata describes {at}")
    return state, metadata["config"], precision
