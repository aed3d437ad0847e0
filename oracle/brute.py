"""Scalar-loop fp64 forward oracle for tiny grids (numpy + Python loops).

Test infrastructure (see ``oracle/__init__.py``).  Written cell by cell from the
update rule of gridnet/backend_torch.py:61-142 with none of the tensor tricks of
the other oracles, so an indexing mistake there shows up here.
"""

import math

import numpy as np


def _act(name: str, u: float) -> float:
    if name == "relu":
        return u if u > 0 else 0.0
    if name == "leaky_relu":
        return u if u > 0 else 0.01 * u
    if name == "silu":
        return u / (1.0 + math.exp(-u))
    if name == "tanh":
        return math.tanh(u)
    raise ValueError(f"unknown activation: {name}")


def gridnet_step_brute(weight, bias, scale, x, inner, bs, eps=1e-5, normalize=True,
                       activation="silu"):
    weight = np.asarray(weight, dtype=np.float64)
    bias = np.asarray(bias, dtype=np.float64)
    scale = np.asarray(scale, dtype=np.float64)
    x = np.asarray(x, dtype=np.float64)
    batch, m, n, k = x.shape
    side = bs + 2
    out = np.empty_like(x)
    for s in range(batch):
        for p in range(0, m, bs):
            for q in range(0, n, bs):
                for r in range(0, k, bs):
                    win = np.zeros((side, side, side))
                    for i in range(side):
                        for j in range(side):
                            for l in range(side):
                                gi, gj, gl = p + i - 1, q + j - 1, r + l - 1
                                if 0 <= gi < m and 0 <= gj < n and 0 <= gl < k:
                                    win[i, j, l] = x[s, gi, gj, gl]
                    for _ in range(inner):
                        if normalize:
                            mu = win.sum() / win.size
                            sd = math.sqrt(((win - mu) ** 2).sum() / win.size)
                            src = (win - mu) / (sd + eps)
                        else:
                            src = win
                        new = win.copy()
                        for i in range(bs):
                            for j in range(bs):
                                for l in range(bs):
                                    u = bias[p + i, q + j, r + l]
                                    for a in range(3):
                                        for b in range(3):
                                            for c in range(3):
                                                u += (
                                                    weight[9 * a + 3 * b + c, p + i, q + j, r + l]
                                                    * src[i + a, j + b, l + c]
                                                )
                                    new[i + 1, j + 1, l + 1] = (
                                        win[i + 1, j + 1, l + 1]
                                        + scale[p + i, q + j, r + l] * _act(activation, u)
                                    )
                        win = new
                    out[s, p : p + bs, q : q + bs, r : r + bs] = win[1:-1, 1:-1, 1:-1]
    return out
