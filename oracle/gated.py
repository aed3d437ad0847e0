"""CPU oracle of the gated variant of the block-local update.

Test infrastructure (see ``oracle/__init__.py``).  Restates
gridnet/backend_torch.py:145-267: weight [27, 2, M, N, K], bias [2, M, N, K]; per inner
iteration and interior cell ``pre = b[0] + sum_t W[t,0] x_nbr``, ``gate = sigmoid(b[1] +
sum_t W[t,1] x_nbr)``, ``x' = gate * x + (1 - gate) * act(pre)``; the halo is frozen, zero
outside the grid, no normalisation, no residual scale.

Pinned in tests/test_oracle_gated.py by the zero-weight scalar recurrence, the centre-tap
recurrence, a scalar-loop brute force and finite differences.
"""

import torch
import torch.nn.functional as F

from .fast import from_blocks, to_windows
from .ref_style import activation_fn, neighbour_gather_index


def _check(weight, bias, x, bs):
    _, m, n, k = x.shape
    assert m % bs == 0 and n % bs == 0 and k % bs == 0, f"block_size={bs} incompatible"
    assert weight.shape == (27, 2, m, n, k), f"weight.shape={tuple(weight.shape)} invalid"
    assert bias.shape == weight.shape[1:], f"bias.shape={tuple(bias.shape)} invalid"


def gated_step_ref(weight, bias, init_activations, inner_iterations, block_size,
                   activation="tanh"):
    """Block loop + gather, the way gridnet/backend_torch.py:178-267 does it."""
    x, bs = init_activations, block_size
    _check(weight, bias, x, bs)
    batch, m, n, k = x.shape
    act = activation_fn(activation)
    index = neighbour_gather_index(bs, x.device)
    padded = F.pad(x, (1,) * 6)
    interiors = []
    for p in range(0, m, bs):
        for q in range(0, n, bs):
            for u in range(0, k, bs):
                win = padded[:, p:p + bs + 2, q:q + bs + 2, u:u + bs + 2]
                w_blk = weight[:, :, p:p + bs, q:q + bs, u:u + bs]
                b_blk = bias[:, p:p + bs, q:q + bs, u:u + bs]
                for _ in range(inner_iterations):
                    flat = win.flatten(1)
                    patches = flat.gather(1, index[None].repeat(batch, 1)).reshape(batch, bs**3, 27)
                    pre = (patches * w_blk[:, 0].flatten(1).t()).sum(-1) + b_blk[0].flatten()
                    gpre = (patches * w_blk[:, 1].flatten(1).t()).sum(-1) + b_blk[1].flatten()
                    gate = torch.sigmoid(gpre)
                    new = gate * win[:, 1:-1, 1:-1, 1:-1].flatten(1) + (1 - gate) * act(pre)
                    out = win.clone()
                    out[:, 1:-1, 1:-1, 1:-1] = new.reshape(-1, bs, bs, bs)
                    win = out
                interiors.append(win[:, 1:-1, 1:-1, 1:-1])
    stacked = torch.stack(interiors).reshape(m // bs, n // bs, k // bs, batch, bs, bs, bs)
    return stacked.permute(3, 0, 4, 1, 5, 2, 6).reshape(batch, m, n, k)


def _blocks5(p, bs):
    """[27 or -, 2, M, N, K] style tensors -> [..., mb, nb, kb, bs, bs, bs]."""
    lead = p.shape[:-3]
    m, n, k = p.shape[-3:]
    nl = len(lead)
    v = p.reshape(*lead, m // bs, bs, n // bs, bs, k // bs, bs)
    return v.permute(*range(nl), nl, nl + 2, nl + 4, nl + 1, nl + 3, nl + 5)


def gated_step_fast(weight, bias, init_activations, inner_iterations, block_size,
                    activation="tanh"):
    """All blocks at once (27 shifted slices); differentiable, fp32/fp64."""
    bs = block_size
    _check(weight, bias, init_activations, bs)
    act = activation_fn(activation)
    win = to_windows(init_activations, bs)
    w_blk = _blocks5(weight, bs)   # [27, 2, mb, nb, kb, bs, bs, bs]
    b_blk = _blocks5(bias, bs)     # [2, mb, nb, kb, bs, bs, bs]
    for _ in range(inner_iterations):
        pre, gpre = b_blk[0], b_blk[1]
        for a in range(3):
            for b in range(3):
                for c in range(3):
                    sl = win[..., a:a + bs, b:b + bs, c:c + bs]
                    pre = pre + w_blk[9 * a + 3 * b + c, 0] * sl
                    gpre = gpre + w_blk[9 * a + 3 * b + c, 1] * sl
        gate = torch.sigmoid(gpre)
        inner = win[..., 1:-1, 1:-1, 1:-1]
        new = gate * inner + (1 - gate) * act(pre)
        win = win + F.pad(new - inner, (1,) * 6)
    return from_blocks(win[..., 1:-1, 1:-1, 1:-1])


def gated_step_brute(weight, bias, x, inner, bs, activation="tanh"):
    """Scalar loops, fp64, tiny grids only."""
    import math

    import numpy as np

    from .brute import _act

    weight, bias, x = (np.asarray(t, dtype=np.float64) for t in (weight, bias, x))
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
                        new = win.copy()
                        for i in range(bs):
                            for j in range(bs):
                                for l in range(bs):
                                    pre = bias[0, p + i, q + j, r + l]
                                    gpre = bias[1, p + i, q + j, r + l]
                                    for a in range(3):
                                        for b in range(3):
                                            for c in range(3):
                                                v = win[i + a, j + b, l + c]
                                                pre += weight[9 * a + 3 * b + c, 0, p + i, q + j, r + l] * v
                                                gpre += weight[9 * a + 3 * b + c, 1, p + i, q + j, r + l] * v
                                    gate = 1.0 / (1.0 + math.exp(-gpre))
                                    new[i + 1, j + 1, l + 1] = (gate * win[i + 1, j + 1, l + 1]
                                                                + (1 - gate) * _act(activation, pre))
                        win = new
                    out[s, p:p + bs, q:q + bs, r:r + bs] = win[1:-1, 1:-1, 1:-1]
    return out
