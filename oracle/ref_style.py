"""Op-for-op CPU restatement of the reference's pure-torch grid update.

Test infrastructure (see ``oracle/__init__.py``); also the timed CPU baseline.

Follows gridnet/backend_torch.py:
  * :48-59   preconditions
  * :61-92   zero-pad the grid by one cell, visit blocks in (M, N, K) order, run
             ``inner_iterations`` updates on each (bs+2)^3 window with a frozen halo
  * :93-106  stitch the block interiors back into a dense [B, M, N, K] tensor
  * :118-140 one update: optional whole-window normalisation, gather 27 neighbours
             per interior cell, multiply by the per-cell weights and sum, add bias,
             activation, residual scale, zero-pad back to the window and add
  * :270-280 activations
  * :283-298 tap order t = 9a + 3b + c, neighbour (i+a-1, j+b-1, k+c-1)
"""

from typing import Callable

import torch
import torch.nn.functional as F

ACTIVATIONS = ("silu", "relu", "leaky_relu", "tanh")


def activation_fn(name: str) -> Callable[[torch.Tensor], torch.Tensor]:
    """gridnet/backend_torch.py:270-280 (leaky slope is torch's default 0.01)."""
    table = {
        "silu": F.silu,
        "relu": F.relu,
        "leaky_relu": F.leaky_relu,
        "tanh": torch.tanh,
    }
    if name not in table:
        raise ValueError(f"unknown activation: {name}")
    return table[name]


def neighbour_gather_index(bs: int, device=None) -> torch.Tensor:
    """Flat window index of every (interior cell, tap) pair.

    gridnet/backend_torch.py:283-298: cells in (i, j, k) raster order, taps in
    (a, b, c) raster order, window side bs + 2, k fastest.
    """
    side = bs + 2
    cell = torch.arange(bs)
    tap = torch.arange(3)
    i, j, k, a, b, c = torch.meshgrid(cell, cell, cell, tap, tap, tap, indexing="ij")
    flat = (k + c) + side * ((j + b) + side * (i + a))
    return flat.reshape(-1).to(device=device, dtype=torch.long)


def check_step_args(weight, bias, residual_scale, x, bs):
    """gridnet/backend_torch.py:48-59."""
    _, m, n, k = x.shape
    assert m % bs == 0 and n % bs == 0 and k % bs == 0, (
        f"block_size={bs} incompatible with init_activations.shape={tuple(x.shape)}"
    )
    assert weight.shape == (27, m, n, k), f"weight.shape={tuple(weight.shape)} invalid"
    assert bias.shape == weight.shape[1:], f"bias.shape={tuple(bias.shape)} invalid"
    assert bias.shape == residual_scale.shape, (
        f"residual_scale.shape={tuple(residual_scale.shape)} invalid"
    )


def window_update(win, w_blk, b_blk, r_blk, index, bs, eps, normalize, act):
    """One inner iteration on one block's window for the whole batch.

    gridnet/backend_torch.py:118-140.  ``win`` is [B, bs+2, bs+2, bs+2].
    """
    batch = win.shape[0]
    flat = win.flatten(1)
    if normalize:
        mu = flat.mean(1, keepdim=True)
        sd = flat.std(1, correction=0, keepdim=True)
        src = (flat - mu) / (sd + eps)
    else:
        src = flat
    patches = src.gather(1, index[None].repeat(batch, 1)).reshape(batch, bs**3, 27)
    pre = (patches * w_blk.flatten(1).t()).sum(-1) + b_blk.flatten()
    delta = act(pre) * r_blk.flatten()
    delta = delta.reshape(-1, bs, bs, bs)
    return F.pad(delta, (1, 1, 1, 1, 1, 1)) + win


def gridnet_step_ref(
    weight: torch.Tensor,
    bias: torch.Tensor,
    residual_scale: torch.Tensor,
    init_activations: torch.Tensor,
    inner_iterations: int,
    block_size: int,
    eps: float = 1e-5,
    normalize: bool = True,
    activation: str = "silu",
) -> torch.Tensor:
    """One outer step, the way gridnet/backend_torch.py:9-106 does it."""
    x = init_activations
    bs = block_size
    check_step_args(weight, bias, residual_scale, x, bs)
    batch, m, n, k = x.shape
    act = activation_fn(activation)
    index = neighbour_gather_index(bs, x.device)
    padded = F.pad(x, (1,) * 6)
    interiors = []
    for p in range(0, m, bs):
        for q in range(0, n, bs):
            for u in range(0, k, bs):
                win = padded[:, p : p + bs + 2, q : q + bs + 2, u : u + bs + 2]
                w_blk = weight[:, p : p + bs, q : q + bs, u : u + bs]
                b_blk = bias[p : p + bs, q : q + bs, u : u + bs]
                r_blk = residual_scale[p : p + bs, q : q + bs, u : u + bs]
                for _ in range(inner_iterations):
                    win = window_update(
                        win, w_blk, b_blk, r_blk, index, bs, eps, normalize, act
                    )
                interiors.append(win[:, 1:-1, 1:-1, 1:-1])
    stacked = torch.stack(interiors).reshape(m // bs, n // bs, k // bs, batch, bs, bs, bs)
    return stacked.permute(3, 0, 4, 1, 5, 2, 6).reshape(batch, m, n, k)
