"""Block-vectorised CPU oracle: every block of the grid advanced at once.

Test infrastructure (see ``oracle/__init__.py``).  Same arithmetic as
``oracle.ref_style`` (gridnet/backend_torch.py:61-142) but the Python loop over
blocks is replaced by one strided view of all (bs+2)^3 windows, and the gather by
27 shifted slices.  Differentiable through torch autograd in fp32 and fp64.
"""

import torch
import torch.nn.functional as F

from .ref_style import activation_fn, check_step_args


def to_windows(x: torch.Tensor, bs: int) -> torch.Tensor:
    """[B, M, N, K] -> [B, M/bs, N/bs, K/bs, bs+2, bs+2, bs+2], zero outside the grid.

    gridnet/backend_torch.py:63-72: the halo is a copy of the *input* grid.
    """
    padded = F.pad(x, (1,) * 6)
    side = bs + 2
    return padded.unfold(1, side, bs).unfold(2, side, bs).unfold(3, side, bs).contiguous()


def to_blocks(p: torch.Tensor, bs: int) -> torch.Tensor:
    """[..., M, N, K] -> [..., M/bs, N/bs, K/bs, bs, bs, bs] (a view where possible)."""
    lead = p.shape[:-3]
    m, n, k = p.shape[-3:]
    nl = len(lead)
    v = p.reshape(*lead, m // bs, bs, n // bs, bs, k // bs, bs)
    return v.permute(*range(nl), nl, nl + 2, nl + 4, nl + 1, nl + 3, nl + 5)


def from_blocks(y: torch.Tensor) -> torch.Tensor:
    """[B, mb, nb, kb, bs, bs, bs] -> [B, M, N, K] (gridnet/backend_torch.py:93-106)."""
    b, mb, nb, kb, bs = y.shape[:5]
    return y.permute(0, 1, 4, 2, 5, 3, 6).reshape(b, mb * bs, nb * bs, kb * bs)


def normalise_windows(win: torch.Tensor, eps: float) -> torch.Tensor:
    """gridnet/backend_torch.py:126-129: whole-window mean, population std, eps on std."""
    flat = win.flatten(-3)
    mu = flat.mean(-1, keepdim=True)
    sd = flat.std(-1, correction=0, keepdim=True)
    return ((flat - mu) / (sd + eps)).reshape(win.shape)


def pre_activation(src: torch.Tensor, w_blk: torch.Tensor, b_blk: torch.Tensor, bs: int):
    """u[c] = bias[c] + sum_t W[t, c] * src[c + off_t], taps in raster order (a, b, c)."""
    acc = None
    for a in range(3):
        for b in range(3):
            for c in range(3):
                term = w_blk[9 * a + 3 * b + c] * src[..., a : a + bs, b : b + bs, c : c + bs]
                acc = term if acc is None else acc + term
    return acc + b_blk


def gridnet_step_fast(
    weight,
    bias,
    residual_scale,
    init_activations,
    inner_iterations: int,
    block_size: int,
    eps: float = 1e-5,
    normalize: bool = True,
    activation: str = "silu",
    watch=None,
):
    """``watch``, when given, is called with the pre-activations of every inner iteration (the
    tests use it to find inputs that keep clear of the kink of relu / leaky_relu)."""
    bs = block_size
    check_step_args(weight, bias, residual_scale, init_activations, bs)
    act = activation_fn(activation)
    win = to_windows(init_activations, bs)
    w_blk = to_blocks(weight, bs)
    b_blk = to_blocks(bias, bs)
    r_blk = to_blocks(residual_scale, bs)
    for _ in range(inner_iterations):
        src = normalise_windows(win, eps) if normalize else win
        u = pre_activation(src, w_blk, b_blk, bs)
        if watch is not None:
            watch(u)
        delta = act(u) * r_blk
        win = win + F.pad(delta, (1,) * 6)
    return from_blocks(win[..., 1:-1, 1:-1, 1:-1])
