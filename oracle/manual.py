"""Hand-derived backward of one outer step and of the LayerNorm (CPU oracle).

Test infrastructure (see ``oracle/__init__.py``).  These are the formulas the HIP
kernels implement, written out in torch so they can be checked against autograd of
``oracle.fast`` on the CPU.  The reference evaluates the same recurrences inside
src/gridnet_cuda_kernels.cu:274-449 (recompute the inner forward, walk it in
reverse, push w*delta onto the 27 neighbours of each cell, add the window of
gradients onto the input grid, sum parameter gradients over the batch).
"""

import torch
import torch.nn.functional as F

from .fast import normalise_windows, pre_activation, to_blocks, to_windows
from .ref_style import check_step_args


def act_and_derivative(name: str, u: torch.Tensor):
    if name == "relu":
        return torch.relu(u), (u > 0).to(u.dtype)
    if name == "leaky_relu":
        one = torch.ones_like(u)
        return torch.where(u > 0, u, 0.01 * u), torch.where(u > 0, one, 0.01 * one)
    if name == "silu":
        s = torch.sigmoid(u)
        return u * s, s * (1 + u * (1 - s))
    if name == "tanh":
        t = torch.tanh(u)
        return t, 1 - t * t
    raise ValueError(f"unknown activation: {name}")


def scatter_to_neighbours(w_blk, delta, bs):
    """dz[c + off_t] += W[t, c] * delta[c] for all 27 taps; returns a full window."""
    shape = delta.shape[:-3] + (bs + 2,) * 3
    dz = delta.new_zeros(shape)
    for a in range(3):
        for b in range(3):
            for c in range(3):
                dz[..., a : a + bs, b : b + bs, c : c + bs] += w_blk[9 * a + 3 * b + c] * delta
    return dz


def fold_windows(g_win: torch.Tensor, bs: int) -> torch.Tensor:
    """Sum every window (halo included) back onto the grid; out-of-grid entries drop."""
    b, mb, nb, kb = g_win.shape[:4]
    m, n, k = mb * bs, nb * bs, kb * bs
    acc = g_win.new_zeros(b, m + 2, n + 2, k + 2)
    for p in range(mb):
        for q in range(nb):
            for u in range(kb):
                acc[:, p * bs : p * bs + bs + 2, q * bs : q * bs + bs + 2,
                    u * bs : u * bs + bs + 2] += g_win[:, p, q, u]
    return acc[:, 1:-1, 1:-1, 1:-1]


def gridnet_step_backward_manual(weight, bias, residual_scale, x, grad_out, inner, bs,
                                 eps=1e-5, normalize=True, activation="silu"):
    """Returns (dweight, dbias, dscale, dx) of one outer step."""
    check_step_args(weight, bias, residual_scale, x, bs)
    w_blk, b_blk, r_blk = to_blocks(weight, bs), to_blocks(bias, bs), to_blocks(residual_scale, bs)
    win = to_windows(x, bs)
    states = []
    for _ in range(inner):
        states.append(win)
        src = normalise_windows(win, eps) if normalize else win
        fu, _ = act_and_derivative(activation, pre_activation(src, w_blk, b_blk, bs))
        win = win + F.pad(fu * r_blk, (1,) * 6)

    g = F.pad(to_blocks(grad_out, bs), (1,) * 6)  # gradient w.r.t. the whole window
    dw = torch.zeros_like(w_blk)
    db = torch.zeros_like(b_blk)
    dr = torch.zeros_like(r_blk)
    nwin = float((bs + 2) ** 3)
    for v in reversed(states):
        if normalize:
            flat = v.flatten(-3)
            mu = flat.mean(-1, keepdim=True)
            sd = flat.std(-1, correction=0, keepdim=True)
            inv = 1.0 / (sd + eps)
            src = ((flat - mu) * inv).reshape(v.shape)
        else:
            src = v
        fu, dfu = act_and_derivative(activation, pre_activation(src, w_blk, b_blk, bs))
        g_own = g[..., 1:-1, 1:-1, 1:-1]
        dr = dr + (fu * g_own).sum(0)
        delta = dfu * g_own * r_blk
        db = db + delta.sum(0)
        for a in range(3):
            for b in range(3):
                for c in range(3):
                    dw[9 * a + 3 * b + c] += (src[..., a : a + bs, b : b + bs, c : c + bs] * delta).sum(0)
        dz = scatter_to_neighbours(w_blk, delta, bs)
        if normalize:
            dzf = dz.flatten(-3)
            cen = flat - mu
            term = inv * (dzf - dzf.mean(-1, keepdim=True))
            proj = (dzf * cen).sum(-1, keepdim=True)
            term = term - proj * cen * inv * inv / (nwin * sd.clamp_min(1e-30))
            g = g + term.reshape(v.shape)
        else:
            g = g + dz
    return (_params_from_blocks(dw), _params_from_blocks(db), _params_from_blocks(dr),
            fold_windows(g, bs))


def _params_from_blocks(p: torch.Tensor) -> torch.Tensor:
    """[..., mb, nb, kb, bs, bs, bs] -> [..., M, N, K]."""
    lead = p.shape[:-6]
    mb, nb, kb, bs = p.shape[-6:-2]
    nl = len(lead)
    v = p.permute(*range(nl), nl, nl + 3, nl + 1, nl + 4, nl + 2, nl + 5)
    return v.reshape(*lead, mb * bs, nb * bs, kb * bs)


def layer_norm_backward_manual(dy, x, gamma, eps=1e-5):
    """Returns (dx, dgamma, dbeta, mean, rstd) of per-sample LayerNorm over all cells."""
    flat = x.flatten(1)
    mu = flat.mean(1, keepdim=True)
    var = ((flat - mu) ** 2).mean(1, keepdim=True)
    rstd = 1.0 / torch.sqrt(var + eps)
    xhat = ((flat - mu) * rstd).reshape(x.shape)
    dbeta = dy.sum(0)
    dgamma = (dy * xhat).sum(0)
    g = (dy * gamma).flatten(1)
    xh = xhat.flatten(1)
    dx = rstd * (g - g.mean(1, keepdim=True) - xh * (g * xh).mean(1, keepdim=True))
    return dx.reshape(x.shape), dgamma, dbeta, mu.flatten(), rstd.flatten()
