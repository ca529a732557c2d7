"""Independent statement of the TGV inpainting layer, written from its energy and not from the
reference's stencil code; used only to pin the oracle.

State (u, v1, v2) per channel.  With forward differences that are zero across the far border,

    z1 = d_x u - v1   (0 in the last column)        z2 = d_y u - v2   (0 in the last row)
    R(u, v) = sum_p huber( sqrt( wx z1^2 + wy z2^2 ) )
            + sum_p huber( sqrt( bx ((d_x v1)^2 + (d_y v1)^2) ) )
            + sum_p huber( sqrt( by ((d_x v2)^2 + (d_y v2)^2) ) )          huber threshold 0.2
    D(u)    = sum_p c_p huber_1(u_p - b_p)

all four weight fields multiplied by L = 1 / (max(32, max_p s_p) + 0.01).  FISTA with unit step:
(u, v) <- y - grad R(y) by autograd, u <- prox_D(u), then the textbook extrapolation on all
three variables.
"""
import numpy as np
import torch

from independent_tv import fista_factors, prox_D

DELTA = float(np.float32(0.2))


def fdiff(f):
    dx = torch.zeros_like(f)
    dy = torch.zeros_like(f)
    dx[..., :, :-1] = f[..., :, 1:] - f[..., :, :-1]
    dy[..., :-1, :] = f[..., 1:, :] - f[..., :-1, :]
    return dx, dy


def huber_of_sqrt(A, delta=DELTA):
    safe = torch.sqrt(torch.clamp(A, min=1e-30))
    return torch.where(A <= delta * delta, 0.5 * A, delta * safe - 0.5 * delta * delta).sum()


def energy_R(u, v1, v2, wxs, wys, bxs, bys):
    """u, v1, v2: (C,H,W); scaled weights (H,W)."""
    ux, uy = fdiff(u)
    mx = torch.ones_like(u); mx[..., :, -1] = 0
    my = torch.ones_like(u); my[..., -1, :] = 0
    z1 = (ux - v1) * mx
    z2 = (uy - v2) * my
    v1x, v1y = fdiff(v1)
    v2x, v2y = fdiff(v2)
    return (huber_of_sqrt(wxs * z1 * z1 + wys * z2 * z2)
            + huber_of_sqrt(bxs * (v1x * v1x + v1y * v1y))
            + huber_of_sqrt(bys * (v2x * v2x + v2y * v2y)))


def lipschitz_scale(dx=None, dy=None, fp32=False):
    """L for weights whose bound stays below 32 (the only case the pins use): 1 / (32 + 0.01f).
    In fp32 the sum is rounded to float before the (double) reciprocal, which is rounded again."""
    if fp32:
        return float(np.float32(1.0 / np.float64(np.float32(np.float32(32.0) + np.float32(0.01)))))
    return 1.0 / (32.0 + float(np.float32(0.01)))


def tgv_layer(dx, dy, c, b, init, its, create_graph=False, L=None):
    """torch float64: dx, dy (2,H,W); c (H,W); b (C,H,W); init (3,C,H,W).  Returns x_K (3,C,H,W)."""
    L = lipschitz_scale(dx, dy) if L is None else L
    wxs, wys, bxs, bys = dx[0] * L, dy[0] * L, dx[1] * L, dy[1] * L
    K = 2 * (its // 2)
    s = fista_factors(max(its, 1))
    x = init
    y = init
    for k in range(K):
        yv = y if y.requires_grad else y.clone().requires_grad_(True)
        (g,) = torch.autograd.grad(energy_R(yv[0], yv[1], yv[2], wxs, wys, bxs, bys), yv, create_graph=create_graph)
        v = yv - g
        if not create_graph:
            v = v.detach()
        xn = torch.stack([prox_D(v[0], c, b), v[1], v[2]])
        y = xn + float(s[k]) * (xn - x)
        x = xn
    return x
