"""Independent statement of the TV inpainting layer, written from its energy and not from the
reference's stencil code; used only to pin the oracle.

Energy (weights already divided by the Lipschitz constant 8, delta = 0.1):

    R(u) = sum_p huber_delta( sqrt( wx_p (u_p - u_right)^2 + wy_p (u_p - u_down)^2 ) )
    D(u) = sum_p c_p huber_1(u_p - b_p)          huber_e(a) = a^2/2 (|a| <= e), e|a| - e^2/2

FISTA with unit step: v = y - grad R(y) (torch autograd supplies the gradient), x+ = prox_D(v),
y+ = x+ + (t-1)/t+ (x+ - x).  Channels never couple.
"""
import numpy as np
import torch

DELTA = float(np.float32(0.1))


def energy_R(u, wxs, wys, delta=DELTA):
    """u: (..., H, W); wxs, wys broadcastable (H, W) scaled weights."""
    dx = torch.zeros_like(u)
    dy = torch.zeros_like(u)
    dx[..., :, :-1] = u[..., :, :-1] - u[..., :, 1:]
    dy[..., :-1, :] = u[..., :-1, :] - u[..., 1:, :]
    A = wxs * dx * dx + wys * dy * dy
    safe = torch.sqrt(torch.clamp(A, min=1e-30))
    return torch.where(A <= delta * delta, 0.5 * A, delta * safe - 0.5 * delta * delta).sum()


def energy_D(u, c, b):
    d = u - b
    ad = d.abs()
    return (c * torch.where(ad <= 1.0, 0.5 * d * d, ad - 0.5)).sum()


def prox_D(v, c, b):
    """argmin_x c*huber_1(x-b) + (x-v)^2/2."""
    d = v - b
    return b + torch.where(d.abs() <= 1.0 + c, d / (1.0 + c), d - c * torch.sign(d))


def fista_factors(its, as_float32=True):
    """(t_k - 1)/t_{k+1} of the textbook recurrence t_{k+1} = (1 + sqrt(1 + 4 t_k^2))/2, t_0 = 1."""
    t, out = 1.0, []
    for _ in range(its):
        tn = (1.0 + np.sqrt(1.0 + 4.0 * t * t)) / 2.0
        out.append(max(0.0, (t - 1.0) / tn))
        t = tn
    out = np.array(out)
    return out.astype(np.float32).astype(np.float64) if as_float32 else out


def tv_layer(wx, wy, c, b, init, its, create_graph=False):
    """All arguments torch float64: wx, wy, c (H,W); b, init (C,H,W).  Returns x_K, K = 2*(its//2)."""
    wxs, wys = wx / 8.0, wy / 8.0
    K = 2 * (its // 2)
    s = fista_factors(max(its, 1))
    x = init
    y = init
    for k in range(K):
        yv = y if y.requires_grad else y.clone().requires_grad_(True)
        (g,) = torch.autograd.grad(energy_R(yv, wxs, wys), yv, create_graph=create_graph)
        v = yv - g
        if not create_graph:
            v = v.detach()
        xn = prox_D(v, c, b)
        y = xn + float(s[k]) * (xn - x)
        x = xn
    return x
