"""Independent model of the layers' hand-unrolled backward pass, used only to pin the oracles' quirk branches.

The forward pass is an unrolled recursion (K iterations, all of them in float64 here):

    x05_k   = G(y_k; w)            gradient step on the regulariser, G = y - grad_y R(y; w)
    x_{k+1} = P(x05_k; c, b)       pointwise prox of the data term (TGV: on u only)
    y_{k+1} = x_{k+1} + s_k (x_{k+1} - x_k)

and its exact adjoint is the recursion (g_x[K] = upstream gradient, partial g_x[K-1] = 0)

    g05[k]    = P'(x05_k)^T g_x[k+1]                 (+ the c and b gradients of that prox)
    g_y[k]    = G'(y_k)^T g05[k]                     (+ the w gradients of that gradient step)
    g_x[k]    = (partial g_x[k]) + (1 + s_{k-1}) g_y[k]
    partial g_x[k-1] = -s_{k-1} g_y[k]

ending with g_init = g_y[0] + partial g_x[0].  Every product with a transposed Jacobian is taken by torch.autograd
from the *energies* in independent_tv / independent_tgv (a vector-Jacobian product of G or P at a given point), so
no stencil code of the reference or of the oracle enters.  With every option at its default the chain is the chain
rule (a test equates it with whole-graph autograd); the options switch on, one at a time, what the reference's
backward does differently:

    lin_y(k+1)   the point at which G' is taken when g05[k+1] is pulled back (the reference does not always use
                 the y_{k+1} of the forward pass);
    skip_iter0   stop after g05[0] and return g_x[1] as the gradient wrt the starting point;
    clamp        clamp every completed g_x[k] to +-clamp;
    jt_extra     a term added to every product G'(y)^T g (the reference's Jacobian differs from G' in one block).
"""
import numpy as np
import torch

from independent_tv import fista_factors


def reference_schedule(its):
    """Checkpoint iterations 2*floor(i*sqrt(its)/2), i < floor(sqrt(its)) (TVInpaintFista.cu:1499-1504)."""
    root = np.sqrt(float(its))
    return [int(2 * np.floor(i * root * 0.5)) for i in range(int(np.floor(root)))]


def rebuilt_y(b, c, xa, xb, t):
    """y_{k+1} as the backward pass rebuilds it from xa = x05[k], xb = x05[k-1] (TVInpaintFista.cu:1149-1165), stated
    with the proxes it amounts to: where |b - xa| <= 1 + c both iterates take the QUADRATIC prox (c b + v)/(1 + c),
    whatever regime x05[k-1] is in; elsewhere both take the prox of the pure L1 data term, v + c sign(b - v) when
    |b - v| >= c and b otherwise."""
    quad = np.abs(b - xa) <= 1.0 + c
    q = lambda v: (c * b + v) / (1.0 + c)
    sgn = lambda v: np.where(b - v < 0, -1.0, 1.0)
    l1 = lambda v: np.where(np.abs(b - v) >= c, v + sgn(v) * c, b)
    xk = np.where(quad, q(xa), l1(xa))
    xkm = np.where(quad, q(xb), l1(xb))
    return xk + t * (xk - xkm)


def forward_history(G, P, init, its):
    """Runs the recursion without building a graph.  Returns lists x[0..K], y[0..K], x05[0..K-1] and the factors."""
    K = 2 * (its // 2)
    s = fista_factors(max(its, 1))
    x, y = [init.detach().clone()], [init.detach().clone()]
    x05 = []
    for k in range(K):
        v = G(y[k]).detach()
        xn = P(v).detach()
        x05.append(v)
        y.append(xn + float(s[k]) * (xn - x[k]))
        x.append(xn)
    return x, y, x05, s


def _vjp(fn, point, cot, params):
    """cot^T d fn / d(point, params) at `point`; params are leaf tensors that fn closes over."""
    p = point.detach().clone().requires_grad_(True)
    out = fn(p)
    grads = torch.autograd.grad(out, [p] + list(params), grad_outputs=cot, allow_unused=True)
    return [g if g is not None else torch.zeros_like(t) for g, t in zip(grads, [p] + list(params))]


def adjoint_chain(G, P, w_params, d_params, hist, gout, lin_y=None, skip_iter0=False, clamp=None, jt_extra=None):
    """G(y) closes over the leaf tensors w_params, P(v) over d_params.  Returns (g_init, [g_w...], [g_d...])."""
    x, y, x05, s = hist
    K = len(x05)
    gw = [torch.zeros_like(t) for t in w_params]
    gd = [torch.zeros_like(t) for t in d_params]
    if K == 0:
        return gout.clone(), gw, gd
    lin_y = lin_y or (lambda k: y[k])
    gx_total = gout.clone()
    g05, *dd = _vjp(P, x05[K - 1], gx_total, d_params)
    gd = [a + b for a, b in zip(gd, dd)]
    gx_partial = torch.zeros_like(gout)
    for k in range(K - 2, -1, -1):  # pulls g05[k+1] back through the gradient step of iteration k+1
        gy, *dw = _vjp(G, lin_y(k + 1), g05, w_params)
        if jt_extra is not None:
            gy = gy + jt_extra(lin_y(k + 1), g05)
        gw = [a + b for a, b in zip(gw, dw)]
        gx_total = gx_partial + (1.0 + float(s[k])) * gy
        if clamp is not None:
            gx_total = torch.clamp(gx_total, -clamp, clamp)
        gx_partial = -float(s[k]) * gy
        g05, *dd = _vjp(P, x05[k], gx_total, d_params)
        gd = [a + b for a, b in zip(gd, dd)]
    if skip_iter0:
        return gx_total, gw, gd
    gy, *dw = _vjp(G, lin_y(0), g05, w_params)
    if jt_extra is not None:
        gy = gy + jt_extra(lin_y(0), g05)
    gw = [a + b for a, b in zip(gw, dw)]
    return gy + gx_partial, gw, gd
