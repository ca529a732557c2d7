"""Independent statements of what the quadratic fit and the histogram median compute, written from
their definitions (not from the reference kernels) in fp64.  They pin the CPU oracle."""
import numpy as np
import torch


def displaced_indices(flow, h, w):
    """Nearest pixel of (x + u, y + v), its clamped 4-neighbours and the inside-the-image mask."""
    ys, xs = torch.meshgrid(torch.arange(h, dtype=flow.dtype), torch.arange(w, dtype=flow.dtype), indexing="ij")
    px, py = xs + flow[:, 0], ys + flow[:, 1]
    inside = (px <= w - 1) & (px >= 0) & (py <= h - 1) & (py >= 0)
    ix = torch.floor(px + 0.5).long().clamp(0, w - 1)
    iy = torch.floor(py + 0.5).long().clamp(0, h - 1)
    return inside, ix, iy


def matching_costs(feat0, feat1, ix, iy):
    """Scalar products of feat0 at the pixel with feat1 at the displaced pixel and its 4-neighbours."""
    n, c, h, w = feat0.shape
    bidx = torch.arange(n).view(n, 1, 1).expand(n, h, w)

    def at(yy, xx):
        g = feat1[bidx, :, yy.clamp(0, h - 1), xx.clamp(0, w - 1)]  # (n,h,w,c)
        return (g * feat0.permute(0, 2, 3, 1)).sum(-1)

    return at(iy, ix), at(iy, ix + 1), at(iy, ix - 1), at(iy + 1, ix), at(iy - 1, ix)


def quadfit(feat0, feat1, flow):
    """(N,3,H,W): offset of the maximum of the parabola through the three costs along x, the same along y,
    and the cost at the centre plus the two parabolas' gains over it.  An axis is fitted only when the
    parabola is strictly concave, its vertex lies within one pixel and the centre is not on the border."""
    n, c, h, w = feat0.shape
    inside, ix, iy = displaced_indices(flow, h, w)
    c0, cxp, cxm, cyp, cym = matching_costs(feat0, feat1, ix, iy)

    def axis(cp, cm, interior):
        a = 0.5 * (cp + cm) - c0  # parabola a t^2 + b t + c0 through t = -1, 0, 1
        b = 0.5 * (cp - cm)
        ok = (a < 0) & (b.abs() <= 2 * a.abs()) & interior
        safe = torch.where(ok, a, -torch.ones_like(a))
        vertex = torch.where(ok, -b / (2 * safe), torch.zeros_like(a))
        gain = torch.where(ok, -b * b / (4 * safe), torch.zeros_like(a))
        return vertex, gain

    fx, gx = axis(cxp, cxm, (ix > 0) & (ix < w - 1))
    fy, gy = axis(cyp, cym, (iy > 0) & (iy < h - 1))
    out = torch.stack([fx, fy, c0 + gx + gy], 1)
    return out * inside.unsqueeze(1)


def polyfit_axis(cm, c0, cp):
    """Vertex and peak value of the least-squares (here: interpolating) parabola, from numpy.polyfit."""
    a, b, c = np.polyfit([-1.0, 0.0, 1.0], [cm, c0, cp], 2)
    return a, b, c


def histogram_median(p):
    """Median of the density that is constant p[c] on [c - 1/2, c + 1/2): inverse of its piecewise-linear CDF."""
    d = len(p)
    cdf = np.concatenate([[0.0], np.cumsum(p)])
    knots = np.arange(d + 1) - 0.5
    return float(np.interp(0.5, cdf, knots))


def normalised_median(vol):
    """Differentiable median of the sum-normalised histogram, and the normalised-free mass of its bin.
    vol: (..., D) torch tensor.  Returns (median, mass)."""
    q = vol / vol.sum(-1, keepdim=True)
    cdf = torch.cumsum(q, -1)
    k = (cdf < 0.5).sum(-1, keepdim=True).clamp(max=vol.shape[-1] - 1)  # first bin whose cdf reaches 1/2
    before = torch.gather(cdf - q, -1, k)
    qk = torch.gather(q, -1, k)
    median = k.to(vol.dtype) - 0.5 + (0.5 - before) / qk
    return median.squeeze(-1), torch.gather(vol, -1, k).squeeze(-1)
