"""Synthetic inputs for the inpainting layers (numpy, deterministic per seed).

The reference ships no data and no example script; these generators produce flow fields,
confidences and edge weights of the kind its README describes (README.md:64-71 of the reference):
a smooth flow, a sparse confidence mask and edge weights exp(-10 |grad I|) in (0, 1].
"""
import numpy as np

try:  # scipy is only needed for the smooth guidance image
    from scipy.ndimage import gaussian_filter
except Exception:  # pragma: no cover
    gaussian_filter = None


def smooth_image(rng, h, w, sigma=4.0):
    """Gaussian-smoothed uniform noise rescaled to [0, 1]."""
    img = rng.random((h, w))
    if gaussian_filter is not None:
        img = gaussian_filter(img, sigma, mode="nearest")
    else:  # separable box blur fallback, three passes
        k = int(2 * sigma) | 1
        ker = np.ones(k) / k
        for _ in range(3):
            img = np.apply_along_axis(lambda r: np.convolve(np.pad(r, k // 2, mode="edge"), ker, "valid"), 1, img)
            img = np.apply_along_axis(lambda r: np.convolve(np.pad(r, k // 2, mode="edge"), ker, "valid"), 0, img)
    img = img - img.min()
    return img / max(img.max(), 1e-12)


def edge_weights(img):
    """wx = exp(-10 |I(h,w+1) - I(h,w)|), wy = exp(-10 |I(h+1,w) - I(h,w)|); last column/row: 1."""
    dxi = np.zeros_like(img)
    dyi = np.zeros_like(img)
    dxi[:, :-1] = np.abs(img[:, 1:] - img[:, :-1])
    dyi[:-1, :] = np.abs(img[1:, :] - img[:-1, :])
    return np.exp(-10.0 * dxi), np.exp(-10.0 * dyi)


def sinusoid_flow(rng, c, h, w, amplitude=8.0, noise=0.5):
    """Sum of 4 random low-frequency sinusoids (<= 3 cycles across the image) spanning +-amplitude."""
    yy, xx = np.meshgrid(np.arange(h) / h, np.arange(w) / w, indexing="ij")
    out = np.zeros((c, h, w))
    for ch in range(c):
        f = np.zeros((h, w))
        for _ in range(4):
            fx, fy = rng.uniform(-3, 3, 2)
            ph = rng.uniform(0, 2 * np.pi)
            f += rng.uniform(0.5, 1.0) * np.sin(2 * np.pi * (fx * xx + fy * yy) + ph)
        f *= amplitude / max(np.abs(f).max(), 1e-12)
        out[ch] = f + rng.normal(0, noise, (h, w))
    return out


def rectangle_flow(rng, c, h, w, count=8, noise=1.0):
    """Piecewise-constant flow: `count` random rectangles with values U(-20, 20), plus noise."""
    out = np.zeros((c, h, w))
    for _ in range(count):
        y0, y1 = sorted(rng.integers(0, h, 2))
        x0, x1 = sorted(rng.integers(0, w, 2))
        for ch in range(c):
            out[ch, y0:y1 + 1, x0:x1 + 1] = rng.uniform(-20, 20)
    return out + rng.normal(0, noise, (c, h, w))


def tv_inputs(n, c, h, w, seed=0, conf_density=0.3, flow="sinusoid", dense_conf=False):
    """Inputs of one TV layer call.

    Returns a dict of float32 arrays: dx, dy, dc (n,1,h,w); db, di, grad (n,c,h,w).
    `di` equals `db` (the README's simplest initialisation).
    """
    rng = np.random.default_rng(seed)
    dx = np.empty((n, 1, h, w), np.float32)
    dy = np.empty((n, 1, h, w), np.float32)
    dc = np.empty((n, 1, h, w), np.float32)
    db = np.empty((n, c, h, w), np.float32)
    for s in range(n):
        db[s] = sinusoid_flow(rng, c, h, w) if flow == "sinusoid" else rectangle_flow(rng, c, h, w)
        if dense_conf:
            conf = rng.random((h, w))
            conf[rng.random((h, w)) < 0.3] = 0.0
        else:
            conf = (rng.random((h, w)) < conf_density) * rng.uniform(0.2, 1.0, (h, w))
        dc[s, 0] = conf
        wx, wy = edge_weights(smooth_image(rng, h, w))
        dx[s, 0], dy[s, 0] = wx, wy
    grad = rng.normal(0, 1, (n, c, h, w)).astype(np.float32)
    return dict(dx=dx, dy=dy, dc=dc, db=db, di=db.copy(), grad=grad)


# The five configurations quoted for this path: (kind, n, c, h, w, its, generator keyword arguments)
CONFIGS = {
    0: dict(kind="tv", n=1, c=2, h=64, w=128, its=20, gen=dict(conf_density=0.3)),
    1: dict(kind="tv", n=4, c=2, h=384, w=1248, its=100, gen=dict(conf_density=0.2)),
    2: dict(kind="tgv", n=4, c=2, h=384, w=1248, its=100, gen=dict(conf_density=0.2)),
    3: dict(kind="tv_hierarchy", n=2, c=2, levels=[(112, 256), (224, 512), (448, 1024)], its=50,
            gen=dict(conf_density=0.25)),
    4: dict(kind="tv", n=16, c=2, h=256, w=512, its=200, gen=dict(flow="rectangles", dense_conf=True)),
    # the two layers upstream of the inpainting layer, at the headline image size
    5: dict(kind="quadfit", n=4, c=32, h=384, w=1248, gen=dict()),
    6: dict(kind="median", n=4, h=384, w=1248, d=33, gen=dict()),
}


def config_inputs(idx, seed=0):
    cfg = CONFIGS[idx]
    if cfg["kind"] == "tv":
        return cfg, tv_inputs(cfg["n"], cfg["c"], cfg["h"], cfg["w"], seed=seed, **cfg["gen"])
    if cfg["kind"] == "tgv":
        return cfg, tgv_inputs(cfg["n"], cfg["c"], cfg["h"], cfg["w"], seed=seed, **cfg["gen"])
    if cfg["kind"] == "quadfit":
        return cfg, quadfit_inputs(cfg["n"], cfg["c"], cfg["h"], cfg["w"], seed=seed, **cfg["gen"])
    if cfg["kind"] == "median":
        return cfg, median_inputs(cfg["n"], cfg["h"], cfg["w"], cfg["d"], seed=seed, **cfg["gen"])
    raise ValueError("config %d is assembled by its caller (hierarchy)" % idx)


def tgv_inputs(n, c, h, w, seed=0, conf_density=0.2, alpha0=1.0, alpha1=2.0):
    """Inputs of one TGV layer call.

    dx, dy: (n,2,h,w) -- channel 0 the edge weight times alpha0, channel 1 the constant alpha1;
    dc: (n,1,h,w); db: (n,c,h,w); di, grad: (n,3c,h,w) in variable-major order (u, v1, v2) with the
    auxiliary variables initialised to zero.
    """
    base = tv_inputs(n, c, h, w, seed=seed, conf_density=conf_density)
    rng = np.random.default_rng(seed + 1000003)
    dx = np.empty((n, 2, h, w), np.float32)
    dy = np.empty((n, 2, h, w), np.float32)
    dx[:, 0], dy[:, 0] = base["dx"][:, 0] * alpha0, base["dy"][:, 0] * alpha0
    dx[:, 1], dy[:, 1] = alpha1, alpha1
    di = np.zeros((n, 3 * c, h, w), np.float32)
    di[:, :c] = base["db"]
    grad = rng.normal(0, 1, (n, 3 * c, h, w)).astype(np.float32)
    return dict(dx=dx, dy=dy, dc=base["dc"], db=base["db"], di=di, grad=grad)


def quadfit_inputs(n, c, h, w, seed=0, flow_channels=2, amplitude=8.0, jitter=0.6):
    """Inputs of one quadratic-fit call: feat1 is a smooth random feature map, feat0 is feat1 looked up
    at the true (smooth, sub-pixel) flow, and the flow handed to the layer is the true flow plus a
    jitter of about half a pixel -- the situation of a matching cost that peaks next to the rounded
    displaced position.  Near the image border part of the displaced pixels fall outside.

    feat0, feat1: (n,c,h,w); flow: (n,flow_channels,h,w); grad: (n,3,h,w).
    """
    from scipy.ndimage import map_coordinates

    rng = np.random.default_rng(seed)
    feat0 = np.empty((n, c, h, w), np.float32)
    feat1 = np.empty((n, c, h, w), np.float32)
    flow = np.zeros((n, flow_channels, h, w), np.float32)
    ys, xs = np.mgrid[0:h, 0:w].astype(np.float64)
    for i in range(n):
        true = sinusoid_flow(rng, 2, h, w, amplitude=amplitude, noise=0.0).astype(np.float64)
        coords = np.stack([ys + true[1], xs + true[0]])
        for k in range(c):
            f = rng.standard_normal((h, w))
            if gaussian_filter is not None:
                f = gaussian_filter(f, 1.5, mode="nearest")
            f = f / max(f.std(), 1e-12)
            feat1[i, k] = f
            feat0[i, k] = map_coordinates(f, coords, order=1, mode="nearest")
        flow[i, 0] = true[0] + rng.normal(0, jitter, (h, w))
        flow[i, 1] = true[1] + rng.normal(0, jitter, (h, w))
        if flow_channels > 2:
            flow[i, 2:] = rng.random((flow_channels - 2, h, w))
    grad = rng.normal(0, 1, (n, 3, h, w)).astype(np.float32)
    return dict(feat0=feat0, feat1=feat1, flow=flow, grad=grad)


def median_inputs(n, h, w, d, seed=0, spread=2.0, empty_fraction=0.02):
    """Inputs of one median call: per pixel a normalised histogram over d displacement bins, a noisy
    bump around a smoothly varying centre; a few pixels carry less than half a unit of mass (the
    layer leaves them at zero).

    vol: (n,h,w,d) with the bins innermost; grad: (n,2,h,w).
    """
    rng = np.random.default_rng(seed)
    vol = np.empty((n, h, w, d), np.float32)
    bins = np.arange(d, dtype=np.float64)
    for i in range(n):
        centre = (d - 1) * (0.5 + 0.4 * sinusoid_flow(rng, 1, h, w, amplitude=1.0, noise=0.0)[0])
        logit = -0.5 * ((bins - centre[..., None]) / spread) ** 2 + 0.5 * rng.standard_normal((h, w, d))
        p = np.exp(logit - logit.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        p[rng.random((h, w)) < empty_fraction] *= 0.3
        vol[i] = p
    grad = rng.normal(0, 1, (n, 2, h, w)).astype(np.float32)
    return dict(vol=vol, grad=grad)
