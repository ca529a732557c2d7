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
}


def config_inputs(idx, seed=0):
    cfg = CONFIGS[idx]
    if cfg["kind"] == "tv":
        return cfg, tv_inputs(cfg["n"], cfg["c"], cfg["h"], cfg["w"], seed=seed, **cfg["gen"])
    if cfg["kind"] == "tgv":
        return cfg, tgv_inputs(cfg["n"], cfg["c"], cfg["h"], cfg["w"], seed=seed, **cfg["gen"])
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
