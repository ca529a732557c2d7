"""Pins what the TGV oracle's backward pass does differently from the chain rule, one deviation at a time, and the
per-pixel Lipschitz bound on weight fields that are not constant.

Deviations of the reference's backward (cudaTGV/cudaCode/TGVInpaintFistaBetas.cu:2621-3063), each behind a toggle of
the oracle:
  * y_{k+1} is rebuilt from the stored half-step values: u by the two-branch rule of the TV layer, v1 and v2 as the
    half-step values themselves, i.e. without their extrapolation (TGVInpaintFistaBetas.cu:1504-1515, 1536-1537);
  * a segment's first iteration k0 takes its Jacobian at the checkpointed y_{k0} (TGVInpaintFistaBetas.cu:2914-2917);
  * iteration 0's Jacobian is never applied (TGVInpaintFistaBetas.cu:2851-2925, 3047);
  * in the main adjoint kernel the rank-one Huber term that the v2 smoothness term of the triangle ABOVE a pixel sends
    to that pixel is scaled by W / hub^2 with hub = rsqrt(B), where all its siblings have W * hub^2
    (TGVInpaintFistaBetas.cu:355) -- i.e. it is B^2 times the true term;
  * completed adjoint iterates are clamped to +-2000 (TGVInpaintFistaBetas.cu:562-583).
Each test switches ONE on (float64, multipliers 1, guard off) and compares the oracle with tests/independent_chain.py,
the exact adjoint recursion whose Jacobian products torch.autograd takes from the layer's energy, with that one
deviation stated in a few lines of Python.
"""
import numpy as np
import pytest
import torch

from independent_chain import adjoint_chain, forward_history, rebuilt_y, reference_schedule
from independent_tgv import DELTA, energy_R, fdiff, lipschitz_scale, tgv_layer
from independent_tv import prox_D

torch.set_default_dtype(torch.float64)

ALL_OFF = dict(end_uses_ckpt_y=0, skip_iter0_adjoint=0, getyk_rebuild=0, scale_factors=0, clamp=0, guard=0, dw_div=0)


@pytest.fixture(scope="module")
def tgv_oracle():
    from oracle.oracle_lib import TGVOracle

    o = TGVOracle()
    o.set_quirks()
    return o


def problem(seed, c=2, h=8, w=9, amp=3.0, conf_density=0.5, beta_hi=3.0, off=0.5, vamp=0.7):
    rng = np.random.default_rng(seed)
    dx = np.stack([rng.uniform(0.05, 1.0, (h, w)), rng.uniform(0.5, beta_hi, (h, w))])[None]
    dy = np.stack([rng.uniform(0.05, 1.0, (h, w)), rng.uniform(0.5, beta_hi, (h, w))])[None]
    cf = (rng.random((1, 1, h, w)) < conf_density) * rng.uniform(0.2, 1.0, (1, 1, h, w))
    b = amp * rng.normal(0, 1, (1, c, h, w))
    u0 = b + rng.normal(0, off, (1, c, h, w))
    v0 = amp * rng.normal(0, vamp, (1, 2 * c, h, w))
    init = np.concatenate([u0, v0], axis=1)
    gout = rng.normal(0, 1, init.shape)
    return dx, dy, cf, b, init, gout


def as3(a, c):
    return a[0].reshape(3, c, *a.shape[2:])


def oracle_grads(o, p, its, pid=5, **quirks):
    dx, dy, cf, b, init, gout = p
    q = dict(ALL_OFF)
    q.update(quirks)
    try:
        o.set_quirks(**q)
        o.reset_id(pid)
        o.forward(dx, dy, cf, b, init, its, pid, f64=True)
        return o.backward(gout.copy(), dx, dy, cf, b, its, pid, f64=True)  # gx, gy, gc, gb, gi
    finally:
        o.set_quirks()


class Model:
    def __init__(self, p, its):
        dx, dy, cf, b, init, gout = p
        self.C = b.shape[1]
        self.dx = torch.tensor(dx[0], requires_grad=True)
        self.dy = torch.tensor(dy[0], requires_grad=True)
        self.c = torch.tensor(cf[0, 0], requires_grad=True)
        self.b = torch.tensor(b[0], requires_grad=True)
        self.init = torch.tensor(as3(init, self.C))
        self.gout = torch.tensor(as3(gout, self.C))
        self.L = lipschitz_scale()
        self.hist = forward_history(self.G, self.P, self.init, its)

    def G(self, y):
        yv = y if y.requires_grad else y.detach().clone().requires_grad_(True)
        L = self.L
        e = energy_R(yv[0], yv[1], yv[2], self.dx[0] * L, self.dy[0] * L, self.dx[1] * L, self.dy[1] * L)
        (g,) = torch.autograd.grad(e, yv, create_graph=True)
        return yv - g

    def P(self, v):
        return torch.stack([prox_D(v[0], self.c, self.b), v[1], v[2]])

    def grads(self, **kw):
        gi, (gdx, gdy), (gc, gb) = adjoint_chain(self.G, self.P, [self.dx, self.dy], [self.c, self.b], self.hist,
                                                 self.gout, **kw)
        n = lambda t: t.detach().numpy()
        return [n(gdx)[None], n(gdy)[None], n(gc)[None, None], n(gb)[None], n(gi).reshape(1, 3 * self.C, *gc.shape)]

    def v2_block_excess(self, y, g):
        """What the division in the v2 block of the upper triangle adds to G'(y)^T g.  The smoothness term of v2 in
        the triangle owned by q is huber(sqrt(B_q)), B_q = by_q |grad+ v2|_q^2, with weight W_q = min(1, delta /
        sqrt(B_q)); the rank-one part of its Hessian sends -(dW_q . g) by_q (v2_p - v2_q) to the pixel p below q
        (dW_q . g = directional derivative of W_q along g).  The reference scales that term by B_q^2."""
        by = (self.dy[1] * self.L).detach()
        v2, g2 = y[2].detach(), g[2].detach()

        def weight(v):
            ddx, ddy = fdiff(v)
            B = by * (ddx * ddx + ddy * ddy)
            return torch.where(B > DELTA * DELTA, DELTA / torch.sqrt(torch.clamp(B, min=1e-30)), torch.ones_like(B))

        _, dWg = torch.autograd.functional.jvp(weight, v2, g2)
        ddx, ddy = fdiff(v2)
        B = by * (ddx * ddx + ddy * ddy)
        true_term = -dWg * by * ddy                      # lands on the pixel below the owner
        excess = torch.where(B > DELTA * DELTA, true_term * (B * B - 1.0), torch.zeros_like(B))
        out = torch.zeros_like(y)
        out[2][..., 1:, :] = excess[..., :-1, :]
        return out


def assert_same(got, ref, tol=1e-9, names=("gx", "gy", "gc", "gb", "gi")):
    for nm, a, r in zip(names, got, ref):
        err = np.abs(a - r).max() / max(np.abs(r).max(), 1e-30)
        assert err <= tol, (nm, err)


def rebuilt_state(m, p, k):
    """(u, v1, v2) of y_{k+1} as the backward pass rebuilds them: u by the TV layer's rule from x05[k], x05[k-1];
    v1, v2 := x05[k] (no extrapolation)."""
    dx, dy, cf, b, init, gout = p
    x, y, x05, s = m.hist
    u = rebuilt_y(b[0], cf[0], x05[k][0].numpy(), x05[k - 1][0].numpy(), float(s[k]))
    return torch.stack([torch.tensor(u), x05[k][1], x05[k][2]])


# ------------------------------------------------------------------------------------------------
def test_the_chain_model_is_the_chain_rule(tgv_oracle):
    its = 6
    p = problem(30)
    m = Model(p, its)
    init_leaf = m.init.clone().requires_grad_(True)
    out = tgv_layer(m.dx, m.dy, m.c, m.b, init_leaf, its, create_graph=True)
    auto = torch.autograd.grad((out * m.gout).sum(), [m.dx, m.dy, m.c, m.b, init_leaf])
    n = lambda t: t.detach().numpy()
    auto = [n(auto[0])[None], n(auto[1])[None], n(auto[2])[None, None], n(auto[3])[None],
            n(auto[4]).reshape(1, 3 * m.C, *m.c.shape)]
    assert_same(m.grads(), auto, 1e-10)
    assert_same(oracle_grads(tgv_oracle, p, its), auto, 1e-9)


# ------------------------------------------------------------------------------------------------
# y rebuild
# ------------------------------------------------------------------------------------------------
def test_rebuilt_u_is_the_true_u_without_a_data_term_and_v_is_not(tgv_oracle):
    # c = 0 makes the u rule exact; what is left of the rebuild is v := x05 (no extrapolation), so the model with
    # ONLY that substitution must reproduce the oracle, and it must differ from the chain rule
    dx, dy, cf, b, init, gout = problem(41)
    p = (dx, dy, 0 * cf, b, init, gout)
    its = 10
    m = Model(p, its)
    x, y, x05, s = m.hist
    k0s = set(reference_schedule(its))
    lin_y = lambda k1: y[k1] if (k1 - 1) in k0s or k1 == 0 else torch.stack([y[k1][0], x05[k1 - 1][1], x05[k1 - 1][2]])
    got = oracle_grads(tgv_oracle, p, its, getyk_rebuild=1)
    assert_same(got, m.grads(lin_y=lin_y))
    plain = oracle_grads(tgv_oracle, p, its)
    assert np.abs(got[0] - plain[0]).max() > 1e-6 * np.abs(plain[0]).max()


def test_rebuild_is_inert_when_no_step_rebuilds(tgv_oracle):
    # its = 3 runs iterations 0 and 1 in one segment: the sweep is [first step][segment start], neither rebuilds y
    p = problem(42)
    assert_same(oracle_grads(tgv_oracle, p, 3, getyk_rebuild=1), oracle_grads(tgv_oracle, p, 3), 1e-13)


@pytest.mark.parametrize("its", [6, 10, 20])
def test_rebuild_rule_in_general(tgv_oracle, its):
    p = problem(43 + its, off=2.5)
    m = Model(p, its)
    x, y, x05, s = m.hist
    k0s = set(reference_schedule(its))
    lin_y = lambda k1: y[k1] if (k1 - 1) in k0s or k1 == 0 else rebuilt_state(m, p, k1 - 1)
    got = oracle_grads(tgv_oracle, p, its, getyk_rebuild=1)
    assert_same(got, m.grads(lin_y=lin_y))


# ------------------------------------------------------------------------------------------------
# checkpointed y at segment starts, skipped iteration 0, clamp
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("its", [2, 5, 10, 20])
def test_segment_starts_take_the_checkpointed_y(tgv_oracle, its):
    p = problem(50 + its)
    m = Model(p, its)
    x, y, x05, s = m.hist
    k0s = set(reference_schedule(its))
    lin_y = lambda k1: y[k1 - 1] if (k1 - 1) in k0s else y[k1]
    got = oracle_grads(tgv_oracle, p, its, end_uses_ckpt_y=1)
    assert_same(got, m.grads(lin_y=lin_y))
    if its >= 5:
        plain = oracle_grads(tgv_oracle, p, its)
        assert np.abs(got[0] - plain[0]).max() > 1e-7 * np.abs(plain[0]).max()


@pytest.mark.parametrize("its", [4, 10])
def test_skipped_iteration_0_is_a_sub_run_started_at_x1(tgv_oracle, its):
    # s_0 = 0, so y_1 = x_1: autograd of iterations 1..K-1 from a leaf x_1 gives the returned "gradient wrt the
    # starting point" and the weight gradients; c and b keep the full run's gradients (iteration 0's prox is
    # back-propagated)
    p = problem(60 + its)
    m = Model(p, its)
    x, y, x05, s = m.hist
    K = 2 * (its // 2)
    x1 = x[1].clone().requires_grad_(True)
    xs, ys = x1, x1
    for k in range(1, K):
        xn = m.P(m.G(ys))
        ys = xn + float(s[k]) * (xn - xs)
        xs = xn
    g_x1, g_dx, g_dy = torch.autograd.grad((xs * m.gout).sum(), [x1, m.dx, m.dy])
    got = oracle_grads(tgv_oracle, p, its, skip_iter0_adjoint=1)
    full = oracle_grads(tgv_oracle, p, its)
    assert_same([got[0], got[1], got[4]],
                [g_dx.numpy()[None], g_dy.numpy()[None], g_x1.numpy().reshape(got[4].shape)], names=("gx", "gy", "gi"))
    assert_same([got[2], got[3]], [full[2], full[3]], 1e-12, names=("gc", "gb"))
    assert_same(got, m.grads(skip_iter0=True))
    assert np.abs(got[4] - full[4]).max() > 1e-3 * np.abs(full[4]).max()


def test_adjoint_iterates_are_clamped_at_2000(tgv_oracle):
    dx, dy, cf, b, init, gout = problem(70)
    p = (dx, dy, cf, b, init, gout * 4.0e3)
    its = 10
    m = Model(p, its)
    got = oracle_grads(tgv_oracle, p, its, clamp=1)
    assert_same(got, m.grads(clamp=2000.0))
    free = oracle_grads(tgv_oracle, p, its)
    assert np.abs(got[4]).max() <= 2000.0 < np.abs(free[4]).max()
    assert np.abs(got[3] - free[3]).max() > 0.05 * np.abs(free[3]).max()


# ------------------------------------------------------------------------------------------------
# the division in the upper triangle's v2 block
# ------------------------------------------------------------------------------------------------
def test_v2_block_division_is_the_true_term_times_B_squared(tgv_oracle):
    dx, dy, cf, b, init, gout = problem(80, c=1, vamp=1.5)
    m = Model((dx, dy, cf, b, init, gout), 2)
    y = m.init
    g = m.gout
    out_q, gw_q = tgv_oracle.jt(dx[0], dy[0], y[:, 0].numpy(), g[:, 0].numpy(), end_form=False, q7=True)
    out_m, gw_m = tgv_oracle.jt(dx[0], dy[0], y[:, 0].numpy(), g[:, 0].numpy(), end_form=False, q7=False)
    excess = m.v2_block_excess(y, g)[:, 0].numpy()
    assert (excess[2] != 0).mean() > 0.3 and not excess[:2].any() and not excess[2, 0].any()
    np.testing.assert_allclose(out_q - out_m, excess, rtol=0, atol=1e-10 * np.abs(excess).max())
    np.testing.assert_array_equal(gw_q, gw_m)


@pytest.mark.parametrize("its", [4, 10])
def test_v2_block_division_through_the_whole_backward(tgv_oracle, its):
    p = problem(81 + its, vamp=1.5)
    m = Model(p, its)
    got = oracle_grads(tgv_oracle, p, its, dw_div=1)
    assert_same(got, m.grads(jt_extra=m.v2_block_excess))
    plain = oracle_grads(tgv_oracle, p, its)
    assert np.abs(got[4] - plain[4]).max() > 1e-6 * np.abs(plain[4]).max()


# ------------------------------------------------------------------------------------------------
# everything at once
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("its,scale", [(10, 1.0), (20, 1.0), (9, 5.0e3)])
def test_all_deviations_together(tgv_oracle, its, scale):
    dx, dy, cf, b, init, gout = problem(90 + its, off=1.5, vamp=1.0)
    p = (dx, dy, cf, b, init, gout * scale)
    m = Model(p, its)
    x, y, x05, s = m.hist
    k0s = set(reference_schedule(its))
    lin_y = lambda k1: y[k1 - 1] if (k1 - 1) in k0s else rebuilt_state(m, p, k1 - 1)
    # the segment-start kernel has its own arithmetic form WITHOUT the division (TGVInpaintFistaBetas.cu:1118-1333)
    extra = lambda yy, gg: m.v2_block_excess(yy, gg) if not any(yy is y[k] for k in k0s) else torch.zeros_like(yy)
    got = oracle_grads(tgv_oracle, p, its, end_uses_ckpt_y=1, skip_iter0_adjoint=1, getyk_rebuild=1, clamp=1, dw_div=1)
    assert_same(got, m.grads(lin_y=lin_y, skip_iter0=True, clamp=2000.0, jt_extra=extra))


# ------------------------------------------------------------------------------------------------
# Lipschitz bound on weight fields that vary
# ------------------------------------------------------------------------------------------------
def lipschitz_brute_force(dx, dy, crossed=True):
    """Per-pixel bound of TGVInpaintFistaBetas.cu:101-148, one pixel at a time, every read written as [row, col].
    The kernel fetches textures at (x = column, y = row).  Its four "previous neighbour" reads of beta are crossed
    over: the one added under `w > 0` is fetched at (column w, row h-1) and the one added under `h > 0` at
    (column w-1, row h); a fetch outside the field returns the border texel (clamp addressing).  crossed=False reads
    them as their names say, for comparison."""
    wgt_x, beta_x = dx
    wgt_y, beta_y = dy
    H, W = wgt_x.shape
    at = lambda f, row, col: f[min(max(row, 0), H - 1), min(max(col, 0), W - 1)]
    up, left = ((0, -1), (-1, 0)) if crossed else ((-1, 0), (0, -1))  # (row, col) offsets read under h > 0 / w > 0
    out = np.zeros((H, W))
    for h in range(H):
        for w in range(W):
            su = s1 = s2 = 0.0
            if h > 0:
                su += 3 * at(wgt_y, h - 1, w)
                s1 += 2 * at(beta_x, h + up[0], w + up[1])
                s2 += 2 * at(beta_y, h + up[0], w + up[1])
            if w > 0:
                su += 3 * at(wgt_x, h, w - 1)
                s1 += 2 * at(beta_x, h + left[0], w + left[1])
                s2 += 2 * at(beta_y, h + left[0], w + left[1])
            own_x = at(wgt_x, h, w) if w < W - 1 else 0.0
            own_y = at(wgt_y, h, w) if h < H - 1 else 0.0
            su += 3 * (own_y + own_x)
            s1 += (2 * at(beta_x, h, w) if w < W - 1 else 0.0) + (2 * at(beta_x, h, w) if h < H - 1 else 0.0) + 3 * own_x
            s2 += (2 * at(beta_y, h, w) if w < W - 1 else 0.0) + (2 * at(beta_y, h, w) if h < H - 1 else 0.0) + 3 * own_y
            out[h, w] = max(su, s1, s2)
    return out


@pytest.mark.parametrize("seed,h,w,beta_hi", [(1, 6, 7, 3.0), (2, 9, 5, 9.0), (3, 1, 8, 9.0), (4, 7, 1, 9.0), (5, 2, 2, 20.0)])
def test_lipschitz_bound_on_varying_fields(tgv_oracle, seed, h, w, beta_hi):
    rng = np.random.default_rng(seed)
    dx = np.stack([rng.uniform(0, 1.0, (h, w)), rng.uniform(0, beta_hi, (h, w))])
    dy = np.stack([rng.uniform(0, 1.0, (h, w)), rng.uniform(0, beta_hi, (h, w))])
    L, st = tgv_oracle.lipschitz(dx, dy, f64=True)
    ref = lipschitz_brute_force(dx, dy)
    np.testing.assert_allclose(st, ref, rtol=1e-14, atol=0)
    assert np.isclose(L, 1.0 / (max(float(np.float32(32.000001)), ref.max()) + float(np.float32(0.01))), rtol=1e-12)
    if h > 2 and w > 2:  # the crossed-over reads matter on fields that vary
        assert np.abs(ref - lipschitz_brute_force(dx, dy, crossed=False)).max() > 0.1
