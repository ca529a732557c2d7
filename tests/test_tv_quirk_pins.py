"""Pins what the TV oracle's backward pass does differently from the chain rule, one deviation at a time.

The reference's hand-written backward (cudaTV/cudaCode/TVInpaintFista.cu:1570-1831) is the chain rule except that
  * the point y_{k+1} at which the gradient step's Jacobian is taken is rebuilt from the stored half-step values by
    a two-branch rule (get_yk, TVInpaintFista.cu:1149-1165) instead of being the forward pass's own y_{k+1};
  * at the first iteration k0 of every checkpoint segment the checkpointed y_{k0} stands in for y_{k0+1}
    (TVInpaintFista.cu:1724-1727);
  * the Jacobian of iteration 0 is never applied and g_x[1] is returned as the gradient wrt the starting point
    (TVInpaintFista.cu:1696-1729, 1816);
  * every completed g_x[k] is clamped to +-1e4 (TVInpaintFista.cu:797-799).
The oracle has one toggle per deviation.  Each test switches ONE on (float64, multipliers 1, guard off) and compares
the oracle with tests/independent_chain.py: the exact adjoint recursion whose Jacobian products torch.autograd takes
from the layer's energy, with that one deviation stated in a line of Python.  A wrong slot index, sign, regime rule
or schedule in the oracle fails these comparisons; special cases that the mathematics fixes without any model (no
data term, regimes that never change, a fixed point, a sub-run started at x_1) are checked as well.
"""
import numpy as np
import pytest
import torch

from independent_chain import adjoint_chain, forward_history, rebuilt_y, reference_schedule
from independent_tv import energy_R, prox_D

torch.set_default_dtype(torch.float64)

ALL_OFF = dict(end_uses_ckpt_y=0, skip_iter0_adjoint=0, getyk_rebuild=0, scale_factors=0, clamp=0, guard=0)


def problem(seed, c=2, h=9, w=11, amp=3.0, conf_density=0.5, off=0.5):
    rng = np.random.default_rng(seed)
    wx = rng.uniform(0.05, 1.0, (1, 1, h, w))
    wy = rng.uniform(0.05, 1.0, (1, 1, h, w))
    cf = (rng.random((1, 1, h, w)) < conf_density) * rng.uniform(0.2, 1.0, (1, 1, h, w))
    b = amp * rng.normal(0, 1, (1, c, h, w))
    init = b + rng.normal(0, off, (1, c, h, w))
    gout = rng.normal(0, 1, (1, c, h, w))
    return wx, wy, cf, b, init, gout


def oracle_grads(o, p, its, pid=5, **quirks):
    wx, wy, cf, b, init, gout = p
    q = dict(ALL_OFF)
    q.update(quirks)
    try:
        o.set_quirks(**q)
        o.reset_id(pid)
        o.forward(wx, wy, cf, b, init, its, pid, f64=True)
        return o.backward(gout.copy(), wx, wy, cf, b, its, pid, f64=True)  # gx, gy, gc, gb, gi
    finally:
        o.set_quirks()


class Model:
    """The layer on one sample, from its energy: gradient step G, prox P, forward history."""

    def __init__(self, p, its):
        wx, wy, cf, b, init, gout = p
        self.wx = torch.tensor(wx[0, 0], requires_grad=True)
        self.wy = torch.tensor(wy[0, 0], requires_grad=True)
        self.c = torch.tensor(cf[0, 0], requires_grad=True)
        self.b = torch.tensor(b[0], requires_grad=True)
        self.init = torch.tensor(init[0])
        self.gout = torch.tensor(gout[0])
        self.hist = forward_history(self.G, self.P, self.init, its)

    def G(self, y):
        yv = y if y.requires_grad else y.detach().clone().requires_grad_(True)
        (g,) = torch.autograd.grad(energy_R(yv, self.wx / 8.0, self.wy / 8.0), yv, create_graph=True)
        return yv - g

    def P(self, v):
        return prox_D(v, self.c, self.b)

    def grads(self, **kw):
        gi, (gwx, gwy), (gc, gb) = adjoint_chain(self.G, self.P, [self.wx, self.wy], [self.c, self.b], self.hist,
                                                 self.gout, **kw)
        return [t.detach().numpy()[None] if t.dim() == 3 else t.detach().numpy()[None, None] for t in (gwx, gwy, gc, gb, gi)]


def assert_same(got, ref, tol=1e-9, names=("gx", "gy", "gc", "gb", "gi")):
    for nm, a, r in zip(names, got, ref):
        scale = max(np.abs(r).max(), 1e-30)
        err = np.abs(a - r).max() / scale
        assert err <= tol, (nm, err)


# ------------------------------------------------------------------------------------------------
# the model itself
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("its", [2, 7, 10])
def test_the_chain_model_is_the_chain_rule(tv_oracle, its):
    # no deviation switched on: whole-graph autograd of an independently written forward == the recursion == oracle
    from independent_tv import tv_layer

    p = problem(30 + its)
    m = Model(p, its)
    init_leaf = m.init.clone().requires_grad_(True)
    out = tv_layer(m.wx, m.wy, m.c, m.b, init_leaf, its, create_graph=True)
    auto = torch.autograd.grad((out * m.gout).sum(), [m.wx, m.wy, m.c, m.b, init_leaf])
    auto = [a.numpy()[None] if a.dim() == 3 else a.numpy()[None, None] for a in auto]
    assert_same(m.grads(), auto, 1e-10)
    assert_same(oracle_grads(tv_oracle, p, its), auto, 1e-9)


# ------------------------------------------------------------------------------------------------
# y rebuild rule
# ------------------------------------------------------------------------------------------------
def test_rebuilt_y_follows_the_two_branch_rule(tv_oracle):
    rng = np.random.default_rng(40)
    c_, h, w = 2, 17, 23
    cf = (rng.random((h, w)) < 0.6) * rng.uniform(0.0, 1.5, (h, w))
    b = rng.normal(0, 2, (c_, h, w))
    xa = b + rng.normal(0, 1.5, (c_, h, w))
    xb = b + rng.normal(0, 1.5, (c_, h, w))
    # exact ties of every comparison in the rule: |b - xa| = 1 + c, |b - xb| = c, b = x05 with and without confidence
    cf[0, :6] = [0.5, 0.5, 0.25, 0.25, 0.0, 0.75]
    b[:, 0, :6] = 1.0
    xa[:, 0, :6] = [2.5, -0.5, 3.0, 3.0, 1.0, 1.0]
    xb[:, 0, :6] = [0.0, 0.0, 1.25, 0.75, 1.0, 1.0]
    t = 0.7
    got = tv_oracle.get_yk(cf, b, xa, xb, t, f64=True)
    ref = rebuilt_y(b, cf, xa, xb, t)
    quad = np.abs(b - xa) <= 1.0 + cf
    assert 0.2 < quad.mean() < 0.95  # both branches are exercised
    assert (np.abs(b - xb)[~quad] < np.broadcast_to(cf, b.shape)[~quad]).any()  # ... and the "b otherwise" case
    np.testing.assert_allclose(got, ref, rtol=0, atol=1e-14)
    # float32 instance: same rule
    got32 = tv_oracle.get_yk(cf, b, xa, xb, t)
    f = lambda a: a.astype(np.float32).astype(np.float64)
    np.testing.assert_allclose(got32, rebuilt_y(f(b), f(cf), f(xa), f(xb), float(np.float32(t))), rtol=0, atol=2e-6)


def test_rebuilt_y_is_the_true_y_without_a_data_term(tv_oracle):
    # c = 0: every prox in the rule and in the forward pass is the identity, so rebuilding changes nothing
    wx, wy, cf, b, init, gout = problem(41)
    p = (wx, wy, 0 * cf, b, init, gout)
    for its in (6, 20):
        assert_same(oracle_grads(tv_oracle, p, its, getyk_rebuild=1), oracle_grads(tv_oracle, p, its), 1e-12)


def test_rebuilt_y_is_the_true_y_while_no_pixel_changes_regime(tv_oracle):
    # pixels that stay in the quadratic regime (|x05 - b| <= 1 + c at every iteration) and pixels that stay in the
    # linear one (b far from everything around it): the rule's proxes are then the forward pass's
    rng = np.random.default_rng(42)
    c_, h, w, its = 2, 9, 11, 12
    wx = rng.uniform(0.05, 1.0, (1, 1, h, w))
    wy = rng.uniform(0.05, 1.0, (1, 1, h, w))
    cf = rng.uniform(0.3, 1.0, (1, 1, h, w))
    b = 0.3 * rng.normal(0, 1, (1, c_, h, w))
    far = rng.random((1, c_, h, w)) < 0.15
    b[far] += 60.0 * rng.choice([-1.0, 1.0], far.sum())
    init = np.where(far, 0.0, b) + 0.1 * rng.normal(0, 1, b.shape)
    gout = rng.normal(0, 1, b.shape)
    p = (wx, wy, cf, b, init, gout)
    m = Model(p, its)
    regimes = np.stack([(np.abs(v.numpy() - b[0]) <= 1.0 + cf[0]) for v in m.hist[2]])
    assert (regimes == regimes[0]).all() and 0.05 < 1.0 - regimes[0].mean() < 0.4
    assert_same(oracle_grads(tv_oracle, p, its, getyk_rebuild=1), oracle_grads(tv_oracle, p, its), 1e-12)


@pytest.mark.parametrize("its", [6, 10, 20])
def test_rebuild_rule_where_regimes_do_switch(tv_oracle, its):
    # general inputs: pixels cross |x05 - b| = 1 + c between iterations.  Model: every step except a segment's first
    # (which never rebuilds) takes its Jacobian at the rebuilt point.
    p = problem(43 + its, amp=3.0, off=2.5)
    wx, wy, cf, b, init, gout = p
    m = Model(p, its)
    x, y, x05, s = m.hist
    regimes = np.stack([(np.abs(v.numpy() - b[0]) <= 1.0 + cf[0]) for v in x05])
    assert (regimes[2:] != regimes[1:-1]).sum() >= 5
    k0s = set(reference_schedule(its))

    def lin_y(k1):  # stands for y_{k1}, used when g05[k1] is pulled back; k = k1 - 1 is the step's iteration
        k = k1 - 1
        if k in k0s or k1 == 0:
            return y[k1]
        return torch.tensor(rebuilt_y(b[0], cf[0], x05[k].numpy(), x05[k - 1].numpy(), float(s[k])))

    got = oracle_grads(tv_oracle, p, its, getyk_rebuild=1)
    assert_same(got, m.grads(lin_y=lin_y))
    plain = oracle_grads(tv_oracle, p, its)
    assert np.abs(got[0] - plain[0]).max() > 1e-6 * np.abs(plain[0]).max()  # the rule does act here


# ------------------------------------------------------------------------------------------------
# checkpointed y at segment starts
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("its", [2, 5, 10, 20, 26])
def test_segment_starts_take_the_checkpointed_y(tv_oracle, its):
    p = problem(50 + its)
    m = Model(p, its)
    x, y, x05, s = m.hist
    k0s = set(reference_schedule(its))
    assert 0 in k0s and all(k % 2 == 0 for k in k0s)
    lin_y = lambda k1: y[k1 - 1] if (k1 - 1) in k0s else y[k1]
    got = oracle_grads(tv_oracle, p, its, end_uses_ckpt_y=1)
    assert_same(got, m.grads(lin_y=lin_y))
    if its >= 5:
        plain = oracle_grads(tv_oracle, p, its)
        assert np.abs(got[0] - plain[0]).max() > 1e-7 * np.abs(plain[0]).max()


def test_checkpointed_y_changes_nothing_at_a_fixed_point(tv_oracle):
    # started at the minimiser every iterate equals it, so y_{k0} = y_{k0+1}
    wx, wy, cf, b, init, gout = problem(56, h=8, w=8, conf_density=0.7)
    star = tv_oracle.forward(wx, wy, cf, b, init, 6000, 5, f64=True)
    again = tv_oracle.forward(wx, wy, cf, b, star, 2, 5, f64=True)
    assert np.abs(again - star).max() < 1e-12
    p = (wx, wy, cf, b, star, gout)
    assert_same(oracle_grads(tv_oracle, p, 12, end_uses_ckpt_y=1), oracle_grads(tv_oracle, p, 12), 1e-8)


# ------------------------------------------------------------------------------------------------
# iteration 0 is not back-propagated
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("its", [4, 10])
def test_skipped_iteration_0_is_a_sub_run_started_at_x1(tv_oracle, its):
    # With s_0 = 0 the second iterate is y_1 = x_1.  Whole-graph autograd of iterations 1..K-1 started at a leaf
    # x_1 = y_1 gives d/dx_1 (returned as the gradient wrt the starting point) and the weight gradients without
    # iteration 0's term; the prox of iteration 0 (x_1 = P(x05_0; c, b)) IS back-propagated, so the c and b
    # gradients are those of the full run.
    p = problem(60 + its)
    m = Model(p, its)
    x, y, x05, s = m.hist
    assert s[0] == 0.0
    K = 2 * (its // 2)
    x1 = x[1].clone().requires_grad_(True)
    xs, ys = x1, x1
    for k in range(1, K):
        xn = m.P(m.G(ys))
        ys = xn + float(s[k]) * (xn - xs)
        xs = xn
    g_x1, g_wx, g_wy = torch.autograd.grad((xs * m.gout).sum(), [x1, m.wx, m.wy])
    got = oracle_grads(tv_oracle, p, its, skip_iter0_adjoint=1)
    full = oracle_grads(tv_oracle, p, its)
    assert_same([got[0], got[1], got[4]], [g_wx.numpy()[None, None], g_wy.numpy()[None, None], g_x1.numpy()[None]],
                names=("gx", "gy", "gi"))
    assert_same([got[2], got[3]], [full[2], full[3]], 1e-12, names=("gc", "gb"))
    assert_same(got, m.grads(skip_iter0=True))
    assert np.abs(got[4] - full[4]).max() > 1e-3 * np.abs(full[4]).max()


# ------------------------------------------------------------------------------------------------
# clamp of the adjoint iterates
# ------------------------------------------------------------------------------------------------
def test_adjoint_iterates_are_clamped(tv_oracle):
    wx, wy, cf, b, init, gout = problem(70)
    gout = gout * 2.0e4  # g_x[K-1] = (1 + s) J^T P' gout passes 1e4 at many pixels
    p = (wx, wy, cf, b, init, gout)
    its = 10
    m = Model(p, its)
    got = oracle_grads(tv_oracle, p, its, clamp=1)
    assert_same(got, m.grads(clamp=1.0e4))
    free = oracle_grads(tv_oracle, p, its)
    assert np.abs(got[4]).max() <= 1.0e4 < np.abs(free[4]).max()
    assert np.abs(got[3] - free[3]).max() > 0.05 * np.abs(free[3]).max()


# ------------------------------------------------------------------------------------------------
# all of them at once: the reference's backward up to its fixed multipliers and the output guard
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("its,scale", [(10, 1.0), (20, 1.0), (9, 3.0e4)])
def test_all_deviations_together(tv_oracle, its, scale):
    wx, wy, cf, b, init, gout = problem(80 + its)
    p = (wx, wy, cf, b, init, gout * scale)
    m = Model(p, its)
    x, y, x05, s = m.hist
    k0s = set(reference_schedule(its))

    def lin_y(k1):
        k = k1 - 1
        if k in k0s:
            return y[k]
        return torch.tensor(rebuilt_y(b[0], cf[0], x05[k].numpy(), x05[k - 1].numpy(), float(s[k])))

    got = oracle_grads(tv_oracle, p, its, end_uses_ckpt_y=1, skip_iter0_adjoint=1, getyk_rebuild=1, clamp=1)
    assert_same(got, m.grads(lin_y=lin_y, skip_iter0=True, clamp=1.0e4))
