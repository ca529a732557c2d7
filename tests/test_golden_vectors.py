"""The committed fixtures of tests/golden (inputs + oracle outputs, written by tests/golden/make_vectors.py
after the oracle was pinned; the reference itself ships no vectors): the CPU oracle must reproduce them bit
for bit (CPU suite), and so must the HIP path through the C ABI (GPU suite; the one order-undefined sum, the
quadratic fit's gradient wrt the second feature map, to 1e-5 of its maximum)."""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    with np.load(os.path.join(GOLDEN, name), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


LAYER_KEYS = ("sol", "gx", "gy", "gc", "gb", "gi")


def test_tv_oracle_reproduces_fixture(tv_oracle):
    v = load("tv_1x2x12x16_its8.npz")
    its = int(v["its"])
    tv_oracle.reset_id(0)
    sol = tv_oracle.forward(v["dx"], v["dy"], v["dc"], v["db"], v["di"], its, 0)
    grads = tv_oracle.backward(v["grad"].copy(), v["dx"], v["dy"], v["dc"], v["db"], its, 0)
    for k, a in zip(LAYER_KEYS, (sol,) + tuple(grads)):
        assert np.array_equal(a, v[k]), k


def test_tgv_oracle_reproduces_fixture():
    from oracle.oracle_lib import TGVOracle

    o = TGVOracle()
    o.set_quirks()
    v = load("tgv_1x1x10x14_its6.npz")
    its = int(v["its"])
    o.reset_id(0)
    sol = o.forward(v["dx"], v["dy"], v["dc"], v["db"], v["di"], its, 0)
    grads = o.backward(v["grad"].copy(), v["dx"], v["dy"], v["dc"], v["db"], its, 0)
    for k, a in zip(LAYER_KEYS, (sol,) + tuple(grads)):
        assert np.array_equal(a, v[k]), k


def test_flow_layer_oracles_reproduce_fixtures(flowaux_oracle):
    o = flowaux_oracle
    v = load("quadfit_1x4x12x18.npz")
    assert np.array_equal(o.quadfit_forward(v["feat0"], v["feat1"], v["flow"]), v["out"])
    g0, g1 = o.quadfit_backward(v["grad"], v["feat0"], v["feat1"], v["flow"])
    assert np.array_equal(g0, v["g0"]) and np.array_equal(g1, v["g1"])
    v = load("median_1x6x9x11.npz")
    assert np.array_equal(o.median_forward(v["vol"]), v["out"])
    assert np.array_equal(o.median_backward(v["grad"], v["vol"]), v["gvol"])
    v = load("hierarchy_1x2x5x7.npz")
    assert np.array_equal(o.upsample2x(v["sol"], 2.0), v["up"])
    wx, wy = o.edge_weights(v["img"], 10.0)
    assert np.array_equal(wx, v["wx"]) and np.array_equal(wy, v["wy"])
    assert np.array_equal(o.upsample2x_adjoint(v["ga"], v["gb"], 2.0), v["g_sol"])


CORRECTED_KEYS = ("corrected_gx", "corrected_gy", "corrected_gc", "corrected_gb", "corrected_gi")


@pytest.mark.parametrize("layer,name", [("tv", "tv_1x2x12x16_its8.npz"), ("tgv", "tgv_1x1x10x14_its6.npz")])
def test_oracles_reproduce_the_corrected_gradient_fixtures(layer, name):
    from oracle.oracle_lib import TGVOracle, TVOracle

    o = TVOracle() if layer == "tv" else TGVOracle()
    v = load(name)
    its = int(v["its"])
    quirks = dict(end_uses_ckpt_y=0, skip_iter0_adjoint=0, getyk_rebuild=0, scale_factors=0, clamp=1, guard=1)
    if layer == "tgv":
        quirks["dw_div"] = 0
    try:
        o.set_quirks(**quirks)
        o.reset_id(0)
        o.forward(v["dx"], v["dy"], v["dc"], v["db"], v["di"], its, 0)
        grads = o.backward(v["grad"].copy(), v["dx"], v["dy"], v["dc"], v["db"], its, 0)
    finally:
        o.set_quirks()
    for k, a in zip(CORRECTED_KEYS, grads):
        assert np.array_equal(a, v[k]), k


@pytest.mark.gpu
@pytest.mark.parametrize("layer,name", [("tv", "tv_1x2x12x16_its8.npz"), ("tgv", "tgv_1x1x10x14_its6.npz")])
def test_inpainting_layers_reproduce_the_corrected_gradient_fixtures_on_the_gpu(layer, name):
    import torch

    if layer == "tv":
        from customnetworklayers_amd.cudaTV import tvInpaint_cuda_ext as ext
    else:
        from customnetworklayers_amd.cudaTGV import tgvInpaint_cuda_ext as ext
    v = load(name)
    its = int(v["its"])
    t = {k: torch.from_numpy(v[k]).cuda() for k in ("dx", "dy", "dc", "db", "di", "grad")}
    try:
        ext.reset_id(0)
        ext.gradient_mode(0, 1)
        (sol,) = ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], its, 0)
        grads = ext.backward(t["grad"], t["dx"], t["dy"], t["dc"], t["db"], its, 0)
        got = [g.cpu().numpy() for g in grads]
    finally:
        ext.reset_id(0)
    assert np.array_equal(sol.cpu().numpy(), v["sol"])
    for k, a in zip(CORRECTED_KEYS, got):
        assert np.array_equal(a, v[k]), k


@pytest.mark.gpu
@pytest.mark.parametrize("layer,name", [("tv", "tv_1x2x12x16_its8.npz"), ("tgv", "tgv_1x1x10x14_its6.npz")])
def test_inpainting_layers_reproduce_fixtures_on_the_gpu(layer, name):
    import torch

    if layer == "tv":
        from customnetworklayers_amd.cudaTV import tvInpaint_cuda_ext as ext
    else:
        from customnetworklayers_amd.cudaTGV import tgvInpaint_cuda_ext as ext
    v = load(name)
    its = int(v["its"])
    t = {k: torch.from_numpy(v[k]).cuda() for k in ("dx", "dy", "dc", "db", "di", "grad")}
    ext.reset_id(0)
    (sol,) = ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], its, 0)
    grads = ext.backward(t["grad"], t["dx"], t["dy"], t["dc"], t["db"], its, 0)
    for k, a in zip(LAYER_KEYS, (sol,) + tuple(grads)):
        assert np.array_equal(a.cpu().numpy(), v[k]), k


@pytest.mark.gpu
def test_flow_layers_reproduce_fixtures_on_the_gpu():
    import torch

    from customnetworklayers_amd import hierarchy
    from customnetworklayers_amd.cudaMedian import median_cuda_ext as med
    from customnetworklayers_amd.cudaQuadFit import QuadFit_cuda_ext as qf

    dev = lambda a: torch.from_numpy(a).cuda()
    v = load("quadfit_1x4x12x18.npz")
    (out,) = qf.forward(dev(v["feat0"]), dev(v["feat1"]), dev(v["flow"]))
    g0, g1 = qf.backward(dev(v["grad"]), dev(v["feat0"]), dev(v["feat1"]), dev(v["flow"]))
    assert np.array_equal(out.cpu().numpy(), v["out"]) and np.array_equal(g0.cpu().numpy(), v["g0"])
    assert np.abs(g1.cpu().numpy() - v["g1"]).max() <= 1e-5 * np.abs(v["g1"]).max()
    v = load("median_1x6x9x11.npz")
    (out,) = med.forward(dev(v["vol"]))
    (g,) = med.backward(dev(v["grad"]), dev(v["vol"]))
    assert np.array_equal(out.cpu().numpy(), v["out"]) and np.array_equal(g.cpu().numpy(), v["gvol"])
    v = load("hierarchy_1x2x5x7.npz")
    up, wx, wy = hierarchy.next_level_forward(dev(v["sol"]), dev(v["img"]))
    assert np.array_equal(up.cpu().numpy(), v["up"])
    assert np.array_equal(wx.cpu().numpy(), v["wx"]) and np.array_equal(wy.cpu().numpy(), v["wy"])
    assert np.array_equal(hierarchy.next_level_backward(dev(v["ga"]), dev(v["gb"])).cpu().numpy(), v["g_sol"])
