"""The quoted TGV workload on the GPU at full size, checked through size-independent properties
(batch independence with per-sample Lipschitz constants, channel independence of the forward pass,
determinism, independence of the id used), plus one full-length sample against the oracle."""
import numpy as np
import pytest
import torch

from customnetworklayers_amd.workloads import CONFIGS, tgv_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ext():
    from customnetworklayers_amd.cudaTGV import tgvInpaint_cuda_ext

    return tgvInpaint_cuda_ext


def gpu_layer(ext, d, its, pid):
    t = {k: torch.from_numpy(np.ascontiguousarray(v)).to(DEV) for k, v in d.items()}
    ext.reset_id(pid)
    (sol,) = ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], its, pid)
    grads = ext.backward(t["grad"], t["dx"], t["dy"], t["dc"], t["db"], its, pid)
    torch.cuda.synchronize()
    return [sol.cpu().numpy()] + [g.cpu().numpy() for g in grads]


def test_tgv_batch_equals_its_samples_run_alone(ext):
    # 4 x 2 x 384 x 1248, 100 iterations: the batch must be 4 independent problems, bit for bit,
    # also when one sample's beta pushes its Lipschitz bound above the constant 32
    cfg = CONFIGS[2]
    c = cfg["c"]
    d = tgv_inputs(cfg["n"], c, cfg["h"], cfg["w"], seed=0, **cfg["gen"])
    d["dx"][3, 1] *= 3.0
    d["dy"][3, 1] *= 3.0
    full = gpu_layer(ext, d, cfg["its"], 0)
    Ls = ext.lipschitz(0, cfg["n"])
    assert Ls[0] == Ls[1] == Ls[2] > Ls[3]
    again = gpu_layer(ext, d, cfg["its"], 1)
    for a, b in zip(full, again):
        np.testing.assert_array_equal(a, b)
    for s in (0, 3):
        one = gpu_layer(ext, {k: v[s:s + 1] for k, v in d.items()}, cfg["its"], 2)
        for a, b in zip(full, one):
            np.testing.assert_array_equal(a[s:s + 1], b)
    assert all(np.isfinite(a).all() for a in full)
    # flow channels never couple in the forward pass; the rhs / init gradients are per channel
    sel = [0, c, 2 * c]  # u, v1, v2 of flow channel 0
    ch0 = {k: v[:1] for k, v in d.items()}
    ch0["db"] = d["db"][:1, :1]
    ch0["di"] = d["di"][:1, sel]
    ch0["grad"] = d["grad"][:1, sel]
    one_ch = gpu_layer(ext, ch0, cfg["its"], 2)
    np.testing.assert_array_equal(one_ch[0][0], full[0][0, sel])
    np.testing.assert_array_equal(one_ch[4][0, 0], full[4][0, 0])  # g_b
    np.testing.assert_array_equal(one_ch[5][0], full[5][0, sel])   # g_init


def test_tgv_full_length_sample_matches_oracle(ext):
    from oracle.oracle_lib import TGVOracle

    o = TGVOracle()
    o.set_quirks()
    cfg = CONFIGS[2]
    d = tgv_inputs(1, cfg["c"], cfg["h"], cfg["w"], seed=3, **cfg["gen"])  # one whole sample, all 100 iterations
    print("case 1x%dx%dx%d its=%d" % (cfg["c"], cfg["h"], cfg["w"], cfg["its"]), flush=True)
    got = gpu_layer(ext, d, cfg["its"], 3)
    o.reset_id(3)
    sol = o.forward(d["dx"], d["dy"], d["dc"], d["db"], d["di"], cfg["its"], 3)
    grads = o.backward(d["grad"].copy(), d["dx"], d["dy"], d["dc"], d["db"], cfg["its"], 3)
    rel = lambda a, r: float(np.abs(a - r).max() / max(np.abs(r).max(), 1e-30))
    errs = [rel(a, r) for a, r in zip(got, [sol] + list(grads))]
    print("\n[tgv 1x2x384x1248 its=100] out %.2e grads %s" % (errs[0], ["%.2e" % e for e in errs[1:]]), flush=True)
    assert errs[0] <= 1e-4 and max(errs[1:]) <= 1e-3


@pytest.mark.parametrize("c,lively", [(3, False), (3, True), (2, True)])
def test_tgv_pair_kernels_match_the_oracle_at_full_image_size(ext, c, lively):
    # 1 x C x 384 x 1248, 20 iterations against the oracle: three channels take the adjoint pairs in four wavefronts at the
    # strip heights and strip counts of config 2's image.  `lively`: auxiliary variables that start far from smooth and a
    # larger beta, so that all three Huber terms are active in many wavefronts and quiet in others (config 2's own data
    # keeps the two smoothness terms below their threshold everywhere, the path on which a wavefront skips their roots)
    from oracle.oracle_lib import TGVOracle

    o = TGVOracle()
    o.set_quirks()
    cfg = CONFIGS[2]
    its = 20
    d = tgv_inputs(1, c, cfg["h"], cfg["w"], seed=30 + c, **cfg["gen"])
    if lively:
        rng = np.random.default_rng(7)
        d["di"][:, c:] = rng.normal(0, 3.0, d["di"][:, c:].shape).astype(np.float32)
        d["di"][:, c:, : cfg["h"] // 2] *= 0.01  # (the upper half stays quiet)
        d["dx"][:, 1] *= 4.0
        d["dy"][:, 1] *= 4.0
    print("case 1x%dx%dx%d its=%d lively=%s" % (c, cfg["h"], cfg["w"], its, lively), flush=True)
    got = gpu_layer(ext, d, its, 3)
    o.reset_id(3)
    sol = o.forward(d["dx"], d["dy"], d["dc"], d["db"], d["di"], its, 3)
    grads = o.backward(d["grad"].copy(), d["dx"], d["dy"], d["dc"], d["db"], its, 3)
    rel = lambda a, r: float(np.abs(a - r).max() / max(np.abs(r).max(), 1e-30))
    errs = [rel(a, r) for a, r in zip(got, [sol] + list(grads))]
    print("\n[tgv 1x%dx384x1248 its=%d] out %.2e grads %s" % (c, its, errs[0], ["%.2e" % e for e in errs[1:]]), flush=True)
    assert errs[0] <= 1e-4 and max(errs[1:]) <= 1e-3  # (the layer's tolerances; the kernels give the oracle's bits)
    for a, r in zip(got, [sol] + list(grads)):
        np.testing.assert_array_equal(a, r)
    ext.reset_id(3)


@pytest.mark.parametrize("c,parts", [(4, ((0, 2), (2, 4))), (3, ((0, 2), (2, 3)))])
def test_tgv_wider_runs_contain_the_narrower_ones(ext, c, parts):
    # 2 x C x 384 x 1248, 100 iterations with three and four channels (adjoint pairs in four wavefronts, two channel groups):
    # the channels couple only through the gradients wrt confidence and weights, so the solution, g_b and g_init of any
    # subset of channels must equal, bit for bit, a run on those channels alone (which takes the two- / one-wavefront kernels)
    cfg = CONFIGS[2]
    n = 2
    d = tgv_inputs(n, c, cfg["h"], cfg["w"], seed=5, **cfg["gen"])
    full = gpu_layer(ext, d, cfg["its"], 0)
    assert all(np.isfinite(a).all() for a in full)
    for lo, hi in parts:
        sel = [v * c + ch for v in range(3) for ch in range(lo, hi)]  # u, v1, v2 of the chosen channels
        sub = dict(d)
        sub["db"] = d["db"][:, lo:hi]
        sub["di"] = d["di"][:, sel]
        sub["grad"] = d["grad"][:, sel]
        part = gpu_layer(ext, sub, cfg["its"], 1)
        np.testing.assert_array_equal(part[0], full[0][:, sel])
        np.testing.assert_array_equal(part[4], full[4][:, lo:hi])  # g_b
        np.testing.assert_array_equal(part[5], full[5][:, sel])    # g_init
    ext.reset_id(0)
    ext.reset_id(1)
