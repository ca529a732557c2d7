"""The output guard on the device against the oracle's, on tensors a backward pass cannot easily be made to produce:
non-finite entries (the running mean restarts at 1000 x the stored mean behind every one of them,
TVInpaintFista.cu:128-175; TGVInpaintFistaHelp.cu:153-216), entries above the tolerance, the rescale and kill
decisions.  The tensors are long enough for the device's passes to be spread over many workgroups.

The means are formed in a different order on the two sides (the reference's sequential running mean in the oracle,
sums of per-workgroup records on the device), hence the relative tolerance 1e-10 on them (observed: 1e-12 where one
entry of 3e9 sits among entries of order 1) and 1e-6 on rescaled float outputs; everything else is exact.
"""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    from customnetworklayers_amd import _lib

    return _lib.lib


def device_guard(lib, layer, g, run, av):
    g = np.ascontiguousarray(g)
    assert g.dtype in (np.float32, np.float64)
    out = np.empty(g.size, np.float32)
    res = np.zeros(7, np.float64)
    fn = lib.tvinpaint_selftest_guard if layer == "tv" else lib.tgvinpaint_selftest_guard
    rc = fn(g.ctypes.data_as(ctypes.c_void_p), g.size, int(g.dtype == np.float32), int(run), float(av),
            out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), res.ctypes.data_as(ctypes.POINTER(ctypes.c_double)))
    assert rc == 0
    return out, res


def check(lib, oracle, layer, g, run, av, name):
    out, res = device_guard(lib, layer, g, run, av)
    ref, av_new, act, st = oracle.guard(g, run=run, av=av, f32=g.dtype == np.float32)
    print("\n[%s %s %s run=%d] device mean %.17g oracle %.17g  invalid %d above %d action %d mult %.6g"
          % (layer, g.dtype, name, run, res[0], st[0], int(res[3]), int(res[2]), int(res[4]), res[6]), flush=True)
    assert res[0] == pytest.approx(st[0], rel=1e-10, abs=0)
    assert res[1] == st[1] and res[2] == st[2] and res[3] == st[3]
    assert int(res[4]) == act
    assert res[5] == pytest.approx(av_new, rel=1e-10, abs=0)
    want = ref.astype(np.float32)
    assert np.array_equal(out == 0, want == 0)
    if act == 0:
        np.testing.assert_array_equal(out, want)
    else:
        np.testing.assert_allclose(out, want, rtol=1e-6, atol=0)
    return res


@pytest.fixture(scope="module")
def oracles():
    from oracle.oracle_lib import TGVOracle, TVOracle

    return {"tv": TVOracle(), "tgv": TGVOracle()}


@pytest.mark.parametrize("layer", ["tv", "tgv"])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("n", [7, 4096, 100003, 1500000])
def test_plain_tensors(lib, oracles, layer, dtype, n):
    g = np.random.default_rng(n).normal(0, 1, n).astype(dtype)
    for run, av in ((0, 0.0), (3, 2.0), (100, 2.0)):
        res = check(lib, oracles[layer], layer, g, run, av, "plain n=%d" % n)
        assert res[4] == 0 and res[6] == 1.0


@pytest.mark.parametrize("layer", ["tv", "tgv"])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("n,where", [
    (1000, [10, 20]),               # one workgroup in the second pass
    (100003, [0]),                  # the whole tensor is the tail
    (100003, [100002]),             # the tail is empty
    (100003, [5, 4097, 77777]),     # the last one counts
    (1500000, [123456, 1499000]),   # many workgroups, a short tail
    (1500000, [3]),                 # many workgroups, a long tail
])
def test_non_finite_entries_restart_the_mean(lib, oracles, layer, dtype, n, where):
    g = np.random.default_rng(n + len(where)).normal(0, 1, n).astype(dtype)
    for i, w in enumerate(where):
        g[w] = (np.nan, np.inf, -np.inf)[i % 3]
    for run, av in ((0, 0.5), (12, 0.25), (12, 1e-4)):
        res = check(lib, oracles[layer], layer, g, run, av, "non-finite at %s" % where)
        assert res[3] == len(where)


@pytest.mark.parametrize("layer", ["tv", "tgv"])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_entries_above_the_tolerance(lib, oracles, layer, dtype):
    # TV zeroes them and counts them in the mean as they are; TGV clamps them, in the mean as well
    g = np.random.default_rng(5).normal(0, 1, 50000).astype(dtype)
    g[5] = 2e7
    g[40000] = -3e9
    g[41000] = 1e4
    res = check(lib, oracles[layer], layer, g, 0, 0.0, "large entries")
    assert res[2] >= 2
    g[30000] = np.nan
    check(lib, oracles[layer], layer, g, 4, 0.7, "large entries behind a NaN")


@pytest.mark.parametrize("layer", ["tv", "tgv"])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_rescale_and_kill(lib, oracles, layer, dtype):
    g = np.random.default_rng(6).normal(0, 1, 200000).astype(dtype)
    mean = float(np.abs(g.astype(np.float64)).mean())
    acts = []
    for run, av in ((10, mean / 20), (10, mean / 60), (9, mean / 60), (10, mean / 2)):
        acts.append(int(check(lib, oracles[layer], layer, g, run, av, "av=mean/%g" % (mean / av))[4]))
    assert acts == [1, 2, 0, 0]


def test_guard_statistics_on_stderr_when_asked(monkeypatch, capfd):
    """INPAINT_STATS_EVERY=N prints the guard's statistics of every Nth backward pass of an id on stderr, in the
    reference's wording (TVInpaintFista.cu:1766-1790 does so on every 75th run); nothing is printed otherwise."""
    from customnetworklayers_amd.cudaTV import tvInpaint_cuda_ext as ext
    from customnetworklayers_amd.workloads import tv_inputs

    d = tv_inputs(1, 2, 24, 70, seed=2, conf_density=0.3)
    t = {k: torch.from_numpy(v).to("cuda:0") for k, v in d.items()}

    def fwd_bwd():
        ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], 8, 6)
        ext.backward(t["grad"].clone(), t["dx"], t["dy"], t["dc"], t["db"], 8, 6)
        torch.cuda.synchronize()

    ext.reset_id(6)
    fwd_bwd()
    assert "Output gradient" not in capfd.readouterr().err
    monkeypatch.setenv("INPAINT_STATS_EVERY", "2")
    try:
        ext.reset_id(6)  # (re-reads the environment; run count 0)
        fwd_bwd()        # run 0: silent
        assert "Output gradient" not in capfd.readouterr().err
        fwd_bwd()        # run 1: 1 % 2 == 1
        err = capfd.readouterr().err
        assert err.count("Output gradient to") == 5 and "gradI" in err
    finally:
        monkeypatch.delenv("INPAINT_STATS_EVERY")
        ext.reset_id(6)
