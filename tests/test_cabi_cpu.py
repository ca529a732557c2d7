"""CPU-side checks of the C-ABI library: it loads without a GPU, exports every symbol that
include/*.h declares, and its host-only helpers (checkpoint schedule, FISTA factors, the guard's
decision rule) agree with the CPU oracle.  No compute entry point is called here."""
import ctypes
import glob
import os
import re

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = []
    for path in sorted(glob.glob(os.path.join(ROOT, "include", "*.h"))):
        text = re.sub(r"/\*.*?\*/", "", open(path).read(), flags=re.S)
        text = re.sub(r"\btypedef\b[^;]*;", "", text)  # (callback types are not symbols)
        names += re.findall(r"\b([a-z_0-9]+)\s*\([^;{]*\)\s*;", text)
    return sorted(set(names))


def test_library_loads_and_exports_every_declared_symbol():
    from customnetworklayers_amd._lib import LIB_PATH

    lib = ctypes.CDLL(LIB_PATH)
    names = declared_symbols()
    assert "tvinpaint_forward" in names and "tvinpaint_backward" in names and len(names) >= 12
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_host_schedule_and_step_sizes_match_the_oracle(tv_oracle):
    from customnetworklayers_amd.cudaTV import tvInpaint_cuda_ext as ext

    for its in (0, 1, 2, 3, 5, 9, 20, 50, 100, 200, 1000, 10200):
        assert ext.schedule(its) == tv_oracle.schedule(its), its
    np.testing.assert_array_equal(np.array(ext.step_sizes(300), np.float32), tv_oracle.step_sizes(300))


def test_host_guard_rule_matches_the_oracle(tv_oracle):
    from customnetworklayers_amd.cudaTV import tvInpaint_cuda_ext as ext

    g = np.abs(np.random.default_rng(0).normal(0, 1, 512)) + 0.1
    mean = float(g.mean())
    for run in (0, 3, 9, 10, 50, 400):
        for ratio in (0.5, 5.0, 20.0, 60.0):
            av0 = mean / ratio
            _, av_ref, act_ref, st = tv_oracle.guard(g, run=run, av=av0)
            act, mult, av = ext.guard_decide(run, float(st[0]), av0)
            assert act == act_ref, (run, ratio)
            np.testing.assert_allclose(av, av_ref, rtol=1e-12)
            assert (mult == 0.0) == (act == 2) and (mult == 1.0) == (act == 0)


def test_bad_arguments_are_rejected_before_any_gpu_work():
    from customnetworklayers_amd._lib import last_error, lib

    # null pointers, bad id, bad sizes: every check happens on the host
    assert lib.tvinpaint_forward(None, None, None, None, None, None, 1, 1, 4, 4, 4, 0, None) == 2
    assert lib.tvinpaint_forward(None, None, None, None, None, None, 1, 1, 4, 4, 4, 10, None) == 1
    assert "id" in last_error()
    assert lib.tvinpaint_backward(*([None] * 10), 1, 1, 4, 4, 4, -1, None) == 1
    assert lib.tvinpaint_slot_bytes(3) == 0


def test_flow_layers_reject_bad_arguments_before_any_gpu_work():
    from customnetworklayers_amd._lib import lib

    assert lib.quadfit_forward(None, None, None, None, 1, 1, 4, 4, 2, None) == 2
    assert lib.quadfit_backward(None, None, None, None, None, None, 1, 1, 4, 4, 2, None, 0, None) == 2
    assert lib.medimax_forward(None, None, 1, 4, 4, 8, None) == 2
    assert lib.medimax_backward(None, None, None, 1, 4, 4, 8, None) == 2
    assert b"null pointer" in lib.flowaux_last_error()
    assert lib.quadfit_backward_workspace_bytes(4, 384, 1248) >= 4 * 384 * 1248 * 4 * 11
    assert lib.quadfit_backward_workspace_bytes(0, 384, 1248) == 0
