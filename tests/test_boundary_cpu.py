"""CPU-side checks of the drop-in boundary: the reference's module names import, the compiled PyTorch bindings load
and refuse bad arguments before any GPU work, `python setup.py build_ext --inplace` builds everything from a clean
copy, and the environment switches are read once."""
import ctypes
import inspect
import os
import shutil
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_reference_module_names_import_with_the_reference_signatures():
    # reference: cudaTV/TVInpainting.py:9,11,32  cudaTGV/TGVInpainting.py:11,14,44  cudaQuadFit/QuadFitting.py  cudaMedian/median.py
    import QuadFit_cuda_ext
    import QuadFitting
    import TGVInpainting
    import TVInpainting
    import median
    import median_cuda_ext
    import tgvInpaint_cuda_ext
    import tvInpaint_cuda_ext

    for m in (tvInpaint_cuda_ext, tgvInpaint_cuda_ext, QuadFit_cuda_ext, median_cuda_ext):
        for name in ("forward", "backward", "dummy", "dummy_only"):  # TVInpaintFista_cuda.cpp:145-150
            assert callable(getattr(m, name)), (m.__name__, name)
    assert list(inspect.signature(tvInpaint_cuda_ext.forward).parameters)[:7] == ["d_x", "d_y", "d_c", "d_b", "d_i", "its", "id"]
    assert list(inspect.signature(tvInpaint_cuda_ext.backward).parameters) == ["d_iGf", "d_x", "d_y", "d_c", "d_b", "its", "id"]
    sig = inspect.signature(TVInpainting.TVInpaint.__init__)
    assert list(sig.parameters)[:4] == ["self", "device", "its", "pid"] and sig.parameters["pid"].default == 6
    sig = inspect.signature(TGVInpainting.TGVInpaint.__init__)
    assert list(sig.parameters)[:4] == ["self", "device", "its", "pid"] and sig.parameters["pid"].default == 3
    assert issubclass(TVInpainting.TVInpaintingFunction, torch.autograd.Function)
    assert issubclass(TGVInpainting.TGVInpaintingFunction, torch.autograd.Function)
    assert list(inspect.signature(TVInpainting.TVInpaint.forward).parameters) == ["self", "t_dx", "t_dy", "t_dc", "t_db", "t_di"]
    assert QuadFitting.QuadFittingFromFlow and QuadFitting.QuadFittingFromFlowFunction and median.Median and median.MedianFunction
    assert tvInpaint_cuda_ext.dummy() == [] and tgvInpaint_cuda_ext.dummy() == []


def test_compiled_bindings_load_and_check_their_arguments_on_the_host():
    from customnetworklayers_amd.cudaTGV import tgvInpaint_hip_ext as tgv
    from customnetworklayers_amd.cudaTV import tvInpaint_hip_ext as tv

    for m in (tv, tgv):
        for name in ("forward", "backward", "dummy", "dummy_only"):
            assert callable(getattr(m, name))
        assert m.dummy() == []
    z = torch.zeros(1, 1, 4, 4)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):  # CHECK_CUDA, TVInpaintFista_cuda.cpp:24
        tv.forward(z, z, z, z, z, 4, 0)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        tgv.backward(z, z, z, z, z, 4, 0)
    with pytest.raises(TypeError):  # the reference's arity: five tensors, its, id
        tv.forward(z, z, z, z, 4, 0)


def test_environment_switches_are_read_once(monkeypatch):
    from customnetworklayers_amd._lib import lib, reload_env

    monkeypatch.delenv("INPAINT_KEEP", raising=False)
    monkeypatch.delenv("INPAINT_KEEP_LAST", raising=False)
    reload_env()
    assert lib.inpaint_keep_override() == -1
    monkeypatch.setenv("INPAINT_KEEP", "1")
    assert lib.inpaint_keep_override() == -1  # not looked at again ...
    reload_env()
    assert lib.inpaint_keep_override() == 1   # ... until somebody asks
    monkeypatch.delenv("INPAINT_KEEP")
    monkeypatch.setenv("INPAINT_KEEP_LAST", "0")
    assert lib.tvinpaint_reset_id(3) == 0     # reset_id asks too
    assert lib.inpaint_keep_override() == 0


def test_planes_beyond_32_bit_offsets_are_refused():
    from customnetworklayers_amd._lib import last_error, lib

    p = ctypes.c_void_p(16)  # never dereferenced: the size check comes first
    assert lib.tvinpaint_forward(p, p, p, p, p, p, 1, 1, 16384, 32768, 4, 0, None) == 2
    assert "2^29" in last_error()
    assert lib.tgvinpaint_forward(p, p, p, p, p, p, 1, 1, 16384, 32768, 4, 0, None) == 2
    assert lib.tvinpaint_forward_noalloc(p, p, p, p, p, p, 1, 1, 16384, 32768, 4, None) == 2


def test_setup_py_builds_everything_from_a_clean_copy(tmp_path):
    # the reference builds with `python setup.py install` (cudaTV/setup.py:16-28); here build_ext --inplace runs hipcc
    # for gfx950 and compiles the two PyTorch bindings
    dst = tmp_path / "copy"
    ignore = shutil.ignore_patterns(".git", "gpurun_out", "_work", "*.so", "*.o", "__pycache__", ".pytest_cache", "profiles", "tests")
    shutil.copytree(ROOT, dst, ignore=ignore)
    r = subprocess.run([sys.executable, "setup.py", "build_ext", "--inplace"], cwd=dst, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    lib = dst / "customnetworklayers_amd" / "libinpaint_hip.so"
    assert lib.exists() and (dst / "customnetworklayers_amd" / "cudaTV" / "tvInpaint_hip_ext.so").exists()
    assert (dst / "customnetworklayers_amd" / "cudaTGV" / "tgvInpaint_hip_ext.so").exists()
    code = ("import sys; sys.path.insert(0, %r); import tvInpaint_cuda_ext, customnetworklayers_amd._lib as l; "
            "from customnetworklayers_amd.cudaTV import tvInpaint_hip_ext; assert l.LIB_PATH.startswith(%r); "
            "print(hasattr(l.lib, 'tvinpaint_forward'))" % (str(dst), str(dst)))
    r = subprocess.run([sys.executable, "-c", code], cwd=tmp_path, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.strip() == "True", r.stdout + r.stderr
