"""Who owns the per-id device blocks (tvinpaint_set_allocator / tgvinpaint_set_allocator): with PyTorch's caching
allocator installed -- the default of this package's modules -- a forward makes torch.cuda.memory_allocated() rise by
the slot's size, the gradients are the bits of a run on hipMalloc'ed memory, and reset_id gives the block back."""
import ctypes

import numpy as np
import pytest
import torch

from customnetworklayers_amd import _lib
from customnetworklayers_amd.workloads import tgv_inputs, tv_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _run(ext, t, its, pid):
    (sol,) = ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], its, pid)
    grads = ext.backward(t["grad"].clone(), t["dx"], t["dy"], t["dc"], t["db"], its, pid)
    torch.cuda.synchronize()
    return [sol] + list(grads)


@pytest.mark.parametrize("layer", ["tv", "tgv"])
def test_slot_memory_lives_in_the_torch_pool(layer):
    if layer == "tv":
        from customnetworklayers_amd.cudaTV import tvInpaint_cuda_ext as ext
        d = tv_inputs(2, 2, 96, 200, seed=4, conf_density=0.3)
    else:
        from customnetworklayers_amd.cudaTGV import tgvInpaint_cuda_ext as ext
        d = tgv_inputs(2, 2, 96, 200, seed=4, conf_density=0.3)
    t = {k: torch.from_numpy(v).to(DEV) for k, v in d.items()}
    its, pid = 20, 5
    ext.reset_id(pid)
    try:
        _lib.use_torch_allocator(False)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        plain = _run(ext, t, its, pid)
        held = ext.slot_bytes(pid)
        assert held > 0
        # (hipMalloc: invisible to PyTorch; only the outputs of this run are counted)
        assert torch.cuda.memory_allocated() - before < held
        ext.reset_id(pid)
        del plain[1:]
        _lib.use_torch_allocator(True)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        (sol,) = ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], its, pid)
        torch.cuda.synchronize()
        assert ext.slot_bytes(pid) == held
        grown = torch.cuda.memory_allocated() - before
        assert held <= grown - sol.numel() * 4 < held + (2 << 20), (held, grown)
        pooled = _run(ext, t, its, pid)  # the same block serves the next calls
        assert torch.equal(pooled[0], plain[0])
        _lib.use_torch_allocator(False)  # the block goes back to the allocator that made it
        del sol
        mid = torch.cuda.memory_allocated()
        ext.reset_id(pid)
        assert mid - torch.cuda.memory_allocated() >= held
        ref = _run(ext, t, its, pid)
        for a, b in zip(pooled, ref):
            assert torch.equal(a, b)
    finally:
        ext.reset_id(pid)
        _lib.use_torch_allocator(True)


def test_allocator_callbacks_come_in_pairs_and_may_refuse():
    lib = _lib.lib
    alloc = ctypes.cast(_lib._torch_alloc_c, ctypes.c_void_p)
    assert lib.tvinpaint_set_allocator(alloc, None, None) == 2 and "both" in _lib.last_error()
    assert lib.tgvinpaint_set_allocator(None, ctypes.cast(_lib._torch_release_c, ctypes.c_void_p), None) == 2
    # an allocator that has nothing to give: the forward fails with the HIP error code and says why; nothing is launched
    refuse = _lib._ALLOC_FN(lambda nbytes, device, stream, user: None)
    noop = _lib._RELEASE_FN(lambda ptr, user: None)
    from customnetworklayers_amd.cudaTV import tvInpaint_cuda_ext as ext

    d = tv_inputs(1, 1, 16, 64, seed=1, conf_density=0.3)
    t = {k: torch.from_numpy(v).to(DEV) for k, v in d.items()}
    ext.reset_id(6)
    try:
        assert lib.tvinpaint_set_allocator(ctypes.cast(refuse, ctypes.c_void_p), ctypes.cast(noop, ctypes.c_void_p), None) == 0
        with pytest.raises(RuntimeError, match="allocator"):
            ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], 4, 6)
    finally:
        _lib.use_torch_allocator(True)
        ext.reset_id(6)
    (sol,) = ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], 4, 6)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(sol).all())
    ext.reset_id(6)
