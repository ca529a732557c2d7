"""tvinpaint_forward_noalloc (the forward pass for callers that cannot allocate device memory) against
tvinpaint_forward through the C ABI: same kernels, so the outputs must be the same bits.  Two calls in a row, the
second on a smaller input, so that what the first left in the library's fixed scratch cannot leak into the second;
then the same in place (the output buffer is the starting point), that a warmed call leaves the device's free memory
as it was, a HIP graph that holds the call and is replayed on changed inputs, and the size limit.  Collected last (the
file name sorts behind every other test file)."""
import ctypes

import numpy as np
import pytest
import torch

from customnetworklayers_amd.workloads import tv_inputs

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _both_forwards(lib, d, its, pid=7):
    dev = torch.device("cuda:0")
    t = {k: torch.from_numpy(v).to(dev) for k, v in d.items()}
    n, c, h, w = d["db"].shape
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    ref = torch.full_like(t["db"], float("nan"))
    out = torch.full_like(t["db"], float("nan"))
    args = [_ptr(t[k]) for k in ("dx", "dy", "dc", "db", "di")]
    assert lib.tvinpaint_reset_id(pid) == 0
    rc = lib.tvinpaint_forward(*args, _ptr(ref), n, c, h, w, its, pid, stream)
    assert rc == 0, lib.tvinpaint_last_error()
    rc = lib.tvinpaint_forward_noalloc(*args, _ptr(out), n, c, h, w, its, stream)
    assert rc == 0, lib.tvinpaint_last_error()
    torch.cuda.synchronize()
    assert lib.tvinpaint_reset_id(pid) == 0
    return out.cpu().numpy(), ref.cpu().numpy()


@pytest.mark.parametrize("first,second", [
    ((2, 2, 130, 200, 50), (1, 2, 37, 101, 20)),   # pair kernels, ragged strips; then a smaller image
    ((1, 5, 40, 70, 9), (1, 3, 9, 63, 4)),         # five channels (two channel groups), odd its; then three channels
    ((1, 1, 33, 64, 1), (1, 1, 5, 3, 0)),          # its in {0, 1}: the output is the starting point
    ((16, 2, 256, 512, 6), (4, 2, 96, 312, 12)),   # exactly the largest field the scratch holds; then a small one
])
def test_noalloc_forward_equals_forward_twice_in_a_row(first, second):
    from customnetworklayers_amd._lib import lib

    for n, c, h, w, its in (first, second):
        print("case n=%d c=%d h=%d w=%d its=%d" % (n, c, h, w, its), flush=True)
        d = tv_inputs(n, c, h, w, seed=h + w + its, conf_density=0.3)
        out, ref = _both_forwards(lib, d, its)
        assert np.isfinite(ref).all()
        assert np.array_equal(out, ref), float(np.abs(out - ref).max())


def _inputs_on_device(d):
    dev = torch.device("cuda:0")
    return {k: torch.from_numpy(v).to(dev) for k, v in d.items()}


@pytest.mark.parametrize("shape,its", [
    ((1, 2, 70, 150), 2),   # one pair launch: it must not read the buffer it writes
    ((2, 3, 33, 130), 3),   # the same with an odd count and the two-wavefront channel count
    ((1, 2, 70, 150), 10),  # several launches: the first reads the buffer, the last writes it
    ((1, 1, 9, 40), 0),     # nothing to do
])
def test_noalloc_forward_in_place(shape, its):
    from customnetworklayers_amd._lib import lib

    n, c, h, w = shape
    print("case in place n=%d c=%d h=%d w=%d its=%d" % (n, c, h, w, its), flush=True)
    d = tv_inputs(n, c, h, w, seed=3 * h + its, conf_density=0.3)
    t = _inputs_on_device(d)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    args = [_ptr(t[k]) for k in ("dx", "dy", "dc", "db")]
    # out of place first (its = 2 takes the single pair launch here too), as the expected result
    expect = torch.full_like(t["db"], float("nan"))
    assert lib.tvinpaint_forward_noalloc(*args, _ptr(t["di"]), _ptr(expect), n, c, h, w, its, stream) == 0, lib.tvinpaint_last_error()
    ref = torch.full_like(t["db"], float("nan"))
    assert lib.tvinpaint_reset_id(7) == 0
    assert lib.tvinpaint_forward(*args, _ptr(t["di"]), _ptr(ref), n, c, h, w, its, 7, stream) == 0, lib.tvinpaint_last_error()
    buf = t["di"].clone()
    assert lib.tvinpaint_forward_noalloc(*args, _ptr(buf), _ptr(buf), n, c, h, w, its, stream) == 0, lib.tvinpaint_last_error()
    torch.cuda.synchronize()
    assert lib.tvinpaint_reset_id(7) == 0
    assert torch.equal(expect, ref)
    assert torch.equal(buf, ref), float((buf - ref).abs().max())


def test_noalloc_forward_leaves_free_memory_as_it_was():
    from customnetworklayers_amd._lib import lib

    d = tv_inputs(2, 2, 96, 200, seed=5, conf_density=0.3)
    t = _inputs_on_device(d)
    n, c, h, w = d["db"].shape
    out = torch.empty_like(t["db"])
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    args = [_ptr(t[k]) for k in ("dx", "dy", "dc", "db", "di")]
    assert lib.tvinpaint_forward_noalloc(*args, _ptr(out), n, c, h, w, 12, stream) == 0  # (resolves the scratch address)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for its in (12, 7, 2):
        assert lib.tvinpaint_forward_noalloc(*args, _ptr(out), n, c, h, w, its, stream) == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before


def test_noalloc_forward_inside_a_hip_graph():
    """The call recorded into a HIP graph (after one eager call has looked the scratch address up) and replayed on
    changed inputs, with eager work and synchronisation between the replays: every replay equals tvinpaint_forward."""
    from customnetworklayers_amd._lib import lib

    n, c, h, w, its = 2, 2, 96, 200, 12
    t = _inputs_on_device(tv_inputs(n, c, h, w, seed=1, conf_density=0.3))
    out = torch.full_like(t["db"], float("nan"))
    args = [_ptr(t[k]) for k in ("dx", "dy", "dc", "db", "di")]
    eager = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.tvinpaint_forward_noalloc(*args, _ptr(out), n, c, h, w, its, eager) == 0, lib.tvinpaint_last_error()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        side = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.tvinpaint_forward_noalloc(*args, _ptr(out), n, c, h, w, its, side)
    assert rc == 0, lib.tvinpaint_last_error()
    for replay in range(3):
        print("replay %d" % replay, flush=True)
        fresh = tv_inputs(n, c, h, w, seed=10 + replay, conf_density=0.3)
        for k in ("dx", "dy", "dc", "db", "di"):
            t[k].copy_(torch.from_numpy(fresh[k]))
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        ref = torch.full_like(out, float("nan"))
        assert lib.tvinpaint_reset_id(7) == 0
        assert lib.tvinpaint_forward(*args, _ptr(ref), n, c, h, w, its, 7, eager) == 0, lib.tvinpaint_last_error()
        torch.cuda.synchronize()
        assert lib.tvinpaint_reset_id(7) == 0
        assert torch.equal(out, ref), "replay %d: %g" % (replay, float((out - ref).abs().max()))


def test_noalloc_forward_rejects_what_does_not_fit_its_scratch():
    from customnetworklayers_amd._lib import last_error, lib

    limit = lib.tvinpaint_forward_noalloc_max_floats()
    assert limit == 1 << 22
    dev = torch.device("cuda:0")
    one = torch.zeros(16, device=dev)
    p = _ptr(one)
    # 1 x 2 x 2048 x 1025 floats is one row of pixels more than the limit: refused on the host, nothing is launched
    assert lib.tvinpaint_forward_noalloc(p, p, p, p, p, p, 1, 2, 2048, 1025, 4, None) == 2
    assert "scratch" in last_error()
    torch.cuda.synchronize()
