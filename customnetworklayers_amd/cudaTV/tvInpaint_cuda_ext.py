"""Binding module of the TV inpainting layer: same name and functions as the reference's pybind
module (cudaTV/TVInpaintFista_cuda.cpp:145-150 of the reference), on top of the C ABI in
include/tvinpaint.h.

Differences from the reference binding, all at its edges: a batch of n >= 1 independent problems
is accepted (the reference prints a message and returns an empty list for n != 1,
TVInpaintFista_cuda.cpp:61-65), and failures raise instead of returning an empty list
(TVInpaintFista_cuda.cpp:80-87).
"""
import ctypes
import os

import torch

from .._lib import last_error, lib, torch_allocator_in_use, use_torch_allocator

# The per-id device blocks come out of PyTorch's caching allocator (t[g]vinpaint_set_allocator), so that
# torch.cuda.memory_allocated() counts them and reset_id() returns them to the pool; INPAINT_TORCH_ALLOCATOR=0 leaves
# them with hipMalloc.
if os.environ.get("INPAINT_TORCH_ALLOCATOR", "1") != "0" and not torch_allocator_in_use():
    use_torch_allocator(True)

_ERRORS = {1: IndexError, 2: ValueError, 3: ValueError, 4: RuntimeError, 5: RuntimeError}


def _check_input(t, name):
    # CHECK_CUDA / CHECK_CONTIGUOUS, TVInpaintFista_cuda.cpp:24-26
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s must be a tensor" % name)
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)
    if t.dtype != torch.float32:  # TVInpaintFista_cuda.cpp:68,86
        raise TypeError("Input/Output type to the operator must be single/float (%s is %s)" % (name, t.dtype))


def _raise(rc, what):
    raise _ERRORS.get(rc, RuntimeError)("%s failed: %s" % (what, last_error()))


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _check_shapes(d_x, d_y, d_c, d_b, others):
    if d_b.dim() != 4:
        raise ValueError("d_b must be (n, c, h, w)")
    n, _, h, w = d_b.shape
    for t, name in ((d_x, "d_x"), (d_y, "d_y"), (d_c, "d_c")):
        if tuple(t.shape) != (n, 1, h, w):
            raise ValueError("%s must have shape (%d, 1, %d, %d), got %s" % (name, n, h, w, tuple(t.shape)))
    for t, name in others:
        if tuple(t.shape) != tuple(d_b.shape):
            raise ValueError("%s must have the shape of d_b %s, got %s" % (name, tuple(d_b.shape), tuple(t.shape)))
    devs = {t.device for t in (d_x, d_y, d_c, d_b) + tuple(o for o, _ in others)}
    if len(devs) != 1:
        raise RuntimeError("all tensors must live on one device")


def forward(d_x, d_y, d_c, d_b, d_i, its, id, keep=None):  # noqa: A002 - the reference's argument name
    """d_x, d_y: edge weights along W / H, d_c: confidence, (n,1,h,w); d_b: right-hand side and d_i:
    starting point, (n,c,h,w).  Returns [solution] after 2*floor(its/2) iterations.
    keep (not in the reference): keep mode for this one call, see keep_iterates; None = the id's own."""
    for t, name in ((d_x, "d_x"), (d_y, "d_y"), (d_c, "d_c"), (d_b, "d_b"), (d_i, "d_i")):
        _check_input(t, name)
    _check_shapes(d_x, d_y, d_c, d_b, ((d_i, "d_i"),))
    n, c, h, w = d_b.shape
    solution = torch.empty_like(d_b)
    if keep is not None:
        _set_keep(id, keep)
    with torch.cuda.device(d_b.device):
        rc = lib.tvinpaint_forward(d_x.data_ptr(), d_y.data_ptr(), d_c.data_ptr(), d_b.data_ptr(), d_i.data_ptr(),
                                   solution.data_ptr(), n, c, h, w, int(its), int(id), _stream(d_b))
    if keep is not None:
        _set_keep(id, _keep_modes.get(int(id), 2))
    if rc:
        _raise(rc, "TVInpaint::forward")
    return [solution]


def backward(d_iGf, d_x, d_y, d_c, d_b, its, id):  # noqa: A002
    """d_iGf: gradient wrt the solution (non-finite entries are zeroed in place, as the reference
    does).  Returns [d_oGx, d_oGy, d_oGc, d_oGb, d_oGi]."""
    for t, name in ((d_x, "d_x"), (d_y, "d_y"), (d_c, "d_c"), (d_b, "d_b"), (d_iGf, "d_iGf")):
        _check_input(t, name)
    _check_shapes(d_x, d_y, d_c, d_b, ((d_iGf, "d_iGf"),))
    n, c, h, w = d_b.shape
    d_oGx, d_oGy, d_oGc = torch.empty_like(d_x), torch.empty_like(d_y), torch.empty_like(d_c)
    d_oGb, d_oGi = torch.empty_like(d_b), torch.empty_like(d_b)
    with torch.cuda.device(d_b.device):
        rc = lib.tvinpaint_backward(d_x.data_ptr(), d_y.data_ptr(), d_c.data_ptr(), d_b.data_ptr(), d_iGf.data_ptr(),
                                    d_oGx.data_ptr(), d_oGy.data_ptr(), d_oGc.data_ptr(), d_oGb.data_ptr(),
                                    d_oGi.data_ptr(), n, c, h, w, int(its), int(id), _stream(d_b))
    if rc:
        _raise(rc, "TVInpaint::backward")
    return [d_oGx, d_oGy, d_oGc, d_oGb, d_oGi]


def forward_noalloc(d_x, d_y, d_c, d_b, d_i, its, out):
    """The forward pass without an id and without any device allocation (not in the reference): the caller passes
    the output tensor, the iterates live in a fixed array inside the library.  For inference under graph capture or
    in loops that must not allocate; no backward can follow.  Raises ValueError when d_b holds more than
    noalloc_max_floats() values.  Calls that overlap on one GPU share the array and race."""
    for t, name in ((d_x, "d_x"), (d_y, "d_y"), (d_c, "d_c"), (d_b, "d_b"), (d_i, "d_i"), (out, "out")):
        _check_input(t, name)
    _check_shapes(d_x, d_y, d_c, d_b, ((d_i, "d_i"), (out, "out")))
    n, c, h, w = d_b.shape
    with torch.cuda.device(d_b.device):
        rc = lib.tvinpaint_forward_noalloc(d_x.data_ptr(), d_y.data_ptr(), d_c.data_ptr(), d_b.data_ptr(), d_i.data_ptr(),
                                           out.data_ptr(), n, c, h, w, int(its), _stream(d_b))
    if rc:
        _raise(rc, "TVInpaint::forward_noalloc")
    return out


def noalloc_max_floats():
    """Largest n*c*h*w forward_noalloc accepts."""
    return int(lib.tvinpaint_forward_noalloc_max_floats())


def dummy():
    print("Input: not present just dummy:")
    return []


def dummy_only():
    print("Dummy call:")


# ---- additions for tests and tooling (no counterpart in the reference module) -------------------
def get_state(id):  # noqa: A002
    """(run, av_GC, av_GX, av_GY, av_GB, av_GI) of the id's guard."""
    buf = (ctypes.c_double * 6)()
    rc = lib.tvinpaint_get_state(int(id), buf)
    if rc:
        _raise(rc, "get_state")
    return list(buf)


def set_state(id, state6):  # noqa: A002
    buf = (ctypes.c_double * 6)(*[float(v) for v in state6])
    rc = lib.tvinpaint_set_state(int(id), buf)
    if rc:
        _raise(rc, "set_state")


def reset_id(id):  # noqa: A002
    rc = lib.tvinpaint_reset_id(int(id))
    if rc:
        _raise(rc, "reset_id")
    _keep_modes.pop(int(id), None)


def gradient_mode(id, mode):  # noqa: A002
    """0 (default): the reference's backward, bit for bit.  1: the corrected gradient -- the adjoint linearised at
    the forward pass's own y, iteration 0 back-propagated, all multipliers 1 (see include/tvinpaint.h)."""
    rc = lib.tvinpaint_gradient_mode(int(id), int(mode))
    if rc:
        _raise(rc, "gradient_mode")


def slot_bytes(id):  # noqa: A002
    """Bytes of device memory the id's slot owns."""
    return int(lib.tvinpaint_slot_bytes(int(id)))


_keep_modes = {}  # id -> mode set through keep_iterates (the library's default is 2)


def _set_keep(id, mode):  # noqa: A002
    rc = lib.tvinpaint_keep_iterates(int(id), int(mode))
    if rc:
        _raise(rc, "keep_iterates")


def keep_iterates(id, mode):  # noqa: A002
    """Which intermediate iterates the forwards on `id` keep for the backward: 0 none (the backward recomputes every
    segment from its checkpoint, as the reference does), 1 the last segment's, 2 all (default: no recompute, `its`
    more fields of memory).  The gradients are the same bits in every mode."""
    _set_keep(id, mode)
    _keep_modes[int(id)] = int(mode)


def guard_stats(id):  # noqa: A002
    """Five rows (C, X, Y, B, I) of [mean |g|, max |g|, count > 1e7, count non-finite, action]."""
    buf = (ctypes.c_double * 25)()
    rc = lib.tvinpaint_guard_stats(int(id), buf)
    if rc:
        _raise(rc, "guard_stats")
    return [list(buf[5 * k:5 * k + 5]) for k in range(5)]


def schedule(its):
    n = max(int(int(its) ** 0.5) + 1, 1)
    buf = (ctypes.c_int * n)()
    m = ctypes.c_int(0)
    cnt = lib.tvinpaint_schedule(int(its), buf, ctypes.byref(m))
    return list(buf[:cnt]), m.value


def step_sizes(its):
    buf = (ctypes.c_float * max(int(its), 1))()
    lib.tvinpaint_step_sizes(int(its), buf)
    return list(buf[:int(its)])


def guard_decide(run, av_gc, av_running):
    """(action, multiplier, new running mean) of the guard's decision rule for one tensor."""
    mult, av = ctypes.c_double(0), ctypes.c_double(0)
    action = lib.tvinpaint_guard_decide(int(run), float(av_gc), float(av_running), ctypes.byref(mult), ctypes.byref(av))
    return action, mult.value, av.value
