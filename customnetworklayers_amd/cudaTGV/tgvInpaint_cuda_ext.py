"""Binding module of the TGV inpainting layer: same name and functions as the reference's pybind
module (cudaTGV/TGVInpaintFista_cuda.cpp:175-180 of the reference), on top of the C ABI in
include/tgvinpaint.h.

Differences from the reference binding, all at its edges: a batch of n >= 1 independent problems
and c >= 1 flow channels are accepted (the reference insists on n == 1 and on a 3-channel starting
point, TGVInpaintFista_cuda.cpp:77-86); the solution and the gradient wrt the starting point have
the 3*c channels the layer really writes (the reference binding allocates only c of them,
TGVInpaintFista_cuda.cpp:91,157); failures raise instead of returning an empty list.
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
from ..cudaTV.tvInpaint_cuda_ext import _check_input, _ERRORS, _stream


def _raise(rc, what):
    raise _ERRORS.get(rc, RuntimeError)("%s failed: %s" % (what, last_error()))


def _check_shapes(d_x, d_y, d_c, d_b, d_s, s_name):
    if d_b.dim() != 4:
        raise ValueError("d_b must be (n, c, h, w)")
    n, c, h, w = d_b.shape
    # TGVInpaintFista_cuda.cpp:69-76: two channels, edge weight and beta
    for t, name in ((d_x, "d_x"), (d_y, "d_y")):
        if tuple(t.shape) != (n, 2, h, w):
            raise ValueError("%s must have shape (%d, 2, %d, %d): the first channel operates on gradients, the "
                             "second on the auxiliary variables; got %s" % (name, n, h, w, tuple(t.shape)))
    if tuple(d_c.shape) != (n, 1, h, w):
        raise ValueError("d_c must have shape (%d, 1, %d, %d), got %s" % (n, h, w, tuple(d_c.shape)))
    # TGVInpaintFista_cuda.cpp:82-86: primary and 2 x auxiliary variables
    if tuple(d_s.shape) != (n, 3 * c, h, w):
        raise ValueError("%s must have shape (%d, %d, %d, %d) (primary and two auxiliary variables per channel), "
                         "got %s" % (s_name, n, 3 * c, h, w, tuple(d_s.shape)))
    if len({t.device for t in (d_x, d_y, d_c, d_b, d_s)}) != 1:
        raise RuntimeError("all tensors must live on one device")


def forward(d_x, d_y, d_c, d_b, d_i, its, id, keep=None):  # noqa: A002 - the reference's argument name
    """d_x, d_y: (n,2,h,w) edge weight and beta along W / H; d_c: (n,1,h,w) confidence; d_b: (n,c,h,w)
    right-hand side; d_i: (n,3c,h,w) starting point (u, v1, v2).  Returns [solution (n,3c,h,w)].
    keep (not in the reference): keep mode for this one call, see keep_iterates; None = the id's own."""
    for t, name in ((d_x, "d_x"), (d_y, "d_y"), (d_c, "d_c"), (d_b, "d_b"), (d_i, "d_i")):
        _check_input(t, name)
    _check_shapes(d_x, d_y, d_c, d_b, d_i, "d_i")
    n, c, h, w = d_b.shape
    solution = torch.empty_like(d_i)
    if keep is not None:
        _set_keep(id, keep)
    with torch.cuda.device(d_b.device):
        rc = lib.tgvinpaint_forward(d_x.data_ptr(), d_y.data_ptr(), d_c.data_ptr(), d_b.data_ptr(), d_i.data_ptr(),
                                    solution.data_ptr(), n, c, h, w, int(its), int(id), _stream(d_b))
    if keep is not None:
        _set_keep(id, _keep_modes.get(int(id), 2))
    if rc:
        _raise(rc, "TGVInpaint::forward")
    return [solution]


def backward(d_iGf, d_x, d_y, d_c, d_b, its, id):  # noqa: A002
    """d_iGf: (n,3c,h,w) gradient wrt the solution.  Returns [d_oGx, d_oGy, d_oGc, d_oGb, d_oGi]; all
    zero (and d_iGf scrubbed in place) when d_iGf holds a non-finite entry or is zero everywhere."""
    for t, name in ((d_x, "d_x"), (d_y, "d_y"), (d_c, "d_c"), (d_b, "d_b"), (d_iGf, "d_iGf")):
        _check_input(t, name)
    _check_shapes(d_x, d_y, d_c, d_b, d_iGf, "d_iGf")
    n, c, h, w = d_b.shape
    d_oGx, d_oGy, d_oGc = torch.empty_like(d_x), torch.empty_like(d_y), torch.empty_like(d_c)
    d_oGb, d_oGi = torch.empty_like(d_b), torch.empty_like(d_iGf)
    with torch.cuda.device(d_b.device):
        rc = lib.tgvinpaint_backward(d_x.data_ptr(), d_y.data_ptr(), d_c.data_ptr(), d_b.data_ptr(), d_iGf.data_ptr(),
                                     d_oGx.data_ptr(), d_oGy.data_ptr(), d_oGc.data_ptr(), d_oGb.data_ptr(),
                                     d_oGi.data_ptr(), n, c, h, w, int(its), int(id), _stream(d_b))
    if rc:
        _raise(rc, "TGVInpaint::backward")
    return [d_oGx, d_oGy, d_oGc, d_oGb, d_oGi]


def dummy():
    print("Input: not present just dummy:")
    return []


def dummy_only():
    print("Dummy call:")


# ---- additions for tests and tooling (no counterpart in the reference module) -------------------
def get_state(id):  # noqa: A002
    buf = (ctypes.c_double * 6)()
    rc = lib.tgvinpaint_get_state(int(id), buf)
    if rc:
        _raise(rc, "get_state")
    return list(buf)


def set_state(id, state6):  # noqa: A002
    buf = (ctypes.c_double * 6)(*[float(v) for v in state6])
    rc = lib.tgvinpaint_set_state(int(id), buf)
    if rc:
        _raise(rc, "set_state")


def reset_id(id):  # noqa: A002
    rc = lib.tgvinpaint_reset_id(int(id))
    if rc:
        _raise(rc, "reset_id")
    _keep_modes.pop(int(id), None)


def gradient_mode(id, mode):  # noqa: A002
    """0 (default): the reference's backward, bit for bit.  1: the corrected gradient -- the adjoint linearised at
    the forward pass's own y, iteration 0 back-propagated, all multipliers 1 (see include/tgvinpaint.h)."""
    rc = lib.tgvinpaint_gradient_mode(int(id), int(mode))
    if rc:
        _raise(rc, "gradient_mode")


def slot_bytes(id):  # noqa: A002
    """Bytes of device memory the id's slot owns."""
    return int(lib.tgvinpaint_slot_bytes(int(id)))


_keep_modes = {}  # id -> mode set through keep_iterates (the library's default is 2)


def _set_keep(id, mode):  # noqa: A002
    rc = lib.tgvinpaint_keep_iterates(int(id), int(mode))
    if rc:
        _raise(rc, "keep_iterates")


def keep_iterates(id, mode):  # noqa: A002
    """Which intermediate iterates the forwards on `id` keep for the backward: 0 none (the backward recomputes every
    segment from its checkpoint, as the reference does), 1 the last segment's, 2 all (default: no recompute, `its`
    more fields of memory).  The gradients are the same bits in every mode."""
    _set_keep(id, mode)
    _keep_modes[int(id)] = int(mode)


def guard_stats(id):  # noqa: A002
    """Five rows (C, X, Y, B, I) of [mean |g|, max |g|, count > 5e6, count non-finite, action]."""
    buf = (ctypes.c_double * 25)()
    rc = lib.tgvinpaint_guard_stats(int(id), buf)
    if rc:
        _raise(rc, "guard_stats")
    return [list(buf[5 * k:5 * k + 5]) for k in range(5)]


def lipschitz(id, n):  # noqa: A002
    """Per-sample step scale L of the last call on this id."""
    buf = (ctypes.c_double * int(n))()
    rc = lib.tgvinpaint_lipschitz(int(id), buf, int(n))
    if rc:
        _raise(rc, "lipschitz")
    return list(buf)


def guard_decide(run, av_gc, av_running):
    mult, av = ctypes.c_double(0), ctypes.c_double(0)
    action = lib.tgvinpaint_guard_decide(int(run), float(av_gc), float(av_running), ctypes.byref(mult), ctypes.byref(av))
    return action, mult.value, av.value
