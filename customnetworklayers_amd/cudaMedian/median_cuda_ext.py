"""Binding module of the median layer: same name and functions as the reference's pybind module
(cudaMedian/median_cuda.cpp:107-112 of the reference), on top of the C ABI in include/flowaux.h.

Differences from the reference binding: every sample of a batch is processed (the reference kernel
is right for n == 1 only, cudaMedian/cudaCode/medimax.cu:23); failures raise instead of returning an
empty list.
"""
import ctypes

import torch

from .._lib import lib

_ERRORS = {1: IndexError, 2: ValueError, 3: ValueError, 4: RuntimeError, 5: RuntimeError}


def _last_error():
    return lib.flowaux_last_error().decode("utf-8", "replace")


def _check_input(t, name):
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s must be a tensor" % name)
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)
    if t.dtype != torch.float32:
        raise TypeError("Input/Output type to the operator must be single/float (%s is %s)" % (name, t.dtype))


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def forward(in_vol):
    """in_vol: (n,h,w,d), the d histogram bins innermost (median_cuda.cpp:43-46).  Returns [(n,2,h,w)]:
    the median's position in bins and the mass of the bin that holds it."""
    _check_input(in_vol, "in_vol")
    if in_vol.dim() != 4:
        raise ValueError("in_vol must be (n, h, w, d)")
    n, h, w, d = in_vol.shape
    solution = torch.empty((n, 2, h, w), dtype=torch.float32, device=in_vol.device)
    with torch.cuda.device(in_vol.device):
        rc = lib.medimax_forward(in_vol.data_ptr(), solution.data_ptr(), n, h, w, d, _stream(in_vol))
    if rc:
        raise _ERRORS.get(rc, RuntimeError)("MediMax::forward failed: %s" % _last_error())
    return [solution]


def backward(d_iGf, in_vol):
    """d_iGf: (n,2,h,w) gradient wrt the result.  Returns [gradient wrt in_vol]."""
    _check_input(in_vol, "in_vol")
    _check_input(d_iGf, "d_iGf")
    if in_vol.dim() != 4:
        raise ValueError("in_vol must be (n, h, w, d)")
    n, h, w, d = in_vol.shape
    if tuple(d_iGf.shape) != (n, 2, h, w):
        raise ValueError("d_iGf must have shape (%d, 2, %d, %d), got %s" % (n, h, w, tuple(d_iGf.shape)))
    if d_iGf.device != in_vol.device:
        raise RuntimeError("all tensors must live on one device")
    outGrad = torch.empty_like(in_vol)
    with torch.cuda.device(in_vol.device):
        rc = lib.medimax_backward(in_vol.data_ptr(), d_iGf.data_ptr(), outGrad.data_ptr(), n, h, w, d, _stream(in_vol))
    if rc:
        raise _ERRORS.get(rc, RuntimeError)("MediMax::backward failed: %s" % _last_error())
    return [outGrad]


def dummy():
    print("Input: not present just dummy:")
    return []


def dummy_only():
    print("Dummy call:")
