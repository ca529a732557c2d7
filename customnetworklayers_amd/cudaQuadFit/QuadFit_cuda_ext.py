"""Binding module of the quadratic-fit layer: same name and functions as the reference's pybind
module (cudaQuadFit/QuadFit_cuda.cpp:117-122 of the reference), on top of the C ABI in
include/flowaux.h.

Differences from the reference binding: the result has 3 channels (offset x, offset y, score) as
the kernel writes them (cudaQuadFit/cudaCode/quadFit.cu:137,315; the reference binding allocates
2, QuadFit_cuda.cpp:60); the flow may have 2 or more channels, of which the first two are read;
failures raise instead of returning an empty list (QuadFit_cuda.cpp:68-74).
"""
import ctypes

import torch

from .._lib import lib

_ERRORS = {1: IndexError, 2: ValueError, 3: ValueError, 4: RuntimeError, 5: RuntimeError}


def _last_error():
    return lib.flowaux_last_error().decode("utf-8", "replace")


def _check_input(t, name):
    # CHECK_CUDA / CHECK_CONTIGUOUS, QuadFit_cuda.cpp:21-23
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s must be a tensor" % name)
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)
    if t.dtype != torch.float32:  # QuadFit_cuda.cpp:57,73
        raise TypeError("Input/Output type to the operator must be single/float (%s is %s)" % (name, t.dtype))


def _check_shapes(featureImage0, featureImage1, flow):
    if featureImage0.dim() != 4:
        raise ValueError("featureImage0 must be (n, c, h, w)")
    n, _, h, w = featureImage0.shape
    if tuple(featureImage1.shape) != tuple(featureImage0.shape):
        raise ValueError("featureImage1 must have the shape of featureImage0 %s, got %s"
                         % (tuple(featureImage0.shape), tuple(featureImage1.shape)))
    if flow.dim() != 4 or flow.shape[0] != n or flow.shape[1] < 2 or tuple(flow.shape[2:]) != (h, w):
        raise ValueError("flow must have shape (%d, >=2, %d, %d), got %s" % (n, h, w, tuple(flow.shape)))
    if len({t.device for t in (featureImage0, featureImage1, flow)}) != 1:
        raise RuntimeError("all tensors must live on one device")


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def forward(featureImage0, featureImage1, flow):
    """featureImage0/1: (n,c,h,w) feature maps; flow: (n,>=2,h,w).  Returns [(n,3,h,w)]: the offsets of the
    fitted maximum in x and y (to be added to the rounded displaced position) and the fitted score."""
    for t, name in ((featureImage0, "featureImage0"), (featureImage1, "featureImage1"), (flow, "flow")):
        _check_input(t, name)
    _check_shapes(featureImage0, featureImage1, flow)
    n, c, h, w = featureImage0.shape
    flowUpdate = torch.empty((n, 3, h, w), dtype=torch.float32, device=flow.device)
    with torch.cuda.device(flow.device):
        rc = lib.quadfit_forward(featureImage0.data_ptr(), featureImage1.data_ptr(), flow.data_ptr(),
                                 flowUpdate.data_ptr(), n, c, h, w, flow.shape[1], _stream(flow))
    if rc:
        raise _ERRORS.get(rc, RuntimeError)("FlowQuadFitting::forward failed: %s" % _last_error())
    return [flowUpdate]


def backward(d_iGf, featureImage0, featureImage1, flow, use_atomics=False):
    """d_iGf: (n,3,h,w) gradient wrt the result.  Returns [d_oFeat0, d_oFeat1].  `use_atomics` selects the
    reference's scatter with float atomics instead of the gather through a scratch buffer."""
    for t, name in ((featureImage0, "featureImage0"), (featureImage1, "featureImage1"), (flow, "flow"),
                    (d_iGf, "d_iGf")):
        _check_input(t, name)
    _check_shapes(featureImage0, featureImage1, flow)
    n, c, h, w = featureImage0.shape
    if tuple(d_iGf.shape) != (n, 3, h, w):
        raise ValueError("d_iGf must have shape (%d, 3, %d, %d), got %s" % (n, h, w, tuple(d_iGf.shape)))
    d_oFeat0, d_oFeat1 = torch.empty_like(featureImage0), torch.empty_like(featureImage1)
    ws_bytes = 0 if use_atomics else lib.quadfit_backward_workspace_bytes(n, h, w)
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=flow.device) if ws_bytes else None
    with torch.cuda.device(flow.device):
        rc = lib.quadfit_backward(featureImage0.data_ptr(), featureImage1.data_ptr(), flow.data_ptr(),
                                  d_iGf.data_ptr(), d_oFeat0.data_ptr(), d_oFeat1.data_ptr(), n, c, h, w,
                                  flow.shape[1], workspace.data_ptr() if ws_bytes else None, ws_bytes, _stream(flow))
    if rc:
        raise _ERRORS.get(rc, RuntimeError)("FlowQuadFitting::backward failed: %s" % _last_error())
    return [d_oFeat0, d_oFeat1]


def dummy():
    print("Input: not present just dummy:")
    return []


def dummy_only():
    print("Dummy call:")
