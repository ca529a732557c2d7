"""Glue between two levels of a coarse-to-fine hierarchy of inpainting layers, on the C ABI of
include/hierarchy.h: the fine level's right-hand side / starting point (2 x bilinear x2 upsampling
of the coarse solution) and its edge weights exp(-alpha |grad I|) in one launch, with the adjoint of
the upsampling for the backward pass.  The reference describes such a hierarchy (README.md:64-71 of
the reference) without shipping this step."""
import ctypes

import torch
from torch.autograd import Function

from ._lib import lib

_ERRORS = {1: IndexError, 2: ValueError, 3: ValueError, 4: RuntimeError, 5: RuntimeError}


def _check(t, name):
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s must be a tensor" % name)
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)
    if t.dtype != torch.float32:
        raise TypeError("%s must be float32, got %s" % (name, t.dtype))


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _raise(rc, what):
    raise _ERRORS.get(rc, RuntimeError)("%s failed: %s" % (what, lib.hierarchy_last_error().decode("utf-8", "replace")))


def next_level_forward(sol, img=None, scale=2.0, alpha=10.0):
    """sol: (n,c,h,w); img: (n,1,2h,2w) or None.  Returns (up, wx, wy); wx, wy are None without an image."""
    _check(sol, "sol")
    if sol.dim() != 4:
        raise ValueError("sol must be (n, c, h, w)")
    n, c, h, w = sol.shape
    up = torch.empty((n, c, 2 * h, 2 * w), dtype=torch.float32, device=sol.device)
    wx = wy = None
    if img is not None:
        _check(img, "img")
        if tuple(img.shape) != (n, 1, 2 * h, 2 * w):
            raise ValueError("img must have shape (%d, 1, %d, %d), got %s" % (n, 2 * h, 2 * w, tuple(img.shape)))
        if img.device != sol.device:
            raise RuntimeError("all tensors must live on one device")
        wx, wy = torch.empty_like(img), torch.empty_like(img)
    with torch.cuda.device(sol.device):
        rc = lib.hierarchy_next_level_forward(sol.data_ptr(), None if img is None else img.data_ptr(), up.data_ptr(),
                                              None if img is None else wx.data_ptr(),
                                              None if img is None else wy.data_ptr(), n, c, h, w, float(scale),
                                              float(alpha), _stream(sol))
    if rc:
        _raise(rc, "hierarchy_next_level_forward")
    return up, wx, wy


def next_level_backward(g_b, g_init=None, scale=2.0):
    """g_b (and g_init, summed): (n,c,2h,2w) gradients wrt the fine level's right-hand side / starting point.
    Returns the gradient wrt the coarse solution, (n,c,h,w)."""
    _check(g_b, "g_b")
    if g_b.dim() != 4 or g_b.shape[2] % 2 or g_b.shape[3] % 2:
        raise ValueError("g_b must be (n, c, 2h, 2w)")
    if g_init is not None:
        _check(g_init, "g_init")
        if tuple(g_init.shape) != tuple(g_b.shape) or g_init.device != g_b.device:
            raise ValueError("g_init must match g_b")
    n, c, h2, w2 = g_b.shape
    g_sol = torch.empty((n, c, h2 // 2, w2 // 2), dtype=torch.float32, device=g_b.device)
    with torch.cuda.device(g_b.device):
        rc = lib.hierarchy_next_level_backward(g_b.data_ptr(), None if g_init is None else g_init.data_ptr(),
                                               g_sol.data_ptr(), n, c, h2 // 2, w2 // 2, float(scale), _stream(g_b))
    if rc:
        _raise(rc, "hierarchy_next_level_backward")
    return g_sol


class NextLevelFunction(Function):
    """(up, wx, wy) = next_level(sol, img).  `up` feeds both the right-hand side and the starting point of the
    next layer; autograd sums their gradients before they arrive here.  The image carries no gradient."""

    @staticmethod
    def forward(ctx, sol, img, scale, alpha):
        ctx.scale = scale
        up, wx, wy = next_level_forward(sol.contiguous(), img.contiguous(), scale, alpha)
        ctx.mark_non_differentiable(wx, wy)
        return up, wx, wy

    @staticmethod
    def backward(ctx, g_up, g_wx, g_wy):
        return next_level_backward(g_up.contiguous(), None, ctx.scale), None, None, None


def next_level(sol, img, scale=2.0, alpha=10.0):
    return NextLevelFunction.apply(sol, img, scale, alpha)
