"""Loader of the HIP library behind the layers.  There is no fallback: if the library is missing
or cannot be loaded the import fails, and the message says how to build it."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libinpaint_hip.so")

_f32p = ctypes.c_void_p  # device pointers travel as integers
_int = ctypes.c_int


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "%s is missing: build it with `make -C %s` (or `python setup.py build_ext`)"
            % (LIB_PATH, os.path.join(_HERE, "csrc")))
    lib = ctypes.CDLL(LIB_PATH)
    lib.tvinpaint_forward.argtypes = [_f32p] * 6 + [_int] * 6 + [ctypes.c_void_p]
    lib.tvinpaint_backward.argtypes = [_f32p] * 10 + [_int] * 6 + [ctypes.c_void_p]
    lib.tvinpaint_forward_noalloc.argtypes = [_f32p] * 6 + [_int] * 5 + [ctypes.c_void_p]
    lib.tvinpaint_forward_noalloc_max_floats.restype = ctypes.c_longlong
    lib.tvinpaint_get_state.argtypes = [_int, ctypes.POINTER(ctypes.c_double)]
    lib.tvinpaint_set_state.argtypes = [_int, ctypes.POINTER(ctypes.c_double)]
    lib.tvinpaint_reset_id.argtypes = [_int]
    lib.tvinpaint_guard_stats.argtypes = [_int, ctypes.POINTER(ctypes.c_double)]
    lib.tvinpaint_keep_iterates.argtypes = [_int, _int]
    lib.tvinpaint_gradient_mode.argtypes = [_int, _int]
    lib.tvinpaint_slot_bytes.argtypes = [_int]
    lib.tvinpaint_slot_bytes.restype = ctypes.c_longlong
    lib.tvinpaint_set_allocator.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    lib.tgvinpaint_set_allocator.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    lib.tvinpaint_schedule.argtypes = [_int, ctypes.POINTER(_int), ctypes.POINTER(_int)]
    lib.tvinpaint_step_sizes.argtypes = [_int, ctypes.POINTER(ctypes.c_float)]
    lib.tvinpaint_step_sizes.restype = None
    lib.tvinpaint_selftest_guard.argtypes = [ctypes.c_void_p, ctypes.c_longlong, _int, _int, ctypes.c_double,
                                             ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_double)]
    lib.tvinpaint_guard_decide.argtypes = [_int, ctypes.c_double, ctypes.c_double,
                                           ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]
    lib.tvinpaint_profile.argtypes = [_int]
    lib.tvinpaint_profile_read.argtypes = [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(_int)]
    lib.inpaint_selftest_math.argtypes = [ctypes.POINTER(ctypes.c_ulonglong), ctypes.c_uint]
    lib.inpaint_selftest_division_pairs.argtypes = [ctypes.c_uint, ctypes.c_uint, ctypes.POINTER(ctypes.c_ulonglong)]
    lib.inpaint_reload_env.restype = None
    lib.inpaint_copy_bandwidth.argtypes = [ctypes.c_longlong, _int, ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]
    lib.inpaint_stream_bandwidth.argtypes = [ctypes.c_longlong, _int, _int, _int, ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]
    lib.tvinpaint_last_error.restype = ctypes.c_char_p
    lib.tgvinpaint_forward.argtypes = [_f32p] * 6 + [_int] * 6 + [ctypes.c_void_p]
    lib.tgvinpaint_backward.argtypes = [_f32p] * 10 + [_int] * 6 + [ctypes.c_void_p]
    lib.tgvinpaint_get_state.argtypes = [_int, ctypes.POINTER(ctypes.c_double)]
    lib.tgvinpaint_set_state.argtypes = [_int, ctypes.POINTER(ctypes.c_double)]
    lib.tgvinpaint_reset_id.argtypes = [_int]
    lib.tgvinpaint_guard_stats.argtypes = [_int, ctypes.POINTER(ctypes.c_double)]
    lib.tgvinpaint_keep_iterates.argtypes = [_int, _int]
    lib.tgvinpaint_gradient_mode.argtypes = [_int, _int]
    lib.tgvinpaint_slot_bytes.argtypes = [_int]
    lib.tgvinpaint_slot_bytes.restype = ctypes.c_longlong
    lib.tgvinpaint_lipschitz.argtypes = [_int, ctypes.POINTER(ctypes.c_double), _int]
    lib.tgvinpaint_selftest_guard.argtypes = [ctypes.c_void_p, ctypes.c_longlong, _int, _int, ctypes.c_double,
                                              ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_double)]
    lib.tgvinpaint_guard_decide.argtypes = [_int, ctypes.c_double, ctypes.c_double,
                                            ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]
    lib.tgvinpaint_profile.argtypes = [_int]
    lib.tgvinpaint_profile_read.argtypes = [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(_int)]
    lib.tgvinpaint_last_error.restype = ctypes.c_char_p
    lib.inpaint_selftest_rsqrt.argtypes = [ctypes.POINTER(ctypes.c_ulonglong), ctypes.c_uint]
    lib.quadfit_forward.argtypes = [_f32p] * 4 + [_int] * 5 + [ctypes.c_void_p]
    lib.quadfit_backward.argtypes = [_f32p] * 6 + [_int] * 5 + [ctypes.c_void_p, ctypes.c_longlong, ctypes.c_void_p]
    lib.quadfit_backward_workspace_bytes.argtypes = [_int] * 3
    lib.quadfit_backward_workspace_bytes.restype = ctypes.c_longlong
    lib.medimax_forward.argtypes = [_f32p] * 2 + [_int] * 4 + [ctypes.c_void_p]
    lib.medimax_backward.argtypes = [_f32p] * 3 + [_int] * 4 + [ctypes.c_void_p]
    lib.flowaux_last_error.restype = ctypes.c_char_p
    lib.hierarchy_next_level_forward.argtypes = [_f32p] * 5 + [_int] * 4 + [ctypes.c_float, ctypes.c_float, ctypes.c_void_p]
    lib.hierarchy_next_level_backward.argtypes = [_f32p] * 3 + [_int] * 4 + [ctypes.c_float, ctypes.c_void_p]
    lib.hierarchy_last_error.restype = ctypes.c_char_p
    lib.flowaux_profile.argtypes = [_int]
    lib.flowaux_profile_read.argtypes = [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(_int)]
    return lib


lib = _load()


# ---- the slots' device memory out of PyTorch's caching allocator (t[g]vinpaint_set_allocator) -------------------
_ALLOC_FN = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_ulonglong, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p)
_RELEASE_FN = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_void_p)


def _torch_alloc(nbytes, device, stream, user):
    try:
        import torch

        return torch.cuda.caching_allocator_alloc(int(nbytes), device, int(stream or 0))
    except Exception:  # out of memory: the library falls back (keep mode 1) or reports the failure itself
        return None


def _torch_release(ptr, user):
    import torch

    torch.cuda.caching_allocator_delete(ptr)


# (kept alive for as long as the library may call them)
_torch_alloc_c, _torch_release_c = _ALLOC_FN(_torch_alloc), _RELEASE_FN(_torch_release)
_torch_allocator_on = False


def use_torch_allocator(enable=True):
    """Take the per-id device blocks of both layers from PyTorch's caching allocator (on by default for the modules of
    this package), so that they show up in torch.cuda.memory_allocated() and return to the pool PyTorch reuses;
    enable=False goes back to hipMalloc / hipFree.  Blocks already handed out stay with the allocator that made them."""
    global _torch_allocator_on
    a, r = (ctypes.cast(_torch_alloc_c, ctypes.c_void_p), ctypes.cast(_torch_release_c, ctypes.c_void_p)) if enable else (None, None)
    for fn in (lib.tvinpaint_set_allocator, lib.tgvinpaint_set_allocator):
        if fn(a, r, None) != 0:
            raise RuntimeError(last_error())
    _torch_allocator_on = bool(enable)


def torch_allocator_in_use():
    return _torch_allocator_on


def reload_env():
    """Re-read the INPAINT_* environment variables (they are read once per process otherwise, and by reset_id)."""
    lib.inpaint_reload_env()


def last_error():
    return lib.tvinpaint_last_error().decode("utf-8", "replace")
