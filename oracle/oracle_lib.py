"""ctypes front end of the CPU oracles.  TEST INFRASTRUCTURE ONLY.

Only the test-suite, the smoke check and the bench's cpu_baseline leg may import this module; the
shipped package never does.  The shared objects are built by ``make -C oracle`` (or by
``__graft_entry__.build()``) from the C++ restatements that sit next to this file.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i32p = ctypes.POINTER(ctypes.c_int)
_int = ctypes.c_int


def build(force=False):
    """Compile the oracle shared objects in place."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


def _load(name):
    path = os.path.join(_HERE, name)
    if not os.path.exists(path):
        build()
    return ctypes.CDLL(path)


def _p32(a):
    return a.ctypes.data_as(_f32p)


def _p64(a):
    return a.ctypes.data_as(_f64p)


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


class TVOracle:
    """Huber-TV FISTA inpainting layer, CPU restatement (oracle/tv_oracle.cpp)."""

    def __init__(self):
        L = self.lib = _load("libtv_oracle.so")
        L.tv_oracle_forward.argtypes = [_f32p] * 6 + [_int] * 6
        L.tv_oracle_backward.argtypes = [_f32p] * 10 + [_int] * 6
        L.tv_oracle_forward_f64.argtypes = [_f64p] * 6 + [_int] * 6
        L.tv_oracle_backward_f64.argtypes = [_f64p] * 10 + [_int] * 6
        L.tv_oracle_set_quirks.argtypes = [_int] * 6
        L.tv_oracle_set_quirks.restype = None
        L.tv_oracle_reset_id.argtypes = [_int]
        L.tv_oracle_reset_id.restype = None
        L.tv_oracle_get_state.argtypes = [_int, _f64p, _int]
        L.tv_oracle_set_state.argtypes = [_int, _f64p]
        L.tv_oracle_schedule.argtypes = [_int, _i32p, _i32p]
        L.tv_oracle_step_sizes.argtypes = [_int, _f32p]
        L.tv_oracle_step_sizes.restype = None
        L.tv_oracle_forward_iter.argtypes = [_f32p] * 8 + [_int] * 3 + [ctypes.c_float]
        L.tv_oracle_forward_iter.restype = None
        L.tv_oracle_forward_iter_f64.argtypes = [_f64p] * 8 + [_int] * 3 + [ctypes.c_double]
        L.tv_oracle_forward_iter_f64.restype = None
        L.tv_oracle_guard_f64.argtypes = [_f64p, ctypes.c_long, _int, _f64p, _f64p]
        L.tv_oracle_guard_f32.argtypes = [_f32p, ctypes.c_long, _int, _f64p, _f64p]
        L.tv_oracle_get_yk.argtypes = [_f32p] * 5 + [_int] * 3 + [ctypes.c_float]
        L.tv_oracle_get_yk.restype = None
        L.tv_oracle_get_yk_f64.argtypes = [_f64p] * 5 + [_int] * 3 + [ctypes.c_double]
        L.tv_oracle_get_yk_f64.restype = None
        L.tv_oracle_set_threads.argtypes = [_int]
        L.tv_oracle_set_threads.restype = None

    # -- whole layer ---------------------------------------------------------------------------
    def forward(self, dx, dy, c, b, init, its, pid=0, f64=False):
        """dx, dy, c: (N,1,H,W); b, init: (N,C,H,W).  Returns x after the last iteration."""
        dt = np.float64 if f64 else np.float32
        dx, dy, c, b, init = (_c(a, dt) for a in (dx, dy, c, b, init))
        n, ic, ih, iw = b.shape
        out = np.empty_like(b)
        P = _p64 if f64 else _p32
        fn = self.lib.tv_oracle_forward_f64 if f64 else self.lib.tv_oracle_forward
        rc = fn(P(dx), P(dy), P(c), P(b), P(init), P(out), n, ic, ih, iw, int(its), int(pid))
        if rc:
            raise RuntimeError("tv_oracle_forward failed with code %d" % rc)
        return out

    def backward(self, gin, dx, dy, c, b, its, pid=0, f64=False):
        """Returns (gx, gy, gc, gb, gi); `gin` (a writable array) is scrubbed in place."""
        dt = np.float64 if f64 else np.float32
        dx, dy, c, b = (_c(a, dt) for a in (dx, dy, c, b))
        if gin.dtype != dt or not gin.flags["C_CONTIGUOUS"]:
            gin = _c(gin, dt).copy()
        n, ic, ih, iw = b.shape
        gx, gy, gc = np.empty_like(dx), np.empty_like(dy), np.empty_like(c)
        gb, gi = np.empty_like(b), np.empty_like(b)
        P = _p64 if f64 else _p32
        fn = self.lib.tv_oracle_backward_f64 if f64 else self.lib.tv_oracle_backward
        rc = fn(P(dx), P(dy), P(c), P(b), P(gin), P(gx), P(gy), P(gc), P(gb), P(gi), n, ic, ih, iw,
                int(its), int(pid))
        if rc:
            raise RuntimeError("tv_oracle_backward failed with code %d" % rc)
        return gx, gy, gc, gb, gi

    # -- pieces --------------------------------------------------------------------------------
    def set_quirks(self, end_uses_ckpt_y=1, skip_iter0_adjoint=1, getyk_rebuild=1, scale_factors=1,
                   clamp=1, guard=1):
        self.lib.tv_oracle_set_quirks(end_uses_ckpt_y, skip_iter0_adjoint, getyk_rebuild,
                                      scale_factors, clamp, guard)

    def reset_id(self, pid):
        self.lib.tv_oracle_reset_id(int(pid))

    def get_state(self, pid, f64=False):
        s = np.zeros(6, np.float64)
        self.lib.tv_oracle_get_state(int(pid), _p64(s), int(f64))
        return s

    def set_state(self, pid, state6):
        s = _c(state6, np.float64)
        self.lib.tv_oracle_set_state(int(pid), _p64(s))

    def schedule(self, its):
        buf = np.zeros(max(int(np.floor(np.sqrt(its))), 1), np.int32)
        m = ctypes.c_int(0)
        n = self.lib.tv_oracle_schedule(int(its), buf.ctypes.data_as(_i32p), ctypes.byref(m))
        return [int(v) for v in buf[:n]], m.value

    def step_sizes(self, its):
        out = np.zeros(its, np.float32)
        self.lib.tv_oracle_step_sizes(int(its), _p32(out))
        return out

    def forward_iter(self, wx_scaled, wy_scaled, c, b, x, y, t, want_x05=False, f64=False):
        """One iteration on one sample: fields (H,W) / (C,H,W).  Returns (x_new, y_new[, x05])."""
        dt = np.float64 if f64 else np.float32
        wx, wy, c, b, y = (_c(a, dt) for a in (wx_scaled, wy_scaled, c, b, y))
        x = _c(x, dt).copy()
        ic, ih, iw = b.shape
        yout = np.empty_like(y)
        x05 = np.empty_like(y) if want_x05 else None
        P = _p64 if f64 else _p32
        fn = self.lib.tv_oracle_forward_iter_f64 if f64 else self.lib.tv_oracle_forward_iter
        fn(P(wx), P(wy), P(c), P(b), P(x), P(y), P(yout), P(x05) if want_x05 else None, ic, ih, iw, t)
        return (x, yout, x05) if want_x05 else (x, yout)

    def get_yk(self, c, b, x05_it, x05_itm1, t, f64=False):
        """The backward pass's rebuild of y_{k+1} from x05[k], x05[k-1] on one sample: c (H,W), the rest (C,H,W)."""
        dt = np.float64 if f64 else np.float32
        c, b, xa, xb = (_c(a, dt) for a in (c, b, x05_it, x05_itm1))
        ic, ih, iw = b.shape
        out = np.empty_like(b)
        P = _p64 if f64 else _p32
        fn = self.lib.tv_oracle_get_yk_f64 if f64 else self.lib.tv_oracle_get_yk
        fn(P(c), P(b), P(xa), P(xb), P(out), ic, ih, iw, t)
        return out

    def guard(self, g, run, av, f32=False):
        """Output guard on one gradient tensor.  Returns (g_new, av_new, action, stats4)."""
        g = _c(g, np.float32 if f32 else np.float64).copy().ravel()
        avv = ctypes.c_double(av)
        stats = np.zeros(4, np.float64)
        fn = self.lib.tv_oracle_guard_f32 if f32 else self.lib.tv_oracle_guard_f64
        act = fn(_p32(g) if f32 else _p64(g), g.size, int(run), ctypes.byref(avv), _p64(stats))
        return g, avv.value, act, stats

    def set_threads(self, n):
        self.lib.tv_oracle_set_threads(int(n))

    def max_threads(self):
        return self.lib.tv_oracle_max_threads()


class TGVOracle:
    """Huber-TGV FISTA inpainting layer, CPU restatement (oracle/tgv_oracle.cpp).

    Shapes: dx, dy (N,2,H,W) with channel 0 = edge weight and channel 1 = beta; c (N,1,H,W);
    b (N,C,H,W); init / output / upstream gradient (N,3*C,H,W) in variable-major order (u, v1, v2).
    """

    def __init__(self):
        L = self.lib = _load("libtgv_oracle.so")
        L.tgv_oracle_forward.argtypes = [_f32p] * 6 + [_int] * 6
        L.tgv_oracle_backward.argtypes = [_f32p] * 10 + [_int] * 6
        L.tgv_oracle_forward_f64.argtypes = [_f64p] * 6 + [_int] * 6
        L.tgv_oracle_backward_f64.argtypes = [_f64p] * 10 + [_int] * 6
        L.tgv_oracle_set_quirks.argtypes = [_int] * 7
        L.tgv_oracle_set_quirks.restype = None
        L.tgv_oracle_reset_id.argtypes = [_int]
        L.tgv_oracle_reset_id.restype = None
        L.tgv_oracle_get_state.argtypes = [_int, _f64p, _int]
        L.tgv_oracle_set_state.argtypes = [_int, _f64p]
        L.tgv_oracle_lipschitz.argtypes = [_f32p, _f32p, _int, _int, _f32p]
        L.tgv_oracle_lipschitz.restype = ctypes.c_double
        L.tgv_oracle_lipschitz_f64.argtypes = [_f64p, _f64p, _int, _int, _f64p]
        L.tgv_oracle_lipschitz_f64.restype = ctypes.c_double
        L.tgv_oracle_forward_iter.argtypes = [_f32p] * 8 + [_int] * 3 + [ctypes.c_float]
        L.tgv_oracle_forward_iter.restype = None
        L.tgv_oracle_forward_iter_f64.argtypes = [_f64p] * 8 + [_int] * 3 + [ctypes.c_double]
        L.tgv_oracle_forward_iter_f64.restype = None
        L.tgv_oracle_guard_f64.argtypes = [_f64p, ctypes.c_long, _int, _f64p, _f64p]
        L.tgv_oracle_guard_f32.argtypes = [_f32p, ctypes.c_long, _int, _f64p, _f64p]
        L.tgv_oracle_set_threads.argtypes = [_int]
        L.tgv_oracle_set_threads.restype = None
        L.tgv_oracle_jt_f64.argtypes = [_f64p] * 4 + [_int] * 4 + [_f64p] * 2
        L.tgv_oracle_jt_f64.restype = None

    def forward(self, dx, dy, c, b, init, its, pid=0, f64=False):
        dt = np.float64 if f64 else np.float32
        dx, dy, c, b, init = (_c(a, dt) for a in (dx, dy, c, b, init))
        n, ic, ih, iw = b.shape
        assert dx.shape == (n, 2, ih, iw) and dy.shape == dx.shape and init.shape == (n, 3 * ic, ih, iw)
        out = np.empty_like(init)
        P = _p64 if f64 else _p32
        fn = self.lib.tgv_oracle_forward_f64 if f64 else self.lib.tgv_oracle_forward
        rc = fn(P(dx), P(dy), P(c), P(b), P(init), P(out), n, ic, ih, iw, int(its), int(pid))
        if rc:
            raise RuntimeError("tgv_oracle_forward failed with code %d" % rc)
        return out

    def backward(self, gin, dx, dy, c, b, its, pid=0, f64=False):
        """Returns (gx, gy, gc, gb, gi); `gin` (a writable array) may be scrubbed in place."""
        dt = np.float64 if f64 else np.float32
        dx, dy, c, b = (_c(a, dt) for a in (dx, dy, c, b))
        if gin.dtype != dt or not gin.flags["C_CONTIGUOUS"]:
            gin = _c(gin, dt).copy()
        n, ic, ih, iw = b.shape
        assert gin.shape == (n, 3 * ic, ih, iw)
        gx, gy, gc = np.empty_like(dx), np.empty_like(dy), np.empty_like(c)
        gb, gi = np.empty_like(b), np.empty_like(gin)
        P = _p64 if f64 else _p32
        fn = self.lib.tgv_oracle_backward_f64 if f64 else self.lib.tgv_oracle_backward
        rc = fn(P(dx), P(dy), P(c), P(b), P(gin), P(gx), P(gy), P(gc), P(gb), P(gi), n, ic, ih, iw,
                int(its), int(pid))
        if rc:
            raise RuntimeError("tgv_oracle_backward failed with code %d" % rc)
        return gx, gy, gc, gb, gi

    def set_quirks(self, end_uses_ckpt_y=1, skip_iter0_adjoint=1, getyk_rebuild=1, scale_factors=1,
                   clamp=1, guard=1, dw_div=1):
        self.lib.tgv_oracle_set_quirks(end_uses_ckpt_y, skip_iter0_adjoint, getyk_rebuild,
                                       scale_factors, clamp, guard, dw_div)

    def reset_id(self, pid):
        self.lib.tgv_oracle_reset_id(int(pid))

    def get_state(self, pid, f64=False):
        s = np.zeros(6, np.float64)
        self.lib.tgv_oracle_get_state(int(pid), _p64(s), int(f64))
        return s

    def set_state(self, pid, state6):
        s = _c(state6, np.float64)
        self.lib.tgv_oracle_set_state(int(pid), _p64(s))

    def lipschitz(self, dx, dy, f64=False):
        """dx, dy: (2,H,W) unscaled.  Returns (L, per-pixel bound (H,W))."""
        dt = np.float64 if f64 else np.float32
        dx, dy = _c(dx, dt), _c(dy, dt)
        _, ih, iw = dx.shape
        st = np.zeros((ih, iw), dt)
        P = _p64 if f64 else _p32
        fn = self.lib.tgv_oracle_lipschitz_f64 if f64 else self.lib.tgv_oracle_lipschitz
        return fn(P(dx), P(dy), ih, iw, P(st)), st

    def forward_iter(self, dx, dy, c, b, x, y, t, want_x05=False, f64=False):
        """One iteration on one sample: dx, dy (2,H,W) unscaled, c (H,W), b (C,H,W), x / y (3,C,H,W)
        (any shape with 3*C*H*W elements).  Returns (x_new, y_new[, x05])."""
        dt = np.float64 if f64 else np.float32
        dx, dy, c, b, y = (_c(a, dt) for a in (dx, dy, c, b, y))
        x = _c(x, dt).copy()
        ic, ih, iw = b.shape
        yout = np.empty_like(y)
        x05 = np.empty_like(y) if want_x05 else None
        P = _p64 if f64 else _p32
        fn = self.lib.tgv_oracle_forward_iter_f64 if f64 else self.lib.tgv_oracle_forward_iter
        fn(P(dx), P(dy), P(c), P(b), P(x), P(y), P(yout), P(x05) if want_x05 else None, ic, ih, iw, t)
        return (x, yout, x05) if want_x05 else (x, yout)

    def jt(self, dx, dy, y, g, end_form=False, q7=False):
        """J(y)^T g of the gradient step (double precision, one channel): dx, dy (2,H,W) unscaled,
        y, g (3,H,W).  Returns (out (3,H,W), weight-gradient increments (4,H,W))."""
        dx, dy, y, g = (_c(a, np.float64) for a in (dx, dy, y, g))
        _, ih, iw = y.shape
        out = np.zeros((3, ih, iw))
        gw = np.zeros((4, ih, iw))
        self.lib.tgv_oracle_jt_f64(_p64(dx), _p64(dy), _p64(y), _p64(g), ih, iw, int(end_form), int(q7),
                                   _p64(out), _p64(gw))
        return out, gw

    def guard(self, g, run, av, f32=False):
        g = _c(g, np.float32 if f32 else np.float64).copy().ravel()
        avv = ctypes.c_double(av)
        stats = np.zeros(4, np.float64)
        fn = self.lib.tgv_oracle_guard_f32 if f32 else self.lib.tgv_oracle_guard_f64
        act = fn(_p32(g) if f32 else _p64(g), g.size, int(run), ctypes.byref(avv), _p64(stats))
        return g, avv.value, act, stats

    def set_threads(self, n):
        self.lib.tgv_oracle_set_threads(int(n))


class FlowAuxOracle:
    """Quadratic sub-pixel fit (cudaQuadFit) and histogram median (cudaMedian), CPU restatement
    (oracle/flowaux_oracle.cpp)."""

    def __init__(self):
        L = self.lib = _load("libflowaux_oracle.so")
        L.quadfit_oracle_forward.argtypes = [_f32p] * 4 + [_int] * 5
        L.quadfit_oracle_forward_f64.argtypes = [_f64p] * 4 + [_int] * 5
        L.quadfit_oracle_backward.argtypes = [_f32p] * 6 + [_int] * 5
        L.quadfit_oracle_backward_f64.argtypes = [_f64p] * 6 + [_int] * 5
        L.median_oracle_forward.argtypes = [_f32p] * 2 + [_int] * 4
        L.median_oracle_forward_f64.argtypes = [_f64p] * 2 + [_int] * 4
        L.median_oracle_backward.argtypes = [_f32p] * 3 + [_int] * 4
        L.median_oracle_backward_f64.argtypes = [_f64p] * 3 + [_int] * 4
        L.flowaux_oracle_set_threads.argtypes = [_int]
        L.flowaux_oracle_set_threads.restype = None
        L.hierarchy_oracle_upsample2x.argtypes = [_f32p] * 2 + [_int] * 3 + [ctypes.c_float]
        L.hierarchy_oracle_upsample2x_f64.argtypes = [_f64p] * 2 + [_int] * 3 + [ctypes.c_double]
        L.hierarchy_oracle_upsample2x_adjoint.argtypes = [_f32p] * 3 + [_int] * 3 + [ctypes.c_float]
        L.hierarchy_oracle_upsample2x_adjoint_f64.argtypes = [_f64p] * 3 + [_int] * 3 + [ctypes.c_double]
        L.hierarchy_oracle_edge_weights.argtypes = [_f32p] * 3 + [_int] * 3 + [ctypes.c_float]
        L.hierarchy_oracle_edge_weights_f64.argtypes = [_f64p] * 3 + [_int] * 3 + [ctypes.c_double]

    def quadfit_forward(self, feat0, feat1, flow, f64=False):
        """feat0, feat1: (N,C,H,W); flow: (N,F,H,W) with F >= 2.  Returns (N,3,H,W) = (fx, fy, score)."""
        dt = np.float64 if f64 else np.float32
        feat0, feat1, flow = (_c(a, dt) for a in (feat0, feat1, flow))
        n, c, h, w = feat0.shape
        out = np.empty((n, 3, h, w), dt)
        P = _p64 if f64 else _p32
        fn = self.lib.quadfit_oracle_forward_f64 if f64 else self.lib.quadfit_oracle_forward
        rc = fn(P(feat0), P(feat1), P(flow), P(out), n, c, h, w, flow.shape[1])
        if rc:
            raise RuntimeError("quadfit_oracle_forward failed with code %d" % rc)
        return out

    def quadfit_backward(self, gin, feat0, feat1, flow, f64=False):
        """gin: (N,3,H,W).  Returns the gradients wrt feat0 and feat1."""
        dt = np.float64 if f64 else np.float32
        gin, feat0, feat1, flow = (_c(a, dt) for a in (gin, feat0, feat1, flow))
        n, c, h, w = feat0.shape
        g0, g1 = np.empty_like(feat0), np.empty_like(feat1)
        P = _p64 if f64 else _p32
        fn = self.lib.quadfit_oracle_backward_f64 if f64 else self.lib.quadfit_oracle_backward
        rc = fn(P(feat0), P(feat1), P(flow), P(gin), P(g0), P(g1), n, c, h, w, flow.shape[1])
        if rc:
            raise RuntimeError("quadfit_oracle_backward failed with code %d" % rc)
        return g0, g1

    def median_forward(self, vol, f64=False):
        """vol: (N,H,W,D).  Returns (N,2,H,W) = (median position, mass of its bin)."""
        dt = np.float64 if f64 else np.float32
        vol = _c(vol, dt)
        n, h, w, d = vol.shape
        out = np.empty((n, 2, h, w), dt)
        P = _p64 if f64 else _p32
        fn = self.lib.median_oracle_forward_f64 if f64 else self.lib.median_oracle_forward
        rc = fn(P(vol), P(out), n, h, w, d)
        if rc:
            raise RuntimeError("median_oracle_forward failed with code %d" % rc)
        return out

    def median_backward(self, gin, vol, f64=False):
        """gin: (N,2,H,W).  Returns the gradient wrt vol."""
        dt = np.float64 if f64 else np.float32
        gin, vol = _c(gin, dt), _c(vol, dt)
        n, h, w, d = vol.shape
        g = np.empty_like(vol)
        P = _p64 if f64 else _p32
        fn = self.lib.median_oracle_backward_f64 if f64 else self.lib.median_oracle_backward
        rc = fn(P(vol), P(gin), P(g), n, h, w, d)
        if rc:
            raise RuntimeError("median_oracle_backward failed with code %d" % rc)
        return g

    def set_threads(self, n):
        self.lib.flowaux_oracle_set_threads(int(n))

    # -- glue between two levels of a hierarchy ----------------------------------------------------
    def upsample2x(self, x, scale=2.0, f64=False):
        """x: (N,C,H,W) -> scale * bilinear x2 upsampling, (N,C,2H,2W)."""
        dt = np.float64 if f64 else np.float32
        x = _c(x, dt)
        n, c, h, w = x.shape
        out = np.empty((n, c, 2 * h, 2 * w), dt)
        P = _p64 if f64 else _p32
        fn = self.lib.hierarchy_oracle_upsample2x_f64 if f64 else self.lib.hierarchy_oracle_upsample2x
        if fn(P(x), P(out), n * c, h, w, scale):
            raise RuntimeError("hierarchy_oracle_upsample2x failed")
        return out

    def upsample2x_adjoint(self, ga, gb=None, scale=2.0, f64=False):
        """ga (and gb, summed): (N,C,2H,2W) -> the adjoint of upsample2x, (N,C,H,W)."""
        dt = np.float64 if f64 else np.float32
        ga = _c(ga, dt)
        gb = None if gb is None else _c(gb, dt)
        n, c, h2, w2 = ga.shape
        out = np.empty((n, c, h2 // 2, w2 // 2), dt)
        P = _p64 if f64 else _p32
        fn = self.lib.hierarchy_oracle_upsample2x_adjoint_f64 if f64 else self.lib.hierarchy_oracle_upsample2x_adjoint
        if fn(P(ga), None if gb is None else P(gb), P(out), n * c, h2 // 2, w2 // 2, scale):
            raise RuntimeError("hierarchy_oracle_upsample2x_adjoint failed")
        return out

    def edge_weights(self, img, alpha=10.0, f64=False):
        """img: (N,1,H,W) -> (wx, wy) = exp(-alpha |forward difference|), 1 in the last column / row."""
        dt = np.float64 if f64 else np.float32
        img = _c(img, dt)
        n, c, h, w = img.shape
        wx, wy = np.empty_like(img), np.empty_like(img)
        P = _p64 if f64 else _p32
        fn = self.lib.hierarchy_oracle_edge_weights_f64 if f64 else self.lib.hierarchy_oracle_edge_weights
        if fn(P(img), P(wx), P(wy), n * c, h, w, alpha):
            raise RuntimeError("hierarchy_oracle_edge_weights failed")
        return wx, wy
