"""CPU checkers for the Deep8 dense-contraction hot path.  TEST INFRASTRUCTURE ONLY.

Only tests/, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import this
package; the product (``deep8_amd``) never does.

Two checkers with the same numpy-level interface:

* ``port``  -- ``libdeep8_oracle.so``, the plain-C restatement in ``deep8_oracle.c``.
* ``ref``   -- ``_ref/libdeep8_ref.so``, Deep8's own CPU (Eigen) sources compiled unmodified and
  wrapped by ``ref_shim.cpp``; ``None`` when it has not been built.

Tensors are numpy float32 arrays whose first axis is Deep8's ``Shape::batch`` and whose remaining
axes are ``Shape::dims`` (deep8/include/model/Shape.h:32-83): a matrix operand is ``(batch, rows)``
or ``(batch, rows, cols)``, an image ``(B, H, W, C)``, a filter ``(1, OC, FH, FW, IC)`` or
``(OC, FH, FW, IC)``.
"""
import contextlib
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
PORT_PATH = os.path.join(_HERE, "libdeep8_oracle.so")
REF_PATH = os.path.join(_HERE, "_ref", "libdeep8_ref.so")

_f32p = ctypes.POINTER(ctypes.c_float)
_i = ctypes.c_int


def build(with_ref=True):
    """Compile the checkers (the reference build only where /root/reference exists)."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "oracle"])
    if with_ref:
        subprocess.check_call(["make", "-s", "-j8", "-C", _HERE, "ref"])


def _p(a):
    return a.ctypes.data_as(_f32p)


def _c(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def _mat(a):
    """(batch, nDims, rows, cols) of a matrix operand."""
    if a.ndim == 2:
        return a.shape[0], 1, a.shape[1], 1
    if a.ndim == 3:
        return a.shape[0], 2, a.shape[1], a.shape[2]
    raise ValueError("matrix operand must be (batch, rows[, cols])")


def matmul_out_shape(x, y):
    """deep8/src/nodes/MatrixMultiply.cpp:10-28"""
    xb, _, xr, xc = _mat(x)
    yb, _, yr, yc = _mat(y)
    if not (xb == yb or xb == 1 or yb == 1) or xc != yr:
        raise ValueError("shape error")
    return (max(xb, yb), xr) if yc == 1 else (max(xb, yb), xr, yc)


def enlarged(shape):
    """(batch, d0, ..) of an array -> the 5-entry form [batch, 1.., dims] (utils/ShapeUtils.h:41-56)"""
    shape = tuple(shape)
    assert 2 <= len(shape) <= 5, "a tensor is (batch, 1..4 dims)"
    return (shape[0],) + (1,) * (5 - len(shape)) + shape[1:]


def broadcast_shape(xs, ys):
    """Deep8's broadcastShape (utils/ShapeUtils.h:19-36) on (batch, dims..) tuples"""
    nd = max(len(xs), len(ys)) - 1
    ex = (xs[0],) + (1,) * (nd - len(xs) + 1) + tuple(xs[1:])
    ey = (ys[0],) + (1,) * (nd - len(ys) + 1) + tuple(ys[1:])
    for a, b in zip(ex, ey):
        if not (a == 1 or b == 1 or a == b):
            raise ValueError("the Shape can not Broadcast")
    return tuple(max(a, b) for a, b in zip(ex, ey))


def kept_shape(shape, axes):
    """keepDims form of the output shape of a reduction of `shape` (batch first) over `axes` (empty: all)"""
    rank = len(shape)
    red = set(range(rank)) if not axes else {(a + rank) % rank for a in axes}
    return tuple(1 if i in red else shape[i] for i in range(rank))


def _i5(shape):
    return (ctypes.c_int * 5)(*enlarged(shape))


def _nd(a):
    return _i(a.shape[0]), _i(a.ndim - 1), (ctypes.c_int * 4)(*(list(a.shape[1:]) + [0] * (5 - a.ndim)))


def _filt(w):
    w = _c(w)
    if w.ndim == 5:
        assert w.shape[0] == 1
        w = w[0]
    return w


# The working precision of the MatrixMultiply / gemm / Conv2d / DeConv2d checkers: float32, or
# float64 inside ``with oracle.float64():`` (every other checker is float32 only).
_WORK = [np.float32]


def _cw(a):
    return np.ascontiguousarray(a, dtype=_WORK[0])


def _filtw(w):
    w = _cw(w)
    if w.ndim == 5:
        assert w.shape[0] == 1
        w = w[0]
    return w


@contextlib.contextmanager
def float64():
    """Inside the block, port.* and ref.* matmul / gemm / conv2d / deconv2d (and their gradients)
    take and return float64: the port's double twins (orc_*_f64) and the reference's own double
    path (deep8/src/math/MatrixMultiply.cpp:119-131 and the Float64 cases of Conv2d.cpp / DeConv2d.cpp)."""
    _WORK[0] = np.float64
    if ref is not None:
        ref.lib.ref_set_double(1)
    try:
        yield
    finally:
        _WORK[0] = np.float32
        if ref is not None:
            ref.lib.ref_set_double(0)


class _Port:
    name = "port"

    def __init__(self, path):
        self.lib = ctypes.CDLL(path)
        self.lib.orc_threads.restype = _i

    def threads(self):
        return self.lib.orc_threads()

    def _f(self, name):
        return getattr(self.lib, name + ("_f64" if _WORK[0] is np.float64 else ""))

    # -- MatrixMultiply ------------------------------------------------------------------
    def matmul(self, x, y):
        x, y = _cw(x), _cw(y)
        z = np.zeros(matmul_out_shape(x, y), _WORK[0])
        xb, _, xr, xc = _mat(x)
        yb, _, yr, yc = _mat(y)
        self._f("orc_matmul")(_p(x), _i(xb), _i(xr), _i(xc), _p(y), _i(yb), _i(yr), _i(yc), _p(z))
        return z

    def matmul_grad_x(self, x, y, dz, dx=None):
        x, y, dz = _cw(x), _cw(y), _cw(dz)
        dx = np.zeros_like(x) if dx is None else _cw(dx).copy()
        xb, _, xr, xc = _mat(x)
        yb, _, yr, yc = _mat(y)
        self._f("orc_matmul_grad_x")(_p(dx), _i(xb), _i(xr), _i(xc), _p(y), _i(yb), _i(yr), _i(yc), _p(dz))
        return dx

    def matmul_grad_y(self, x, y, dz, dy=None):
        x, y, dz = _cw(x), _cw(y), _cw(dz)
        dy = np.zeros_like(y) if dy is None else _cw(dy).copy()
        xb, _, xr, xc = _mat(x)
        yb, _, yr, yc = _mat(y)
        self._f("orc_matmul_grad_y")(_p(x), _i(xb), _i(xr), _i(xc), _p(dy), _i(yb), _i(yr), _i(yc), _p(dz))
        return dy

    def gemm(self, ta, tb, A, B, C=None, beta=0.0):
        A, B = _cw(A), _cw(B)
        M, K = (A.shape[1], A.shape[0]) if ta else A.shape
        N = B.shape[0] if tb else B.shape[1]
        C = np.zeros((M, N), _WORK[0]) if C is None else _cw(C).copy()
        self._f("orc_gemm")(_i(ta), _i(tb), _i(M), _i(N), _i(K), _p(A), _i(A.shape[1]), _p(B), _i(B.shape[1]),
                          ctypes.c_float(beta), _p(C), _i(N))
        return C

    # -- geometry --------------------------------------------------------------------------
    def conv2d_geometry(self, IH, IW, FH, FW, covered, sy, sx, dy, dx):
        out = (ctypes.c_int * 4)()
        self.lib.orc_conv2d_geometry(IH, IW, FH, FW, int(covered), sy, sx, dy, dx, out)
        return tuple(out)

    def deconv2d_geometry(self, IH, IW, FH, FW, covered, sy, sx):
        out = (ctypes.c_int * 4)()
        self.lib.orc_deconv2d_geometry(IH, IW, FH, FW, int(covered), sy, sx, out)
        return tuple(out)

    # -- Conv2d ----------------------------------------------------------------------------
    def conv2d(self, x, w, covered=True, sy=1, sx=1, dy=1, dx=1):
        x, w = _cw(x), _filtw(w)
        B, IH, IW, IC = x.shape
        OC, FH, FW, _ = w.shape
        OH, OW, _, _ = self.conv2d_geometry(IH, IW, FH, FW, covered, sy, sx, dy, dx)
        z = np.zeros((B, OH, OW, OC), _WORK[0])
        self._f("orc_conv2d")(_p(x), B, IH, IW, IC, _p(w), OC, FH, FW, _p(z), int(covered), sy, sx, dy, dx)
        return z

    def conv2d_grad_x(self, x, w, gz, covered=True, sy=1, sx=1, dy=1, dx=1, gx=None):
        x, w, gz = _cw(x), _filtw(w), _cw(gz)
        B, IH, IW, IC = x.shape
        OC, FH, FW, _ = w.shape
        gx = np.zeros_like(x) if gx is None else _cw(gx).copy()
        self._f("orc_conv2d_grad_x")(_p(gx), B, IH, IW, IC, _p(w), OC, FH, FW, _p(gz), int(covered), sy, sx, dy, dx)
        return gx

    def conv2d_grad_y(self, x, w, gz, covered=True, sy=1, sx=1, dy=1, dx=1, gw=None):
        x, w, gz = _cw(x), _filtw(w), _cw(gz)
        B, IH, IW, IC = x.shape
        OC, FH, FW, _ = w.shape
        gw = np.zeros_like(w) if gw is None else _filtw(gw).copy()
        self._f("orc_conv2d_grad_y")(_p(x), B, IH, IW, IC, _p(gw), OC, FH, FW, _p(gz), int(covered), sy, sx, dy, dx)
        return gw

    # -- DeConv2d --------------------------------------------------------------------------
    def deconv2d(self, x, w, covered=False, sy=1, sx=1):
        x, w = _cw(x), _filtw(w)
        B, IH, IW, IC = x.shape
        OC, FH, FW, _ = w.shape
        OH, OW, _, _ = self.deconv2d_geometry(IH, IW, FH, FW, covered, sy, sx)
        z = np.zeros((B, OH, OW, OC), _WORK[0])
        self._f("orc_deconv2d")(_p(x), B, IH, IW, IC, _p(w), OC, FH, FW, _p(z), int(covered), sy, sx)
        return z

    def deconv2d_grad_x(self, x, w, gz, covered=False, sy=1, sx=1, gx=None):
        x, w, gz = _cw(x), _filtw(w), _cw(gz)
        B, IH, IW, IC = x.shape
        OC, FH, FW, _ = w.shape
        gx = np.zeros_like(x) if gx is None else _cw(gx).copy()
        self._f("orc_deconv2d_grad_x")(_p(gx), B, IH, IW, IC, _p(w), OC, FH, FW, _p(gz), int(covered), sy, sx)
        return gx

    def deconv2d_grad_y(self, x, w, gz, covered=False, sy=1, sx=1, gw=None):
        x, w, gz = _cw(x), _filtw(w), _cw(gz)
        B, IH, IW, IC = x.shape
        OC, FH, FW, _ = w.shape
        gw = np.zeros_like(w) if gw is None else _filtw(gw).copy()
        self._f("orc_deconv2d_grad_y")(_p(x), B, IH, IW, IC, _p(gw), OC, FH, FW, _p(gz), int(covered), sy, sx)
        return gw

    # -- gather / scatter maps ---------------------------------------------------------------
    def im2col(self, im, OH, OW, FH, FW, sy, sx, dy, dx, padTop, padLeft):
        im = _c(im)
        B, IH, IW, C = im.shape
        col = np.empty((B * OH * OW, FH * FW * C), np.float32)
        self.lib.orc_im2col(_p(im), _p(col), B, IH, IW, C, OH, OW, FH, FW, sy, sx, dy, dx, padTop, padLeft)
        return col

    def col2im(self, col, im, OH, OW, FH, FW, sy, sx, dy, dx, padTop, padLeft):
        """returns im + col2im(col)"""
        col, im = _c(col), _c(im).copy()
        B, IH, IW, C = im.shape
        self.lib.orc_col2im(_p(col), _p(im), B, IH, IW, C, OH, OW, FH, FW, sy, sx, dy, dx, padTop, padLeft)
        return im

    def deconv_col2im(self, zmat, B, IH, IW, OH, OW, OC, FH, FW, sy, sx, padTop, padLeft):
        zmat = _c(zmat)
        z = np.empty((B, OH, OW, OC), np.float32)
        self.lib.orc_deconv_col2im(_p(zmat), _p(z), B, IH, IW, OH, OW, OC, FH, FW, sy, sx, padTop, padLeft)
        return z

    def deconv_im2col(self, dz, IH, IW, FH, FW, sy, sx, padTop, padLeft):
        dz = _c(dz)
        B, OH, OW, OC = dz.shape
        m = np.empty((B * IH * IW, OC * FH * FW), np.float32)
        self.lib.orc_deconv_im2col(_p(dz), _p(m), B, IH, IW, OH, OW, OC, FH, FW, sy, sx, padTop, padLeft)
        return m


    # -- Add / ReLu (arrays are (batch, 1..4 dims)) ---------------------------------------------
    def add(self, x, y):
        x, y = _c(x), _c(y)
        z = np.zeros(broadcast_shape(x.shape, y.shape), np.float32)
        self.lib.orc_add(_p(x), _i5(x.shape), _p(y), _i5(y.shape), _p(z), _i5(z.shape))
        return z

    def add_grad(self, like, dz, g=None):
        """g (shaped like `like`) += dz summed over the broadcast axes"""
        dz = _c(dz)
        g = np.zeros(np.shape(like), np.float32) if g is None else _c(g).copy()
        nd = dz.ndim
        gs = (g.shape[0],) + (1,) * (nd - g.ndim) + tuple(g.shape[1:])
        self.lib.orc_add_grad(_p(g), _i5(gs), _p(dz), _i5(dz.shape))
        return g

    def relu(self, x):
        x = _c(x)
        y = np.zeros_like(x)
        self.lib.orc_relu(_p(x), _p(y), ctypes.c_long(x.size))
        return y

    def relu_grad(self, x, dy, dx=None):
        x, dy = _c(x), _c(dy)
        dx = np.zeros_like(x) if dx is None else _c(dx).copy()
        self.lib.orc_relu_grad(_p(x), _p(dx), _p(dy), ctypes.c_long(x.size))
        return dx

    # -- Minus, L1Norm / L2Norm, ReduceMean, AXPBY ---------------------------------------------
    def minus(self, x, y):
        x, y = _c(x), _c(y)
        z = np.zeros(broadcast_shape(x.shape, y.shape), np.float32)
        self.lib.orc_minus(_p(x), _i5(x.shape), _p(y), _i5(y.shape), _p(z), _i5(z.shape))
        return z

    def minus_grad_y(self, like, dz, g=None):
        """g (shaped like `like`) -= dz summed over the broadcast axes"""
        dz = _c(dz)
        g = np.zeros(np.shape(like), np.float32) if g is None else _c(g).copy()
        gs = (g.shape[0],) + (1,) * (dz.ndim - g.ndim) + tuple(g.shape[1:])
        self.lib.orc_minus_grad_y(_p(g), _i5(gs), _p(dz), _i5(dz.shape))
        return g

    def l1norm(self, x):
        x = _c(x)
        y = np.zeros((x.shape[0], 1), np.float32)
        self.lib.orc_l1norm(_p(x), _p(y), _i(x.shape[0]), ctypes.c_long(x.size // x.shape[0]))
        return y

    def l1norm_grad(self, x, dy, dx=None):
        x, dy = _c(x), _c(dy)
        dx = np.zeros_like(x) if dx is None else _c(dx).copy()
        self.lib.orc_l1norm_grad(_p(x), _p(dx), _p(dy), _i(x.shape[0]), ctypes.c_long(x.size // x.shape[0]))
        return dx

    def l2norm(self, x):
        x = _c(x)
        y = np.zeros((x.shape[0], 1), np.float32)
        self.lib.orc_l2norm(_p(x), _p(y), _i(x.shape[0]), ctypes.c_long(x.size // x.shape[0]))
        return y

    def l2norm_grad(self, x, y, dy, dx=None):
        x, y, dy = _c(x), _c(y), _c(dy)
        dx = np.zeros_like(x) if dx is None else _c(dx).copy()
        self.lib.orc_l2norm_grad(_p(x), _p(dx), _p(y), _p(dy), _i(x.shape[0]), ctypes.c_long(x.size // x.shape[0]))
        return dx

    def reduce_mean(self, x, axes=()):
        """mean over `axes` (batch is axis 0; empty = all); returns the keepDims form"""
        x = _c(x)
        ys = kept_shape(x.shape, axes)
        y = np.zeros(ys, np.float32)
        self.lib.orc_reduce_mean(_p(x), _i5(x.shape), _p(y), _i5(ys))
        return y

    def reduce_mean_grad(self, dx, dy):
        dx, dy = _c(dx).copy(), _c(dy)
        self.lib.orc_reduce_mean_grad(_p(dx), _i5(dx.shape), _p(dy), _i5(dy.shape))
        return dx

    def axpby(self, x, alpha, y, beta):
        x, y = _c(x), _c(y)
        z = np.zeros_like(x)
        self.lib.orc_axpby(_p(x), ctypes.c_float(alpha), _p(y), ctypes.c_float(beta), _p(z), ctypes.c_long(x.size))
        return z

    def pool2d(self, is_max, x, FH, FW, covered=False, sy=1, sx=1):
        x = _c(x)
        B, IH, IW, C = x.shape
        OH, OW, _, _ = self.conv2d_geometry(IH, IW, FH, FW, covered, sy, sx, 1, 1)
        y = np.zeros((B, OH, OW, C), np.float32)
        self.lib.orc_pool2d(_i(int(is_max)), _p(x), _p(y), B, IH, IW, C, FH, FW, int(covered), sy, sx)
        return y

    def pool2d_grad(self, is_max, x, dy, FH, FW, covered=False, sy=1, sx=1, dx=None):
        x, dy = _c(x), _c(dy)
        dx = np.zeros_like(x) if dx is None else _c(dx).copy()
        B, IH, IW, C = x.shape
        self.lib.orc_pool2d_grad(_i(int(is_max)), _p(x), _p(dx), _p(dy), B, IH, IW, C, FH, FW, int(covered), sy, sx)
        return dx

    def adam_update(self, value, gradient, m, v, beta1, beta2, epsilon, learning_rate, weight_decay, steps):
        a = [_c(t).copy() for t in (value, gradient, m, v)]
        cf = ctypes.c_float
        self.lib.orc_adam_update(_p(a[0]), _p(a[1]), _p(a[2]), _p(a[3]), cf(beta1), cf(beta2), cf(epsilon), cf(learning_rate),
                                 cf(weight_decay), ctypes.c_long(steps), ctypes.c_long(a[0].size))
        return tuple(a)


class _Ref:
    """Deep8's own CPU path (float; double for the contraction path inside ``float64()``)."""
    name = "reference"

    def __init__(self, path):
        self.lib = ctypes.CDLL(path)
        self.lib.ref_last_error.restype = ctypes.c_char_p
        self.lib.ref_threads.restype = _i

    def threads(self):
        return self.lib.ref_threads()

    def _chk(self, rc):
        if rc == 1:
            raise ValueError(self.lib.ref_last_error().decode())
        if rc:
            raise RuntimeError(self.lib.ref_last_error().decode())

    def matmul(self, x, y, z_shape=None):
        x, y = _cw(x), _cw(y)
        z = np.zeros(matmul_out_shape(x, y) if z_shape is None else z_shape, _WORK[0])
        self._chk(self.lib.ref_matmul(_p(x), *map(_i, _mat(x)), _p(y), *map(_i, _mat(y)), _p(z), *map(_i, _mat(z))))
        return z

    def matmul_grad_x(self, x, y, dz, dx=None):
        x, y, dz = _cw(x), _cw(y), _cw(dz)
        dx = np.zeros_like(x) if dx is None else _cw(dx).copy()
        z = np.zeros_like(dz)
        self._chk(self.lib.ref_matmul_grad_x(_p(x), _p(dx), *map(_i, _mat(x)), _p(y), *map(_i, _mat(y)),
                                             _p(z), _p(dz), *map(_i, _mat(dz))))
        return dx

    def matmul_grad_y(self, x, y, dz, dy=None):
        x, y, dz = _cw(x), _cw(y), _cw(dz)
        dy = np.zeros_like(y) if dy is None else _cw(dy).copy()
        z = np.zeros_like(dz)
        self._chk(self.lib.ref_matmul_grad_y(_p(x), *map(_i, _mat(x)), _p(y), _p(dy), *map(_i, _mat(y)),
                                             _p(z), _p(dz), *map(_i, _mat(dz))))
        return dy

    def conv2d(self, x, w, covered=True, sy=1, sx=1, dy=1, dx=1, out_hw=None):
        x, w = _cw(x), _filtw(w)
        B, IH, IW, IC = x.shape
        OC, FH, FW, _ = w.shape
        OH, OW = out_hw if out_hw else port.conv2d_geometry(IH, IW, FH, FW, covered, sy, sx, dy, dx)[:2]
        z = np.zeros((B, OH, OW, OC), _WORK[0])
        self._chk(self.lib.ref_conv2d(_p(x), B, IH, IW, IC, _p(w), OC, FH, FW, _p(z), OH, OW,
                                      int(covered), sy, sx, dy, dx))
        return z

    def conv2d_grad_x(self, x, w, gz, covered=True, sy=1, sx=1, dy=1, dx=1, gx=None):
        x, w, gz = _cw(x), _filtw(w), _cw(gz)
        B, IH, IW, IC = x.shape
        OC, FH, FW, _ = w.shape
        _, OH, OW, _ = gz.shape
        gx = np.zeros_like(x) if gx is None else _cw(gx).copy()
        z = np.zeros_like(gz)
        self._chk(self.lib.ref_conv2d_grad_x(_p(x), _p(gx), B, IH, IW, IC, _p(w), OC, FH, FW, _p(z), _p(gz),
                                             OH, OW, int(covered), sy, sx, dy, dx))
        return gx

    def conv2d_grad_y(self, x, w, gz, covered=True, sy=1, sx=1, dy=1, dx=1, gw=None):
        x, w, gz = _cw(x), _filtw(w), _cw(gz)
        B, IH, IW, IC = x.shape
        OC, FH, FW, _ = w.shape
        _, OH, OW, _ = gz.shape
        gw = np.zeros_like(w) if gw is None else _filtw(gw).copy()
        z = np.zeros_like(gz)
        self._chk(self.lib.ref_conv2d_grad_y(_p(x), B, IH, IW, IC, _p(w), _p(gw), OC, FH, FW, _p(z), _p(gz),
                                             OH, OW, int(covered), sy, sx, dy, dx))
        return gw

    def deconv2d(self, x, w, covered=False, sy=1, sx=1, out_hw=None):
        x, w = _cw(x), _filtw(w)
        B, IH, IW, IC = x.shape
        OC, FH, FW, _ = w.shape
        OH, OW = out_hw if out_hw else port.deconv2d_geometry(IH, IW, FH, FW, covered, sy, sx)[:2]
        z = np.zeros((B, OH, OW, OC), _WORK[0])
        self._chk(self.lib.ref_deconv2d(_p(x), B, IH, IW, IC, _p(w), OC, FH, FW, _p(z), OH, OW,
                                        int(covered), sy, sx))
        return z

    def deconv2d_grad_x(self, x, w, gz, covered=False, sy=1, sx=1, gx=None):
        x, w, gz = _cw(x), _filtw(w), _cw(gz)
        B, IH, IW, IC = x.shape
        OC, FH, FW, _ = w.shape
        _, OH, OW, _ = gz.shape
        gx = np.zeros_like(x) if gx is None else _cw(gx).copy()
        z = np.zeros_like(gz)
        self._chk(self.lib.ref_deconv2d_grad_x(_p(x), _p(gx), B, IH, IW, IC, _p(w), OC, FH, FW, _p(z), _p(gz),
                                               OH, OW, int(covered), sy, sx))
        return gx

    def deconv2d_grad_y(self, x, w, gz, covered=False, sy=1, sx=1, gw=None):
        x, w, gz = _cw(x), _filtw(w), _cw(gz)
        B, IH, IW, IC = x.shape
        OC, FH, FW, _ = w.shape
        _, OH, OW, _ = gz.shape
        gw = np.zeros_like(w) if gw is None else _filtw(gw).copy()
        z = np.zeros_like(gz)
        self._chk(self.lib.ref_deconv2d_grad_y(_p(x), B, IH, IW, IC, _p(w), _p(gw), OC, FH, FW, _p(z), _p(gz),
                                               OH, OW, int(covered), sy, sx))
        return gw

    def image_patches(self, im, FH, FW, sy, sx, dy, dx, iy, ix, pt, pb, pl, pr, OH, OW):
        """Materialised Eigen extract_image_patches(...).reshape([B*OH*OW, FH*FW*C])."""
        im = _c(im)
        B, H, W, C = im.shape
        out = np.empty((B * OH * OW, FH * FW * C), np.float32)
        self._chk(self.lib.ref_image_patches(_p(im), B, H, W, C, FH, FW, sy, sx, dy, dx, iy, ix,
                                             pt, pb, pl, pr, OH, OW, _p(out)))
        return out

    def add(self, x, y, z_shape=None):
        x, y = _c(x), _c(y)
        z = np.zeros(broadcast_shape(x.shape, y.shape) if z_shape is None else z_shape, np.float32)
        self._chk(self.lib.ref_add(_p(x), *_nd(x), _p(y), *_nd(y), _p(z), *_nd(z)))
        return z

    def add_grad(self, which, x, y, dz, g=None):
        """which 0: AddGradX, 1: AddGradY; returns g + gradient"""
        x, y, dz = _c(x), _c(y), _c(dz)
        like = x if which == 0 else y
        g = np.zeros_like(like) if g is None else _c(g).copy()
        z = np.zeros_like(dz)
        self._chk(self.lib.ref_add_grad(_i(which), _p(x), *_nd(x), _p(y), *_nd(y), _p(g), _p(z), _p(dz), *_nd(dz)))
        return g

    def relu(self, x):
        x = _c(x)
        y = np.zeros_like(x)
        self._chk(self.lib.ref_relu(_p(x), _p(y), *_nd(x)))
        return y

    def relu_grad(self, x, dy, dx=None):
        x, dy = _c(x), _c(dy)
        dx = np.zeros_like(x) if dx is None else _c(dx).copy()
        y = np.maximum(x, 0)
        self._chk(self.lib.ref_relu_grad(_p(x), _p(dx), _p(y), _p(dy), *_nd(x)))
        return dx

    # -- Minus, L1Norm / L2Norm, ReduceMean, AXPBY through the reference's Math:: functions -------
    def minus(self, x, y):
        x, y = _c(x), _c(y)
        z = np.zeros(broadcast_shape(x.shape, y.shape), np.float32)
        self._chk(self.lib.ref_minus(_p(x), *_nd(x), _p(y), *_nd(y), _p(z), *_nd(z)))
        return z

    def minus_grad(self, which, x, y, dz, g=None):
        """which 0: MinusGradX, 1: MinusGradY; returns g + gradient"""
        x, y, dz = _c(x), _c(y), _c(dz)
        like = x if which == 0 else y
        g = np.zeros_like(like) if g is None else _c(g).copy()
        z = np.zeros_like(dz)
        self._chk(self.lib.ref_minus_grad(_i(which), _p(x), *_nd(x), _p(y), *_nd(y), _p(g), _p(z), _p(dz), *_nd(dz)))
        return g

    def norm(self, which, x):
        """which 1: L1Norm, 2: L2Norm; x (batch, dims..) -> (batch, 1)"""
        x = _c(x)
        y = np.zeros((x.shape[0], 1), np.float32)
        self._chk(self.lib.ref_norm(_i(which), _p(x), *_nd(x), _p(y)))
        return y

    def norm_grad(self, which, x, y, dy, dx=None):
        x, y, dy = _c(x), _c(y), _c(dy)
        dx = np.zeros_like(x) if dx is None else _c(dx).copy()
        self._chk(self.lib.ref_norm_grad(_i(which), _p(x), _p(dx), *_nd(x), _p(y), _p(dy)))
        return dx

    def reduce_mean(self, x, axes=(), keep=True):
        x = _c(x)
        ys = kept_shape(x.shape, axes)
        y = np.zeros(ys, np.float32)
        ax = (ctypes.c_int * max(1, len(axes)))(*axes)
        self._chk(self.lib.ref_reduce_mean(_p(x), *_nd(x), _p(y), ax, _i(len(axes)), _i(int(keep))))
        return y

    def reduce_mean_grad(self, x, y, dy, axes=(), keep=True, dx=None):
        x, y, dy = _c(x), _c(y), _c(dy)
        dx = np.zeros_like(x) if dx is None else _c(dx).copy()
        ax = (ctypes.c_int * max(1, len(axes)))(*axes)
        self._chk(self.lib.ref_reduce_mean_grad(_p(x), _p(dx), *_nd(x), _p(y), _p(dy), ax, _i(len(axes)), _i(int(keep))))
        return dx

    def axpby(self, x, alpha, y, beta):
        x, y = _c(x), _c(y)
        z = np.zeros_like(x)
        self._chk(self.lib.ref_axpby(_p(x), ctypes.c_float(alpha), _p(y), ctypes.c_float(beta), _p(z), *_nd(x)))
        return z

    def pool2d(self, is_max, x, FH, FW, covered=False, sy=1, sx=1):
        x = _c(x)
        B, IH, IW, C = x.shape
        OH, OW, _, _ = port.conv2d_geometry(IH, IW, FH, FW, covered, sy, sx, 1, 1)
        y = np.zeros((B, OH, OW, C), np.float32)
        self._chk(self.lib.ref_pool2d(_i(int(is_max)), _p(x), _p(y), B, IH, IW, C, OH, OW, FH, FW, int(covered), sy, sx))
        return y

    def pool2d_grad(self, is_max, x, dy, FH, FW, covered=False, sy=1, sx=1, dx=None):
        x, dy = _c(x), _c(dy)
        dx = np.zeros_like(x) if dx is None else _c(dx).copy()
        B, IH, IW, C = x.shape
        _, OH, OW, _ = dy.shape
        y = np.zeros_like(dy)
        self._chk(self.lib.ref_pool2d_grad(_i(int(is_max)), _p(x), _p(dx), _p(y), _p(dy), B, IH, IW, C, OH, OW, FH, FW,
                                           int(covered), sy, sx))
        return dx

    def adam_update(self, value, gradient, m, v, beta1, beta2, epsilon, learning_rate, weight_decay, steps):
        a = [_c(t).copy() for t in (value, gradient, m, v)]
        cf = ctypes.c_float
        self._chk(self.lib.ref_adam_update(_p(a[0]), _p(a[1]), _p(a[2]), _p(a[3]), cf(beta1), cf(beta2), cf(epsilon),
                                           cf(learning_rate), cf(weight_decay), ctypes.c_long(steps), *_nd(a[0])))
        return tuple(a)


port = _Port(PORT_PATH) if os.path.exists(PORT_PATH) else None
ref = _Ref(REF_PATH) if os.path.exists(REF_PATH) else None


def rel_fro(got, want):
    """||got - want||_F / ||want||_F in double."""
    g = np.asarray(got, np.float64).ravel()
    w = np.asarray(want, np.float64).ravel()
    d = np.linalg.norm(w)
    return float(np.linalg.norm(g - w) / d) if d else float(np.linalg.norm(g))
