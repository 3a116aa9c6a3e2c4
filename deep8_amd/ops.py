"""numpy-in / numpy-out drivers of the C ABI, used by the parity tests, smoke() and bench.py.

Every function copies its operands to the GPU, calls one entry point of libdeep8_hip.so and copies
the result back.  Tensors follow Deep8's layout: first axis = Shape::batch, then Shape::dims
(matrix: (batch, rows[, cols]); image: (B, H, W, C); filter: (OC, FH, FW, IC)).
float32 and float16 arrays are accepted (float64 too by gemm, the gather maps, matmul*, conv2d* and
deconv2d*); all operands of one call must share the dtype.
"""
import ctypes

import numpy as np

from . import capi
from .capi import DeviceArray, check


def _same_dtype(*arrays):
    dt = arrays[0].dtype
    for a in arrays:
        if a.dtype != dt:
            raise ValueError("the data type must be same")
    return capi.dtype_id(dt)


def _mat(a):
    if a.ndim == 2:
        return a.shape[0], a.shape[1], 1
    if a.ndim == 3:
        return a.shape
    raise ValueError("the shape is error")


def matmul_out_shape(x, y):
    xb, xr, xc = _mat(x)
    yb, yr, yc = _mat(y)
    if not (xb == yb or xb == 1 or yb == 1) or xc != yr:
        raise ValueError("the shape is error")
    return (max(xb, yb), xr) if y.ndim == 2 else (max(xb, yb), xr, yc)


def _scratch(nbytes):
    return DeviceArray((max(int(nbytes), 16),), np.uint8)


def gemm(ta, tb, A, B, C=None, beta=0.0, use_workspace=True):
    """C = op(A) op(B) + beta C for 2-D (or batched 3-D, broadcast by a leading 1) arrays."""
    lib = capi.init()
    A, B = np.ascontiguousarray(A), np.ascontiguousarray(B)
    dt = _same_dtype(A, B)
    A3 = A if A.ndim == 3 else A[None]
    B3 = B if B.ndim == 3 else B[None]
    K, M = (A3.shape[1], A3.shape[2]) if ta else (A3.shape[2], A3.shape[1])
    N = B3.shape[1] if tb else B3.shape[2]
    batch = max(A3.shape[0], B3.shape[0])
    if C is None:
        C3 = np.zeros((batch, M, N), A.dtype)
    else:
        C3 = np.ascontiguousarray(C)
        C3 = C3 if C3.ndim == 3 else C3[None]
    sA = 0 if A3.shape[0] == 1 else A3.shape[1] * A3.shape[2]
    sB = 0 if B3.shape[0] == 1 else B3.shape[1] * B3.shape[2]
    sC = 0 if C3.shape[0] == 1 else M * N
    dA, dB, dC = DeviceArray.from_numpy(A3), DeviceArray.from_numpy(B3), DeviceArray.from_numpy(C3)
    wsb = lib.d8_gemm_workspace_bytes(dt, ta, tb, M, N, K, batch, sC) if use_workspace else 0
    ws = _scratch(wsb) if wsb else None
    check(lib.d8_gemm(dt, ta, tb, M, N, K, dA.ptr, A3.shape[2], sA, dB.ptr, B3.shape[2], sB, beta,
                      dC.ptr, N, sC, batch, ws.ptr if ws else None, wsb, None))
    out = dC.numpy()
    squeeze = (np.ndim(C) == 2) if C is not None else (A.ndim == 2 and B.ndim == 2)
    return out[0] if squeeze else out


# ---- MatrixMultiply ----------------------------------------------------------------------------
def _mm(which, x, y, z, overwrite=False):
    lib = capi.init()
    dt = _same_dtype(x, y, z)
    xb, xr, xc = _mat(x)
    yb, yr, yc = _mat(y)
    dx_, dy_, dz_ = DeviceArray.from_numpy(x), DeviceArray.from_numpy(y), DeviceArray.from_numpy(z)
    nb = lib.d8_matmul_scratch_bytes(dt, which, xb, xr, xc, yb, yr, yc)
    ws = _scratch(nb) if nb else None
    fn = (lib.d8_matmul, lib.d8_matmul_grad_x_overwrite if overwrite else lib.d8_matmul_grad_x,
          lib.d8_matmul_grad_y_overwrite if overwrite else lib.d8_matmul_grad_y)[which]
    check(fn(dt, dx_.ptr, xb, xr, xc, dy_.ptr, yb, yr, yc, dz_.ptr, ws.ptr if ws else None, nb, None))
    return (dz_, dx_, dy_)[which].numpy()


def matmul(x, y):
    x, y = np.ascontiguousarray(x), np.ascontiguousarray(y)
    z = np.zeros(matmul_out_shape(x, y), x.dtype)
    return _mm(0, x, y, z)


def matmul_grad_x(x, y, dz, dx=None, overwrite=False):
    """returns dx + dz * y^T (dx defaults to zeros of x's shape; x only supplies the shape); with
    overwrite the destination's old contents are ignored: dz * y^T"""
    y, dz = np.ascontiguousarray(y), np.ascontiguousarray(dz)
    dx = np.zeros(np.shape(x), y.dtype) if dx is None else np.ascontiguousarray(dx)
    return _mm(1, dx, y, dz, overwrite)


def matmul_grad_y(x, y, dz, dy=None, overwrite=False):
    x, dz = np.ascontiguousarray(x), np.ascontiguousarray(dz)
    dy = np.zeros(np.shape(y), x.dtype) if dy is None else np.ascontiguousarray(dy)
    return _mm(2, x, dy, dz, overwrite)


def matmul_grad_xy(x, y, dz, dx=None, dy=None, overwrite_x=False, overwrite_y=False):
    """both gradients from one call (d8_matmul_grad_xy): returns (dx + dz * y^T, dy + x^T * dz)"""
    lib = capi.init()
    x, y, dz = np.ascontiguousarray(x), np.ascontiguousarray(y), np.ascontiguousarray(dz)
    dx = np.zeros(x.shape, x.dtype) if dx is None else np.ascontiguousarray(dx)
    dy = np.zeros(y.shape, y.dtype) if dy is None else np.ascontiguousarray(dy)
    dt = _same_dtype(x, y, dz, dx, dy)
    xb, xr, xc = _mat(x)
    yb, yr, yc = _mat(y)
    x_, y_, dz_ = DeviceArray.from_numpy(x), DeviceArray.from_numpy(y), DeviceArray.from_numpy(dz)
    dx_, dy_ = DeviceArray.from_numpy(dx), DeviceArray.from_numpy(dy)
    nb = lib.d8_matmul_scratch_bytes(dt, 3, xb, xr, xc, yb, yr, yc)
    ws = _scratch(nb) if nb else None
    check(lib.d8_matmul_grad_xy(dt, x_.ptr, dx_.ptr, xb, xr, xc, y_.ptr, dy_.ptr, yb, yr, yc, dz_.ptr,
                                int(overwrite_x) | int(overwrite_y) << 1, ws.ptr if ws else None, nb, None))
    return dx_.numpy(), dy_.numpy()


# ---- geometry -------------------------------------------------------------------------------------
def conv2d_geometry(IH, IW, FH, FW, covered, sy, sx, dy, dx):
    out = (ctypes.c_int * 4)()
    check(capi.load().d8_conv2d_geometry(IH, IW, FH, FW, int(covered), sy, sx, dy, dx, out))
    return tuple(out)


def deconv2d_geometry(IH, IW, FH, FW, covered, sy, sx):
    out = (ctypes.c_int * 4)()
    check(capi.load().d8_deconv2d_geometry(IH, IW, FH, FW, int(covered), sy, sx, out))
    return tuple(out)


# ---- Conv2d ------------------------------------------------------------------------------------------
def _filt(w):
    w = np.ascontiguousarray(w)
    return w[0] if w.ndim == 5 else w


def conv2d(x, w, covered=True, sy=1, sx=1, dy=1, dx=1):
    lib = capi.init()
    x, w = np.ascontiguousarray(x), _filt(w)
    dt = _same_dtype(x, w)
    B, IH, IW, IC = x.shape
    OC, FH, FW, _ = w.shape
    OH, OW, _, _ = conv2d_geometry(IH, IW, FH, FW, covered, sy, sx, dy, dx)
    dx_, dw_ = DeviceArray.from_numpy(x), DeviceArray.from_numpy(w)
    dz_ = DeviceArray((B, OH, OW, OC), x.dtype)
    nb = lib.d8_conv2d_scratch_bytes(dt, 0, B, IH, IW, IC, OC, FH, FW, int(covered), sy, sx, dy, dx)
    ws = _scratch(nb)
    check(lib.d8_conv2d(dt, dx_.ptr, B, IH, IW, IC, dw_.ptr, OC, FH, FW, dz_.ptr, int(covered), sy, sx, dy, dx,
                        ws.ptr, nb, None))
    return dz_.numpy()


def conv2d_bias_relu(x, w, bias, relu=True, covered=True, sy=1, sx=1, dy=1, dx=1):
    """relu?(conv2d(x, w) + bias) from one call (bias: OC values or None)"""
    lib = capi.init()
    x, w = np.ascontiguousarray(x), _filt(w)
    dt = _same_dtype(x, w)
    B, IH, IW, IC = x.shape
    OC, FH, FW, _ = w.shape
    OH, OW, _, _ = conv2d_geometry(IH, IW, FH, FW, covered, sy, sx, dy, dx)
    dx_, dw_ = DeviceArray.from_numpy(x), DeviceArray.from_numpy(w)
    db = DeviceArray.from_numpy(np.ascontiguousarray(bias, dtype=x.dtype).reshape(OC)) if bias is not None else None
    dz_ = DeviceArray((B, OH, OW, OC), x.dtype)
    nb = lib.d8_conv2d_scratch_bytes(dt, 0, B, IH, IW, IC, OC, FH, FW, int(covered), sy, sx, dy, dx)
    ws = _scratch(nb)
    check(lib.d8_conv2d_bias_relu(dt, dx_.ptr, B, IH, IW, IC, dw_.ptr, OC, FH, FW, db.ptr if db else None, int(relu), dz_.ptr,
                                  int(covered), sy, sx, dy, dx, ws.ptr, nb, None))
    return dz_.numpy()


def matmul_bias_relu(x, y, bias, relu=True):
    """relu?(matmul(x, y) + bias) from one call (bias: one value per column of the result, or None)"""
    lib = capi.init()
    x, y = np.ascontiguousarray(x), np.ascontiguousarray(y)
    dt = _same_dtype(x, y)
    zs = matmul_out_shape(x, y)
    xb, xr, xc = _mat(x)
    yb, yr, yc = _mat(y)
    dx_, dy_, dz_ = DeviceArray.from_numpy(x), DeviceArray.from_numpy(y), DeviceArray(zs, x.dtype)
    db = DeviceArray.from_numpy(np.ascontiguousarray(bias, dtype=x.dtype).reshape(zs[-1])) if bias is not None else None
    nb = lib.d8_matmul_scratch_bytes(dt, 0, xb, xr, xc, yb, yr, yc)
    ws = _scratch(nb) if nb else None
    check(lib.d8_matmul_bias_relu(dt, dx_.ptr, xb, xr, xc, dy_.ptr, yb, yr, yc, db.ptr if db else None, int(relu), dz_.ptr,
                                  ws.ptr if ws else None, nb, None))
    return dz_.numpy()


def bias_relu_grad(z, dz, dbias=None, use_scratch=True, in_place=False):
    """returns (dpre, dbias): dpre = dz where z > 0 else 0; dbias (+)= column sums of dpre over all leading axes"""
    lib = capi.init()
    z, dz = np.ascontiguousarray(z), np.ascontiguousarray(dz)
    dt = _same_dtype(z, dz)
    cols = z.shape[-1]
    rows = z.size // cols
    dz_, dg_ = DeviceArray.from_numpy(z), DeviceArray.from_numpy(dz)
    dp_ = dg_ if in_place else DeviceArray(z.shape, z.dtype)
    acc = dbias is not None
    db_ = DeviceArray.from_numpy(np.ascontiguousarray(dbias, dtype=z.dtype).reshape(cols)) if acc else DeviceArray.from_numpy(np.full(cols, np.nan, z.dtype))
    nb = lib.d8_bias_relu_grad_scratch_bytes(dt, rows, cols) if use_scratch else 0
    ws = _scratch(nb)
    check(lib.d8_bias_relu_grad(dt, dz_.ptr, dg_.ptr, dp_.ptr, db_.ptr, rows, cols, int(acc), ws.ptr if nb else None, nb, None))
    return dp_.numpy(), db_.numpy()


def conv2d_grad_x(x, w, gz, covered=True, sy=1, sx=1, dy=1, dx=1, gx=None, overwrite=False):
    lib = capi.init()
    w, gz = _filt(w), np.ascontiguousarray(gz)
    dt = _same_dtype(w, gz)
    B, IH, IW, IC = np.shape(x)
    OC, FH, FW, _ = w.shape
    gx = np.zeros((B, IH, IW, IC), w.dtype) if gx is None else np.ascontiguousarray(gx)
    dgx, dw_, dgz = DeviceArray.from_numpy(gx), DeviceArray.from_numpy(w), DeviceArray.from_numpy(gz)
    nb = lib.d8_conv2d_scratch_bytes(dt, 1, B, IH, IW, IC, OC, FH, FW, int(covered), sy, sx, dy, dx)
    ws = _scratch(nb)
    check((lib.d8_conv2d_grad_x_overwrite if overwrite else lib.d8_conv2d_grad_x)(dt, dgx.ptr, B, IH, IW, IC, dw_.ptr, OC, FH, FW, dgz.ptr, int(covered),
                               sy, sx, dy, dx, ws.ptr, nb, None))
    return dgx.numpy()


def conv2d_grad_y(x, w, gz, covered=True, sy=1, sx=1, dy=1, dx=1, gw=None, overwrite=False):
    lib = capi.init()
    x, gz = np.ascontiguousarray(x), np.ascontiguousarray(gz)
    dt = _same_dtype(x, gz)
    B, IH, IW, IC = x.shape
    OC, FH, FW, _ = np.shape(_filt(w)) if not isinstance(w, tuple) else w
    gw = np.zeros((OC, FH, FW, IC), x.dtype) if gw is None else _filt(gw)
    dx_, dgw, dgz = DeviceArray.from_numpy(x), DeviceArray.from_numpy(gw), DeviceArray.from_numpy(gz)
    nb = lib.d8_conv2d_scratch_bytes(dt, 2, B, IH, IW, IC, OC, FH, FW, int(covered), sy, sx, dy, dx)
    ws = _scratch(nb)
    check((lib.d8_conv2d_grad_y_overwrite if overwrite else lib.d8_conv2d_grad_y)(dt, dx_.ptr, B, IH, IW, IC, dgw.ptr, OC, FH, FW, dgz.ptr, int(covered),
                               sy, sx, dy, dx, ws.ptr, nb, None))
    return dgw.numpy()


# ---- DeConv2d -----------------------------------------------------------------------------------------
def deconv2d(x, w, covered=False, sy=1, sx=1):
    lib = capi.init()
    x, w = np.ascontiguousarray(x), _filt(w)
    dt = _same_dtype(x, w)
    B, IH, IW, IC = x.shape
    OC, FH, FW, _ = w.shape
    OH, OW, _, _ = deconv2d_geometry(IH, IW, FH, FW, covered, sy, sx)
    dx_, dw_ = DeviceArray.from_numpy(x), DeviceArray.from_numpy(w)
    dz_ = DeviceArray((B, OH, OW, OC), x.dtype)
    nb = lib.d8_deconv2d_scratch_bytes(dt, 0, B, IH, IW, IC, OC, FH, FW, int(covered), sy, sx)
    ws = _scratch(nb)
    check(lib.d8_deconv2d(dt, dx_.ptr, B, IH, IW, IC, dw_.ptr, OC, FH, FW, dz_.ptr, int(covered), sy, sx,
                          ws.ptr, nb, None))
    return dz_.numpy()


def deconv2d_grad_x(x, w, gz, covered=False, sy=1, sx=1, gx=None, overwrite=False):
    lib = capi.init()
    w, gz = _filt(w), np.ascontiguousarray(gz)
    dt = _same_dtype(w, gz)
    B, IH, IW, IC = np.shape(x)
    OC, FH, FW, _ = w.shape
    gx = np.zeros((B, IH, IW, IC), w.dtype) if gx is None else np.ascontiguousarray(gx)
    dgx, dw_, dgz = DeviceArray.from_numpy(gx), DeviceArray.from_numpy(w), DeviceArray.from_numpy(gz)
    nb = lib.d8_deconv2d_scratch_bytes(dt, 1, B, IH, IW, IC, OC, FH, FW, int(covered), sy, sx)
    ws = _scratch(nb)
    check((lib.d8_deconv2d_grad_x_overwrite if overwrite else lib.d8_deconv2d_grad_x)(dt, dgx.ptr, B, IH, IW, IC, dw_.ptr, OC, FH, FW, dgz.ptr, int(covered),
                                 sy, sx, ws.ptr, nb, None))
    return dgx.numpy()


def deconv2d_grad_y(x, w, gz, covered=False, sy=1, sx=1, gw=None, overwrite=False):
    lib = capi.init()
    x, gz = np.ascontiguousarray(x), np.ascontiguousarray(gz)
    dt = _same_dtype(x, gz)
    B, IH, IW, IC = x.shape
    OC, FH, FW, _ = np.shape(_filt(w))
    gw = np.zeros((OC, FH, FW, IC), x.dtype) if gw is None else _filt(gw)
    dx_, dgw, dgz = DeviceArray.from_numpy(x), DeviceArray.from_numpy(gw), DeviceArray.from_numpy(gz)
    nb = lib.d8_deconv2d_scratch_bytes(dt, 2, B, IH, IW, IC, OC, FH, FW, int(covered), sy, sx)
    ws = _scratch(nb)
    check((lib.d8_deconv2d_grad_y_overwrite if overwrite else lib.d8_deconv2d_grad_y)(dt, dx_.ptr, B, IH, IW, IC, dgw.ptr, OC, FH, FW, dgz.ptr, int(covered),
                                 sy, sx, ws.ptr, nb, None))
    return dgw.numpy()


def _both(overwrite_x, overwrite_w):
    return (1 if overwrite_x else 0) | (2 if overwrite_w else 0)


def conv2d_grad_xy(x, w, gz, covered=True, sy=1, sx=1, dy=1, dx=1, gx=None, gw=None, overwrite_x=False, overwrite_w=False):
    """both gradients of Conv2d from one call (d8_conv2d_grad_xy): returns (gx, gw)"""
    lib = capi.init()
    x, w, gz = np.ascontiguousarray(x), _filt(w), np.ascontiguousarray(gz)
    dt = _same_dtype(x, w, gz)
    B, IH, IW, IC = x.shape
    OC, FH, FW, _ = w.shape
    gx = np.zeros(x.shape, x.dtype) if gx is None else np.ascontiguousarray(gx)
    gw = np.zeros(w.shape, x.dtype) if gw is None else _filt(gw)
    dx_, dw_, dgz = DeviceArray.from_numpy(x), DeviceArray.from_numpy(w), DeviceArray.from_numpy(gz)
    dgx, dgw = DeviceArray.from_numpy(gx), DeviceArray.from_numpy(gw)
    nb = lib.d8_conv2d_scratch_bytes(dt, 3, B, IH, IW, IC, OC, FH, FW, int(covered), sy, sx, dy, dx)
    ws = _scratch(nb)
    check(lib.d8_conv2d_grad_xy(dt, dx_.ptr, dgx.ptr, B, IH, IW, IC, dw_.ptr, dgw.ptr, OC, FH, FW, dgz.ptr, int(covered),
                                sy, sx, dy, dx, _both(overwrite_x, overwrite_w), ws.ptr, nb, None))
    return dgx.numpy(), dgw.numpy()


def deconv2d_grad_xy(x, w, gz, covered=False, sy=1, sx=1, gx=None, gw=None, overwrite_x=False, overwrite_w=False, geometry=None):
    """both gradients of DeConv2d from one call (d8_deconv2d_grad_xy, or d8_deconv2d_grad_xy_ex with
    geometry = (OH, OW, padTop, padLeft)): returns (gx, gw)"""
    lib = capi.init()
    x, w, gz = np.ascontiguousarray(x), _filt(w), np.ascontiguousarray(gz)
    dt = _same_dtype(x, w, gz)
    B, IH, IW, IC = x.shape
    OC, FH, FW, _ = w.shape
    gx = np.zeros(x.shape, x.dtype) if gx is None else np.ascontiguousarray(gx)
    gw = np.zeros(w.shape, x.dtype) if gw is None else _filt(gw)
    dx_, dw_, dgz = DeviceArray.from_numpy(x), DeviceArray.from_numpy(w), DeviceArray.from_numpy(gz)
    dgx, dgw = DeviceArray.from_numpy(gx), DeviceArray.from_numpy(gw)
    if geometry is None:
        nb = lib.d8_deconv2d_scratch_bytes(dt, 3, B, IH, IW, IC, OC, FH, FW, int(covered), sy, sx)
        ws = _scratch(nb)
        check(lib.d8_deconv2d_grad_xy(dt, dx_.ptr, dgx.ptr, B, IH, IW, IC, dw_.ptr, dgw.ptr, OC, FH, FW, dgz.ptr, int(covered),
                                      sy, sx, _both(overwrite_x, overwrite_w), ws.ptr, nb, None))
    else:
        nb = lib.d8_deconv2d_scratch_bytes_ex(dt, 3, B, IH, IW, IC, OC, FH, FW, *geometry, sy, sx)
        ws = _scratch(nb)
        check(lib.d8_deconv2d_grad_xy_ex(dt, dx_.ptr, dgx.ptr, B, IH, IW, IC, dw_.ptr, dgw.ptr, OC, FH, FW, dgz.ptr, *geometry,
                                         sy, sx, _both(overwrite_x, overwrite_w), ws.ptr, nb, None))
    return dgx.numpy(), dgw.numpy()


# ---- the four maps ---------------------------------------------------------------------------------------
def deconv2d_ex(which, x, w, gz, OH, OW, padTop, padLeft, sy, sx, acc=None, overwrite=False):
    """DeConv2d at an explicit geometry: which 0 forward (gz unused), 1 gradient of x, 2 gradient of w; gradients are
    added to `acc` (zeros by default) unless overwrite"""
    lib = capi.init()
    x, w = np.ascontiguousarray(x), _filt(w)
    dt = _same_dtype(x, w)
    B, IH, IW, IC = x.shape
    OC, FH, FW, _ = w.shape
    nb = lib.d8_deconv2d_scratch_bytes_ex(dt, which, B, IH, IW, IC, OC, FH, FW, OH, OW, padTop, padLeft, sy, sx)
    ws = _scratch(nb)
    dx_, dw_ = DeviceArray.from_numpy(x), DeviceArray.from_numpy(w)
    if which == 0:
        dz_ = DeviceArray((B, OH, OW, OC), x.dtype)
        check(lib.d8_deconv2d_ex(dt, dx_.ptr, B, IH, IW, IC, dw_.ptr, OC, FH, FW, dz_.ptr, OH, OW, padTop, padLeft, sy, sx,
                                 ws.ptr, nb, None))
        return dz_.numpy()
    dgz = DeviceArray.from_numpy(np.ascontiguousarray(gz))
    like = x if which == 1 else w
    out = DeviceArray.from_numpy(np.zeros_like(like) if acc is None else np.ascontiguousarray(acc, dtype=like.dtype))
    if which == 1:
        check(lib.d8_deconv2d_grad_x_ex(dt, out.ptr, B, IH, IW, IC, dw_.ptr, OC, FH, FW, dgz.ptr, OH, OW, padTop, padLeft, sy, sx,
                                        int(overwrite), ws.ptr, nb, None))
    else:
        check(lib.d8_deconv2d_grad_y_ex(dt, dx_.ptr, B, IH, IW, IC, out.ptr, OC, FH, FW, dgz.ptr, OH, OW, padTop, padLeft, sy, sx,
                                        int(overwrite), ws.ptr, nb, None))
    return out.numpy()


def im2col(im, OH, OW, FH, FW, sy, sx, dy, dx, padTop, padLeft):
    lib = capi.init()
    im = np.ascontiguousarray(im)
    B, IH, IW, C = im.shape
    dim_ = DeviceArray.from_numpy(im)
    col = DeviceArray((B * OH * OW, FH * FW * C), im.dtype)
    check(lib.d8_im2col(capi.dtype_id(im.dtype), dim_.ptr, col.ptr, B, IH, IW, C, OH, OW, FH, FW,
                        sy, sx, dy, dx, padTop, padLeft, None))
    return col.numpy()


def col2im(col, im, OH, OW, FH, FW, sy, sx, dy, dx, padTop, padLeft):
    """returns im + col2im(col)"""
    lib = capi.init()
    col, im = np.ascontiguousarray(col), np.ascontiguousarray(im)
    dt = _same_dtype(col, im)
    B, IH, IW, C = im.shape
    dcol, dim_ = DeviceArray.from_numpy(col), DeviceArray.from_numpy(im)
    check(lib.d8_col2im(dt, dcol.ptr, dim_.ptr, B, IH, IW, C, OH, OW, FH, FW, sy, sx, dy, dx, padTop, padLeft, None))
    return dim_.numpy()


def deconv_col2im(zmat, B, IH, IW, OH, OW, OC, FH, FW, sy, sx, padTop, padLeft):
    lib = capi.init()
    zmat = np.ascontiguousarray(zmat)
    dzm = DeviceArray.from_numpy(zmat)
    z = DeviceArray((B, OH, OW, OC), zmat.dtype)
    check(lib.d8_deconv_col2im(capi.dtype_id(zmat.dtype), dzm.ptr, z.ptr, B, IH, IW, OH, OW, OC, FH, FW,
                               sy, sx, padTop, padLeft, None))
    return z.numpy()


def deconv_im2col(dz, IH, IW, FH, FW, sy, sx, padTop, padLeft):
    lib = capi.init()
    dz = np.ascontiguousarray(dz)
    B, OH, OW, OC = dz.shape
    ddz = DeviceArray.from_numpy(dz)
    m = DeviceArray((B * IH * IW, OC * FH * FW), dz.dtype)
    check(lib.d8_deconv_im2col(capi.dtype_id(dz.dtype), ddz.ptr, m.ptr, B, IH, IW, OH, OW, OC, FH, FW,
                               sy, sx, padTop, padLeft, None))
    return m.numpy()


# ---- Add (broadcasting) / ReLu ---------------------------------------------------------------------
def _enlarged(shape):
    """(batch, 1..4 dims) -> ctypes int[5] in Deep8's enlarged form [batch, 1.., dims]"""
    shape = tuple(shape)
    if not 2 <= len(shape) <= 5:
        raise ValueError("a tensor is (batch, 1..4 dims)")
    return (ctypes.c_int * 5)(*((shape[0],) + (1,) * (5 - len(shape)) + shape[1:]))


def _broadcast(xs, ys):
    nd = max(len(xs), len(ys)) - 1
    ex = (xs[0],) + (1,) * (nd - len(xs) + 1) + tuple(xs[1:])
    ey = (ys[0],) + (1,) * (nd - len(ys) + 1) + tuple(ys[1:])
    return tuple(max(a, b) for a, b in zip(ex, ey))


def add(x, y):
    lib = capi.init()
    x, y = np.ascontiguousarray(x), np.ascontiguousarray(y)
    dt = _same_dtype(x, y)
    zs = _broadcast(x.shape, y.shape)
    dx_, dy_, dz_ = DeviceArray.from_numpy(x), DeviceArray.from_numpy(y), DeviceArray(zs, x.dtype)
    check(lib.d8_add(dt, dx_.ptr, _enlarged(x.shape), dy_.ptr, _enlarged(y.shape), dz_.ptr, _enlarged(zs), None))
    return dz_.numpy()


def add_grad(g, dz, use_scratch=True, overwrite=False):
    """returns g + dz summed over the axes g is broadcast along (g: (batch, dims..), right-aligned to dz);
    overwrite: g's contents are ignored"""
    lib = capi.init()
    g, dz = np.ascontiguousarray(g), np.ascontiguousarray(dz)
    dt = _same_dtype(g, dz)
    gs = (g.shape[0],) + (1,) * (dz.ndim - g.ndim) + tuple(g.shape[1:])
    gd, zd = _enlarged(gs), _enlarged(dz.shape)
    dg, ddz = DeviceArray.from_numpy(g), DeviceArray.from_numpy(dz)
    nb = lib.d8_add_grad_scratch_bytes(dt, gd, zd) if use_scratch else 0
    ws = _scratch(nb)
    fn = lib.d8_add_grad_overwrite if overwrite else lib.d8_add_grad
    check(fn(dt, dg.ptr, gd, ddz.ptr, zd, ws.ptr if nb else None, nb, None))
    return dg.numpy()


def relu(x):
    lib = capi.init()
    x = np.ascontiguousarray(x)
    dx_, dy_ = DeviceArray.from_numpy(x), DeviceArray(x.shape, x.dtype)
    check(lib.d8_relu(capi.dtype_id(x.dtype), dx_.ptr, dy_.ptr, x.size, None))
    return dy_.numpy()


def relu_grad(x, dy, dx=None, overwrite=False):
    lib = capi.init()
    x, dy = np.ascontiguousarray(x), np.ascontiguousarray(dy)
    dt = _same_dtype(x, dy)
    dx = np.zeros_like(x) if dx is None else np.ascontiguousarray(dx)
    a, b, c = DeviceArray.from_numpy(x), DeviceArray.from_numpy(dx), DeviceArray.from_numpy(dy)
    check((lib.d8_relu_grad_overwrite if overwrite else lib.d8_relu_grad)(dt, a.ptr, b.ptr, c.ptr, x.size, None))
    return b.numpy()


# ---- Minus, L1Norm / L2Norm, ReduceMean, AXPBY ----------------------------------------------------
def minus(x, y):
    lib = capi.init()
    x, y = np.ascontiguousarray(x), np.ascontiguousarray(y)
    dt = _same_dtype(x, y)
    zs = _broadcast(x.shape, y.shape)
    dx_, dy_, dz_ = DeviceArray.from_numpy(x), DeviceArray.from_numpy(y), DeviceArray(zs, x.dtype)
    check(lib.d8_minus(dt, dx_.ptr, _enlarged(x.shape), dy_.ptr, _enlarged(y.shape), dz_.ptr, _enlarged(zs), None))
    return dz_.numpy()


def minus_grad_y(g, dz, use_scratch=True):
    """returns g - dz summed over the axes g is broadcast along"""
    lib = capi.init()
    g, dz = np.ascontiguousarray(g), np.ascontiguousarray(dz)
    dt = _same_dtype(g, dz)
    gs = (g.shape[0],) + (1,) * (dz.ndim - g.ndim) + tuple(g.shape[1:])
    gd, zd = _enlarged(gs), _enlarged(dz.shape)
    dg, ddz = DeviceArray.from_numpy(g), DeviceArray.from_numpy(dz)
    nb = lib.d8_add_grad_scratch_bytes(dt, gd, zd) if use_scratch else 0
    ws = _scratch(nb)
    check(lib.d8_minus_grad_y(dt, dg.ptr, gd, ddz.ptr, zd, ws.ptr if nb else None, nb, None))
    return dg.numpy()


def _norm(fn_name, x, use_scratch):
    lib = capi.init()
    x = np.ascontiguousarray(x)
    dt = capi.dtype_id(x.dtype)
    batch, size = x.shape[0], int(np.prod(x.shape[1:]))
    dx_, dy_ = DeviceArray.from_numpy(x), DeviceArray((batch, 1), x.dtype)
    nb = lib.d8_add_grad_scratch_bytes(dt, _enlarged((batch, 1)), _enlarged((batch, size))) if use_scratch else 0
    ws = _scratch(nb)
    check(getattr(lib, fn_name)(dt, dx_.ptr, dy_.ptr, batch, size, ws.ptr if nb else None, nb, None))
    return dy_.numpy()


def l1norm(x, use_scratch=True):
    """x: (batch, dims..) -> (batch, 1)"""
    return _norm("d8_l1norm", x, use_scratch)


def l2norm(x, use_scratch=True):
    return _norm("d8_l2norm", x, use_scratch)


def l1norm_grad(x, dy, dx=None):
    lib = capi.init()
    x, dy = np.ascontiguousarray(x), np.ascontiguousarray(dy)
    dt = _same_dtype(x, dy)
    dx = np.zeros_like(x) if dx is None else np.ascontiguousarray(dx)
    a, b, c = DeviceArray.from_numpy(x), DeviceArray.from_numpy(dx), DeviceArray.from_numpy(dy)
    check(lib.d8_l1norm_grad(dt, a.ptr, b.ptr, c.ptr, x.shape[0], int(np.prod(x.shape[1:])), None))
    return b.numpy()


def l2norm_grad(x, y, dy, dx=None):
    lib = capi.init()
    x, y, dy = np.ascontiguousarray(x), np.ascontiguousarray(y), np.ascontiguousarray(dy)
    dt = _same_dtype(x, dy)
    dx = np.zeros_like(x) if dx is None else np.ascontiguousarray(dx)
    a, b, c, d = DeviceArray.from_numpy(x), DeviceArray.from_numpy(dx), DeviceArray.from_numpy(y), DeviceArray.from_numpy(dy)
    check(lib.d8_l2norm_grad(dt, a.ptr, b.ptr, c.ptr, d.ptr, x.shape[0], int(np.prod(x.shape[1:])), None))
    return b.numpy()


def _kept_shape(shape, axes):
    """keepDims form of the output shape of a reduction of `shape` (batch first) over `axes` (empty: all)"""
    rank = len(shape)
    red = set(range(rank)) if not axes else {(a + rank) % rank for a in axes}
    return tuple(1 if i in red else shape[i] for i in range(rank))


def reduce_mean(x, axes=(), use_scratch=True):
    """mean over `axes` of x (batch is axis 0; empty = every axis); returns the keepDims form"""
    lib = capi.init()
    x = np.ascontiguousarray(x)
    dt = capi.dtype_id(x.dtype)
    ys = _kept_shape(x.shape, axes)
    xd, yd = _enlarged(x.shape), _enlarged(ys)
    dx_, dy_ = DeviceArray.from_numpy(x), DeviceArray(ys, x.dtype)
    nb = lib.d8_add_grad_scratch_bytes(dt, yd, xd) if use_scratch else 0
    ws = _scratch(nb)
    check(lib.d8_reduce_mean(dt, dx_.ptr, xd, dy_.ptr, yd, ws.ptr if nb else None, nb, None))
    return dy_.numpy()


def reduce_mean_grad(dx, dy):
    """returns dx + dy / count with dy (keepDims form) broadcast over the reduced axes"""
    lib = capi.init()
    dx, dy = np.ascontiguousarray(dx), np.ascontiguousarray(dy)
    dt = _same_dtype(dx, dy)
    a, b = DeviceArray.from_numpy(dx), DeviceArray.from_numpy(dy)
    check(lib.d8_reduce_mean_grad(dt, a.ptr, _enlarged(dx.shape), b.ptr, _enlarged(dy.shape), None))
    return a.numpy()


def axpby(x, alpha, y, beta):
    lib = capi.init()
    x, y = np.ascontiguousarray(x), np.ascontiguousarray(y)
    dt = _same_dtype(x, y)
    a, b, c = DeviceArray.from_numpy(x), DeviceArray.from_numpy(y), DeviceArray(x.shape, x.dtype)
    check(lib.d8_axpby(dt, a.ptr, alpha, b.ptr, beta, c.ptr, x.size, None))
    return c.numpy()


def adam_update(value, gradient, m, v, beta1, beta2, epsilon, learning_rate, weight_decay, steps):
    """one Adam step; returns the updated (value, gradient, m, v)"""
    lib = capi.init()
    arrs = [np.ascontiguousarray(a) for a in (value, gradient, m, v)]
    dt = _same_dtype(*arrs)
    dev = [DeviceArray.from_numpy(a) for a in arrs]
    check(lib.d8_adam_update(dt, dev[0].ptr, dev[1].ptr, dev[2].ptr, dev[3].ptr, beta1, beta2, epsilon, learning_rate,
                             weight_decay, steps, arrs[0].size, None))
    return tuple(d.numpy() for d in dev)


# ---- MaxPooling2d / AvgPooling2d ------------------------------------------------------------------
def _pool(kind, x, FH, FW, covered, sy, sx):
    lib = capi.init()
    x = np.ascontiguousarray(x)
    B, IH, IW, C = x.shape
    OH, OW, _, _ = conv2d_geometry(IH, IW, FH, FW, covered, sy, sx, 1, 1)
    dx_, dy_ = DeviceArray.from_numpy(x), DeviceArray((B, OH, OW, C), x.dtype)
    fn = lib.d8_maxpool2d if kind == "max" else lib.d8_avgpool2d
    check(fn(capi.dtype_id(x.dtype), dx_.ptr, dy_.ptr, B, IH, IW, C, FH, FW, int(covered), sy, sx, None))
    return dy_.numpy()


def maxpool2d(x, FH, FW, covered=False, sy=1, sx=1):
    return _pool("max", x, FH, FW, covered, sy, sx)


def avgpool2d(x, FH, FW, covered=False, sy=1, sx=1):
    return _pool("avg", x, FH, FW, covered, sy, sx)


def maxpool2d_grad(x, dy, FH, FW, covered=False, sy=1, sx=1, dx=None, overwrite=False):
    """returns dx + the gradient of maxpool2d at x"""
    lib = capi.init()
    x, dy = np.ascontiguousarray(x), np.ascontiguousarray(dy)
    dt = _same_dtype(x, dy)
    dx = np.zeros_like(x) if dx is None else np.ascontiguousarray(dx)
    B, IH, IW, C = x.shape
    a, b, c = DeviceArray.from_numpy(x), DeviceArray.from_numpy(dx), DeviceArray.from_numpy(dy)
    fn = lib.d8_maxpool2d_grad_overwrite if overwrite else lib.d8_maxpool2d_grad
    check(fn(dt, a.ptr, b.ptr, c.ptr, B, IH, IW, C, FH, FW, int(covered), sy, sx, None))
    return b.numpy()


def avgpool2d_grad(xshape, dy, FH, FW, covered=False, sy=1, sx=1, dx=None, overwrite=False):
    lib = capi.init()
    dy = np.ascontiguousarray(dy)
    dx = np.zeros(xshape, dy.dtype) if dx is None else np.ascontiguousarray(dx)
    dt = _same_dtype(dx, dy)
    B, IH, IW, C = dx.shape
    b, c = DeviceArray.from_numpy(dx), DeviceArray.from_numpy(dy)
    fn = lib.d8_avgpool2d_grad_overwrite if overwrite else lib.d8_avgpool2d_grad
    check(fn(dt, b.ptr, c.ptr, B, IH, IW, C, FH, FW, int(covered), sy, sx, None))
    return b.numpy()
