"""ctypes binding of libdeep8_hip.so (the C ABI declared in include/deep8_hip.h).

Loading fails loudly when the library has not been built: there is no CPU fallback.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdeep8_hip.so")

FLOAT16 = 10
FLOAT32 = 11
FLOAT64 = 12
STATIC_SCRATCH_BYTES = 32 << 20  # D8_STATIC_SCRATCH_BYTES of include/deep8_hip.h

c_int, c_long, c_size_t, c_float, c_void_p = (ctypes.c_int, ctypes.c_long, ctypes.c_size_t, ctypes.c_float,
                                              ctypes.c_void_p)
_I, _L, _Z, _F, _P = c_int, c_long, c_size_t, c_float, c_void_p
_PP = ctypes.POINTER(c_void_p)

# name -> (restype, argtypes); mirrors include/deep8_hip.h declaration by declaration
_IP = ctypes.POINTER(ctypes.c_int)

SIGNATURES = {
    "d8_last_error": (ctypes.c_char_p, []),
    "d8_device_init": (_I, [_I]),
    "d8_device_count": (_I, [ctypes.POINTER(_I)]),
    "d8_device_info": (_I, [ctypes.POINTER(_I), ctypes.POINTER(_I), ctypes.POINTER(_Z), ctypes.c_char_p, _I]),
    "d8_mem_info": (_I, [ctypes.POINTER(_Z), ctypes.POINTER(_Z)]),
    "d8_malloc": (_I, [_PP, _Z]),
    "d8_free": (_I, [_P]),
    "d8_host_malloc": (_I, [_PP, _Z]),
    "d8_host_free": (_I, [_P]),
    "d8_memset": (_I, [_P, _I, _Z, _P]),
    "d8_fill": (_I, [_I, _P, _Z, _F, _P]),
    "d8_memcpy_h2d": (_I, [_P, _P, _Z]),
    "d8_memcpy_d2h": (_I, [_P, _P, _Z]),
    "d8_memcpy_d2d": (_I, [_P, _P, _Z, _P]),
    "d8_stream_create": (_I, [_PP]),
    "d8_stream_destroy": (_I, [_P]),
    "d8_stream_sync": (_I, [_P]),
    "d8_graph_begin": (_I, [_P]),
    "d8_graph_end": (_I, [_P, _PP]),
    "d8_graph_launch": (_I, [_P, _P]),
    "d8_graph_destroy": (_I, [_P]),
    "d8_event_create": (_I, [_PP]),
    "d8_event_destroy": (_I, [_P]),
    "d8_event_record": (_I, [_P, _P]),
    "d8_event_elapsed_ms": (_I, [_P, _P, ctypes.POINTER(_F)]),
    "d8_gemm_workspace_bytes": (_Z, [_I, _I, _I, _I, _I, _I, _I, _L]),
    "d8_gemm": (_I, [_I, _I, _I, _I, _I, _I, _P, _I, _L, _P, _I, _L, _F, _P, _I, _L, _I, _P, _Z, _P]),
    "d8_im2col": (_I, [_I, _P, _P] + [_I] * 14 + [_P]),
    "d8_col2im": (_I, [_I, _P, _P] + [_I] * 14 + [_P]),
    "d8_deconv_col2im": (_I, [_I, _P, _P] + [_I] * 12 + [_P]),
    "d8_deconv_im2col": (_I, [_I, _P, _P] + [_I] * 12 + [_P]),
    "d8_matmul_scratch_bytes": (_Z, [_I, _I, _I, _I, _I, _I, _I, _I]),
    "d8_matmul": (_I, [_I, _P, _I, _I, _I, _P, _I, _I, _I, _P, _P, _Z, _P]),
    "d8_matmul_grad_x": (_I, [_I, _P, _I, _I, _I, _P, _I, _I, _I, _P, _P, _Z, _P]),
    "d8_matmul_grad_y": (_I, [_I, _P, _I, _I, _I, _P, _I, _I, _I, _P, _P, _Z, _P]),
    "d8_deconv2d_scratch_bytes_ex": (_Z, [_I] * 15),
    "d8_deconv2d_ex": (_I, [_I, _P, _I, _I, _I, _I, _P, _I, _I, _I, _P] + [_I] * 6 + [_P, _Z, _P]),
    "d8_deconv2d_grad_x_ex": (_I, [_I, _P, _I, _I, _I, _I, _P, _I, _I, _I, _P] + [_I] * 7 + [_P, _Z, _P]),
    "d8_deconv2d_grad_y_ex": (_I, [_I, _P, _I, _I, _I, _I, _P, _I, _I, _I, _P] + [_I] * 7 + [_P, _Z, _P]),
    "d8_matmul_bias_relu": (_I, [_I, _P, _I, _I, _I, _P, _I, _I, _I, _P, _I, _P, _P, _Z, _P]),
    "d8_conv2d_bias_relu": (_I, [_I, _P, _I, _I, _I, _I, _P, _I, _I, _I, _P, _I, _P] + [_I] * 5 + [_P, _Z, _P]),
    "d8_bias_relu_grad_scratch_bytes": (_Z, [_I, _L, _I]),
    "d8_bias_relu_grad": (_I, [_I, _P, _P, _P, _P, _L, _I, _I, _P, _Z, _P]),
    "d8_matmul_grad_y_static": (_I, [_I, _P, _I, _I, _I, _P, _I, _I, _I, _P, _P]),
    "d8_matmul_grad_x_overwrite": (_I, [_I, _P, _I, _I, _I, _P, _I, _I, _I, _P, _P, _Z, _P]),
    "d8_matmul_grad_y_overwrite": (_I, [_I, _P, _I, _I, _I, _P, _I, _I, _I, _P, _P, _Z, _P]),
    "d8_matmul_grad_xy": (_I, [_I, _P, _P, _I, _I, _I, _P, _P, _I, _I, _I, _P, _I, _P, _Z, _P]),
    "d8_conv2d_geometry": (_I, [_I] * 9 + [ctypes.POINTER(_I)]),
    "d8_deconv2d_geometry": (_I, [_I] * 7 + [ctypes.POINTER(_I)]),
    "d8_conv2d_scratch_bytes": (_Z, [_I] * 14),
    "d8_conv2d": (_I, [_I, _P, _I, _I, _I, _I, _P, _I, _I, _I, _P, _I, _I, _I, _I, _I, _P, _Z, _P]),
    "d8_conv_grad_pair_launches": (ctypes.c_ulong, []),
    "d8_matmul_grad_pair_launches": (ctypes.c_ulong, []),
    "d8_conv2d_grad_xy": (_I, [_I, _P, _P, _I, _I, _I, _I, _P, _P, _I, _I, _I, _P] + [_I] * 6 + [_P, _Z, _P]),
    "d8_deconv2d_grad_xy": (_I, [_I, _P, _P, _I, _I, _I, _I, _P, _P, _I, _I, _I, _P] + [_I] * 4 + [_P, _Z, _P]),
    "d8_deconv2d_grad_xy_ex": (_I, [_I, _P, _P, _I, _I, _I, _I, _P, _P, _I, _I, _I, _P] + [_I] * 7 + [_P, _Z, _P]),
    "d8_conv2d_grad_x": (_I, [_I, _P, _I, _I, _I, _I, _P, _I, _I, _I, _P, _I, _I, _I, _I, _I, _P, _Z, _P]),
    "d8_conv2d_grad_y": (_I, [_I, _P, _I, _I, _I, _I, _P, _I, _I, _I, _P, _I, _I, _I, _I, _I, _P, _Z, _P]),
    "d8_conv2d_grad_x_overwrite": (_I, [_I, _P, _I, _I, _I, _I, _P, _I, _I, _I, _P, _I, _I, _I, _I, _I, _P, _Z, _P]),
    "d8_conv2d_grad_y_overwrite": (_I, [_I, _P, _I, _I, _I, _I, _P, _I, _I, _I, _P, _I, _I, _I, _I, _I, _P, _Z, _P]),
    "d8_deconv2d_scratch_bytes": (_Z, [_I] * 12),
    "d8_deconv2d": (_I, [_I, _P, _I, _I, _I, _I, _P, _I, _I, _I, _P, _I, _I, _I, _P, _Z, _P]),
    "d8_deconv2d_grad_x": (_I, [_I, _P, _I, _I, _I, _I, _P, _I, _I, _I, _P, _I, _I, _I, _P, _Z, _P]),
    "d8_deconv2d_grad_y": (_I, [_I, _P, _I, _I, _I, _I, _P, _I, _I, _I, _P, _I, _I, _I, _P, _Z, _P]),
    "d8_deconv2d_grad_x_overwrite": (_I, [_I, _P, _I, _I, _I, _I, _P, _I, _I, _I, _P, _I, _I, _I, _P, _Z, _P]),
    "d8_deconv2d_grad_y_overwrite": (_I, [_I, _P, _I, _I, _I, _I, _P, _I, _I, _I, _P, _I, _I, _I, _P, _Z, _P]),
    "d8_add": (_I, [_I, _P, _IP, _P, _IP, _P, _IP, _P]),
    "d8_add_grad_scratch_bytes": (_Z, [_I, _IP, _IP]),
    "d8_add_grad": (_I, [_I, _P, _IP, _P, _IP, _P, _Z, _P]),
    "d8_add_grad_overwrite": (_I, [_I, _P, _IP, _P, _IP, _P, _Z, _P]),
    "d8_relu": (_I, [_I, _P, _P, ctypes.c_long, _P]),
    "d8_relu_grad": (_I, [_I, _P, _P, _P, ctypes.c_long, _P]),
    "d8_relu_grad_overwrite": (_I, [_I, _P, _P, _P, ctypes.c_long, _P]),
    "d8_minus": (_I, [_I, _P, _IP, _P, _IP, _P, _IP, _P]),
    "d8_minus_grad_y": (_I, [_I, _P, _IP, _P, _IP, _P, _Z, _P]),
    "d8_l1norm": (_I, [_I, _P, _P, _I, ctypes.c_long, _P, _Z, _P]),
    "d8_l1norm_grad": (_I, [_I, _P, _P, _P, _I, ctypes.c_long, _P]),
    "d8_l2norm": (_I, [_I, _P, _P, _I, ctypes.c_long, _P, _Z, _P]),
    "d8_l2norm_grad": (_I, [_I, _P, _P, _P, _P, _I, ctypes.c_long, _P]),
    "d8_reduce_mean": (_I, [_I, _P, _IP, _P, _IP, _P, _Z, _P]),
    "d8_reduce_mean_grad": (_I, [_I, _P, _IP, _P, _IP, _P]),
    "d8_axpby": (_I, [_I, _P, _F, _P, _F, _P, ctypes.c_long, _P]),
    "d8_maxpool2d": (_I, [_I, _P, _P] + [_I] * 9 + [_P]),
    "d8_maxpool2d_grad": (_I, [_I, _P, _P, _P] + [_I] * 9 + [_P]),
    "d8_maxpool2d_grad_overwrite": (_I, [_I, _P, _P, _P] + [_I] * 9 + [_P]),
    "d8_avgpool2d": (_I, [_I, _P, _P] + [_I] * 9 + [_P]),
    "d8_avgpool2d_grad": (_I, [_I, _P, _P] + [_I] * 9 + [_P]),
    "d8_avgpool2d_grad_overwrite": (_I, [_I, _P, _P] + [_I] * 9 + [_P]),
    "d8_adam_update": (_I, [_I, _P, _P, _P, _P, _F, _F, _F, _F, _F, ctypes.c_long, ctypes.c_long, _P]),
    "d8_gemm_phase_record": (_I, [_P, _Z]),
    "d8_mfma_stream_out_bytes": (_Z, []),
    "d8_mfma_stream": (_I, [_I, _P, _Z, _P, _I, ctypes.POINTER(ctypes.c_double), _P]),
}


class Deep8HipError(RuntimeError):
    pass


_lib = None


def load():
    """Load the shared library and declare every entry point.  No GPU call is made."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise Deep8HipError(
            "%s is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(there is no CPU fallback)" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc):
    if rc != 0:
        raise Deep8HipError("deep8_hip error %d: %s" % (rc, load().d8_last_error().decode()))


_initialised = False


def init(device=0):
    global _initialised
    lib = load()
    if not _initialised:
        check(lib.d8_device_init(device))
        _initialised = True
    return lib


def dtype_id(np_dtype):
    np_dtype = np.dtype(np_dtype)
    if np_dtype == np.float32:
        return FLOAT32
    if np_dtype == np.float16:
        return FLOAT16
    if np_dtype == np.float64:  # the contraction path only; every other entry point rejects it
        return FLOAT64
    raise Deep8HipError("type %s is not support" % np_dtype)


class DeviceArray:
    """A device allocation with a numpy-like shape/dtype; frees itself."""

    def __init__(self, shape, dtype=np.float32, zero=False):
        lib = init()
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = c_void_p()
        check(lib.d8_malloc(ctypes.byref(p), max(self.nbytes, 16)))
        self.ptr = p.value
        if zero:
            self.zero_()

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        d = cls(a.shape, a.dtype)
        check(load().d8_memcpy_h2d(d.ptr, a.ctypes.data, d.nbytes))
        return d

    def numpy(self):
        out = np.empty(self.shape, self.dtype)
        check(load().d8_memcpy_d2h(out.ctypes.data, self.ptr, self.nbytes))
        return out

    def zero_(self, stream=None):
        check(load().d8_memset(self.ptr, 0, self.nbytes, stream))
        return self

    def copy_from(self, a):
        a = np.ascontiguousarray(a, dtype=self.dtype)
        assert a.nbytes == self.nbytes
        check(load().d8_memcpy_h2d(self.ptr, a.ctypes.data, self.nbytes))
        return self

    def free(self):
        if getattr(self, "ptr", None):
            load().d8_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Timer:
    """HIP-event timing on a given stream (None = default stream)."""

    def __init__(self, stream=None):
        lib = init()
        self.stream = stream
        self.a, self.b = c_void_p(), c_void_p()
        check(lib.d8_event_create(ctypes.byref(self.a)))
        check(lib.d8_event_create(ctypes.byref(self.b)))

    def start(self):
        check(load().d8_event_record(self.a, self.stream))

    def stop_ms(self):
        lib = load()
        check(lib.d8_event_record(self.b, self.stream))
        ms = c_float()
        check(lib.d8_event_elapsed_ms(self.a, self.b, ctypes.byref(ms)))
        return ms.value


def sync(stream=None):
    check(load().d8_stream_sync(stream))
