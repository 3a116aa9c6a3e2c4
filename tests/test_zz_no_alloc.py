"""d8_matmul_grad_y_static (the entry point that allocates nothing) against d8_matmul_grad_y.

Both run the same kernels over the same split of the reduction, so the results must agree bit for bit,
on integers and on reals.  Two calls in a row share the device's static array; the second is smaller,
so anything the first left there must not leak into it.
"""
import numpy as np
import pytest

from deep8_amd import capi
from deep8_amd.capi import DeviceArray, check

def _grad_y(fn_name, x, dy0, dz, with_scratch):
    lib = capi.init()
    dt = capi.dtype_id(x.dtype)
    xb, xr, xc = x.shape
    yb, yr, yc = dy0.shape
    dx_, dy_, dz_ = DeviceArray.from_numpy(x), DeviceArray.from_numpy(dy0), DeviceArray.from_numpy(dz)
    if with_scratch:
        nb = lib.d8_matmul_scratch_bytes(dt, 2, xb, xr, xc, yb, yr, yc)
        ws = DeviceArray((max(nb, 16),), np.uint8)
        check(getattr(lib, fn_name)(dt, dx_.ptr, xb, xr, xc, dy_.ptr, yb, yr, yc, dz_.ptr, ws.ptr, nb, None))
    else:
        check(getattr(lib, fn_name)(dt, dx_.ptr, xb, xr, xc, dy_.ptr, yb, yr, yc, dz_.ptr, None))
    capi.sync()
    return dy_.numpy()


def _case(rng, dtype, xb, xr, xc, yc, integers):
    if integers:
        hi = 3 if dtype == np.float16 else 8
        x = rng.integers(0, hi, (xb, xr, xc)).astype(dtype)
        dz = rng.integers(0, hi, (xb, xr, yc)).astype(dtype)
        dy0 = rng.integers(0, hi, (1, xc, yc)).astype(dtype)
    else:
        x = rng.uniform(-1, 1, (xb, xr, xc)).astype(dtype)
        dz = rng.uniform(-1, 1, (xb, xr, yc)).astype(dtype)
        dy0 = rng.uniform(-1, 1, (1, xc, yc)).astype(dtype)
    return x, dy0, dz


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("integers", [True, False])
def test_two_calls_in_a_row_match_the_scratch_taking_entry_point(dtype, integers, oracle_port):
    rng = np.random.default_rng(7)
    lib = capi.init()
    # first: 32 x [256 x 384]^T . [256 x 256], reduction over 8192 rows -> split; second: smaller, also split
    shapes = [(32, 256, 384, 256), (8, 128, 128, 192)]
    for i, (xb, xr, xc, yc) in enumerate(shapes):
        nb = lib.d8_matmul_scratch_bytes(capi.dtype_id(dtype), 2, xb, xr, xc, 1, xc, yc)
        assert 0 < nb <= capi.STATIC_SCRATCH_BYTES, (i, nb)  # the case must exercise the static array
        x, dy0, dz = _case(rng, dtype, xb, xr, xc, yc, integers)
        want = _grad_y("d8_matmul_grad_y", x, dy0, dz, True)
        got = _grad_y("d8_matmul_grad_y_static", x, dy0, dz, False)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (i, dtype)
        # and the existing entry point itself agrees with the CPU checker
        ref = oracle_port.matmul_grad_y(x.astype(np.float32), dy0.astype(np.float32), dz.astype(np.float32),
                                        dy0.astype(np.float32))
        err = np.linalg.norm(got.astype(np.float64) - ref) / max(np.linalg.norm(ref), 1e-30)
        assert err <= (1e-5 if dtype == np.float32 else 2e-3), (i, err)


@pytest.mark.gpu
def test_the_static_call_leaves_free_device_memory_unchanged():
    """allocates and frees nothing: hipMemGetInfo's free bytes are the same before and after the call, the first
    one on this device included (the look-up of the array's address allocates nothing either)"""
    import ctypes
    lib = capi.init()
    rng = np.random.default_rng(9)
    xb, xr, xc, yc = 16, 256, 256, 256
    assert lib.d8_matmul_scratch_bytes(capi.FLOAT32, 2, xb, xr, xc, 1, xc, yc) > 0
    x, dy0, dz = _case(rng, np.float32, xb, xr, xc, yc, True)
    dx_, dy_, dz_ = DeviceArray.from_numpy(x), DeviceArray.from_numpy(dy0), DeviceArray.from_numpy(dz)

    def free_bytes():
        capi.sync()
        f, t = ctypes.c_size_t(), ctypes.c_size_t()
        check(lib.d8_mem_info(ctypes.byref(f), ctypes.byref(t)))
        return f.value

    before = free_bytes()
    for _ in range(3):
        check(lib.d8_matmul_grad_y_static(capi.FLOAT32, dx_.ptr, xb, xr, xc, dy_.ptr, 1, xc, yc, dz_.ptr, None))
    assert free_bytes() == before
    want = dy0 + 3 * np.einsum("brk,brn->kn", x.astype(np.float64), dz.astype(np.float64))[None]
    assert np.array_equal(dy_.numpy().astype(np.float64), want)


@pytest.mark.gpu
def test_unsplit_shape_needs_no_scratch():
    rng = np.random.default_rng(8)
    x, dy0, dz = _case(rng, np.float32, 1, 64, 128, 256, True)
    want = _grad_y("d8_matmul_grad_y", x, dy0, dz, True)
    got = _grad_y("d8_matmul_grad_y_static", x, dy0, dz, False)
    assert np.array_equal(got, want)


def test_every_shape_the_planner_splits_fits_the_static_scratch():
    """The refusal in d8_matmul_grad_y_static is a guard: the planner never cuts a reduction into more pieces
    than two per compute unit, and 2 x 256 tiles of 128 x 128 fp32 partial sums are exactly 32 MiB."""
    lib = capi.load()  # size queries launch nothing, so this runs without a GPU too
    worst = 0
    for dt in (capi.FLOAT16, capi.FLOAT32, capi.FLOAT64):
        for xb in (1, 8, 64):
            for xr in (1, 64, 1024, 4096, 65536):
                for xc in (25, 64, 147, 512, 1024, 1500, 4096):
                    for yc in (1, 3, 64, 200, 512, 1024, 1500):
                        for yb in (1, xb):
                            worst = max(worst, lib.d8_matmul_scratch_bytes(dt, 2, xb, xr, xc, yb, xc, yc))
    assert 0 < worst <= capi.STATIC_SCRATCH_BYTES
