"""Add (broadcasting) and ReLu through the C ABI against the oracle: additions and selections of
single elements are exact in either precision, and the broadcast-gradient sums are exact on integer
inputs (order cannot matter) and within tolerance on seeded reals."""
import numpy as np
import pytest

from util import FP16_TOL, FP32_TOL, f, h, ints, nrm, rel_fro, rng

pytestmark = pytest.mark.gpu

# (x shape, y shape) as (batch, dims..); test/AddTest.h uses Shape(10,{500,200}) + Shape(1,{200})-like pairs
PAIRS = [
    ((4, 50, 20), (4, 50, 20)),            # same shape
    ((4, 50, 20), (1, 20)),                # bias along the last axis, shared over the batch
    ((2, 14, 14, 64), (1, 64)),            # conv output + per-channel bias (the Conv2d -> Add step)
    ((2, 14, 14, 64), (2, 1, 1, 64)),      # per-image bias: [K0][R][C] reduction
    ((3, 33, 7), (3, 1, 7)),               # odd extents: scalar paths
    ((1, 6, 1), (5, 1, 9)),                # both operands broadcast, different axes
    ((5, 8, 16), (5, 8, 1)),               # broadcast along the last axis: row sums
    ((3, 4, 5, 6, 8), (1, 4, 1, 6, 1)),    # alternating kept / summed axes: the general kernel
    ((2, 3), (1, 1)),                      # scalar y
    ((1, 1), (1, 1)),
    ((8, 512, 64), (1, 64)),               # long reduction, two-pass with scratch
]


def _ex(a, nd):
    return a.reshape((a.shape[0],) + (1,) * (nd - a.ndim) + a.shape[1:])


@pytest.mark.parametrize("xs,ys", PAIRS)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_add_forward_and_gradients(oracle_port, xs, ys, dtype):
    from deep8_amd import ops
    r = rng(sum(xs) + 3 * sum(ys))
    c = (lambda a: h(a)) if dtype == np.float16 else (lambda a: a)
    x, y = c(nrm(r, xs)), c(nrm(r, ys))
    want = oracle_port.add(f(x), f(y))
    got = ops.add(x, y)
    assert got.dtype == dtype and got.shape == want.shape
    assert np.array_equal(got, want.astype(dtype))          # one rounding of an exact fp32 sum
    # gradients: integers exact, with and without the two-pass scratch
    hi = 3 if dtype == np.float16 else 50
    dz = ints(r, want.shape, hi)
    if dtype == np.float16 and dz.size > 4000:
        dz = dz * (r.random(dz.shape) < 0.2)
    for like in (x, y):
        g0 = ints(r, like.shape, hi)
        w = oracle_port.add_grad(g0, dz, g0)
        assert dtype == np.float32 or np.abs(w).max() < 2048
        for use_scratch in (True, False):
            assert np.array_equal(f(ops.add_grad(c(g0), c(dz), use_scratch)), w), (like.shape, use_scratch)
            # the overwrite form never reads what the destination held
            nan = np.full(g0.shape, np.nan, dtype)
            assert np.array_equal(f(ops.add_grad(nan, c(dz), use_scratch, overwrite=True)), w - g0), (like.shape, use_scratch)
    # reals within tolerance
    dzr = c(nrm(r, want.shape))
    tol = FP16_TOL if dtype == np.float16 else FP32_TOL
    for like in (x, y):
        w = oracle_port.add_grad(f(like), f(dzr), f(like))
        assert rel_fro(f(ops.add_grad(like, dzr)), w) <= tol


@pytest.mark.parametrize("shape", [(3, 5, 7), (2, 14, 14, 64), (1, 1), (4, 4096)])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_relu_forward_and_gradient(oracle_port, shape, dtype):
    from deep8_amd import ops
    r = rng(sum(shape))
    c = (lambda a: h(a)) if dtype == np.float16 else (lambda a: a)
    x = c(nrm(r, shape))
    x.flat[0] = 0.0          # x == 0 passes no gradient (x > 0 is strict, deep8/src/math/ReLu.cpp:54-58)
    if x.size > 1:
        x.flat[1] = -0.0
    got = ops.relu(x)
    assert np.array_equal(got, oracle_port.relu(f(x)).astype(dtype)) and not np.signbit(got).any()
    dy, dx0 = c(nrm(r, shape)), c(nrm(r, shape))
    want = oracle_port.relu_grad(f(x), f(dy), f(dx0))
    assert np.array_equal(ops.relu_grad(x, dy, dx0), want.astype(dtype))
    nan = np.full(shape, np.nan, dtype)
    assert np.array_equal(ops.relu_grad(x, dy, nan, overwrite=True), oracle_port.relu_grad(f(x), f(dy)).astype(dtype))


def test_full_size_bias_and_relu_after_config4(oracle_port):
    """The element-wise steps at benchmark configuration 4's output size (32 x 56 x 56 x 64, fp32)."""
    from deep8_amd import ops
    r = rng(404)
    z, b = nrm(r, (32, 56, 56, 64)), nrm(r, (1, 64))
    out = ops.add(z, b)
    assert np.array_equal(out, z + b.reshape(1, 1, 1, 64))
    act = ops.relu(out)
    assert np.array_equal(act, np.maximum(out, 0))
    gz = nrm(r, z.shape)
    gpre = ops.relu_grad(out, gz)
    assert np.array_equal(gpre, np.where(out > 0, gz, 0).astype(np.float32))
    gb = ops.add_grad(np.zeros_like(b), gpre)
    want = gpre.astype(np.float64).sum(axis=(0, 1, 2)).reshape(1, 64)
    assert rel_fro(gb, want) <= FP32_TOL
    assert np.array_equal(ops.add_grad(np.zeros_like(z), gpre), gpre)


def test_elementwise_argument_errors():
    import ctypes
    from deep8_amd import capi
    lib = capi.init()
    a = capi.DeviceArray((16,), np.float32, zero=True)
    d = lambda *v: (ctypes.c_int * 5)(*v)
    rc = lib.d8_add(capi.FLOAT32, a.ptr, d(1, 1, 1, 1, 3), a.ptr, d(1, 1, 1, 1, 4), a.ptr, d(1, 1, 1, 1, 4), None)
    assert rc == 10001 and b"shape" in lib.d8_last_error()
    rc = lib.d8_add(12, a.ptr, d(1, 1, 1, 1, 4), a.ptr, d(1, 1, 1, 1, 4), a.ptr, d(1, 1, 1, 1, 4), None)
    assert rc == 10002
    rc = lib.d8_add_grad(capi.FLOAT32, a.ptr, d(1, 1, 1, 2, 4), a.ptr, d(1, 1, 1, 1, 4), None, 0, None)
    assert rc == 10001
    assert lib.d8_relu(capi.FLOAT32, None, None, 0, None) == 0
