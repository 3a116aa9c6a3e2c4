"""Minus, L1Norm / L2Norm, ReduceMean and AXPBY through the C ABI against the oracle: what a loss
and a trainer step need after the dense operators.  Integer inputs make every sum exact (order
cannot matter), seeded reals must agree within the tolerance."""
import numpy as np
import pytest

from util import FP16_TOL, FP32_TOL, f, h, ints, nrm, rel_fro, rng

pytestmark = pytest.mark.gpu

PAIRS = [((4, 50, 20), (4, 50, 20)), ((4, 50, 20), (1, 20)), ((2, 14, 14, 64), (2, 1, 1, 64)), ((3, 33, 7), (3, 1, 7)),
         ((1, 6, 1), (5, 1, 9)), ((3, 4, 5, 6, 8), (1, 4, 1, 6, 1)), ((2, 3), (1, 1)), ((8, 512, 64), (1, 64)),
         ((1, 2), (1, 2))]


def _c(dtype):
    return (lambda a: h(a)) if dtype == np.float16 else (lambda a: np.asarray(a, np.float32))


@pytest.mark.parametrize("xs,ys", PAIRS)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_minus_forward_and_gradients(oracle_port, xs, ys, dtype):
    from deep8_amd import ops
    r = rng(sum(xs) + 5 * sum(ys))
    c = _c(dtype)
    x, y = c(nrm(r, xs)), c(nrm(r, ys))
    want = oracle_port.minus(f(x), f(y))
    got = ops.minus(x, y)
    assert got.dtype == dtype and np.array_equal(got, want.astype(dtype))
    hi = 3 if dtype == np.float16 else 50
    dz = ints(r, want.shape, hi)
    if dtype == np.float16 and dz.size > 4000:
        dz = dz * (r.random(dz.shape) < 0.2)
    g0 = ints(r, y.shape, hi)
    w = oracle_port.minus_grad_y(g0, dz, g0)
    assert dtype == np.float32 or np.abs(w).max() < 2048
    for use_scratch in (True, False):
        assert np.array_equal(f(ops.minus_grad_y(c(g0), c(dz), use_scratch)), w)
    dzr = c(nrm(r, want.shape))
    tol = FP16_TOL if dtype == np.float16 else FP32_TOL
    assert rel_fro(f(ops.minus_grad_y(y, dzr)), oracle_port.minus_grad_y(f(y), f(dzr), f(y))) <= tol


@pytest.mark.parametrize("shape", [(3, 17), (1, 1), (1, 100000), (4, 5, 6, 8), (7, 1), (64, 1000), (2, 56, 56, 64)])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_l1_and_l2_norm(oracle_port, shape, dtype):
    from deep8_amd import ops
    r = rng(sum(shape) + 1)
    c = _c(dtype)
    tol = FP16_TOL if dtype == np.float16 else FP32_TOL
    # integers -1..1, thinned for half so that every row sum stays an exact fp16 integer
    xi = ints(r, shape, 3) - 1
    if dtype == np.float16:
        xi = xi * (r.random(shape) < min(1.0, 1500.0 / max(1, np.prod(shape[1:]))))
    want1 = oracle_port.l1norm(xi)
    assert dtype == np.float32 or want1.max() < 2048
    for use_scratch in (True, False):
        assert np.array_equal(f(ops.l1norm(c(xi), use_scratch)), want1)
    dy = ints(r, (shape[0], 1), 4) + 1
    dx0 = ints(r, shape, 4)
    assert np.array_equal(f(ops.l1norm_grad(c(xi), c(dy), c(dx0))), oracle_port.l1norm_grad(xi, dy, dx0))
    # reals
    x = c(nrm(r, shape) / (4 if dtype == np.float16 else 1))
    for use_scratch in (True, False):
        assert rel_fro(f(ops.l1norm(x, use_scratch)), oracle_port.l1norm(f(x))) <= tol
        assert rel_fro(f(ops.l2norm(x, use_scratch)), oracle_port.l2norm(f(x))) <= tol
    y2 = oracle_port.l2norm(f(x)) + 0.5
    dyr = nrm(r, (shape[0], 1))
    assert rel_fro(f(ops.l2norm_grad(x, c(y2), c(dyr), c(dx0))), oracle_port.l2norm_grad(f(x), f(c(y2)), f(c(dyr)), dx0)) <= tol


@pytest.mark.parametrize("shape,axes", [((3, 8), ()), ((3, 8), (0,)), ((3, 8), (1,)), ((2, 4, 5, 8), (1, 3)), ((2, 4, 5, 6), (-1,)),
                                        ((2, 3, 4, 5, 6), (0, 2, 4)), ((1, 12), (0, 1)), ((16, 1), ()), ((32, 56, 56, 64), (0, 1, 2)),
                                        ((4, 4096), ())])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_reduce_mean_and_gradient(oracle_port, shape, axes, dtype):
    from deep8_amd import ops
    r = rng(sum(shape) + len(axes) + 7)
    c = _c(dtype)
    tol = FP16_TOL if dtype == np.float16 else FP32_TOL
    x = c(nrm(r, shape))
    want = oracle_port.reduce_mean(f(x), axes)
    for use_scratch in (True, False):
        got = ops.reduce_mean(x, axes, use_scratch)
        assert got.shape == want.shape and rel_fro(f(got), want) <= tol
    # a constant tensor has exactly that mean when the count is a power of two
    count = x.size // want.size
    if count & (count - 1) == 0:
        k = c(np.full(shape, 3.0))
        assert np.array_equal(f(ops.reduce_mean(k, axes)), np.full(want.shape, 3.0, np.float32))
    dm, dx0 = c(nrm(r, want.shape)), c(nrm(r, shape))
    assert rel_fro(f(ops.reduce_mean_grad(dx0, dm)), oracle_port.reduce_mean_grad(f(dx0), f(dm))) <= tol


@pytest.mark.parametrize("n", [1, 7, 4096, 100003])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_axpby(oracle_port, n, dtype):
    from deep8_amd import ops
    r = rng(n)
    c = _c(dtype)
    x, y = c(nrm(r, (1, n))), c(nrm(r, (1, n)))
    want = oracle_port.axpby(f(x), -0.01, f(y), 0.999)
    got = ops.axpby(x, -0.01, y, 0.999)
    if dtype == np.float32:
        assert rel_fro(got, want) <= 1e-7  # an fma may replace the two roundings of mul + add
    else:
        assert rel_fro(f(got), want) <= FP16_TOL


def test_loss_op_argument_errors():
    import ctypes
    from deep8_amd import capi
    lib = capi.init()
    a = capi.DeviceArray((16,), np.float32, zero=True)
    d = lambda *v: (ctypes.c_int * 5)(*v)
    assert lib.d8_minus(capi.FLOAT32, a.ptr, d(1, 1, 1, 1, 3), a.ptr, d(1, 1, 1, 1, 4), a.ptr, d(1, 1, 1, 1, 4), None) == 10001
    assert lib.d8_reduce_mean(capi.FLOAT32, a.ptr, d(1, 1, 1, 2, 4), a.ptr, d(1, 1, 1, 3, 1), None, 0, None) == 10001
    assert lib.d8_l1norm(12, a.ptr, a.ptr, 1, 4, None, 0, None) == 10002
    assert lib.d8_l2norm(capi.FLOAT32, a.ptr, a.ptr, 0, 4, None, 0, None) == 10001
    assert lib.d8_axpby(capi.FLOAT32, None, 1.0, None, 1.0, None, 0, None) == 0


@pytest.mark.parametrize("n", [1, 7, 4096, 100003])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_adam_update(oracle_port, n, dtype):
    """d8_adam_update against the oracle over three steps (the state of one step feeds the next)."""
    from deep8_amd import ops
    r = rng(n + 3)
    c = _c(dtype)
    st = [c(nrm(r, (1, n))), None, c(np.zeros((1, n))), c(np.zeros((1, n)))]
    ref = [f(st[0]), None, f(st[2]), f(st[3])]
    tol = 1e-5 if dtype == np.float32 else 4e-3
    for step in (1, 2, 3):
        g = c(nrm(r, (1, n)))
        st = list(ops.adam_update(st[0], g, st[2], st[3], 0.9, 0.999, 1e-7, 0.01, 0.001, step))
        ref = list(oracle_port.adam_update(ref[0], f(g), ref[2], ref[3], 0.9, 0.999, 1e-7, 0.01, 0.001, step))
        for k in range(4):
            assert rel_fro(f(st[k]), ref[k]) <= tol, (step, k)
        if dtype == np.float16:
            ref = [f(t) for t in st]  # follow the half-rounded state
