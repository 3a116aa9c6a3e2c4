"""MaxPooling2d / AvgPooling2d through the C ABI against the oracle: maxima and routed gradients are
selections and sums of a few elements (exact on integers, maximum exact always), means within the
tolerance."""
import numpy as np
import pytest

from util import FP16_TOL, FP32_TOL, f, h, ints, nrm, rel_fro, rng

pytestmark = pytest.mark.gpu

# B, IH, IW, C, FH, FW, covered, sy, sx
CASES = [(2, 8, 8, 3, 2, 2, False, 2, 2), (1, 9, 9, 4, 3, 3, False, 2, 2), (2, 7, 7, 2, 3, 3, True, 2, 2), (1, 6, 6, 5, 3, 3, True, 1, 1),
         (1, 10, 10, 8, 4, 4, True, 3, 3), (2, 12, 10, 16, 3, 2, False, 1, 2), (1, 5, 5, 1, 5, 5, False, 1, 1), (1, 1, 1, 4, 1, 1, False, 1, 1),
         (4, 28, 28, 64, 2, 2, False, 2, 2), (2, 15, 15, 24, 3, 3, True, 2, 2),
         # windows that do not overlap: rows and columns no window reaches, strides above the filter, padded borders
         (2, 9, 9, 8, 2, 2, False, 2, 2), (2, 11, 10, 8, 2, 2, False, 3, 3), (1, 7, 9, 4, 3, 3, True, 3, 3), (1, 9, 7, 4, 2, 2, True, 2, 2),
         (1, 10, 12, 4, 2, 3, True, 3, 4), (3, 13, 13, 3, 1, 1, False, 2, 2), (2, 8, 8, 5, 2, 2, True, 4, 4), (1, 6, 6, 16, 3, 3, False, 3, 3)]


@pytest.mark.parametrize("cfg", CASES)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_pooling_forward_and_gradients(oracle_port, cfg, dtype):
    from deep8_amd import ops
    B, IH, IW, C, FH, FW, cov, sy, sx = cfg
    a = (FH, FW, cov, sy, sx)
    r = rng(sum(int(v) for v in cfg) + 2)
    c = (lambda t: h(t)) if dtype == np.float16 else (lambda t: np.asarray(t, np.float32))
    tol = FP16_TOL if dtype == np.float16 else FP32_TOL
    x = c(nrm(r, (B, IH, IW, C)) - (0.5 if cov else 0.0))
    # maximum: a selection, exact in either precision
    assert np.array_equal(ops.maxpool2d(x, *a), oracle_port.pool2d(True, f(x), *a).astype(dtype))
    assert rel_fro(f(ops.avgpool2d(x, *a)), oracle_port.pool2d(False, f(x), *a)) <= tol
    # gradients on small integers: exact
    xi = c(ints(r, (B, IH, IW, C), 5) - 2)          # many ties: the first maximum must win
    OH, OW = oracle_port.pool2d(True, f(xi), *a).shape[1:3]
    dy, dx0 = c(ints(r, (B, OH, OW, C), 4)), c(ints(r, (B, IH, IW, C), 4))
    assert np.array_equal(f(ops.maxpool2d_grad(xi, dy, *a, dx=dx0)), oracle_port.pool2d_grad(True, f(xi), f(dy), *a, dx=f(dx0)))
    nan = np.full(xi.shape, np.nan, dtype)  # the overwrite forms never read what the destination held
    assert np.array_equal(f(ops.maxpool2d_grad(xi, dy, *a, dx=nan, overwrite=True)), oracle_port.pool2d_grad(True, f(xi), f(dy), *a))
    assert np.array_equal(f(ops.avgpool2d_grad(xi.shape, c(np.zeros((B, OH, OW, C))), *a, dx=nan, overwrite=True)), np.zeros(xi.shape, np.float32))
    dyr = c(nrm(r, (B, OH, OW, C)))
    assert rel_fro(f(ops.avgpool2d_grad(x.shape, dyr, *a, dx=nan, overwrite=True)), oracle_port.pool2d_grad(False, f(x), f(dyr), *a)) <= tol
    assert rel_fro(f(ops.maxpool2d_grad(x, dyr, *a, dx=nan, overwrite=True)), oracle_port.pool2d_grad(True, f(x), f(dyr), *a)) <= tol
    assert rel_fro(f(ops.avgpool2d_grad(x.shape, dyr, *a, dx=dx0)), oracle_port.pool2d_grad(False, f(x), f(dyr), *a, dx=f(dx0))) <= tol
    assert rel_fro(f(ops.maxpool2d_grad(x, dyr, *a)), oracle_port.pool2d_grad(True, f(x), f(dyr), *a)) <= tol


def test_pooling_after_config4_full_size(oracle_port):
    """2 x 2 / 2 pooling at benchmark configuration 4's activation size, against numpy reshapes."""
    from deep8_amd import ops
    r = rng(56)
    x = nrm(r, (32, 56, 56, 64))
    blocks = x.reshape(32, 28, 2, 28, 2, 64)
    assert np.array_equal(ops.maxpool2d(x, 2, 2, False, 2, 2), blocks.max(axis=(2, 4)))
    assert rel_fro(ops.avgpool2d(x, 2, 2, False, 2, 2), blocks.astype(np.float64).mean(axis=(2, 4))) <= FP32_TOL
    dy = nrm(r, (32, 28, 28, 64))
    g = ops.maxpool2d_grad(x, dy, 2, 2, False, 2, 2)
    assert np.array_equal(g.reshape(32, 28, 2, 28, 2, 64).sum(axis=(2, 4)), dy)          # each window passes dy to one element
    assert np.array_equal((g != 0) <= (x == np.repeat(np.repeat(blocks.max(axis=(2, 4)), 2, 1), 2, 2)), np.ones_like(x, bool))
    ga = ops.avgpool2d_grad(x.shape, dy, 2, 2, False, 2, 2)
    assert np.array_equal(ga, np.repeat(np.repeat(dy * np.float32(0.25), 2, 1), 2, 2))


def test_pooling_argument_errors():
    from deep8_amd import capi
    lib = capi.init()
    a = capi.DeviceArray((64,), np.float32, zero=True)
    assert lib.d8_maxpool2d(capi.FLOAT32, a.ptr, a.ptr, 1, 4, 4, 1, 0, 2, 0, 1, 1, None) == 10001
    assert lib.d8_avgpool2d(12, a.ptr, a.ptr, 1, 4, 4, 1, 2, 2, 0, 1, 1, None) == 10002
    assert lib.d8_maxpool2d(capi.FLOAT32, a.ptr, a.ptr, 1, 2, 2, 1, 3, 3, 0, 1, 1, None) == 10001  # filter larger than the image
