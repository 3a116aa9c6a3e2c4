"""A seeded sweep over shapes nobody picked by hand: d8_gemm, the MatrixMultiply operator and the two convolutions
with both gradients, fp32 and half, against the oracle on integer inputs (bit-exact).  The shapes are drawn so that
every route is hit: small-product kernel, any-shape kernel, tiled kernels with ragged tiles, split reductions,
patch-matrix operands, residue classes, and the im2col / col2im fallbacks."""
import numpy as np
import pytest

from util import f, h

pytestmark = pytest.mark.gpu


def _case(r, port, ops):
    pick = lambda *o: o[r.integers(0, len(o))]
    ints = lambda shape, hi: r.integers(0, hi, size=shape).astype(np.float32)
    kind = pick("gemm", "gemm", "conv", "deconv", "matmul")
    half = r.random() < 0.4
    hi = 3 if half else 20
    c = h if half else (lambda a: a)
    small = lambda *ts: not half or max(np.abs(t).max() for t in ts) < 2048  # half holds the results exactly
    if kind == "gemm":
        M = int(pick(1, 7, 32, 33, 64, 100, 128, 129, 200, 256, 300, 512, 700))
        N = int(pick(1, 5, 32, 64, 72, 128, 136, 256, 264, 576))
        K = int(pick(1, 8, 16, 31, 32, 64, 96, 128, 192, 256, 512, 1024, 2048))
        K = min(K, 256) if half else K
        ta, tb = pick((0, 0), (0, 1), (1, 0))
        A, B = ints((K, M) if ta else (M, K), hi), ints((N, K) if tb else (K, N), hi)
        C0, beta = ints((M, N), hi), float(pick(0, 1))
        want = [port.gemm(ta, tb, A, B, C0, beta)]
        if not small(*want):
            return None
        got = [f(ops.gemm(ta, tb, c(A), c(B), c(C0), beta)).reshape(want[0].shape)]
        return (kind, half, ta, tb, M, N, K, beta), got, want
    if kind == "matmul":
        xb, yb = pick((1, 1), (4, 1), (1, 4), (3, 3), (8, 1))
        M, K, N = int(pick(1, 16, 40, 64, 128, 130)), int(pick(8, 30, 64, 128, 256)), int(pick(1, 9, 64, 128, 200))
        K = min(K, 64) if half else K
        x, y = ints((xb, M, K), hi), ints((yb, K, N), hi)
        z = port.matmul(x, y)
        dz = ints(z.shape, hi)
        want = [z, port.matmul_grad_x(x, y, dz, x), port.matmul_grad_y(x, y, dz, y)]
        if not small(*want):
            return None
        got = [ops.matmul(c(x), c(y)), ops.matmul_grad_x(c(x), c(y), c(dz), c(x)), ops.matmul_grad_y(c(x), c(y), c(dz), c(y))]
        return (kind, half, x.shape, y.shape), [f(g).reshape(w.shape) for g, w in zip(got, want)], want
    B, IH, IW = int(pick(1, 2, 3, 5)), int(pick(5, 8, 9, 12, 16, 17)), int(pick(5, 8, 10, 12, 16))
    IC, OC = int(pick(3, 8, 16, 32, 64, 128)), int(pick(4, 8, 32, 64, 72, 128))
    FH, FW = int(pick(1, 2, 3, 4, 5)), int(pick(1, 2, 3, 4))
    sy, sx, cov = int(pick(1, 1, 2, 3)), int(pick(1, 1, 2, 3)), bool(pick(0, 1))
    hi = 2 if half else hi
    thin = (lambda t, p: t * (r.random(t.shape) < p)) if half else (lambda t, p: t)
    x, w = thin(ints((B, IH, IW, IC), hi), 0.3), thin(ints((OC, FH, FW, IC), hi), 0.3)
    if kind == "conv":
        dy, dx = int(pick(1, 1, 2)), int(pick(1, 1, 2))
        if not cov and (FH + (FH - 1) * (dy - 1) > IH or FW + (FW - 1) * (dx - 1) > IW):
            return None
        a = (cov, sy, sx, dy, dx)
        fwd, gx, gy = (port.conv2d, port.conv2d_grad_x, port.conv2d_grad_y), ops.conv2d_grad_x, ops.conv2d_grad_y
        run = ops.conv2d
    else:
        a = (cov, sy, sx)
        fwd, gx, gy = (port.deconv2d, port.deconv2d_grad_x, port.deconv2d_grad_y), ops.deconv2d_grad_x, ops.deconv2d_grad_y
        run = ops.deconv2d
    z = fwd[0](x, w, *a)
    gz = thin(ints(z.shape, hi), 0.2)
    want = [z, fwd[1](x, w, gz, *a, x), fwd[2](x, w, gz, *a, w)]
    if not small(*want):
        return None
    got = [run(c(x), c(w), *a), gx(c(x), c(w), c(gz), *a, c(x)), gy(c(x), c(w), c(gz), *a, c(w))]
    return (kind, half, x.shape, w.shape, a), [f(g) for g in got], want


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_shapes_against_the_oracle(oracle_port, seed):
    from deep8_amd import ops
    r = np.random.default_rng(seed)
    ran = 0
    for _ in range(250):
        case = _case(r, oracle_port, ops)
        if case is None:
            continue
        desc, got, want = case
        ran += 1
        for k, (g, w) in enumerate(zip(got, want)):
            assert np.array_equal(g, w), (desc, k)
    assert ran > 150


@pytest.mark.parametrize("seed", [21, 22])
def test_random_pooling_geometries_against_the_oracle(oracle_port, seed):
    """Pooling gradients over drawn geometries, overlapping windows (the gather kernel) and non-overlapping ones
    (a thread per window writes its stride cell), accumulate and overwrite forms, fp32 and half; integer inputs
    with many ties, so the first maximum must win: bit-exact."""
    from deep8_amd import ops
    r = np.random.default_rng(seed)
    pick = lambda *o: o[r.integers(0, len(o))]
    ran = 0
    for _ in range(120):
        B, IH, IW, C = int(pick(1, 2, 3)), int(pick(1, 4, 7, 8, 13, 16)), int(pick(1, 5, 8, 9, 16)), int(pick(1, 3, 4, 8, 16, 24))
        FH, FW, sy, sx, cov = int(pick(1, 2, 3)), int(pick(1, 2, 3)), int(pick(1, 2, 3, 4)), int(pick(1, 2, 3)), bool(pick(0, 1))
        if FH > IH or FW > IW:
            continue
        half = r.random() < 0.4
        c = h if half else (lambda a: np.asarray(a, np.float32))
        a = (FH, FW, cov, sy, sx)
        x = c(r.integers(-2, 3, size=(B, IH, IW, C)).astype(np.float32))
        y = oracle_port.pool2d(True, f(x), *a)
        dy = c(r.integers(0, 4, size=y.shape).astype(np.float32))
        dx0 = c(r.integers(0, 4, size=x.shape).astype(np.float32))
        nan = np.full(x.shape, np.nan, x.dtype)
        desc = (B, IH, IW, C, FH, FW, cov, sy, sx, half)
        assert np.array_equal(f(ops.maxpool2d(x, *a)), y), desc
        assert np.array_equal(f(ops.maxpool2d_grad(x, dy, *a, dx=dx0)), oracle_port.pool2d_grad(True, f(x), f(dy), *a, dx=f(dx0))), desc
        assert np.array_equal(f(ops.maxpool2d_grad(x, dy, *a, dx=nan, overwrite=True)), oracle_port.pool2d_grad(True, f(x), f(dy), *a)), desc
        if FH * FW in (1, 2, 4):  # dy / (FH * FW) is exact
            assert np.array_equal(f(ops.avgpool2d_grad(x.shape, dy, *a, dx=dx0)), oracle_port.pool2d_grad(False, f(x), f(dy), *a, dx=f(dx0))), desc
            assert np.array_equal(f(ops.avgpool2d_grad(x.shape, dy, *a, dx=nan, overwrite=True)), oracle_port.pool2d_grad(False, f(x), f(dy), *a)), desc
        ran += 1
    assert ran > 80


@pytest.mark.parametrize("seed", [31])
def test_random_double_products_against_numpy(seed):
    """fp64 d8_gemm over drawn shapes, among them small outputs with long reductions (split through the workspace)
    and outputs large enough for the 128 x 128 tiles; integer inputs: bit-exact."""
    from deep8_amd import ops
    r = np.random.default_rng(seed)
    pick = lambda *o: o[r.integers(0, len(o))]
    for _ in range(60):
        M, N = int(pick(1, 7, 33, 64, 100, 128, 257, 700, 1800)), int(pick(1, 5, 64, 72, 136, 576, 1700))
        K = int(pick(1, 15, 16, 17, 100, 1000, 4097, 30000))
        if M * N * K > 3e9:
            continue
        ta, tb = pick((0, 0), (0, 1), (1, 0))
        A = r.integers(0, 9, size=(K, M) if ta else (M, K)).astype(np.float64)
        B = r.integers(0, 9, size=(N, K) if tb else (K, N)).astype(np.float64)
        C0, beta = r.integers(0, 9, size=(M, N)).astype(np.float64), float(pick(0, 1))
        want = (A.T if ta else A) @ (B.T if tb else B) + beta * C0
        assert np.array_equal(ops.gemm(ta, tb, A, B, C0, beta), want), (ta, tb, M, N, K, beta)
