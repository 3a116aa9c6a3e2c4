"""Pins of the CPU oracle (oracle/deep8_oracle.c).  No GPU.

Every oracle function is fixed by something that is not a retyping of its own formula:
  * golden vectors written by Deep8's own CPU (Eigen) build (tests/golden/deep8_cpu_reference.npz),
  * the same library live, on integer inputs, when oracle/_ref is present,
  * numpy / torch CPU routines (matmul, conv2d + autograd, conv_transpose2d),
  * identities: adjointness of the gather maps, 1x1 conv == GEMM, outer product, accumulate twice.
"""
import os

import numpy as np
import pytest

from util import ints, nrm, rel_fro, rng, uni

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "deep8_cpu_reference.npz"))
TOL = 2e-6  # oracle (double accumulation) vs Eigen (float accumulation) on O(10..100)-term sums


def _n(prefix):
    return sorted({int(k[len(prefix):].split("_")[0]) for k in GOLD.files if k.startswith(prefix) and k[len(prefix)].isdigit()})


# ---- golden vectors -----------------------------------------------------------------------------------
@pytest.mark.parametrize("i", _n("mm"))
def test_matmul_against_golden(oracle_port, i):
    g = lambda k: GOLD["mm%d_%s" % (i, k)]
    z = oracle_port.matmul(g("x"), g("y"))
    assert z.shape == g("z").shape and rel_fro(z, g("z")) <= TOL
    assert rel_fro(oracle_port.matmul_grad_x(g("x"), g("y"), g("dz"), g("dx0")), g("dx")) <= TOL
    assert rel_fro(oracle_port.matmul_grad_y(g("x"), g("y"), g("dz"), g("dy0")), g("dy")) <= TOL


@pytest.mark.parametrize("i", _n("conv"))
def test_conv2d_against_golden(oracle_port, i):
    g = lambda k: GOLD["conv%d_%s" % (i, k)]
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx, dy, dx = (int(v) for v in g("cfg"))
    a = (bool(cov), sy, sx, dy, dx)
    z = oracle_port.conv2d(g("x"), g("w"), *a)
    assert z.shape == g("z").shape and rel_fro(z, g("z")) <= TOL
    assert rel_fro(oracle_port.conv2d_grad_x(g("x"), g("w"), g("gz"), *a, gx=g("gx0")), g("gx")) <= TOL
    assert rel_fro(oracle_port.conv2d_grad_y(g("x"), g("w"), g("gz"), *a, gw=g("gw0")), g("gw")) <= TOL
    # im2col == the patch matrix Eigen builds, bit for bit
    OH, OW, pt, pl = oracle_port.conv2d_geometry(IH, IW, FH, FW, cov, sy, sx, dy, dx)
    col = oracle_port.im2col(g("x"), OH, OW, FH, FW, sy, sx, dy, dx, pt, pl)
    assert np.array_equal(col.view(np.uint32), g("patches").view(np.uint32))


@pytest.mark.parametrize("i", _n("deconv"))
def test_deconv2d_against_golden(oracle_port, i):
    g = lambda k: GOLD["deconv%d_%s" % (i, k)]
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx = (int(v) for v in g("cfg"))
    a = (bool(cov), sy, sx)
    z = oracle_port.deconv2d(g("x"), g("w"), *a)
    assert z.shape == g("z").shape and rel_fro(z, g("z")) <= TOL
    assert rel_fro(oracle_port.deconv2d_grad_x(g("x"), g("w"), g("gz"), *a, gx=g("gx0")), g("gx")) <= TOL
    assert rel_fro(oracle_port.deconv2d_grad_y(g("x"), g("w"), g("gz"), *a, gw=g("gw0")), g("gw")) <= TOL
    # deconv im2col is a pure permutation of the patches Eigen extracts from dz with the flipped filter:
    # dzmat[r, oc*FH*FW + fy*FW + fx] == patches[r, ((FH-1-fy)*FW + (FW-1-fx))*OC + oc]
    OH, OW, pt, pl = oracle_port.deconv2d_geometry(IH, IW, FH, FW, cov, sy, sx)
    m = oracle_port.deconv_im2col(g("gz"), IH, IW, FH, FW, sy, sx, pt, pl).reshape(-1, OC, FH, FW)
    p = g("gpatches").reshape(-1, FH, FW, OC)[:, ::-1, ::-1, :].transpose(0, 3, 1, 2)
    assert np.array_equal(m.view(np.uint32), np.ascontiguousarray(p).view(np.uint32))


# ---- the reference library, live -------------------------------------------------------------------------
MM_SHAPES = [((10, 40, 20), (1, 20, 30)), ((1, 30, 10), (10, 10)), ((4, 8, 6), (4, 6, 5)), ((1, 8, 6), (4, 6, 5)),
             ((4, 8, 6), (4, 6)), ((3, 17), (1, 1, 9))]


@pytest.mark.parametrize("xs,ys", MM_SHAPES)
def test_matmul_against_reference_live(oracle_port, oracle_ref, xs, ys):
    r = rng(1)
    x, y = ints(r, xs), ints(r, ys)
    z = oracle_ref.matmul(x, y)
    assert np.array_equal(oracle_port.matmul(x, y), z)
    dz = ints(r, z.shape)
    assert np.array_equal(oracle_port.matmul_grad_x(x, y, dz), oracle_ref.matmul_grad_x(x, y, dz))
    assert np.array_equal(oracle_port.matmul_grad_y(x, y, dz), oracle_ref.matmul_grad_y(x, y, dz))


@pytest.mark.parametrize("cov", [True, False])
@pytest.mark.parametrize("s,d,F", [(1, 1, 3), (2, 2, 4), (2, 1, 3), (1, 2, 3), (3, 1, 5)])
def test_conv2d_against_reference_live(oracle_port, oracle_ref, cov, s, d, F):
    r = rng(2)
    x, w = ints(r, (2, 17, 17, 5)), ints(r, (6, F, F, 5))
    a = (cov, s, s, d, d)
    z = oracle_ref.conv2d(x, w, *a)
    assert np.array_equal(oracle_port.conv2d(x, w, *a), z)
    gz = ints(r, z.shape)
    assert np.array_equal(oracle_port.conv2d_grad_x(x, w, gz, *a), oracle_ref.conv2d_grad_x(x, w, gz, *a))
    assert np.array_equal(oracle_port.conv2d_grad_y(x, w, gz, *a), oracle_ref.conv2d_grad_y(x, w, gz, *a))


@pytest.mark.parametrize("cov", [True, False])
@pytest.mark.parametrize("s,F", [(1, 3), (2, 4), (3, 4), (2, 3), (3, 2)])
def test_deconv2d_against_reference_live(oracle_port, oracle_ref, cov, s, F):
    r = rng(3)
    x, w = ints(r, (2, 9, 9, 5)), ints(r, (6, F, F, 5))
    a = (cov, s, s)
    z = oracle_ref.deconv2d(x, w, *a)
    assert np.array_equal(oracle_port.deconv2d(x, w, *a), z)
    gz = ints(r, z.shape)
    assert np.array_equal(oracle_port.deconv2d_grad_x(x, w, gz, *a), oracle_ref.deconv2d_grad_x(x, w, gz, *a))
    assert np.array_equal(oracle_port.deconv2d_grad_y(x, w, gz, *a), oracle_ref.deconv2d_grad_y(x, w, gz, *a))


def test_reference_rejects_bad_shapes(oracle_ref):
    with pytest.raises(ValueError):
        oracle_ref.matmul(np.zeros((1, 3, 4), np.float32), np.zeros((1, 4, 5), np.float32), z_shape=(1, 3, 6))


# ---- numpy / torch -------------------------------------------------------------------------------------------
@pytest.mark.parametrize("xs,ys", MM_SHAPES)
def test_matmul_against_numpy(oracle_port, xs, ys):
    r = rng(4)
    x, y = uni(r, xs), uni(r, ys)
    x3 = x.astype(np.float64).reshape(xs[0], xs[1], xs[2] if len(xs) == 3 else 1)
    y3 = y.astype(np.float64).reshape(ys[0], ys[1], ys[2] if len(ys) == 3 else 1)
    zb = max(xs[0], ys[0])
    X, Y = np.broadcast_to(x3, (zb,) + x3.shape[1:]), np.broadcast_to(y3, (zb,) + y3.shape[1:])
    z = oracle_port.matmul(x, y)
    want = np.matmul(X, Y)
    assert rel_fro(z.reshape(want.shape), want) <= 1e-6
    dz = uni(r, z.shape)
    DZ = dz.astype(np.float64).reshape(want.shape)
    dX = np.matmul(DZ, Y.transpose(0, 2, 1))
    dY = np.matmul(X.transpose(0, 2, 1), DZ)
    if xs[0] == 1:
        dX = dX.sum(0, keepdims=True)
    if ys[0] == 1:
        dY = dY.sum(0, keepdims=True)
    assert rel_fro(oracle_port.matmul_grad_x(x, y, dz).reshape(dX.shape), dX) <= 1e-6
    assert rel_fro(oracle_port.matmul_grad_y(x, y, dz).reshape(dY.shape), dY) <= 1e-6


CONV = [(2, 12, 12, 4, 5, 3, 3, True, 1, 1, 1, 1), (2, 13, 12, 3, 4, 4, 4, True, 2, 2, 2, 2),
        (1, 11, 11, 3, 2, 3, 3, False, 2, 2, 1, 1), (1, 10, 9, 2, 3, 5, 3, True, 1, 2, 1, 1),
        (2, 9, 9, 4, 4, 2, 2, True, 3, 3, 1, 1)]


@pytest.mark.parametrize("cfg", CONV)
def test_conv2d_against_torch(oracle_port, cfg):
    torch = pytest.importorskip("torch")
    F = torch.nn.functional
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx, dy, dx = cfg
    r = rng(5)
    x, w = nrm(r, (B, IH, IW, IC)), nrm(r, (OC, FH, FW, IC))
    OH, OW, pt, pl = oracle_port.conv2d_geometry(IH, IW, FH, FW, cov, sy, sx, dy, dx)
    rfh, rfw = FH + (FH - 1) * (dy - 1), FW + (FW - 1) * (dx - 1)
    py, px = max(0, (OH - 1) * sy + rfh - IH), max(0, (OW - 1) * sx + rfw - IW)
    tx = torch.tensor(x, dtype=torch.float64).permute(0, 3, 1, 2).requires_grad_(True)
    tw = torch.tensor(w, dtype=torch.float64).permute(0, 3, 1, 2).requires_grad_(True)
    tz = F.conv2d(F.pad(tx, (pl, px - pl, pt, py - pt)), tw, stride=(sy, sx), dilation=(dy, dx))
    a = (cov, sy, sx, dy, dx)
    z = oracle_port.conv2d(x, w, *a)
    assert z.shape == (B, OH, OW, OC) == tuple(tz.permute(0, 2, 3, 1).shape)
    assert rel_fro(z, tz.detach().permute(0, 2, 3, 1).numpy()) <= 1e-6
    gz = nrm(r, z.shape)
    tz.backward(torch.tensor(gz, dtype=torch.float64).permute(0, 3, 1, 2))
    assert rel_fro(oracle_port.conv2d_grad_x(x, w, gz, *a), tx.grad.permute(0, 2, 3, 1).numpy()) <= 1e-6
    assert rel_fro(oracle_port.conv2d_grad_y(x, w, gz, *a), tw.grad.permute(0, 2, 3, 1).numpy()) <= 1e-6


DECONV = [(2, 5, 5, 3, 4, 4, 4, False, 2, 2), (2, 5, 5, 3, 4, 4, 4, True, 2, 2), (1, 6, 4, 2, 3, 3, 3, True, 3, 3),
          (1, 4, 6, 2, 3, 4, 4, False, 3, 3), (2, 5, 5, 2, 2, 3, 3, False, 1, 1), (2, 5, 5, 2, 2, 4, 4, True, 1, 1)]


@pytest.mark.parametrize("cfg", DECONV)
def test_deconv2d_against_torch(oracle_port, cfg):
    """Deep8's DeConv2d == conv_transpose2d with the spatially flipped filter, cropped at FH-1-padTop."""
    torch = pytest.importorskip("torch")
    F = torch.nn.functional
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx = cfg
    r = rng(6)
    x, w = nrm(r, (B, IH, IW, IC)), nrm(r, (OC, FH, FW, IC))
    OH, OW, pt, pl = oracle_port.deconv2d_geometry(IH, IW, FH, FW, cov, sy, sx)
    tx = torch.tensor(x, dtype=torch.float64).permute(0, 3, 1, 2).requires_grad_(True)
    tw = torch.tensor(w, dtype=torch.float64).requires_grad_(True)
    wt = torch.flip(tw, (1, 2)).permute(3, 0, 1, 2)  # [IC, OC, FH, FW]
    full = F.conv_transpose2d(tx, wt, stride=(sy, sx))
    oy, ox = FH - 1 - pt, FW - 1 - pl
    tz = full[:, :, oy:oy + OH, ox:ox + OW]
    a = (cov, sy, sx)
    z = oracle_port.deconv2d(x, w, *a)
    assert z.shape == (B, OH, OW, OC) == tuple(tz.permute(0, 2, 3, 1).shape)
    assert rel_fro(z, tz.detach().permute(0, 2, 3, 1).numpy()) <= 1e-6
    gz = nrm(r, z.shape)
    tz.backward(torch.tensor(gz, dtype=torch.float64).permute(0, 3, 1, 2))
    assert rel_fro(oracle_port.deconv2d_grad_x(x, w, gz, *a), tx.grad.permute(0, 2, 3, 1).numpy()) <= 1e-6
    assert rel_fro(oracle_port.deconv2d_grad_y(x, w, gz, *a), tw.grad.numpy()) <= 1e-6


# ---- identities ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("cfg", CONV)
def test_im2col_brute_force_and_adjoint(oracle_port, cfg):
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx, dy, dx = cfg
    OH, OW, pt, pl = oracle_port.conv2d_geometry(IH, IW, FH, FW, cov, sy, sx, dy, dx)
    r = rng(7)
    im = ints(r, (B, IH, IW, IC))
    col = oracle_port.im2col(im, OH, OW, FH, FW, sy, sx, dy, dx, pt, pl)
    # brute force through a zero-padded copy and numpy fancy indexing
    big = np.zeros((B, IH + 2 * 64, IW + 2 * 64, IC), np.float32)
    big[:, 64:64 + IH, 64:64 + IW] = im
    want = np.empty((B, OH, OW, FH, FW, IC), np.float32)
    for fy in range(FH):
        for fx in range(FW):
            ys = 64 - pt + fy * dy + sy * np.arange(OH)
            xs = 64 - pl + fx * dx + sx * np.arange(OW)
            want[:, :, :, fy, fx, :] = big[:, ys][:, :, xs]
    assert np.array_equal(col, want.reshape(col.shape))
    # <im2col(im), c> == <im, col2im(c)> exactly on integers
    c = ints(r, col.shape, 10)
    back = oracle_port.col2im(c, np.zeros_like(im), OH, OW, FH, FW, sy, sx, dy, dx, pt, pl)
    assert float(np.sum(col.astype(np.float64) * c)) == float(np.sum(im.astype(np.float64) * back))
    # col2im adds into its destination
    twice = oracle_port.col2im(c, back, OH, OW, FH, FW, sy, sx, dy, dx, pt, pl)
    assert np.array_equal(twice, 2 * back)


@pytest.mark.parametrize("cfg", DECONV)
def test_deconv_maps_adjoint(oracle_port, cfg):
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx = cfg
    OH, OW, pt, pl = oracle_port.deconv2d_geometry(IH, IW, FH, FW, cov, sy, sx)
    r = rng(8)
    zmat = ints(r, (B * IH * IW, OC * FH * FW), 10)
    dz = ints(r, (B, OH, OW, OC), 10)
    z = oracle_port.deconv_col2im(zmat, B, IH, IW, OH, OW, OC, FH, FW, sy, sx, pt, pl)
    m = oracle_port.deconv_im2col(dz, IH, IW, FH, FW, sy, sx, pt, pl)
    assert float(np.sum(z.astype(np.float64) * dz)) == float(np.sum(zmat.astype(np.float64) * m))


@pytest.mark.parametrize("cfg", CONV)
def test_conv2d_equals_im2col_gemm_col2im(oracle_port, cfg):
    """The direct loops and the lowering the GPU path uses agree (integers: exactly)."""
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx, dy, dx = cfg
    OH, OW, pt, pl = oracle_port.conv2d_geometry(IH, IW, FH, FW, cov, sy, sx, dy, dx)
    r = rng(9)
    x, w, gz = ints(r, (B, IH, IW, IC), 20), ints(r, (OC, FH, FW, IC), 20), ints(r, (B, OH, OW, OC), 20)
    a = (cov, sy, sx, dy, dx)
    g = (OH, OW, FH, FW, sy, sx, dy, dx, pt, pl)
    col = oracle_port.im2col(x, *g)
    wm = w.reshape(OC, -1)
    assert np.array_equal(oracle_port.gemm(0, 1, col, wm).reshape(B, OH, OW, OC), oracle_port.conv2d(x, w, *a))
    dxcol = oracle_port.gemm(0, 0, gz.reshape(-1, OC), wm)
    assert np.array_equal(oracle_port.col2im(dxcol, np.zeros_like(x), *g), oracle_port.conv2d_grad_x(x, w, gz, *a))
    assert np.array_equal(oracle_port.gemm(1, 0, gz.reshape(-1, OC), col).reshape(w.shape),
                          oracle_port.conv2d_grad_y(x, w, gz, *a))


@pytest.mark.parametrize("cfg", DECONV)
def test_deconv2d_equals_gemm_and_maps(oracle_port, cfg):
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx = cfg
    OH, OW, pt, pl = oracle_port.deconv2d_geometry(IH, IW, FH, FW, cov, sy, sx)
    r = rng(10)
    x, w, gz = ints(r, (B, IH, IW, IC), 20), ints(r, (OC, FH, FW, IC), 20), ints(r, (B, OH, OW, OC), 20)
    a = (cov, sy, sx)
    wm = w.reshape(OC * FH * FW, IC)
    zmat = oracle_port.gemm(0, 1, x.reshape(-1, IC), wm)
    assert np.array_equal(oracle_port.deconv_col2im(zmat, B, IH, IW, OH, OW, OC, FH, FW, sy, sx, pt, pl),
                          oracle_port.deconv2d(x, w, *a))
    dzmat = oracle_port.deconv_im2col(gz, IH, IW, FH, FW, sy, sx, pt, pl)
    assert np.array_equal(oracle_port.gemm(0, 0, dzmat, wm).reshape(x.shape), oracle_port.deconv2d_grad_x(x, w, gz, *a))
    assert np.array_equal(oracle_port.gemm(1, 0, dzmat, x.reshape(-1, IC)).reshape(w.shape),
                          oracle_port.deconv2d_grad_y(x, w, gz, *a))


def test_special_cases(oracle_port):
    r = rng(11)
    # 1x1 filter, stride 1: conv is a GEMM over pixels
    x, w = ints(r, (2, 5, 6, 7)), ints(r, (3, 1, 1, 7))
    assert np.array_equal(oracle_port.conv2d(x, w).reshape(-1, 3), x.reshape(-1, 7) @ w.reshape(3, 7).T)
    # K = 1: outer product; identity operand
    a, b = ints(r, (1, 9, 1)), ints(r, (1, 1, 4))
    assert np.array_equal(oracle_port.matmul(a, b)[0], np.outer(a[0, :, 0], b[0, 0]))
    m = ints(r, (1, 6, 6))
    assert np.array_equal(oracle_port.matmul(m, np.eye(6, dtype=np.float32)[None]), m)
    # gradients accumulate: running twice doubles
    y, dz = ints(r, (1, 6, 5)), ints(r, (1, 6, 5))
    once = oracle_port.matmul_grad_x(m, y, dz)
    assert np.array_equal(oracle_port.matmul_grad_x(m, y, dz, once), 2 * once)
    # stride >= filter: col2im never overlaps, every element is copied once
    im = np.zeros((1, 6, 6, 2), np.float32)
    col = ints(r, (9, 2 * 2 * 2)) + 1
    out = oracle_port.col2im(col, im, 3, 3, 2, 2, 2, 2, 1, 1, 0, 0)
    assert sorted(out.ravel()) == sorted(col.ravel())
    # geometry of the benchmark configurations
    assert oracle_port.conv2d_geometry(56, 56, 3, 3, True, 1, 1, 1, 1) == (56, 56, 1, 1)
    assert oracle_port.deconv2d_geometry(28, 28, 4, 4, False, 2, 2) == (58, 58, 3, 3)
    assert oracle_port.deconv2d_geometry(28, 28, 4, 4, True, 2, 2) == (55, 55, 1, 1)


# ---- Add / ReLu ------------------------------------------------------------------------------------------------------
ADD_PAIRS = [((2, 3, 4), (2, 3, 4)), ((10, 50, 20), (1, 20)), ((2, 5, 6, 8), (1, 8)), ((1, 4, 1), (3, 1, 5)),
             ((3, 7), (1, 1)), ((2, 2, 3, 4, 5), (2, 1, 3, 1, 5)), ((2, 6, 6, 8), (2, 1, 1, 8))]


def _ex(a, nd):
    return a.reshape((a.shape[0],) + (1,) * (nd - a.ndim) + a.shape[1:])


@pytest.mark.parametrize("xs,ys", ADD_PAIRS)
def test_add_against_numpy_and_reference(oracle_port, oracle_ref, xs, ys):
    """numpy broadcasting (batch axis first, dims right-aligned) fixes the index map; np.sum over the
    broadcast axes fixes the gradient; the live reference build must agree wherever it is present."""
    r = rng(sum(xs) + sum(ys))
    x, y = ints(r, xs), ints(r, ys)
    nd = max(x.ndim, y.ndim)
    ex, ey = _ex(x, nd), _ex(y, nd)
    z = oracle_port.add(x, y)
    assert np.array_equal(z, ex + ey)
    dz = ints(r, z.shape)
    for which, a, ea in ((0, x, ex), (1, y, ey)):
        axes = tuple(i for i in range(nd) if ea.shape[i] == 1 and z.shape[i] != 1)
        want = dz.sum(axis=axes, keepdims=True).reshape(a.shape) + a
        assert np.array_equal(oracle_port.add_grad(a, dz, a), want)
        if oracle_ref is not None:
            assert np.array_equal(oracle_ref.add_grad(which, x, y, dz, a), want)
    if oracle_ref is not None:
        assert np.array_equal(oracle_ref.add(x, y), z)
        xr, yr, dzr = nrm(r, xs), nrm(r, ys), nrm(r, z.shape)
        assert np.array_equal(oracle_ref.add(xr, yr), oracle_port.add(xr, yr))
        assert rel_fro(oracle_ref.add_grad(1, xr, yr, dzr), oracle_port.add_grad(yr, dzr)) <= 1e-6


def test_relu_against_numpy_and_reference(oracle_port, oracle_ref):
    r = rng(12)
    x, dy, dx0 = nrm(r, (3, 9, 11)), nrm(r, (3, 9, 11)), nrm(r, (3, 9, 11))
    x[0, 0, :3] = (0.0, -0.0, 1e-30)
    assert np.array_equal(oracle_port.relu(x), np.maximum(x, 0))
    want = dx0 + np.where(x > 0, dy, 0).astype(np.float32)
    assert np.array_equal(oracle_port.relu_grad(x, dy, dx0), want)
    if oracle_ref is not None:
        assert np.array_equal(oracle_ref.relu(x), np.maximum(x, 0))
        assert np.array_equal(oracle_ref.relu_grad(x, dy, dx0), want)


# ---- Minus / L1Norm / L2Norm / ReduceMean / AXPBY ------------------------------------------------------------
@pytest.mark.parametrize("i", _n("loss"))
def test_loss_ops_against_golden(oracle_port, i):
    """Outputs of the reference's own CPU build for Minus, the two norms, ReduceMean and AXPBY."""
    g = lambda k: GOLD["loss%d_%s" % (i, k)]
    x, y, axes = g("x"), g("y"), tuple(int(a) for a in g("axes"))
    assert np.array_equal(oracle_port.minus(x, y), g("z"))
    assert rel_fro(oracle_port.add_grad(x, g("dz"), g("dx0")), g("minus_gx")) <= TOL
    assert rel_fro(oracle_port.minus_grad_y(y, g("dz"), g("dy0")), g("minus_gy")) <= TOL
    assert rel_fro(oracle_port.l1norm(x), g("l1")) <= TOL
    assert rel_fro(oracle_port.l2norm(x), g("l2")) <= TOL
    assert rel_fro(oracle_port.l1norm_grad(x, g("dn"), g("dx0")), g("l1_gx")) <= TOL
    assert rel_fro(oracle_port.l2norm_grad(x, g("l2"), g("dn"), g("dx0")), g("l2_gx")) <= TOL
    m = oracle_port.reduce_mean(x, axes)
    assert m.size == g("mean").size and rel_fro(m.ravel(), g("mean").ravel()) <= TOL
    assert rel_fro(oracle_port.reduce_mean_grad(g("dx0"), g("dm").reshape(m.shape)), g("mean_gx")) <= TOL
    assert rel_fro(oracle_port.axpby(x, -0.01, g("dx0"), 0.999), g("axpby")) <= 1e-7


@pytest.mark.parametrize("xs,ys", ADD_PAIRS)
def test_minus_against_numpy_and_reference(oracle_port, oracle_ref, xs, ys):
    r = rng(sum(xs) * 3 + sum(ys))
    x, y = ints(r, xs), ints(r, ys)
    nd = max(x.ndim, y.ndim)
    ex, ey = _ex(x, nd), _ex(y, nd)
    z = oracle_port.minus(x, y)
    assert np.array_equal(z, ex - ey)
    dz = ints(r, z.shape)
    axes = tuple(i for i in range(nd) if ey.shape[i] == 1 and z.shape[i] != 1)
    want = y - dz.sum(axis=axes, keepdims=True).reshape(y.shape)
    assert np.array_equal(oracle_port.minus_grad_y(y, dz, y), want)
    if oracle_ref is not None:
        assert np.array_equal(oracle_ref.minus(x, y), z)
        assert np.array_equal(oracle_ref.minus_grad(1, x, y, dz, y), want)
        assert np.array_equal(oracle_ref.minus_grad(0, x, y, dz, x), oracle_port.add_grad(x, dz, x))


@pytest.mark.parametrize("shape", [(3, 17), (1, 1000), (4, 5, 6, 7), (7, 1)])
def test_norms_against_numpy_and_reference(oracle_port, oracle_ref, shape):
    """np.abs().sum / np.sqrt((x*x).sum) per batch row; gradients by their closed forms, including
    sign(0) = 0 for L1 and the accumulate-twice identity."""
    r = rng(sum(shape))
    x = ints(r, shape, 7) - 3  # integers -3..3, zeros included
    flat = x.reshape(shape[0], -1).astype(np.float64)
    assert np.array_equal(oracle_port.l1norm(x), np.abs(flat).sum(1, keepdims=True).astype(np.float32))
    l2 = oracle_port.l2norm(x)
    assert rel_fro(l2, np.sqrt((flat * flat).sum(1, keepdims=True))) <= 1e-7
    dy = ints(r, (shape[0], 1), 5) + 1
    bshape = (shape[0],) + (1,) * (len(shape) - 1)
    g1 = oracle_port.l1norm_grad(x, dy)
    assert np.array_equal(g1, (np.sign(x) * dy.reshape(bshape)).astype(np.float32))
    assert np.array_equal(oracle_port.l1norm_grad(x, dy, g1), 2 * g1)
    xr = nrm(r, shape) + 0.1
    l2r = oracle_port.l2norm(xr)
    g2 = oracle_port.l2norm_grad(xr, l2r, dy)
    assert rel_fro(g2, xr * (dy / l2r).reshape(bshape)) <= 1e-6
    if oracle_ref is not None:
        assert np.array_equal(oracle_ref.norm(1, x), oracle_port.l1norm(x))
        assert np.array_equal(oracle_ref.norm_grad(1, x, oracle_port.l1norm(x), dy), g1)
        assert rel_fro(oracle_ref.norm(2, xr), l2r) <= 1e-6
        assert rel_fro(oracle_ref.norm_grad(2, xr, l2r, dy), g2) <= 1e-6


@pytest.mark.parametrize("shape,axes", [((3, 8), ()), ((3, 8), (0,)), ((3, 8), (1,)), ((2, 4, 5, 6), (1, 3)), ((2, 4, 5, 6), (-1,)),
                                        ((2, 3, 4, 5, 6), (0, 2, 4)), ((1, 12), (0, 1))])
def test_reduce_mean_against_numpy_and_reference(oracle_port, oracle_ref, shape, axes):
    r = rng(sum(shape) + len(axes))
    x = ints(r, shape, 9)
    ax = tuple(range(len(shape))) if not axes else tuple((a + len(shape)) % len(shape) for a in axes)
    want = x.astype(np.float64).mean(axis=ax, keepdims=True)
    m = oracle_port.reduce_mean(x, axes)
    assert m.shape == want.shape and rel_fro(m, want) <= 1e-7
    dm, dx0 = ints(r, m.shape, 9), ints(r, shape, 9)
    count = x.size // m.size
    g = oracle_port.reduce_mean_grad(dx0, dm)
    assert rel_fro(g, dx0 + np.broadcast_to(dm, shape) / count) <= 1e-7
    if oracle_ref is not None:
        for keep in (True, False):
            assert rel_fro(oracle_ref.reduce_mean(x, axes, keep).ravel(), m.ravel()) <= 1e-6
            assert rel_fro(oracle_ref.reduce_mean_grad(x, m, dm, axes, keep, dx0), g) <= 1e-6


def test_axpby_against_numpy_and_reference(oracle_port, oracle_ref):
    r = rng(5)
    x, y = nrm(r, (3, 50)), nrm(r, (3, 50))
    z = oracle_port.axpby(x, -0.01, y, 0.999)
    assert np.array_equal(z, x * np.float32(-0.01) + y * np.float32(0.999))
    if oracle_ref is not None:
        assert rel_fro(oracle_ref.axpby(x, -0.01, y, 0.999), z) <= 1e-7


# ---- AdamUpdate -------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("i", _n("adam"))
def test_adam_update_against_golden(oracle_port, i):
    """Three consecutive steps of the reference's CPU AdamUpdate (weight decay 0.001)."""
    g = lambda k: GOLD["adam%d_%s" % (i, k)]
    st = [g("value0"), None, np.zeros_like(g("value0")), np.zeros_like(g("value0"))]
    for step in (1, 2, 3):
        st = list(oracle_port.adam_update(st[0], g("grad%d" % step), st[2], st[3], 0.9, 0.999, 1e-7, 0.01, 0.001, step))
        want = g("step%d" % step)
        for k in range(4):
            assert rel_fro(st[k], want[k]) <= 1e-6, (step, k)


def test_adam_update_against_textbook_and_reference(oracle_port, oracle_ref):
    """Bias-corrected Adam in float64 numpy: m_hat = m / (1 - b1^t), v_hat = v / (1 - b2^t),
    x -= lr * m_hat / (sqrt(v_hat) + eps'), which equals the reference's ratio form when epsilon is
    scaled by sqrt(1 - b2^t); with epsilon = 0 the two coincide exactly."""
    r = rng(77)
    x, g = nrm(r, (2, 33)), nrm(r, (2, 33))
    m, v = np.zeros_like(x), np.zeros_like(x)
    b1, b2, lr = float(np.float32(0.9)), float(np.float32(0.999)), 0.01  # the betas as the float code sees them
    X, M, V = x.astype(np.float64), m.astype(np.float64), v.astype(np.float64)
    st = [x, None, m, v]
    for t in (1, 2, 3, 4):
        gt = nrm(r, x.shape)
        st = list(oracle_port.adam_update(st[0], gt, st[2], st[3], b1, b2, 0.0, lr, 0.0, t))
        M = b1 * M + (1 - b1) * gt
        V = b2 * V + (1 - b2) * gt.astype(np.float64) ** 2
        X = X - lr * (M / (1 - b1 ** t)) / np.sqrt(V / (1 - b2 ** t))
        assert rel_fro(st[0], X) <= 1e-5 and rel_fro(st[2], M) <= 1e-6 and rel_fro(st[3], V) <= 1e-6
    # steps <= 0 count as 1; weight decay adds wd * value to the gradient first
    a = oracle_port.adam_update(x, g, m, v, b1, b2, 1e-7, lr, 0.5, 0)
    b = oracle_port.adam_update(x, g + 0.5 * x, m, v, b1, b2, 1e-7, lr, 0.0, 1)
    assert rel_fro(a[0], b[0]) <= 1e-6 and rel_fro(a[1], b[1]) <= 1e-7
    if oracle_ref is not None:
        want = oracle_ref.adam_update(x, g, m, v, b1, b2, 1e-7, lr, 0.001, 3)
        got = oracle_port.adam_update(x, g, m, v, b1, b2, 1e-7, lr, 0.001, 3)
        for k in range(4):
            assert rel_fro(got[k], want[k]) <= 1e-6


# ---- MaxPooling2d / AvgPooling2d ---------------------------------------------------------------------------------
@pytest.mark.parametrize("i", _n("pool"))
def test_pooling_against_golden(oracle_port, i):
    g = lambda k: GOLD["pool%d_%s" % (i, k)]
    B, IH, IW, C, FH, FW, cov, sy, sx = (int(v) for v in g("cfg"))
    a = (FH, FW, bool(cov), sy, sx)
    assert np.array_equal(oracle_port.pool2d(True, g("x"), *a), g("max"))
    assert rel_fro(oracle_port.pool2d(False, g("x"), *a), g("avg")) <= TOL
    assert np.array_equal(oracle_port.pool2d_grad(True, g("x"), g("dy"), *a, dx=g("dx0")), g("max_gx"))
    assert rel_fro(oracle_port.pool2d_grad(False, g("x"), g("dy"), *a, dx=g("dx0")), g("avg_gx")) <= TOL


@pytest.mark.parametrize("cfg", [(2, 8, 8, 3, 2, 2, 2, 2), (1, 9, 9, 4, 3, 3, 2, 2), (2, 12, 10, 5, 3, 2, 1, 2), (1, 7, 7, 2, 7, 7, 1, 1)])
def test_pooling_inside_the_image_against_torch(oracle_port, cfg):
    """Windows that stay inside the image (covered = false): torch's max_pool2d / avg_pool2d and their
    autograd gradients (distinct values, so the maximum is unique)."""
    import torch
    import torch.nn.functional as F
    B, IH, IW, C, FH, FW, sy, sx = cfg
    r = rng(sum(cfg))
    x = r.permutation(B * IH * IW * C).astype(np.float32).reshape(B, IH, IW, C) - 100.0
    for is_max in (True, False):
        xt = torch.tensor(x).permute(0, 3, 1, 2).clone().requires_grad_(True)
        yt = F.max_pool2d(xt, (FH, FW), (sy, sx)) if is_max else F.avg_pool2d(xt, (FH, FW), (sy, sx))
        y = oracle_port.pool2d(is_max, x, FH, FW, False, sy, sx)
        assert rel_fro(y, yt.detach().permute(0, 2, 3, 1).numpy()) <= 1e-6
        dy = nrm(r, y.shape)
        yt.backward(torch.tensor(dy).permute(0, 3, 1, 2))
        want = xt.grad.permute(0, 2, 3, 1).numpy()
        assert rel_fro(oracle_port.pool2d_grad(is_max, x, dy, FH, FW, False, sy, sx), want) <= 1e-6


@pytest.mark.parametrize("cfg", [(2, 7, 7, 2, 3, 3, 2, 2), (1, 6, 6, 3, 3, 3, 1, 1), (1, 10, 10, 2, 4, 4, 3, 3), (1, 5, 5, 1, 2, 2, 2, 2)])
def test_pooling_with_padding_against_padded_copy_and_reference(oracle_port, oracle_ref, cfg):
    """covered = true: the forward pass equals pooling (inside the image) of a zero-padded copy -- so a
    window of negative values that touches the border yields 0 -- while the max gradient ignores the
    padding; ties go to the first element in scan order."""
    B, IH, IW, C, FH, FW, sy, sx = cfg
    r = rng(sum(cfg) + 1)
    x = -np.abs(nrm(r, (B, IH, IW, C))) - 0.5  # all negative: padding zeros win every border window
    OH, OW, pt, pl = oracle_port.conv2d_geometry(IH, IW, FH, FW, True, sy, sx, 1, 1)
    py, px = max(0, (OH - 1) * sy + FH - IH), max(0, (OW - 1) * sx + FW - IW)
    xp = np.zeros((B, IH + py, IW + px, C), np.float32)
    xp[:, pt:pt + IH, pl:pl + IW] = x
    for is_max in (True, False):
        y = oracle_port.pool2d(is_max, x, FH, FW, True, sy, sx)
        assert np.array_equal(y, oracle_port.pool2d(is_max, xp, FH, FW, False, sy, sx)[:, :OH, :OW])
        if is_max and (py or px):
            assert (y[:, -1] == 0).all()
    # gradient: brute force over windows with numpy argmax on the clipped window
    dy = ints(r, (B, OH, OW, C), 9) + 1
    want = np.zeros_like(x)
    wavg = np.zeros_like(x)
    for b in range(B):
        for oh in range(OH):
            for ow in range(OW):
                h0, h1 = max(0, oh * sy - pt), min(IH, oh * sy - pt + FH)
                w0, w1 = max(0, ow * sx - pl), min(IW, ow * sx - pl + FW)
                for c in range(C):
                    win = x[b, h0:h1, w0:w1, c]
                    k = int(np.argmax(win))  # first maximum in row-major order
                    want[b, h0 + k // (w1 - w0), w0 + k % (w1 - w0), c] += dy[b, oh, ow, c]
                    wavg[b, h0:h1, w0:w1, c] += dy[b, oh, ow, c] / np.float32(FH * FW)
    assert np.array_equal(oracle_port.pool2d_grad(True, x, dy, FH, FW, True, sy, sx), want)
    assert rel_fro(oracle_port.pool2d_grad(False, x, dy, FH, FW, True, sy, sx), wavg) <= 1e-6
    # ties: a constant image sends every window's gradient to its first in-image element
    k = np.ones((1, 4, 4, 1), np.float32)
    g = oracle_port.pool2d_grad(True, k, np.ones((1, 2, 2, 1), np.float32), 2, 2, False, 2, 2)
    assert np.array_equal(g[0, :, :, 0], np.array([[1, 0, 1, 0], [0, 0, 0, 0], [1, 0, 1, 0], [0, 0, 0, 0]], np.float32))
    if oracle_ref is not None:
        for is_max in (True, False):
            assert rel_fro(oracle_ref.pool2d(is_max, x, FH, FW, True, sy, sx), oracle_port.pool2d(is_max, x, FH, FW, True, sy, sx)) <= 1e-6
            assert rel_fro(oracle_ref.pool2d_grad(is_max, x, dy, FH, FW, True, sy, sx),
                           oracle_port.pool2d_grad(is_max, x, dy, FH, FW, True, sy, sx)) <= 1e-6


# ---- the double twins of the contraction path (orc_*_f64) ----------------------------------------------------
# Same loops as the float functions, compiled for double.  Pinned by: the float path on integer inputs
# (exact in both), numpy / torch in float64 on real inputs, and the reference's own Float64 CPU path live.
F64_TOL = 1e-13


def _torch_conv2d(port, x, w, gz, cfg):
    import torch
    F = torch.nn.functional
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx, dy, dx = cfg
    OH, OW, pt, pl = port.conv2d_geometry(IH, IW, FH, FW, cov, sy, sx, dy, dx)
    rfh, rfw = FH + (FH - 1) * (dy - 1), FW + (FW - 1) * (dx - 1)
    py, px = max(0, (OH - 1) * sy + rfh - IH), max(0, (OW - 1) * sx + rfw - IW)
    tx = torch.tensor(x, dtype=torch.float64).permute(0, 3, 1, 2).requires_grad_(True)
    tw = torch.tensor(w, dtype=torch.float64).permute(0, 3, 1, 2).requires_grad_(True)
    tz = F.conv2d(F.pad(tx, (pl, px - pl, pt, py - pt)), tw, stride=(sy, sx), dilation=(dy, dx))
    tz.backward(torch.tensor(gz, dtype=torch.float64).permute(0, 3, 1, 2))
    return (tz.detach().permute(0, 2, 3, 1).numpy(), tx.grad.permute(0, 2, 3, 1).numpy(), tw.grad.permute(0, 2, 3, 1).numpy())


def _torch_deconv2d(port, x, w, gz, cfg):
    import torch
    F = torch.nn.functional
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx = cfg
    OH, OW, pt, pl = port.deconv2d_geometry(IH, IW, FH, FW, cov, sy, sx)
    tx = torch.tensor(x, dtype=torch.float64).permute(0, 3, 1, 2).requires_grad_(True)
    tw = torch.tensor(w, dtype=torch.float64).requires_grad_(True)
    full = F.conv_transpose2d(tx, torch.flip(tw, (1, 2)).permute(3, 0, 1, 2), stride=(sy, sx))
    oy, ox = FH - 1 - pt, FW - 1 - pl
    tz = full[:, :, oy:oy + OH, ox:ox + OW]
    tz.backward(torch.tensor(gz, dtype=torch.float64).permute(0, 3, 1, 2))
    return tz.detach().permute(0, 2, 3, 1).numpy(), tx.grad.permute(0, 2, 3, 1).numpy(), tw.grad.numpy()


@pytest.mark.parametrize("xs,ys", MM_SHAPES)
def test_double_matmul(oracle_port, oracle_ref, oracle, xs, ys):
    r = rng(40)
    xi, yi = ints(r, xs), ints(r, ys)
    zi = oracle_port.matmul(xi, yi)
    dzi = ints(r, zi.shape)
    x, y = r.standard_normal(xs), r.standard_normal(ys)
    x3 = x.reshape(xs[0], xs[1], xs[2] if len(xs) == 3 else 1)
    y3 = y.reshape(ys[0], ys[1], ys[2] if len(ys) == 3 else 1)
    zb = max(xs[0], ys[0])
    X, Y = np.broadcast_to(x3, (zb,) + x3.shape[1:]), np.broadcast_to(y3, (zb,) + y3.shape[1:])
    want = np.matmul(X, Y)
    dz = r.standard_normal(zi.shape)
    DZ = dz.reshape(want.shape)
    dX, dY = np.matmul(DZ, Y.transpose(0, 2, 1)), np.matmul(X.transpose(0, 2, 1), DZ)
    dX = dX.sum(0, keepdims=True) if xs[0] == 1 else dX
    dY = dY.sum(0, keepdims=True) if ys[0] == 1 else dY
    f32 = (zi, oracle_port.matmul_grad_x(xi, yi, dzi), oracle_port.matmul_grad_y(xi, yi, dzi))
    with oracle.float64():
        got_i = (oracle_port.matmul(xi, yi), oracle_port.matmul_grad_x(xi, yi, dzi), oracle_port.matmul_grad_y(xi, yi, dzi))
        got = (oracle_port.matmul(x, y), oracle_port.matmul_grad_x(x, y, dz), oracle_port.matmul_grad_y(x, y, dz))
        live = (oracle_ref.matmul(x, y), oracle_ref.matmul_grad_x(x, y, dz), oracle_ref.matmul_grad_y(x, y, dz))
    for a, b in zip(got_i, f32):
        assert a.dtype == np.float64 and np.array_equal(a, b.astype(np.float64))
    for a, b, c in zip(got, (want, dX, dY), live):
        assert rel_fro(a.reshape(b.shape), b) <= F64_TOL
        assert c.dtype == np.float64 and rel_fro(a, c) <= F64_TOL
    # beta = 1: the old value takes part
    with oracle.float64():
        twice = oracle_port.matmul_grad_x(x, y, dz, dx=got[1])
    assert rel_fro(twice, 2 * got[1]) <= F64_TOL


@pytest.mark.parametrize("cfg", CONV)
def test_double_conv2d(oracle_port, oracle, cfg):
    pytest.importorskip("torch")
    B, IH, IW, IC, OC, FH, FW = cfg[:7]
    a = cfg[7:]
    r = rng(41)
    xi, wi = ints(r, (B, IH, IW, IC), 8), ints(r, (OC, FH, FW, IC), 8)
    zi = oracle_port.conv2d(xi, wi, *a)
    gzi = ints(r, zi.shape, 8)
    f32 = (zi, oracle_port.conv2d_grad_x(xi, wi, gzi, *a), oracle_port.conv2d_grad_y(xi, wi, gzi, *a))
    x, w, gz = r.standard_normal(xi.shape), r.standard_normal(wi.shape), r.standard_normal(zi.shape)
    want = _torch_conv2d(oracle_port, x, w, gz, cfg)
    with oracle.float64():
        got_i = (oracle_port.conv2d(xi, wi, *a), oracle_port.conv2d_grad_x(xi, wi, gzi, *a), oracle_port.conv2d_grad_y(xi, wi, gzi, *a))
        got = (oracle_port.conv2d(x, w, *a), oracle_port.conv2d_grad_x(x, w, gz, *a), oracle_port.conv2d_grad_y(x, w, gz, *a))
    for p, q in zip(got_i, f32):
        assert p.dtype == np.float64 and np.array_equal(p, q.astype(np.float64))
    for p, q in zip(got, want):
        assert rel_fro(p, q) <= F64_TOL


@pytest.mark.parametrize("cfg", DECONV)
def test_double_deconv2d(oracle_port, oracle, cfg):
    pytest.importorskip("torch")
    B, IH, IW, IC, OC, FH, FW = cfg[:7]
    a = cfg[7:]
    r = rng(42)
    xi, wi = ints(r, (B, IH, IW, IC), 8), ints(r, (OC, FH, FW, IC), 8)
    zi = oracle_port.deconv2d(xi, wi, *a)
    gzi = ints(r, zi.shape, 8)
    f32 = (zi, oracle_port.deconv2d_grad_x(xi, wi, gzi, *a), oracle_port.deconv2d_grad_y(xi, wi, gzi, *a))
    x, w, gz = r.standard_normal(xi.shape), r.standard_normal(wi.shape), r.standard_normal(zi.shape)
    want = _torch_deconv2d(oracle_port, x, w, gz, cfg)
    with oracle.float64():
        got_i = (oracle_port.deconv2d(xi, wi, *a), oracle_port.deconv2d_grad_x(xi, wi, gzi, *a), oracle_port.deconv2d_grad_y(xi, wi, gzi, *a))
        got = (oracle_port.deconv2d(x, w, *a), oracle_port.deconv2d_grad_x(x, w, gz, *a), oracle_port.deconv2d_grad_y(x, w, gz, *a))
    for p, q in zip(got_i, f32):
        assert p.dtype == np.float64 and np.array_equal(p, q.astype(np.float64))
    for p, q in zip(got, want):
        assert rel_fro(p, q) <= F64_TOL


def test_double_gemm_against_numpy(oracle_port, oracle):
    r = rng(43)
    A, B, C = r.standard_normal((37, 23)), r.standard_normal((23, 41)), r.standard_normal((37, 41))
    with oracle.float64():
        assert rel_fro(oracle_port.gemm(0, 0, A, B), A @ B) <= F64_TOL
        assert rel_fro(oracle_port.gemm(0, 1, A, np.ascontiguousarray(B.T)), A @ B) <= F64_TOL
        assert rel_fro(oracle_port.gemm(1, 0, np.ascontiguousarray(A.T), B, C, 1.0), A @ B + C) <= F64_TOL


# The reference's Float64 CPU path, live, on the shapes of the float live tests above (square images: its patch
# expression pads the wrong axis when the two pads differ).
@pytest.mark.parametrize("cov", [True, False])
@pytest.mark.parametrize("s,d,F", [(1, 1, 3), (2, 2, 4), (2, 1, 3), (1, 2, 3), (3, 1, 5)])
def test_double_conv2d_against_reference_live(oracle_port, oracle_ref, oracle, cov, s, d, F):
    r = rng(44)
    x, w = r.standard_normal((2, 17, 17, 5)), r.standard_normal((6, F, F, 5))
    a = (cov, s, s, d, d)
    with oracle.float64():
        z = oracle_ref.conv2d(x, w, *a)
        assert z.dtype == np.float64 and rel_fro(oracle_port.conv2d(x, w, *a), z) <= F64_TOL
        gz = r.standard_normal(z.shape)
        assert rel_fro(oracle_port.conv2d_grad_x(x, w, gz, *a), oracle_ref.conv2d_grad_x(x, w, gz, *a)) <= F64_TOL
        assert rel_fro(oracle_port.conv2d_grad_y(x, w, gz, *a), oracle_ref.conv2d_grad_y(x, w, gz, *a)) <= F64_TOL


@pytest.mark.parametrize("cov", [True, False])
@pytest.mark.parametrize("s,F", [(1, 3), (2, 4), (3, 4), (2, 3), (3, 2)])
def test_double_deconv2d_against_reference_live(oracle_port, oracle_ref, oracle, cov, s, F):
    r = rng(45)
    x, w = r.standard_normal((2, 9, 9, 5)), r.standard_normal((6, F, F, 5))
    a = (cov, s, s)
    with oracle.float64():
        z = oracle_ref.deconv2d(x, w, *a)
        assert z.dtype == np.float64 and rel_fro(oracle_port.deconv2d(x, w, *a), z) <= F64_TOL
        gz = r.standard_normal(z.shape)
        assert rel_fro(oracle_port.deconv2d_grad_x(x, w, gz, *a), oracle_ref.deconv2d_grad_x(x, w, gz, *a)) <= F64_TOL
        assert rel_fro(oracle_port.deconv2d_grad_y(x, w, gz, *a), oracle_ref.deconv2d_grad_y(x, w, gz, *a)) <= F64_TOL
