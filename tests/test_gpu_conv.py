"""Conv2d / DeConv2d through the C ABI against the oracle.

* the four gather maps must be bit-exact (pure copies, or float additions in the reference
  kernels' own order);
* whole operators: integer inputs bit-exact, seeded real inputs within tolerance;
* geometry variants follow the reference's tests (test/Conv2dTest.h: stride 2 + dilation 2
  covered, 5x5 stride 1, not covered; test/DeConv2dTest.h: stride 3 4x4, covered and not).
"""
import numpy as np
import pytest

from util import FP16_TOL, FP32_TOL, f, h, ints, nrm, rel_fro, rng, uni

pytestmark = pytest.mark.gpu

# (B, IH, IW, IC, OC, FH, FW, covered, sy, sx, dy, dx)
CONV = [
    (2, 32, 32, 64, 32, 4, 4, True, 2, 2, 2, 2),    # Conv2dTest forwardCPU_float
    (2, 16, 16, 8, 6, 5, 5, True, 1, 1, 1, 1),      # backwardCPU_float-like
    (2, 17, 13, 5, 7, 3, 3, False, 1, 1, 1, 1),     # not covered, odd channel counts (scalar paths)
    (1, 9, 9, 4, 4, 3, 3, True, 2, 2, 1, 1),
    (3, 12, 12, 16, 8, 3, 3, False, 2, 2, 2, 2),
    (2, 8, 8, 16, 16, 1, 1, True, 1, 1, 1, 1),      # 1x1: conv == GEMM
    (2, 14, 14, 32, 24, 3, 3, True, 1, 1, 1, 1),    # same padding like BASELINE config 4
    (1, 10, 10, 3, 5, 2, 2, True, 3, 3, 1, 1),      # stride > filter: holes in col2im
]
# (B, IH, IW, IC, OC, FH, FW, covered, sy, sx)
DECONV = [
    (2, 8, 8, 16, 8, 4, 4, False, 3, 3),    # DeConv2dTest forwardCPU geometry (smaller)
    (2, 8, 8, 16, 8, 4, 4, True, 3, 3),     # backwardCPU geometry
    (2, 7, 7, 8, 16, 4, 4, False, 2, 2),    # BASELINE config 5 family -> 2*7+2
    (2, 7, 7, 8, 16, 4, 4, True, 2, 2),
    (1, 5, 6, 3, 5, 3, 3, False, 1, 1),
    (2, 6, 5, 4, 3, 3, 2, True, 2, 2),
    (1, 4, 4, 2, 2, 2, 2, False, 3, 3),     # stride > filter
]


@pytest.mark.parametrize("cfg", CONV)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_im2col_col2im_bit_exact(oracle_port, cfg, dtype):
    from deep8_amd import ops
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx, dy, dx = cfg
    OH, OW, pt, pl = oracle_port.conv2d_geometry(IH, IW, FH, FW, cov, sy, sx, dy, dx)
    assert ops.conv2d_geometry(IH, IW, FH, FW, cov, sy, sx, dy, dx) == (OH, OW, pt, pl)
    r = rng(B + IH + FH)
    im = nrm(r, (B, IH, IW, IC)).astype(dtype)
    want = oracle_port.im2col(f(im), OH, OW, FH, FW, sy, sx, dy, dx, pt, pl)
    got = ops.im2col(im, OH, OW, FH, FW, sy, sx, dy, dx, pt, pl)
    assert got.dtype == dtype
    assert np.array_equal(got.view(np.uint16 if dtype == np.float16 else np.uint32),
                          want.astype(dtype).view(np.uint16 if dtype == np.float16 else np.uint32))
    if dtype == np.float32:
        col = nrm(r, want.shape)
        im0 = nrm(r, im.shape)
        w = oracle_port.col2im(col, im0, OH, OW, FH, FW, sy, sx, dy, dx, pt, pl)
        g = ops.col2im(col, im0, OH, OW, FH, FW, sy, sx, dy, dx, pt, pl)
        assert np.array_equal(g.view(np.uint32), w.view(np.uint32))
    else:
        col = h(ints(r, want.shape, 8))
        im0 = h(ints(r, im.shape, 8))
        w = oracle_port.col2im(f(col), f(im0), OH, OW, FH, FW, sy, sx, dy, dx, pt, pl)
        g = ops.col2im(col, im0, OH, OW, FH, FW, sy, sx, dy, dx, pt, pl)
        assert np.array_equal(f(g), w)


@pytest.mark.parametrize("cfg", DECONV)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_deconv_maps_bit_exact(oracle_port, cfg, dtype):
    from deep8_amd import ops
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx = cfg
    OH, OW, pt, pl = oracle_port.deconv2d_geometry(IH, IW, FH, FW, cov, sy, sx)
    assert ops.deconv2d_geometry(IH, IW, FH, FW, cov, sy, sx) == (OH, OW, pt, pl)
    r = rng(B + IH + FH + 1)
    dz = nrm(r, (B, OH, OW, OC)).astype(dtype)
    want = oracle_port.deconv_im2col(f(dz), IH, IW, FH, FW, sy, sx, pt, pl)
    got = ops.deconv_im2col(dz, IH, IW, FH, FW, sy, sx, pt, pl)
    assert np.array_equal(f(got), want)
    if dtype == np.float32:
        zmat = nrm(r, (B * IH * IW, OC * FH * FW))
        w = oracle_port.deconv_col2im(zmat, B, IH, IW, OH, OW, OC, FH, FW, sy, sx, pt, pl)
        g = ops.deconv_col2im(zmat, B, IH, IW, OH, OW, OC, FH, FW, sy, sx, pt, pl)
        assert np.array_equal(g.view(np.uint32), w.view(np.uint32))
    else:
        zmat = h(ints(r, (B * IH * IW, OC * FH * FW), 8))
        w = oracle_port.deconv_col2im(f(zmat), B, IH, IW, OH, OW, OC, FH, FW, sy, sx, pt, pl)
        g = ops.deconv_col2im(zmat, B, IH, IW, OH, OW, OC, FH, FW, sy, sx, pt, pl)
        assert np.array_equal(f(g), w)


@pytest.mark.parametrize("cfg", CONV)
def test_conv2d_integer_exact(oracle_port, cfg):
    from deep8_amd import ops
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx, dy, dx = cfg
    r = rng(B + IH + OC)
    x, w = ints(r, (B, IH, IW, IC)), ints(r, (OC, FH, FW, IC))
    want = oracle_port.conv2d(x, w, cov, sy, sx, dy, dx)
    got = ops.conv2d(x, w, cov, sy, sx, dy, dx)
    assert got.shape == want.shape and np.array_equal(got, want)
    gz = ints(r, want.shape, 10)
    gx0, gw0 = ints(r, x.shape), ints(r, w.shape)
    assert np.array_equal(ops.conv2d_grad_x(x, w, gz, cov, sy, sx, dy, dx, gx0),
                          oracle_port.conv2d_grad_x(x, w, gz, cov, sy, sx, dy, dx, gx0))
    assert np.array_equal(ops.conv2d_grad_y(x, w, gz, cov, sy, sx, dy, dx, gw0),
                          oracle_port.conv2d_grad_y(x, w, gz, cov, sy, sx, dy, dx, gw0))


@pytest.mark.parametrize("cfg", CONV)
def test_conv2d_real_tolerance(oracle_port, cfg):
    from deep8_amd import ops
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx, dy, dx = cfg
    r = rng(B + IH + OC + 5)
    x, w = nrm(r, (B, IH, IW, IC)), nrm(r, (OC, FH, FW, IC), np.sqrt(2.0 / (FH * FW * IC)))
    want = oracle_port.conv2d(x, w, cov, sy, sx, dy, dx)
    gz = nrm(r, want.shape)
    a = (cov, sy, sx, dy, dx)
    assert rel_fro(ops.conv2d(x, w, *a), want) <= FP32_TOL
    assert rel_fro(ops.conv2d_grad_x(x, w, gz, *a), oracle_port.conv2d_grad_x(x, w, gz, *a)) <= FP32_TOL
    assert rel_fro(ops.conv2d_grad_y(x, w, gz, *a), oracle_port.conv2d_grad_y(x, w, gz, *a)) <= FP32_TOL
    xh, wh, gzh = h(x), h(w), h(gz)
    assert rel_fro(f(ops.conv2d(xh, wh, *a)), oracle_port.conv2d(f(xh), f(wh), *a)) <= FP16_TOL
    assert rel_fro(f(ops.conv2d_grad_x(xh, wh, gzh, *a)),
                   oracle_port.conv2d_grad_x(f(xh), f(wh), f(gzh), *a)) <= FP16_TOL
    assert rel_fro(f(ops.conv2d_grad_y(xh, wh, gzh, *a)),
                   oracle_port.conv2d_grad_y(f(xh), f(wh), f(gzh), *a)) <= FP16_TOL


@pytest.mark.parametrize("cfg", DECONV)
def test_deconv2d_integer_exact(oracle_port, cfg):
    from deep8_amd import ops
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx = cfg
    r = rng(B + IH + OC + 9)
    x, w = ints(r, (B, IH, IW, IC)), ints(r, (OC, FH, FW, IC))
    want = oracle_port.deconv2d(x, w, cov, sy, sx)
    got = ops.deconv2d(x, w, cov, sy, sx)
    assert got.shape == want.shape and np.array_equal(got, want)
    gz = ints(r, want.shape, 10)
    gx0, gw0 = ints(r, x.shape), ints(r, w.shape)
    assert np.array_equal(ops.deconv2d_grad_x(x, w, gz, cov, sy, sx, gx0),
                          oracle_port.deconv2d_grad_x(x, w, gz, cov, sy, sx, gx0))
    assert np.array_equal(ops.deconv2d_grad_y(x, w, gz, cov, sy, sx, gw0),
                          oracle_port.deconv2d_grad_y(x, w, gz, cov, sy, sx, gw0))


@pytest.mark.parametrize("cfg", DECONV)
def test_deconv2d_real_tolerance(oracle_port, cfg):
    from deep8_amd import ops
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx = cfg
    r = rng(B + IH + OC + 13)
    x, w = nrm(r, (B, IH, IW, IC)), nrm(r, (OC, FH, FW, IC), np.sqrt(2.0 / (FH * FW * IC)))
    a = (cov, sy, sx)
    want = oracle_port.deconv2d(x, w, *a)
    gz = nrm(r, want.shape)
    assert rel_fro(ops.deconv2d(x, w, *a), want) <= FP32_TOL
    assert rel_fro(ops.deconv2d_grad_x(x, w, gz, *a), oracle_port.deconv2d_grad_x(x, w, gz, *a)) <= FP32_TOL
    assert rel_fro(ops.deconv2d_grad_y(x, w, gz, *a), oracle_port.deconv2d_grad_y(x, w, gz, *a)) <= FP32_TOL
    xh, wh, gzh = h(x), h(w), h(gz)
    assert rel_fro(f(ops.deconv2d(xh, wh, *a)), oracle_port.deconv2d(f(xh), f(wh), *a)) <= FP16_TOL
    assert rel_fro(f(ops.deconv2d_grad_x(xh, wh, gzh, *a)),
                   oracle_port.deconv2d_grad_x(f(xh), f(wh), f(gzh), *a)) <= FP16_TOL
    assert rel_fro(f(ops.deconv2d_grad_y(xh, wh, gzh, *a)),
                   oracle_port.deconv2d_grad_y(f(xh), f(wh), f(gzh), *a)) <= FP16_TOL
