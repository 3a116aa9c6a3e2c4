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
    (2, 14, 14, 32, 24, 3, 3, True, 1, 1, 1, 1),    # same padding like benchmark configuration 4
    (1, 10, 10, 3, 5, 2, 2, True, 3, 3, 1, 1),      # stride > filter: holes in col2im
]
# (B, IH, IW, IC, OC, FH, FW, covered, sy, sx)
DECONV = [
    (2, 8, 8, 64, 3, 4, 4, False, 2, 2),    # few output channels (an RGB output)
    (2, 10, 10, 128, 1, 3, 3, True, 1, 1),
    (2, 8, 8, 16, 8, 4, 4, False, 3, 3),    # DeConv2dTest forwardCPU geometry (smaller)
    (2, 8, 8, 16, 8, 4, 4, True, 3, 3),     # backwardCPU geometry
    (2, 7, 7, 8, 16, 4, 4, False, 2, 2),    # benchmark configuration 5 family -> 2*7+2
    (2, 7, 7, 8, 16, 4, 4, True, 2, 2),
    (1, 5, 6, 3, 5, 3, 3, False, 1, 1),
    (2, 6, 5, 4, 3, 3, 2, True, 2, 2),
    (1, 4, 4, 2, 2, 2, 2, False, 3, 3),     # stride > filter
    (2, 8, 8, 64, 64, 4, 4, False, 2, 2),   # wide enough for the tiled GEMMs and the implicit dX
    (2, 7, 7, 128, 32, 3, 3, True, 2, 2),
    (1, 12, 12, 72, 64, 4, 4, False, 3, 3),
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


# shapes for the gather maps' staged kernels: channel counts that move in 16-byte pieces, the filters the im2col kernel
# with the in-register block transpose is built for (4 x 4, 3 x 3, 2 x 2) at strides 1, 2, 3, a 5 x 3 filter for the
# kernel that walks filter windows, rows that are not a multiple of the workgroup, pads on and off
DECONV_MAPS = [
    (2, 6, 6, 16, 16, 2, 2, False, 2, 2),
    (2, 9, 7, 8, 24, 3, 3, True, 2, 2),
    (1, 10, 10, 8, 40, 4, 4, False, 1, 1),
    (2, 5, 9, 8, 8, 4, 4, True, 3, 3),
    (3, 7, 5, 8, 72, 3, 3, False, 1, 1),
    (1, 6, 6, 8, 16, 5, 3, False, 2, 1),
    (2, 6, 7, 8, 16, 4, 2, False, 2, 2),
    (2, 28, 28, 16, 64, 4, 4, False, 2, 2),
    (1, 3, 33, 8, 128, 2, 2, True, 2, 2),
]


@pytest.mark.parametrize("cfg", DECONV + DECONV_MAPS)
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
    # the overwrite forms ignore what the destination held
    assert np.array_equal(ops.conv2d_grad_x(x, w, gz, cov, sy, sx, dy, dx, gx0 - 500, overwrite=True),
                          oracle_port.conv2d_grad_x(x, w, gz, cov, sy, sx, dy, dx))
    assert np.array_equal(ops.conv2d_grad_y(x, w, gz, cov, sy, sx, dy, dx, gw0 - 500, overwrite=True),
                          oracle_port.conv2d_grad_y(x, w, gz, cov, sy, sx, dy, dx))


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
    assert np.array_equal(ops.deconv2d_grad_x(x, w, gz, cov, sy, sx, gx0 - 500, overwrite=True),
                          oracle_port.deconv2d_grad_x(x, w, gz, cov, sy, sx))
    assert np.array_equal(ops.deconv2d_grad_y(x, w, gz, cov, sy, sx, gw0 - 500, overwrite=True),
                          oracle_port.deconv2d_grad_y(x, w, gz, cov, sy, sx))


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


def test_config4_full_size_properties(oracle_port):
    """benchmark configuration 4 (Conv2d fp32, B32 56x56x64, 3x3x64 -> 64, same padding) at full size:
    two sampled images against the oracle (forward and dX are independent per image), dW through
    its additivity over the batch, and the adjoint identity <z, dz> == <x, dx> == <w, dw>."""
    from deep8_amd import ops
    r = rng(44)
    B = 32
    x, w = nrm(r, (B, 56, 56, 64)), nrm(r, (64, 3, 3, 64), np.sqrt(2.0 / 576))
    gz = nrm(r, (B, 56, 56, 64))
    a = (True, 1, 1, 1, 1)
    z, gx, gw = ops.conv2d(x, w, *a), ops.conv2d_grad_x(x, w, gz, *a), ops.conv2d_grad_y(x, w, gz, *a)
    assert z.shape == (B, 56, 56, 64)
    pick = [3, 30]
    assert rel_fro(z[pick], oracle_port.conv2d(x[pick], w, *a)) <= FP32_TOL
    assert rel_fro(gx[pick], oracle_port.conv2d_grad_x(x[pick], w, gz[pick], *a)) <= FP32_TOL
    halves = ops.conv2d_grad_y(x[:16], w, gz[:16], *a) + ops.conv2d_grad_y(x[16:], w, gz[16:], *a)
    assert rel_fro(gw, halves) <= FP32_TOL
    assert rel_fro(ops.conv2d_grad_y(x[pick], w, gz[pick], *a), oracle_port.conv2d_grad_y(x[pick], w, gz[pick], *a)) <= FP32_TOL
    ip = lambda u, v: float(np.sum(u.astype(np.float64) * v.astype(np.float64)))
    t = ip(z, gz)
    assert abs(ip(x, gx) - t) <= 1e-5 * abs(t) + 1e-2 and abs(ip(w, gw) - t) <= 1e-5 * abs(t) + 1e-2


@pytest.mark.parametrize("cov", [False, True])
def test_config5_full_size_properties(oracle_port, cov):
    """benchmark configuration 5 (DeConv2d half, B16 28x28x128, 4x4 stride 2 -> 64 channels) at Deep8's two
    legal output sizes (58 when not covered, 55 when covered)."""
    from deep8_amd import ops
    r = rng(55)
    B = 16
    x, w = h(nrm(r, (B, 28, 28, 128))), h(nrm(r, (64, 4, 4, 128), np.sqrt(2.0 / 2048)))
    a = (cov, 2, 2)
    z = ops.deconv2d(x, w, *a)
    assert z.shape == (B, 58, 58, 64) if not cov else (B, 55, 55, 64)
    gz = h(nrm(r, z.shape))
    gx, gw = ops.deconv2d_grad_x(x, w, gz, *a), ops.deconv2d_grad_y(x, w, gz, *a)
    pick = [0, 9]
    xf, wf, gzf = f(x), f(w), f(gz)
    assert rel_fro(f(z[pick]), oracle_port.deconv2d(xf[pick], wf, *a)) <= FP16_TOL
    assert rel_fro(f(gx[pick]), oracle_port.deconv2d_grad_x(xf[pick], wf, gzf[pick], *a)) <= FP16_TOL
    assert rel_fro(f(ops.deconv2d_grad_y(x[pick], w, gz[pick], *a)),
                   oracle_port.deconv2d_grad_y(xf[pick], wf, gzf[pick], *a)) <= FP16_TOL
    ip = lambda u, v: float(np.sum(f(u).astype(np.float64) * f(v).astype(np.float64)))
    t = ip(z, gz)
    assert abs(ip(x, gx) - t) <= 4e-3 * abs(t) + 1.0 and abs(ip(w, gw) - t) <= 4e-3 * abs(t) + 1.0


def test_config5_literal_56x56_through_explicit_pads(oracle_port):
    """The config's literal geometry (28 -> 56, PyTorch's ConvTranspose2d(k=4, s=2, p=1)) is not a
    shape Deep8's DeConv2d admits, but the kernel-level entry points take explicit pads:
    padTop = padLeft = 2 gives it.  GEMM + gather map here against torch's conv_transpose2d."""
    torch = pytest.importorskip("torch")
    from deep8_amd import ops
    r = rng(56)
    B, IH, IC, OC, FH, S, OH, P = 2, 28, 128, 64, 4, 2, 56, 2
    x, w = h(nrm(r, (B, IH, IH, IC))), h(nrm(r, (OC, FH, FH, IC), np.sqrt(2.0 / 2048)))
    zmat = ops.gemm(0, 1, x.reshape(B * IH * IH, IC), w.reshape(OC * FH * FH, IC))        # [B*IH*IW, OC*FH*FW]
    z = ops.deconv_col2im(zmat, B, IH, IH, OH, OH, OC, FH, FH, S, S, P, P)
    assert np.array_equal(f(z), oracle_port.deconv_col2im(f(zmat), B, IH, IH, OH, OH, OC, FH, FH, S, S, P, P).astype(np.float16).astype(np.float32))
    tx = torch.tensor(f(x), dtype=torch.float64).permute(0, 3, 1, 2)
    wt = torch.flip(torch.tensor(f(w), dtype=torch.float64), (1, 2)).permute(3, 0, 1, 2)
    tz = torch.nn.functional.conv_transpose2d(tx, wt, stride=S, padding=FH - 1 - P)
    assert tuple(tz.shape) == (B, OC, OH, OH)
    assert rel_fro(f(z), tz.permute(0, 2, 3, 1).numpy()) <= FP16_TOL
    # and the gradient-side gather with the same pads is the exact transpose of the forward one
    dz = h(ints(r, (B, OH, OH, OC), 4))
    dzmat = ops.deconv_im2col(dz, IH, IH, FH, FH, S, S, P, P)
    assert np.array_equal(f(dzmat), oracle_port.deconv_im2col(f(dz), IH, IH, FH, FH, S, S, P, P))
    zi = h(ints(r, zmat.shape, 4))
    lhs = float(np.sum(f(dzmat).astype(np.float64) * f(zi)))
    rhs = float(np.sum(f(dz).astype(np.float64) * f(ops.deconv_col2im(zi, B, IH, IH, OH, OH, OC, FH, FH, S, S, P, P))))
    assert lhs == rhs


# Shapes whose patch matrix is read by the GEMM's tile loader straight from the image (channel
# counts that are multiples of the K step; 64-wide or wider outputs).  (cfg, passes expected implicit
# for fp32, for half)
IMPLICIT = [
    ((2, 16, 16, 64, 64, 3, 3, True, 1, 1, 1, 1), (0, 1, 2), (0, 1, 2)),
    ((2, 16, 16, 64, 128, 3, 3, False, 1, 1, 1, 1), (0, 1), (0, 1)),       # 392 patch rows: ragged tiles, explicit dW
    ((4, 16, 16, 32, 64, 3, 3, True, 2, 2, 1, 1), (0, 1, 2), (1, 2)),      # stride 2: dX by residue classes of input pixels (32 channels wide)
    ((2, 20, 12, 64, 96, 5, 3, True, 1, 1, 2, 2), (0, 1, 2), (0,)),       # dilation, 5x3 filter, non-square image
    ((8, 8, 8, 64, 192, 2, 2, False, 1, 1, 1, 1), (0, 1), (0, 1)),
    ((1, 16, 16, 128, 64, 3, 3, True, 1, 1, 1, 1), (0, 1, 2), (0, 1, 2)),
]


@pytest.mark.parametrize("IC,FH,FW,dil", [(4, 7, 7, 1), (8, 5, 5, 1), (12, 5, 3, 2), (20, 3, 3, 1), (40, 2, 2, 1), (96, 3, 3, 1)])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_conv2d_filter_gradient_with_few_input_channels(oracle_port, monkeypatch, IC, FH, FW, dil, dtype):
    """The filter gradient's patch loader where one 32-column pass of a tile spans several taps (fewer than 32
    input channels) or straddles a tap's end (40, 96): bit for bit against the oracle on integers, accumulate and
    overwrite forms, on the route that stages nothing."""
    from deep8_amd import capi, ops
    lib = capi.init()
    B, IH, IW, OC = 2, 16, 16, 64
    a = (True, 1, 1, dil, dil)
    OH, OW, _, _ = ops.conv2d_geometry(IH, IW, FH, FW, *a)
    if IC % (16 // np.dtype(dtype).itemsize) == 0:  # the channels of a tap move in 16-byte pieces
        q = lambda: lib.d8_conv2d_scratch_bytes(capi.dtype_id(np.dtype(dtype)), 2, B, IH, IW, IC, OC, FH, FW, 1, 1, 1, dil, dil)
        monkeypatch.setenv("D8_CONV_EXPLICIT", "1")
        explicit = q()
        monkeypatch.delenv("D8_CONV_EXPLICIT")
        assert q() < explicit, (q(), explicit)
    r = rng(IC + FH)
    c = (lambda v: h(v)) if dtype == np.float16 else (lambda v: v)
    hi = 3 if dtype == np.float16 else 20
    x, w, gz = ints(r, (B, IH, IW, IC), hi), ints(r, (OC, FH, FW, IC), hi), ints(r, (B, OH, OW, OC), hi)
    if dtype == np.float16:
        x, gz = x * (r.random(x.shape) < 0.3), gz * (r.random(gz.shape) < 0.1)
    want = oracle_port.conv2d_grad_y(x, w, gz, *a, w)
    assert dtype == np.float32 or np.abs(want).max() < 2048
    assert np.array_equal(f(ops.conv2d_grad_y(c(x), c(w), c(gz), *a, c(w))), want)
    assert np.array_equal(f(ops.conv2d_grad_y(c(x), c(w), c(gz), *a, c(w), overwrite=True)), want - w)


@pytest.mark.parametrize("cfg,imp32,imp16", IMPLICIT)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_conv2d_implicit_route(oracle_port, monkeypatch, cfg, imp32, imp16, dtype):
    """The implicit route against the oracle (integers bit-exact, reals within tolerance) and
    against the im2col route forced through the same entry points."""
    from deep8_amd import capi, ops
    lib = capi.init()
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx, dy, dx = cfg
    a = (cov, sy, sx, dy, dx)
    OH, OW, _, _ = ops.conv2d_geometry(IH, IW, FH, FW, *a)
    for which in range(3):  # the implicit route asks for a different scratch size than the im2col route
        q = lambda: lib.d8_conv2d_scratch_bytes(capi.dtype_id(np.dtype(dtype)), which, B, IH, IW, IC, OC, FH, FW, int(cov), sy, sx, dy, dx)
        monkeypatch.setenv("D8_CONV_EXPLICIT", "1")
        explicit = q()
        assert explicit >= B * OH * OW * FH * FW * IC * np.dtype(dtype).itemsize
        monkeypatch.delenv("D8_CONV_EXPLICIT")
        assert (q() != explicit) == (which in (imp32 if dtype == np.float32 else imp16)), (which, q(), explicit)
    r = rng(B + IH + OC + 77)
    c = (lambda v: h(v)) if dtype == np.float16 else (lambda v: v)
    hi = 3 if dtype == np.float16 else 20
    tol = FP16_TOL if dtype == np.float16 else FP32_TOL
    # integers, thinned for half so that every sum stays exact
    x, w = ints(r, (B, IH, IW, IC), hi), ints(r, (OC, FH, FW, IC), hi)
    gz = ints(r, (B, OH, OW, OC), hi)
    if dtype == np.float16:
        x, w, gz = x * (r.random(x.shape) < 0.3), w * (r.random(w.shape) < 0.3), gz * (r.random(gz.shape) < 0.1)
    want = (oracle_port.conv2d(x, w, *a), oracle_port.conv2d_grad_x(x, w, gz, *a, x), oracle_port.conv2d_grad_y(x, w, gz, *a, w))
    assert dtype == np.float32 or max(np.abs(t).max() for t in want) < 2048
    got = (ops.conv2d(c(x), c(w), *a), ops.conv2d_grad_x(c(x), c(w), c(gz), *a, c(x)), ops.conv2d_grad_y(c(x), c(w), c(gz), *a, c(w)))
    for g_, w_ in zip(got, want):
        assert np.array_equal(f(g_), w_)
    assert np.array_equal(f(ops.conv2d_grad_x(c(x), c(w), c(gz), *a, c(x), overwrite=True)), want[1] - x)
    assert np.array_equal(f(ops.conv2d_grad_y(c(x), c(w), c(gz), *a, c(w), overwrite=True)), want[2] - w)
    # reals: both routes within tolerance of the oracle
    x, w = c(nrm(r, (B, IH, IW, IC))), c(nrm(r, (OC, FH, FW, IC), np.sqrt(2.0 / (FH * FW * IC))))
    gz = c(nrm(r, (B, OH, OW, OC)))
    want = (oracle_port.conv2d(f(x), f(w), *a), oracle_port.conv2d_grad_x(f(x), f(w), f(gz), *a), oracle_port.conv2d_grad_y(f(x), f(w), f(gz), *a))
    for route in ("implicit", "explicit"):
        if route == "explicit":
            monkeypatch.setenv("D8_CONV_EXPLICIT", "1")
        got = (ops.conv2d(x, w, *a), ops.conv2d_grad_x(x, w, gz, *a), ops.conv2d_grad_y(x, w, gz, *a))
        for k, (g_, w_) in enumerate(zip(got, want)):
            assert rel_fro(f(g_), w_) <= tol, (route, k)


# ---- DeConv2d forward by residue classes of output pixels (no interim matrix): shapes that take it (channel
# counts that are multiples of the K step, 64 or more output channels, every class tile-sized, a tap for
# every class) and, last, shapes that must fall back.  (B, IH, IW, IC, OC, FH, FW, covered, sy, sx), fp32?, half?
DECONV_CLASSES = [
    ((2, 9, 8, 64, 64, 4, 4, False, 2, 2), True, True),
    ((3, 9, 8, 64, 96, 4, 4, True, 2, 2), True, True),      # covered: pads shift the classes' taps
    ((2, 12, 11, 64, 64, 4, 4, False, 3, 3), True, True),   # stride 3: classes with 2x2, 2x1, 1x2 and 1x1 taps
    ((2, 12, 11, 64, 64, 4, 4, True, 3, 3), True, True),
    ((2, 10, 10, 128, 128, 3, 3, True, 2, 2), True, True),  # 3x3 stride 2: 2 or 1 taps per axis; 128-wide tiles
    ((2, 9, 9, 64, 64, 5, 3, False, 2, 1), True, True),     # different strides per axis, 5x3 filter
    ((3, 8, 8, 32, 64, 2, 2, False, 2, 2), True, False),    # 32 channels: one fp32 K step, too few for half
    ((1, 16, 16, 64, 64, 4, 4, False, 1, 1), True, True),   # stride 1: a single class with all 16 taps
    ((2, 16, 16, 64, 72, 4, 4, True, 4, 4), True, True),    # 16 classes of one tap each
    ((2, 9, 8, 64, 64, 2, 2, False, 3, 3), True, True),     # stride > filter: some classes have no tap, their pixels stay zero
    ((2, 9, 9, 64, 64, 1, 1, True, 2, 2), True, True),      # a 1 x 1 filter at stride 2: one class in four has a tap
    ((1, 6, 6, 64, 64, 4, 4, False, 2, 2), False, False),   # classes smaller than a tile
]


@pytest.mark.parametrize("cfg,imp32,imp16", DECONV_CLASSES)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_deconv2d_forward_by_classes(oracle_port, monkeypatch, cfg, imp32, imp16, dtype):
    from deep8_amd import capi, ops
    from deep8_amd.capi import DeviceArray, check
    lib = capi.init()
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx = cfg
    dt = capi.dtype_id(np.dtype(dtype))
    OH, OW, _, _ = ops.deconv2d_geometry(IH, IW, FH, FW, cov, sy, sx)
    nb = lib.d8_deconv2d_scratch_bytes(dt, 0, B, IH, IW, IC, OC, FH, FW, int(cov), sy, sx)
    assert (nb == 0) == (imp32 if dtype == np.float32 else imp16)
    monkeypatch.setenv("D8_CONV_EXPLICIT", "1")
    assert lib.d8_deconv2d_scratch_bytes(dt, 0, B, IH, IW, IC, OC, FH, FW, int(cov), sy, sx) >= B * IH * IW * FH * FW * OC * np.dtype(dtype).itemsize
    monkeypatch.delenv("D8_CONV_EXPLICIT")

    def forward(x, w):  # into an output pre-filled with NaN: every pixel must be written
        dx_, dw_ = DeviceArray.from_numpy(x), DeviceArray.from_numpy(w)
        dz_ = DeviceArray.from_numpy(np.full((B, OH, OW, OC), np.nan, dtype))
        ws = DeviceArray((max(nb, 16),), np.uint8)
        check(lib.d8_deconv2d(dt, dx_.ptr, B, IH, IW, IC, dw_.ptr, OC, FH, FW, dz_.ptr, int(cov), sy, sx, ws.ptr if nb else None, nb, None))
        return dz_.numpy()

    r = rng(B + IH + OC + 91)
    c = (lambda v: h(v)) if dtype == np.float16 else (lambda v: v)
    hi = 3 if dtype == np.float16 else 20
    x, w = ints(r, (B, IH, IW, IC), hi), ints(r, (OC, FH, FW, IC), hi)
    if dtype == np.float16:
        x, w = x * (r.random(x.shape) < 0.3), w * (r.random(w.shape) < 0.3)
    want = oracle_port.deconv2d(x, w, cov, sy, sx)
    assert dtype == np.float32 or np.abs(want).max() < 2048
    got = forward(c(x), c(w))
    assert got.shape == want.shape and np.array_equal(f(got), want)
    x, w = c(nrm(r, (B, IH, IW, IC))), c(nrm(r, (OC, FH, FW, IC), np.sqrt(2.0 / (FH * FW * IC))))
    want = oracle_port.deconv2d(f(x), f(w), cov, sy, sx)
    tol = FP16_TOL if dtype == np.float16 else FP32_TOL
    assert rel_fro(f(forward(x, w)), want) <= tol
    monkeypatch.setenv("D8_CONV_EXPLICIT", "1")
    assert rel_fro(f(ops.deconv2d(x, w, cov, sy, sx)), want) <= tol


# ---- DeConv2d filter gradient without the interim matrix (the patch matrix of dz read by the tile loader, the
# result stored transposed per tap): needs B*IH*IW a multiple of the K step and 64 or more input channels
DECONV_DW = [
    ((2, 8, 8, 64, 64, 4, 4, False, 2, 2), True, True),
    ((4, 8, 8, 64, 96, 4, 4, True, 2, 2), True, True),
    ((2, 8, 8, 128, 64, 3, 3, True, 2, 2), True, True),
    ((1, 16, 8, 64, 64, 4, 4, False, 3, 3), True, True),
    ((2, 8, 8, 64, 64, 5, 3, False, 2, 1), True, True),
    ((2, 16, 16, 64, 64, 2, 2, False, 3, 3), True, True),   # stride > filter
    ((1, 8, 4, 64, 64, 4, 4, False, 2, 2), True, False),    # 32 input pixels: one fp32 K step
    ((2, 7, 7, 64, 64, 4, 4, False, 2, 2), False, False),   # 98 input pixels: not a multiple of the K step
]


@pytest.mark.parametrize("cfg,imp32,imp16", DECONV_DW)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_deconv2d_filter_gradient_without_interim(oracle_port, monkeypatch, cfg, imp32, imp16, dtype):
    from deep8_amd import capi, ops
    lib = capi.init()
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx = cfg
    a = (cov, sy, sx)
    dt = capi.dtype_id(np.dtype(dtype))
    OH, OW, _, _ = ops.deconv2d_geometry(IH, IW, FH, FW, *a)
    q = lambda: lib.d8_deconv2d_scratch_bytes(dt, 2, B, IH, IW, IC, OC, FH, FW, int(cov), sy, sx)
    interim = B * IH * IW * FH * FW * OC * np.dtype(dtype).itemsize
    monkeypatch.setenv("D8_CONV_EXPLICIT", "1")
    assert q() >= interim
    monkeypatch.delenv("D8_CONV_EXPLICIT")
    expect = imp32 if dtype == np.float32 else imp16
    assert (q() < interim) == expect or (not expect and q() >= interim)
    r = rng(B + IH + OC + 93)
    c = (lambda v: h(v)) if dtype == np.float16 else (lambda v: v)
    hi = 3 if dtype == np.float16 else 20
    x, w, gz = ints(r, (B, IH, IW, IC), hi), ints(r, (OC, FH, FW, IC), hi), ints(r, (B, OH, OW, OC), hi)
    if dtype == np.float16:
        x, gz = x * (r.random(x.shape) < 0.3), gz * (r.random(gz.shape) < 0.2)
    want = oracle_port.deconv2d_grad_y(x, w, gz, *a, w)
    assert dtype == np.float32 or np.abs(want).max() < 2048
    assert np.array_equal(f(ops.deconv2d_grad_y(c(x), c(w), c(gz), *a, c(w))), want)
    assert np.array_equal(f(ops.deconv2d_grad_y(c(x), c(w), c(gz), *a, c(w) - 2, overwrite=True)), want - w)
    x, w, gz = c(nrm(r, (B, IH, IW, IC))), c(nrm(r, (OC, FH, FW, IC))), c(nrm(r, (B, OH, OW, OC)))
    want = oracle_port.deconv2d_grad_y(f(x), f(w), f(gz), *a)
    tol = FP16_TOL if dtype == np.float16 else FP32_TOL
    assert rel_fro(f(ops.deconv2d_grad_y(x, w, gz, *a)), want) <= tol
    monkeypatch.setenv("D8_CONV_EXPLICIT", "1")
    assert rel_fro(f(ops.deconv2d_grad_y(x, w, gz, *a)), want) <= tol


# ---- Conv2d gradient of x for a stride above 1, by residue classes of input pixels (no patch matrix)
CONV_DX_CLASSES = [
    ((2, 16, 16, 64, 64, 3, 3, True, 2, 2, 1, 1), True),
    ((3, 17, 15, 64, 128, 3, 3, False, 2, 2, 1, 1), True),   # not covered: border pixels that no patch reaches
    ((4, 18, 18, 128, 64, 4, 4, True, 3, 3, 1, 1), True),
    ((2, 16, 16, 64, 64, 5, 3, True, 2, 1, 1, 1), True),     # stride 2 down, 1 across
    ((4, 16, 16, 64, 64, 2, 2, False, 2, 2, 1, 1), True),    # filter == stride: one tap per class
    ((2, 16, 16, 64, 64, 3, 3, True, 2, 2, 2, 2), True),     # dilation 2 at stride 2: only even rows and columns of x are read at all
    ((2, 16, 16, 64, 64, 1, 1, True, 2, 2, 1, 1), True),     # filter smaller than the stride: classes without a tap
    ((2, 32, 32, 64, 32, 4, 4, True, 2, 2, 2, 2), True),     # Conv2dTest forwardCPU_float's geometry (fp32: 32 output channels are one K step)
    ((2, 18, 17, 64, 64, 3, 3, True, 2, 2, 3, 3), True),     # dilation 3 at stride 2: every class has taps, two filter rows apart
    ((3, 25, 25, 64, 64, 3, 3, False, 3, 3, 2, 2), True),    # stride 3, dilation 2, not covered
    ((2, 40, 20, 64, 64, 5, 5, True, 4, 2, 2, 3), True),     # stride 4 x 2, dilation 2 x 3: a common factor down, none across
    ((2, 24, 24, 64, 64, 3, 3, True, 6, 6, 1, 1), False),    # 36 classes: more than a launch takes
]


@pytest.mark.parametrize("cfg,classes", CONV_DX_CLASSES)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_conv2d_strided_gradient_of_x(oracle_port, monkeypatch, cfg, classes, dtype):
    from deep8_amd import capi, ops
    lib = capi.init()
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx, dy, dx = cfg
    a = (cov, sy, sx, dy, dx)
    OH, OW, _, _ = ops.conv2d_geometry(IH, IW, FH, FW, *a)
    nb = lib.d8_conv2d_scratch_bytes(capi.dtype_id(np.dtype(dtype)), 1, B, IH, IW, IC, OC, FH, FW, int(cov), sy, sx, dy, dx)
    assert (nb == 0) == (classes and OC % (64 if dtype == np.float16 else 32) == 0)  # (a K step stays inside one tap)
    r = rng(B + IH + OC + 95)
    c = (lambda v: h(v)) if dtype == np.float16 else (lambda v: v)
    hi = 3 if dtype == np.float16 else 20
    x, w, gz = ints(r, (B, IH, IW, IC), hi), ints(r, (OC, FH, FW, IC), hi), ints(r, (B, OH, OW, OC), hi)
    if dtype == np.float16:
        w, gz = w * (r.random(w.shape) < 0.3), gz * (r.random(gz.shape) < 0.3)
    want = oracle_port.conv2d_grad_x(x, w, gz, *a, x)
    assert dtype == np.float32 or np.abs(want).max() < 2048
    assert np.array_equal(f(ops.conv2d_grad_x(c(x), c(w), c(gz), *a, c(x))), want)
    nan = np.full(x.shape, np.nan, dtype)  # the overwrite form must write every pixel, reached by a patch or not
    assert np.array_equal(f(ops.conv2d_grad_x(c(x), c(w), c(gz), *a, nan, overwrite=True)), want - x)
    x, w, gz = c(nrm(r, (B, IH, IW, IC))), c(nrm(r, (OC, FH, FW, IC), np.sqrt(2.0 / (FH * FW * IC)))), c(nrm(r, (B, OH, OW, OC)))
    want = oracle_port.conv2d_grad_x(f(x), f(w), f(gz), *a)
    tol = FP16_TOL if dtype == np.float16 else FP32_TOL
    assert rel_fro(f(ops.conv2d_grad_x(x, w, gz, *a)), want) <= tol
    monkeypatch.setenv("D8_CONV_EXPLICIT", "1")
    assert rel_fro(f(ops.conv2d_grad_x(x, w, gz, *a)), want) <= tol


# first layers: a patch row of 25, 27, 54, 147 ... elements cannot be moved in 16-byte pieces; with an output channel
# count that can, the operator pads the patch matrix's rows (and a copy of the filter) to the next multiple
FIRST_LAYERS = [(2, 12, 12, 3, 8, 3, 3, True, 1, 1, 1, 1), (2, 16, 16, 1, 16, 5, 5, True, 1, 1, 1, 1),
                (1, 20, 20, 3, 64, 7, 7, True, 2, 2, 1, 1), (1, 12, 12, 3, 8, 3, 3, False, 1, 1, 2, 2),
                (2, 9, 11, 6, 24, 3, 3, True, 2, 1, 1, 1), (3, 28, 28, 1, 32, 5, 5, False, 1, 1, 1, 1),
                (16, 32, 32, 3, 32, 3, 3, True, 1, 1, 1, 1), (2, 10, 10, 3, 8, 5, 5, True, 1, 1, 1, 1),
                (1, 14, 14, 3, 16, 6, 6, True, 1, 1, 1, 1), (2, 13, 9, 5, 40, 4, 4, False, 1, 2, 1, 1)]


# last layers: few output channels (an RGB or a one-channel output); the forward pass still reads its patch rows
# straight from the image, the filter's rows past the last one arriving as zeros
LAST_LAYERS = [(2, 16, 16, 64, 3, 3, 3, True, 1, 1, 1, 1), (2, 12, 12, 32, 1, 1, 1, True, 1, 1, 1, 1),
               (1, 16, 16, 64, 5, 3, 3, False, 1, 1, 1, 1), (2, 14, 14, 128, 3, 5, 5, True, 1, 1, 1, 1),
               (4, 20, 20, 64, 16, 3, 3, True, 2, 2, 1, 1), (2, 16, 16, 16, 64, 3, 3, True, 1, 1, 1, 1)]


@pytest.mark.parametrize("cfg", FIRST_LAYERS + LAST_LAYERS)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_conv2d_first_layers_padded_patch_rows(oracle_port, cfg, dtype):
    from deep8_amd import ops
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx, dy, dx = cfg
    a = (cov, sy, sx, dy, dx)
    r = rng(B + IH + OC + 31)
    half = dtype == np.float16
    c = h if half else (lambda t: t)
    hi = 2 if half else 20
    thin = (lambda t, p: t * (r.random(t.shape) < p)) if half else (lambda t, p: t)
    x, w = thin(ints(r, (B, IH, IW, IC), hi), 0.5), thin(ints(r, (OC, FH, FW, IC), hi), 0.5)
    want = oracle_port.conv2d(x, w, *a)
    gz = thin(ints(r, want.shape, hi), 0.1 if half else 1.0)
    gx0, gw0 = ints(r, x.shape, hi), ints(r, w.shape, hi)
    wants = [want, oracle_port.conv2d_grad_x(x, w, gz, *a, gx0), oracle_port.conv2d_grad_y(x, w, gz, *a, gw0),
             oracle_port.conv2d_grad_x(x, w, gz, *a), oracle_port.conv2d_grad_y(x, w, gz, *a)]
    assert not half or max(np.abs(t).max() for t in wants) < 2048
    nan = lambda t: np.full(t.shape, np.nan, dtype)
    gots = [ops.conv2d(c(x), c(w), *a), ops.conv2d_grad_x(c(x), c(w), c(gz), *a, c(gx0)), ops.conv2d_grad_y(c(x), c(w), c(gz), *a, c(gw0)),
            ops.conv2d_grad_x(c(x), c(w), c(gz), *a, nan(x), overwrite=True), ops.conv2d_grad_y(c(x), c(w), c(gz), *a, nan(w), overwrite=True)]
    for k, (g, t) in enumerate(zip(gots, wants)):
        assert np.array_equal(f(g), t), (cfg, k)
    # reals within the tolerance
    xr, wr = c(nrm(r, x.shape)), c(nrm(r, w.shape, np.sqrt(2.0 / (FH * FW * IC))))
    gzr = c(nrm(r, want.shape))
    tol = FP16_TOL if half else FP32_TOL
    assert rel_fro(f(ops.conv2d(xr, wr, *a)), oracle_port.conv2d(f(xr), f(wr), *a)) <= tol
    assert rel_fro(f(ops.conv2d_grad_x(xr, wr, gzr, *a)), oracle_port.conv2d_grad_x(f(xr), f(wr), f(gzr), *a)) <= tol
    assert rel_fro(f(ops.conv2d_grad_y(xr, wr, gzr, *a)), oracle_port.conv2d_grad_y(f(xr), f(wr), f(gzr), *a)) <= tol


# ---- DeConv2d at an explicit geometry (d8_deconv2d*_ex) ------------------------------------------------------------
def _torch_deconv(x, w, gz, S, P, OH):
    """torch's conv_transpose2d and its autograd gradients in Deep8's layout and filter convention (flipped kernel,
    padding = F - 1 - padTop), float64"""
    import torch
    F = w.shape[1]
    tx = torch.tensor(f(x), dtype=torch.float64).permute(0, 3, 1, 2).clone().requires_grad_(True)
    tw = torch.tensor(f(w), dtype=torch.float64).requires_grad_(True)
    wt = torch.flip(tw, (1, 2)).permute(3, 0, 1, 2)
    tz = torch.nn.functional.conv_transpose2d(tx, wt, stride=S, padding=F - 1 - P)
    assert tuple(tz.shape[2:]) == (OH, OH)
    tz.backward(torch.tensor(f(gz), dtype=torch.float64).permute(0, 3, 1, 2))
    return tz.detach().permute(0, 2, 3, 1).numpy(), tx.grad.permute(0, 2, 3, 1).numpy(), tw.grad.numpy()


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_config5_as_written_at_operator_level(dtype):
    """Benchmark configuration 5 literally: B16 28x28x128 -> 56x56x64, 4x4, stride 2, PyTorch's pad 1 (padTop = 2 here),
    forward and both gradients through d8_deconv2d*_ex at full size, against torch's conv_transpose2d in float64."""
    pytest.importorskip("torch")
    from deep8_amd import ops
    r = rng(556)
    B, IH, IC, OC, F, S, OH, P = 16, 28, 128, 64, 4, 2, 56, 2
    c = (lambda a: h(a)) if dtype == np.float16 else (lambda a: a)
    tol = FP16_TOL if dtype == np.float16 else FP32_TOL
    x, w = c(nrm(r, (B, IH, IH, IC))), c(nrm(r, (OC, F, F, IC), np.sqrt(2.0 / 2048)))
    gz = c(nrm(r, (B, OH, OH, OC)))
    tz, tgx, tgw = _torch_deconv(x, w, gz, S, P, OH)
    z = ops.deconv2d_ex(0, x, w, None, OH, OH, P, P, S, S)
    assert z.shape == (B, OH, OH, OC) and rel_fro(f(z), tz) <= tol
    assert rel_fro(f(ops.deconv2d_ex(1, x, w, gz, OH, OH, P, P, S, S)), tgx) <= tol
    assert rel_fro(f(ops.deconv2d_ex(2, x, w, gz, OH, OH, P, P, S, S)), tgw) <= tol
    # accumulate and overwrite forms
    junk = c(nrm(r, x.shape))
    got = ops.deconv2d_ex(1, x, w, gz, OH, OH, P, P, S, S, acc=junk, overwrite=True)
    assert rel_fro(f(got), tgx) <= tol
    got = ops.deconv2d_ex(1, x, w, gz, OH, OH, P, P, S, S, acc=junk)
    assert rel_fro(f(got), tgx + f(junk)) <= tol


@pytest.mark.parametrize("cfg", [
    # B, IH, IC, OC, F, S, OH, P  (square; OH and P free)
    (2, 7, 16, 8, 4, 2, 14, 2),     # k4 s2 p1 at a size that takes the im2col / col2im route
    (2, 6, 64, 64, 3, 2, 12, 1),    # ConvTranspose2d(k3, s2, p1, output_padding 1): OH = 2 IH
    (1, 5, 3, 2, 5, 3, 13, 3),
    (2, 9, 64, 64, 4, 2, 18, 2),    # implicit route
    (3, 8, 32, 64, 2, 2, 16, 1),    # filter = stride: no overlaps (p0 -> padTop = k - 1)
])
def test_deconv2d_ex_integer_exact(oracle_port, cfg):
    """Small explicit geometries, integers, bit for bit against the kernel-level route through the oracle:
    zmat = X W^T, then the oracle's deconv_col2im with the same pads; gradients via the oracle's deconv_im2col."""
    from deep8_amd import ops
    B, IH, IC, OC, F, S, OH, P = cfg
    r = rng(sum(cfg))
    x, w = ints(r, (B, IH, IH, IC), 4), ints(r, (OC, F, F, IC), 4)
    gz = ints(r, (B, OH, OH, OC), 4)
    zmat = x.reshape(-1, IC) @ w.reshape(OC * F * F, IC).T
    want_z = oracle_port.deconv_col2im(zmat, B, IH, IH, OH, OH, OC, F, F, S, S, P, P)
    dzmat = oracle_port.deconv_im2col(gz, IH, IH, F, F, S, S, P, P)
    want_gx = (dzmat @ w.reshape(OC * F * F, IC)).reshape(x.shape)
    want_gw = (dzmat.T @ x.reshape(-1, IC)).reshape(w.shape)
    for dtype in (np.float32, np.float16):
        if dtype == np.float16 and max(np.abs(want_z).max(), np.abs(want_gx).max(), np.abs(want_gw).max()) >= 2048:
            continue
        c = lambda a: a.astype(dtype)
        assert np.array_equal(f(ops.deconv2d_ex(0, c(x), c(w), None, OH, OH, P, P, S, S)), want_z)
        assert np.array_equal(f(ops.deconv2d_ex(1, c(x), c(w), c(gz), OH, OH, P, P, S, S)), want_gx)
        assert np.array_equal(f(ops.deconv2d_ex(2, c(x), c(w), c(gz), OH, OH, P, P, S, S)), want_gw)
    # Deep8's own geometry through the _ex entry points is the operator itself
    OHd, OWd, pt, pl = ops.deconv2d_geometry(IH, IH, F, F, False, S, S)
    assert np.array_equal(ops.deconv2d_ex(0, x, w, None, OHd, OWd, pt, pl, S, S), ops.deconv2d(x, w, False, S, S))


def test_conv2d_tensor_view_at_an_odd_offset(oracle_port):
    """A tensor that is not 16-byte aligned cannot be read by the tile loader: the operator takes the staged route.
    With the staged route's scratch the result is the same; with the scratch the size query names (it plans for
    aligned tensors) the call fails and says why."""
    from deep8_amd import capi
    from deep8_amd.capi import DeviceArray, check
    lib = capi.init()
    r = rng(77)
    B, IH, IC, OC, F = 2, 12, 64, 64, 3
    x, w = ints(r, (B, IH, IH, IC), 5), ints(r, (OC, F, F, IC), 5)
    gz = ints(r, (B, IH, IH, OC), 5)
    want = (oracle_port.conv2d(x, w), oracle_port.conv2d_grad_x(x, w, gz), oracle_port.conv2d_grad_y(x, w, gz))
    args = (1, 1, 1, 1, 1)
    asked = lib.d8_conv2d_scratch_bytes(capi.FLOAT32, 0, B, IH, IH, IC, OC, F, F, *args)
    assert asked < 4 * B * IH * IH * F * F * IC           # the query plans for the route that stages nothing
    small = DeviceArray((max(asked, 16),), np.uint8)
    raw = DeviceArray((x.size + 1,), np.float32)          # x lives 4 bytes into this allocation
    check(lib.d8_memcpy_h2d(raw.ptr + 4, x.ctypes.data, x.nbytes))
    dw, dgz = DeviceArray.from_numpy(w), DeviceArray.from_numpy(gz)
    z, gx_raw, gw = DeviceArray(gz.shape, np.float32), DeviceArray((x.size + 1,), np.float32, zero=True), DeviceArray(w.shape, np.float32, zero=True)
    rc = lib.d8_conv2d(capi.FLOAT32, raw.ptr + 4, B, IH, IH, IC, dw.ptr, OC, F, F, z.ptr, *args, small.ptr, asked, None)
    assert rc == 10001 and b"not 16-byte aligned" in lib.d8_last_error()
    nb = 4 * B * IH * IH * F * F * IC + (32 << 20)        # the interim matrix + room for any split workspace
    ws = DeviceArray((nb,), np.uint8)
    check(lib.d8_conv2d(capi.FLOAT32, raw.ptr + 4, B, IH, IH, IC, dw.ptr, OC, F, F, z.ptr, *args, ws.ptr, nb, None))
    assert np.array_equal(z.numpy(), want[0])
    check(lib.d8_conv2d_grad_x(capi.FLOAT32, gx_raw.ptr + 4, B, IH, IH, IC, dw.ptr, OC, F, F, dgz.ptr, *args, ws.ptr, nb, None))
    assert np.array_equal(gx_raw.numpy()[1:].reshape(x.shape), want[1])
    check(lib.d8_conv2d_grad_y(capi.FLOAT32, raw.ptr + 4, B, IH, IH, IC, gw.ptr, OC, F, F, dgz.ptr, *args, ws.ptr, nb, None))
    assert np.array_equal(gw.numpy(), want[2])


def test_conv_sizes_beyond_int_range_are_refused():
    """Pixel and patch-row counts are ints inside the library: a geometry whose products pass 2^31 - 1 is refused
    with a message (no launch), by the operators and by their scratch queries alike."""
    from deep8_amd import capi
    lib = capi.init()
    a = capi.DeviceArray((64,), np.float32, zero=True)
    big = (capi.FLOAT32, a.ptr, 40000, 300, 300, 4, a.ptr, 4, 3, 3, a.ptr)  # 3.6e9 pixels
    assert lib.d8_conv2d(*big, 1, 1, 1, 1, 1, None, 0, None) == 10001 and b"exceed" in lib.d8_last_error()
    assert lib.d8_conv2d_scratch_bytes(capi.FLOAT32, 0, 40000, 300, 300, 4, 4, 3, 3, 1, 1, 1, 1, 1) == 0
    assert lib.d8_deconv2d(*big, 0, 2, 2, None, 0, None) == 10001 and b"exceed" in lib.d8_last_error()
    # a DeConv2d whose input fits but whose output does not: 2e9 input pixels x stride 2 x 2
    assert lib.d8_deconv2d(capi.FLOAT32, a.ptr, 20000, 300, 300, 4, a.ptr, 4, 2, 2, a.ptr, 0, 2, 2, None, 0, None) == 10001
    assert b"output pixels" in lib.d8_last_error()
    assert lib.d8_deconv2d_scratch_bytes(capi.FLOAT32, 0, 20000, 300, 300, 4, 4, 2, 2, 0, 2, 2) == 0
