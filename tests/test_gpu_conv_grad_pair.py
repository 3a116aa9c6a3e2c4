"""d8_conv2d_grad_xy / d8_deconv2d_grad_xy(_ex): both gradients of a convolution from one call.  The reference runs
Conv2d::backward / DeConv2d::backward once per input (deep8/src/nodes/Conv2d.cpp:85-151,
deep8/src/nodes/DeConv2d.cpp:74-126); the call must leave bit for bit what the two separate calls leave, in every
accumulate / overwrite combination, whether the two products share a launch (small layers, both read their patch
matrices inside the GEMM) or run one after the other -- and, on integers, exactly what the oracle computes."""
import numpy as np
import pytest

from test_gpu_conv import CONV, DECONV
from util import FP16_TOL, FP32_TOL, f, h, ints, nrm, rel_fro, rng

pytestmark = pytest.mark.gpu

# Layers whose two gradient products share a launch.  Columns after the shape: whether they do in fp32; in half; whether
# in half the gradient of x runs whole only because it has company (alone it is cut into pieces whose sums are added in
# another order: equal within rounding, not bit for bit); whether they do in fp32 once the environment forces it.
# (B, IH, IW, IC, OC, FH, FW, covered, sy, sx, dy, dx)
CONV_SHARED = [
    ((2, 16, 16, 64, 64, 3, 3, True, 1, 1, 1, 1), False, True, False, True),      # dX on 128 x 64 tiles, dW on 64 x 64
    ((1, 16, 16, 128, 64, 3, 3, True, 1, 1, 1, 1), False, True, False, True),     # dX 64 x 128, dW 64 x 128
    ((4, 28, 28, 128, 128, 3, 3, True, 1, 1, 1, 1), False, True, False, True),    # dX 64 x 128 (half tiles), dW 128 x 128 in pieces
    ((8, 20, 20, 96, 64, 3, 3, False, 1, 1, 2, 2), False, True, False, True),     # dilation, not covered
    ((12, 24, 24, 32, 64, 5, 5, True, 1, 1, 1, 1), False, True, True, True),      # 32 input channels, 5 x 5
    ((16, 28, 28, 64, 64, 3, 3, True, 1, 1, 1, 1), False, True, False, False),
]
# (B, IH, IW, IC, OC, FH, FW, covered, sy, sx)
DECONV_SHARED = [
    ((2, 8, 8, 64, 64, 4, 4, False, 2, 2), False, True, False, True),
    ((2, 8, 8, 128, 64, 3, 3, True, 2, 2), False, True, False, True),
    ((16, 28, 28, 128, 64, 4, 4, False, 2, 2), True, True, False, True),          # benchmark configuration 5
    ((1, 16, 8, 64, 64, 4, 4, False, 3, 3), False, True, False, True),
    ((8, 16, 16, 64, 128, 4, 4, False, 3, 3), False, True, True, True),
    ((4, 32, 32, 64, 64, 4, 4, False, 2, 2), False, True, False, True),
]


def _row(cfg, shared_list):
    for row in shared_list:
        if row[0] == cfg:
            return row
    return (cfg, False, False, False, False)


def _expected(cfg, shared_list, dtype):
    row = _row(cfg, shared_list)
    return 4 if (dtype == np.float32 and row[1]) or (dtype == np.float16 and row[2]) else 0


def _x_matches(cfg, shared_list, dtype, got, alone):
    """bit for bit, or (half, a gradient of x that runs whole only in company) within the half tolerance"""
    if dtype == np.float16 and _row(cfg, shared_list)[3]:
        return rel_fro(f(got), f(alone)) <= FP16_TOL
    return _same(got, alone)


def _bits(a):
    return a.view({2: np.uint16, 4: np.uint32, 8: np.uint64}[a.dtype.itemsize])


def _same(a, b):
    return a.shape == b.shape and np.array_equal(_bits(a), _bits(b))


def _data(r, B, IH, IW, IC, OC, FH, FW, OH, OW, dtype):
    c = (lambda v: h(v)) if dtype == np.float16 else (lambda v: v.astype(dtype))
    x, w = c(nrm(r, (B, IH, IW, IC))), c(nrm(r, (OC, FH, FW, IC), np.sqrt(2.0 / (FH * FW * IC))))
    gz = c(nrm(r, (B, OH, OW, OC)))
    gx0, gw0 = c(nrm(r, x.shape)), c(nrm(r, w.shape))
    return x, w, gz, gx0, gw0


@pytest.mark.parametrize("cfg", CONV + [row[0] for row in CONV_SHARED])
@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.float64])
def test_conv2d_both_gradients_from_one_call(cfg, dtype):
    from deep8_amd import capi, ops
    lib = capi.init()
    B, IH, IW, IC, OC, FH, FW = cfg[:7]
    a = cfg[7:]
    OH, OW, _, _ = ops.conv2d_geometry(IH, IW, FH, FW, *a)
    x, w, gz, gx0, gw0 = _data(rng(sum(cfg[:7]) + 5), B, IH, IW, IC, OC, FH, FW, OH, OW, dtype)
    before = lib.d8_conv_grad_pair_launches()
    for ox, ow in ((False, False), (True, True), (True, False), (False, True)):
        gx, gw = ops.conv2d_grad_xy(x, w, gz, *a, gx0, gw0, ox, ow)
        assert _x_matches(cfg, CONV_SHARED, dtype, gx, ops.conv2d_grad_x(x, w, gz, *a, gx0, overwrite=ox)), (ox, ow)
        assert _same(gw, ops.conv2d_grad_y(x, w, gz, *a, gw0, overwrite=ow)), (ox, ow)
    shared = lib.d8_conv_grad_pair_launches() - before
    assert shared == _expected(cfg, CONV_SHARED, dtype), shared


@pytest.mark.parametrize("cfg", DECONV + [row[0] for row in DECONV_SHARED[1:]])
@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.float64])
def test_deconv2d_both_gradients_from_one_call(cfg, dtype):
    from deep8_amd import capi, ops
    lib = capi.init()
    B, IH, IW, IC, OC, FH, FW = cfg[:7]
    a = cfg[7:]
    OH, OW, _, _ = ops.deconv2d_geometry(IH, IW, FH, FW, *a)
    x, w, gz, gx0, gw0 = _data(rng(sum(cfg[:7]) + 6), B, IH, IW, IC, OC, FH, FW, OH, OW, dtype)
    before = lib.d8_conv_grad_pair_launches()
    for ox, ow in ((False, False), (True, True), (True, False), (False, True)):
        gx, gw = ops.deconv2d_grad_xy(x, w, gz, *a, gx0, gw0, ox, ow)
        assert _x_matches(cfg, DECONV_SHARED, dtype, gx, ops.deconv2d_grad_x(x, w, gz, *a, gx0, overwrite=ox)), (ox, ow)
        assert _same(gw, ops.deconv2d_grad_y(x, w, gz, *a, gw0, overwrite=ow)), (ox, ow)
    shared = lib.d8_conv_grad_pair_launches() - before
    assert shared == _expected(cfg, DECONV_SHARED, dtype), shared


@pytest.mark.parametrize("cfg", [row[0] for row in CONV_SHARED])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_conv2d_shared_launch_against_the_oracle(oracle_port, monkeypatch, cfg, dtype):
    """integers (thinned for half so that every sum stays exact): bit for bit; reals within tolerance; and the same
    call with the shared launch switched off gives the same bits.  In fp32 the shared launch is forced (the gradient
    of x runs whole beside the filter gradient's pieces whatever its length), so that its kernels are covered too."""
    from deep8_amd import capi, ops
    monkeypatch.setenv("D8_CONV_PAIR_STEPS", "1000000")
    before = capi.init().d8_conv_grad_pair_launches()
    B, IH, IW, IC, OC, FH, FW = cfg[:7]
    a = cfg[7:]
    OH, OW, _, _ = ops.conv2d_geometry(IH, IW, FH, FW, *a)
    r = rng(sum(cfg[:7]) + 7)
    c = (lambda v: h(v)) if dtype == np.float16 else (lambda v: v)
    hi = 3 if dtype == np.float16 else 20
    x, w, gz = ints(r, (B, IH, IW, IC), hi), ints(r, (OC, FH, FW, IC), hi), ints(r, (B, OH, OW, OC), hi)
    if dtype == np.float16:
        x, w, gz = x * (r.random(x.shape) < 0.3), w * (r.random(w.shape) < 0.3), gz * (r.random(gz.shape) < 0.05)
    want = (oracle_port.conv2d_grad_x(x, w, gz, *a, x), oracle_port.conv2d_grad_y(x, w, gz, *a, w))
    assert dtype == np.float32 or max(np.abs(t).max() for t in want) < 2048
    gx, gw = ops.conv2d_grad_xy(c(x), c(w), c(gz), *a, c(x), c(w))
    assert np.array_equal(f(gx), want[0]) and np.array_equal(f(gw), want[1])
    gx, gw = ops.conv2d_grad_xy(c(x), c(w), c(gz), *a, c(x) * 0 - 9, c(w) * 0 + 9, True, True)
    assert np.array_equal(f(gx), want[0] - x) and np.array_equal(f(gw), want[1] - w)
    xr, wr, gzr, _, _ = _data(r, B, IH, IW, IC, OC, FH, FW, OH, OW, dtype)
    gx, gw = ops.conv2d_grad_xy(xr, wr, gzr, *a)
    tol = FP16_TOL if dtype == np.float16 else FP32_TOL
    assert rel_fro(f(gx), oracle_port.conv2d_grad_x(f(xr), f(wr), f(gzr), *a)) <= tol
    assert rel_fro(f(gw), oracle_port.conv2d_grad_y(f(xr), f(wr), f(gzr), *a)) <= tol
    shares = dtype == np.float16 or _row(cfg, CONV_SHARED)[4]
    assert capi.init().d8_conv_grad_pair_launches() == before + (3 if shares else 0)
    monkeypatch.setenv("D8_CONV_GRADS_APART", "1")
    ax, aw = ops.conv2d_grad_xy(xr, wr, gzr, *a)
    assert _same(aw, gw) and rel_fro(f(ax), f(gx)) <= tol  # (alone, the gradient of x may be cut into pieces)
    assert capi.init().d8_conv_grad_pair_launches() == before + (3 if shares else 0)


@pytest.mark.parametrize("cfg", [row[0] for row in DECONV_SHARED])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_deconv2d_shared_launch_against_the_oracle(oracle_port, monkeypatch, cfg, dtype):
    from deep8_amd import capi, ops
    monkeypatch.setenv("D8_CONV_PAIR_STEPS", "1000000")
    before = capi.init().d8_conv_grad_pair_launches()
    B, IH, IW, IC, OC, FH, FW = cfg[:7]
    a = cfg[7:]
    OH, OW, _, _ = ops.deconv2d_geometry(IH, IW, FH, FW, *a)
    r = rng(sum(cfg[:7]) + 8)
    c = (lambda v: h(v)) if dtype == np.float16 else (lambda v: v)
    hi = 3 if dtype == np.float16 else 20
    keep = min(1.0, 40.0 / np.sqrt(B * IH * IW))  # half: every sum of the filter gradient stays below 2048
    x, w, gz = ints(r, (B, IH, IW, IC), hi), ints(r, (OC, FH, FW, IC), hi), ints(r, (B, OH, OW, OC), hi)
    if dtype == np.float16:
        x, w, gz = x * (r.random(x.shape) < 0.3 * keep), w * (r.random(w.shape) < 0.3), gz * (r.random(gz.shape) < 0.2 * keep)
    want = (oracle_port.deconv2d_grad_x(x, w, gz, *a, x), oracle_port.deconv2d_grad_y(x, w, gz, *a, w))
    assert dtype == np.float32 or max(np.abs(t).max() for t in want) < 2048
    gx, gw = ops.deconv2d_grad_xy(c(x), c(w), c(gz), *a, c(x), c(w))
    assert np.array_equal(f(gx), want[0]) and np.array_equal(f(gw), want[1])
    xr, wr, gzr, _, _ = _data(r, B, IH, IW, IC, OC, FH, FW, OH, OW, dtype)
    gx, gw = ops.deconv2d_grad_xy(xr, wr, gzr, *a, overwrite_x=True, overwrite_w=True)
    tol = FP16_TOL if dtype == np.float16 else FP32_TOL
    assert rel_fro(f(gx), oracle_port.deconv2d_grad_x(f(xr), f(wr), f(gzr), *a)) <= tol
    assert rel_fro(f(gw), oracle_port.deconv2d_grad_y(f(xr), f(wr), f(gzr), *a)) <= tol
    assert capi.init().d8_conv_grad_pair_launches() == before + 2
    monkeypatch.setenv("D8_CONV_GRADS_APART", "1")
    ax, aw = ops.deconv2d_grad_xy(xr, wr, gzr, *a, overwrite_x=True, overwrite_w=True)
    assert _same(aw, gw) and rel_fro(f(ax), f(gx)) <= tol


def test_deconv2d_both_gradients_at_an_explicit_geometry():
    """benchmark configuration 5 as written (28 x 28 -> 56 x 56, pads 1): the _ex form against the two _ex calls"""
    from deep8_amd import capi, ops
    lib = capi.init()
    B, IH, IW, IC, OC, FH, FW, sy, sx = 16, 28, 28, 128, 64, 4, 4, 2, 2
    geo = (56, 56, 1, 1)
    x, w, gz, gx0, gw0 = _data(rng(56), B, IH, IW, IC, OC, FH, FW, 56, 56, np.float16)
    before = lib.d8_conv_grad_pair_launches()
    gx, gw = ops.deconv2d_grad_xy(x, w, gz, False, sy, sx, gx0, gw0, False, True, geometry=geo)
    assert lib.d8_conv_grad_pair_launches() == before + 1
    assert _same(gx, ops.deconv2d_ex(1, x, w, gz, *geo, sy, sx, gx0))
    assert _same(gw, ops.deconv2d_ex(2, x, w, gz, *geo, sy, sx, gw0, overwrite=True))


def test_large_half_layer_shares_a_launch_when_the_scratch_has_room():
    """benchmark configuration 4's layer in half (B32 56 x 56 x 64, 3 x 3): more workgroups than the chip holds at once,
    and a gradient of x whose remainder band rides in its launch.  With the scratch of the which = 3 query both
    gradients share a launch; with the larger of the two single queries they run apart; both leave the bits of the
    two calls."""
    from deep8_amd import capi, ops
    from deep8_amd.capi import DeviceArray, check
    lib = capi.init()
    B, IH, IW, IC, OC, FH, FW = 32, 56, 56, 64, 64, 3, 3
    a = (1, 1, 1, 1, 1)
    dt = capi.FLOAT16
    x, w, gz, gx0, gw0 = _data(rng(404), B, IH, IW, IC, OC, FH, FW, 56, 56, np.float16)
    want_x = ops.conv2d_grad_x(x, w, gz, True, 1, 1, 1, 1, gx0)
    want_w = ops.conv2d_grad_y(x, w, gz, True, 1, 1, 1, 1, gw0, overwrite=True)
    dx_, dw_, dgz = DeviceArray.from_numpy(x), DeviceArray.from_numpy(w), DeviceArray.from_numpy(gz)
    q = lambda which: lib.d8_conv2d_scratch_bytes(dt, which, B, IH, IW, IC, OC, FH, FW, *a)
    assert q(3) >= q(1) + q(2) > max(q(1), q(2)) > 0
    for nb, shared in ((q(3), 1), (max(q(1), q(2)), 0)):
        ws = DeviceArray((nb,), np.uint8)
        dgx, dgw = DeviceArray.from_numpy(gx0), DeviceArray.from_numpy(gw0)
        before = lib.d8_conv_grad_pair_launches()
        check(lib.d8_conv2d_grad_xy(dt, dx_.ptr, dgx.ptr, B, IH, IW, IC, dw_.ptr, dgw.ptr, OC, FH, FW, dgz.ptr, *a, 2, ws.ptr, nb, None))
        assert lib.d8_conv_grad_pair_launches() - before == shared
        assert _same(dgx.numpy(), want_x) and _same(dgw.numpy(), want_w), shared
