"""The HIP path against the vectors Deep8's own CPU (Eigen) build wrote (tests/golden/deep8_cpu_reference.npz,
made by tests/golden/make_golden.py from deep8/src/math/{MatrixMultiply,Conv2d,DeConv2d,...}.cpp), with no
checker in between: inputs from the file go through the C ABI, results are compared with the stored outputs.

fp32 results within a relative Frobenius error of 1e-5; the patch matrices bit for bit (the uint32 views are
compared), which is the sentence "im2col bit-exact against Deep8's own CPU Eigen path" taken literally.
"""
import os

import numpy as np
import pytest

from util import FP32_TOL, rel_fro

pytestmark = pytest.mark.gpu

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "deep8_cpu_reference.npz"))


def _n(prefix):
    return sorted({int(k[len(prefix):].split("_")[0]) for k in GOLD.files if k.startswith(prefix) and k[len(prefix)].isdigit()})


@pytest.mark.parametrize("i", _n("mm"))
def test_matmul_golden(i):
    from deep8_amd import ops
    g = lambda k: GOLD["mm%d_%s" % (i, k)]
    z = ops.matmul(g("x"), g("y"))
    assert z.shape == g("z").shape and rel_fro(z, g("z")) <= FP32_TOL
    assert rel_fro(ops.matmul_grad_x(g("x"), g("y"), g("dz"), g("dx0")), g("dx")) <= FP32_TOL
    assert rel_fro(ops.matmul_grad_y(g("x"), g("y"), g("dz"), g("dy0")), g("dy")) <= FP32_TOL


@pytest.mark.parametrize("i", _n("conv"))
def test_conv2d_golden(i):
    from deep8_amd import ops
    g = lambda k: GOLD["conv%d_%s" % (i, k)]
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx, dy, dx = (int(v) for v in g("cfg"))
    a = (bool(cov), sy, sx, dy, dx)
    z = ops.conv2d(g("x"), g("w"), *a)
    assert z.shape == g("z").shape and rel_fro(z, g("z")) <= FP32_TOL
    assert rel_fro(ops.conv2d_grad_x(g("x"), g("w"), g("gz"), *a, gx=g("gx0")), g("gx")) <= FP32_TOL
    assert rel_fro(ops.conv2d_grad_y(g("x"), g("w"), g("gz"), *a, gw=g("gw0")), g("gw")) <= FP32_TOL
    # d8_im2col == the patch matrix Eigen's extract_image_patches builds, bit for bit
    OH, OW, pt, pl = ops.conv2d_geometry(IH, IW, FH, FW, cov, sy, sx, dy, dx)
    col = ops.im2col(g("x"), OH, OW, FH, FW, sy, sx, dy, dx, pt, pl)
    assert col.shape == g("patches").shape
    assert np.array_equal(col.view(np.uint32), g("patches").view(np.uint32))


@pytest.mark.parametrize("i", _n("deconv"))
def test_deconv2d_golden(i):
    from deep8_amd import ops
    g = lambda k: GOLD["deconv%d_%s" % (i, k)]
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx = (int(v) for v in g("cfg"))
    a = (bool(cov), sy, sx)
    z = ops.deconv2d(g("x"), g("w"), *a)
    assert z.shape == g("z").shape and rel_fro(z, g("z")) <= FP32_TOL
    assert rel_fro(ops.deconv2d_grad_x(g("x"), g("w"), g("gz"), *a, gx=g("gx0")), g("gx")) <= FP32_TOL
    assert rel_fro(ops.deconv2d_grad_y(g("x"), g("w"), g("gz"), *a, gw=g("gw0")), g("gw")) <= FP32_TOL
    # d8_deconv_im2col is a pure permutation of the patches Eigen cuts from dz for the flipped filter:
    # dzmat[r, oc*FH*FW + fy*FW + fx] == patches[r, ((FH-1-fy)*FW + (FW-1-fx))*OC + oc]
    OH, OW, pt, pl = ops.deconv2d_geometry(IH, IW, FH, FW, cov, sy, sx)
    m = ops.deconv_im2col(g("gz"), IH, IW, FH, FW, sy, sx, pt, pl).reshape(-1, OC, FH, FW)
    p = g("gpatches").reshape(-1, FH, FW, OC)[:, ::-1, ::-1, :].transpose(0, 3, 1, 2)
    assert np.array_equal(m.view(np.uint32), np.ascontiguousarray(p).view(np.uint32))


@pytest.mark.parametrize("i", _n("loss"))
def test_loss_ops_golden(i):
    from deep8_amd import ops
    g = lambda k: GOLD["loss%d_%s" % (i, k)]
    x, y, axes = g("x"), g("y"), tuple(int(a) for a in g("axes"))
    assert np.array_equal(ops.minus(x, y), g("z"))
    assert rel_fro(ops.l1norm(x), g("l1")) <= FP32_TOL
    assert rel_fro(ops.l2norm(x), g("l2")) <= FP32_TOL
    assert rel_fro(ops.l1norm_grad(x, g("dn"), g("dx0")), g("l1_gx")) <= FP32_TOL
    assert rel_fro(ops.l2norm_grad(x, g("l2"), g("dn"), g("dx0")), g("l2_gx")) <= FP32_TOL
    m = ops.reduce_mean(x, axes)
    assert m.size == g("mean").size and rel_fro(m.ravel(), g("mean").ravel()) <= FP32_TOL
    assert rel_fro(ops.axpby(x, -0.01, g("dx0"), 0.999), g("axpby")) <= FP32_TOL


@pytest.mark.parametrize("i", _n("pool"))
def test_pooling_golden(i):
    from deep8_amd import ops
    g = lambda k: GOLD["pool%d_%s" % (i, k)]
    B, IH, IW, C, FH, FW, cov, sy, sx = (int(v) for v in g("cfg"))
    a = (FH, FW, bool(cov), sy, sx)
    assert np.array_equal(ops.maxpool2d(g("x"), *a), g("max"))
    assert rel_fro(ops.avgpool2d(g("x"), *a), g("avg")) <= FP32_TOL
    # overlapping windows add several dy into one dx: the reference scatters window by window, the HIP kernel
    # gathers pixel by pixel, so on real-valued data the last bit of such a sum may differ
    assert rel_fro(ops.maxpool2d_grad(g("x"), g("dy"), *a, dx=g("dx0")), g("max_gx")) <= 1e-6
    assert rel_fro(ops.avgpool2d_grad(g("x").shape, g("dy"), *a, dx=g("dx0")), g("avg_gx")) <= FP32_TOL
