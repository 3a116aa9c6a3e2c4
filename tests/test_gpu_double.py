"""The Float64 contraction path (d8_gemm, the gather maps, d8_matmul*, d8_conv2d*, d8_deconv2d* with D8_FLOAT64)
against the oracle's double twins: integer inputs bit for bit, seeded real inputs to 1e-12 relative Frobenius
error (sums are carried in double on both sides; only the order differs).  The reference's counterpart is the
`double` branch of its GPU dispatchers (deep8/src/math/MatrixMultiply.cu:142-175 and the Float64 cases of
Conv2d.cu / DeConv2d.cu)."""
import numpy as np
import pytest

from test_gpu_conv import CONV, DECONV
from test_gpu_gemm import SHAPES, TRANS
from test_gpu_matmul import CASES
from util import ints, rel_fro, rng

pytestmark = pytest.mark.gpu

F64_TOL = 1e-12


def d(a):
    return np.asarray(a, dtype=np.float64)


@pytest.mark.parametrize("ta,tb", TRANS)
@pytest.mark.parametrize("M,N,K", SHAPES + [(96, 80, 4099)])
def test_gemm_f64(oracle, oracle_port, ta, tb, M, N, K):
    from deep8_amd import ops
    r = rng(M * 7 + N * 3 + K + 2)
    sa, sb = ((K, M) if ta else (M, K)), ((N, K) if tb else (K, N))
    Ai, Bi, Ci = d(ints(r, sa)), d(ints(r, sb)), d(ints(r, (M, N)))
    A, B, C = r.standard_normal(sa), r.standard_normal(sb), r.standard_normal((M, N))
    with oracle.float64():
        for beta, c in ((0.0, None), (1.0, Ci)):
            got = ops.gemm(ta, tb, Ai, Bi, c, beta)
            assert got.dtype == np.float64 and np.array_equal(got, oracle_port.gemm(ta, tb, Ai, Bi, c, beta)), (beta,)
        assert rel_fro(ops.gemm(ta, tb, A, B, C, 1.0), oracle_port.gemm(ta, tb, A, B, C, 1.0)) <= F64_TOL


def test_gemm_f64_batched_broadcast_and_summed():
    from deep8_amd import ops
    r = rng(77)
    A, B = r.standard_normal((5, 70, 33)), r.standard_normal((5, 33, 90))
    assert rel_fro(ops.gemm(0, 0, A, B), A @ B) <= F64_TOL
    assert rel_fro(ops.gemm(0, 0, A, B[:1]), A @ B[0]) <= F64_TOL
    assert rel_fro(ops.gemm(0, 0, A[:1], B), A[0] @ B) <= F64_TOL
    Ai, Bi = d(ints(r, (5, 70, 33))), d(ints(r, (5, 33, 90)))
    assert np.array_equal(ops.gemm(0, 1, Ai, np.ascontiguousarray(Bi.transpose(0, 2, 1))), Ai @ Bi)
    assert np.array_equal(ops.gemm(1, 0, np.ascontiguousarray(Ai.transpose(0, 2, 1)), Bi), Ai @ Bi)


@pytest.mark.parametrize("ta,tb", TRANS)
@pytest.mark.parametrize("M,N,K,batch", [(64, 576, 20000, 1), (70, 33, 9001, 1), (40, 50, 5000, 3), (128, 128, 70000, 1)])
def test_gemm_f64_long_reduction_is_split(ta, tb, M, N, K, batch):
    """A small output with a long reduction runs in pieces through the workspace; the pieces must add up to the
    same result as the whole (bit for bit on integers), with beta = 1 too, and without a workspace."""
    from deep8_amd import capi, ops
    lib = capi.init()
    assert lib.d8_gemm_workspace_bytes(capi.FLOAT64, ta, tb, M, N, K, batch, M * N if batch > 1 else 0) >= 2 * batch * M * N * 8
    r = rng(M + N + K + batch)
    sa, sb = ((batch, K, M) if ta else (batch, M, K)), ((batch, N, K) if tb else (batch, K, N))
    Ai, Bi, Ci = d(ints(r, sa, 4)), d(ints(r, sb, 4)), d(ints(r, (batch, M, N)))
    want = (Ai.transpose(0, 2, 1) if ta else Ai) @ (Bi.transpose(0, 2, 1) if tb else Bi)
    assert np.array_equal(ops.gemm(ta, tb, Ai, Bi), want)
    assert np.array_equal(ops.gemm(ta, tb, Ai, Bi, Ci, 1.0), want + Ci)
    assert np.array_equal(ops.gemm(ta, tb, Ai, Bi, use_workspace=False), want)
    A, B = r.standard_normal(sa), r.standard_normal(sb)
    wantr = (A.transpose(0, 2, 1) if ta else A) @ (B.transpose(0, 2, 1) if tb else B)
    assert rel_fro(ops.gemm(ta, tb, A, B), wantr) <= F64_TOL


def test_gemm_f64_summed_batch_is_split():
    """strideC = 0: the products of the whole batch are summed into one C, in pieces over products x K steps"""
    from deep8_amd import ops
    r = rng(79)
    Ai, Bi = d(ints(r, (9, 48, 1000), 4)), d(ints(r, (9, 1000, 40), 4))
    C0 = d(ints(r, (48, 40)))
    assert np.array_equal(ops.gemm(0, 0, Ai, Bi, C0, 1.0), np.einsum("bmk,bkn->mn", Ai, Bi) + C0)


def test_gemm_f64_large_against_numpy():
    from deep8_amd import ops
    r = rng(78)
    A, B = r.standard_normal((1024, 768)), r.standard_normal((768, 1536))
    assert rel_fro(ops.gemm(0, 0, A, B), A @ B) <= F64_TOL


@pytest.mark.parametrize("xs,ys", CASES)
def test_matmul_f64(oracle, oracle_port, xs, ys):
    from deep8_amd import ops
    r = rng(sum(xs) + sum(ys) + 9)
    xi, yi = d(ints(r, xs)), d(ints(r, ys))
    x, y = r.standard_normal(xs), r.standard_normal(ys)
    with oracle.float64():
        want = oracle_port.matmul(xi, yi)
        z = ops.matmul(xi, yi)
        assert z.dtype == np.float64 and z.shape == want.shape and np.array_equal(z, want)
        dz = d(ints(r, z.shape))
        dx0, dy0 = d(ints(r, xs)), d(ints(r, ys))
        assert np.array_equal(ops.matmul_grad_x(xi, yi, dz, dx0), oracle_port.matmul_grad_x(xi, yi, dz, dx0))
        assert np.array_equal(ops.matmul_grad_y(xi, yi, dz, dy0), oracle_port.matmul_grad_y(xi, yi, dz, dy0))
        assert np.array_equal(ops.matmul_grad_x(xi, yi, dz, dx0 - 500, overwrite=True), oracle_port.matmul_grad_x(xi, yi, dz))
        assert np.array_equal(ops.matmul_grad_y(xi, yi, dz, dy0 - 500, overwrite=True), oracle_port.matmul_grad_y(xi, yi, dz))
        g = r.standard_normal(z.shape)
        assert rel_fro(ops.matmul(x, y), oracle_port.matmul(x, y)) <= F64_TOL
        assert rel_fro(ops.matmul_grad_x(x, y, g), oracle_port.matmul_grad_x(x, y, g)) <= F64_TOL
        assert rel_fro(ops.matmul_grad_y(x, y, g), oracle_port.matmul_grad_y(x, y, g)) <= F64_TOL


# 128 input channels or more: the gradient of x reads its patch rows of dz inside the GEMM as well (stride 1:
# one product per tap; stride 2: by residue classes of input pixels)
CONV_WIDE = [
    (2, 12, 12, 128, 24, 3, 3, True, 1, 1, 1, 1),
    (1, 10, 10, 136, 8, 3, 3, False, 1, 1, 2, 2),
    (2, 12, 12, 128, 16, 3, 3, True, 2, 2, 1, 1),
    (1, 11, 9, 130, 5, 4, 3, False, 2, 1, 1, 1),
    (2, 12, 12, 128, 16, 3, 3, True, 2, 2, 2, 2),   # strided and dilated: classes of input pixels, some without a tap
]


@pytest.mark.parametrize("cfg", CONV + CONV_WIDE)
def test_conv2d_f64(oracle, oracle_port, cfg):
    from deep8_amd import ops
    B, IH, IW, IC, OC, FH, FW = cfg[:7]
    a = cfg[7:]
    r = rng(B + IH + OC + 3)
    xi, wi = d(ints(r, (B, IH, IW, IC))), d(ints(r, (OC, FH, FW, IC)))
    x, w = r.standard_normal(xi.shape), r.standard_normal(wi.shape)
    with oracle.float64():
        want = oracle_port.conv2d(xi, wi, *a)
        got = ops.conv2d(xi, wi, *a)
        assert got.dtype == np.float64 and got.shape == want.shape and np.array_equal(got, want)
        gz = d(ints(r, want.shape, 10))
        gx0, gw0 = d(ints(r, xi.shape)), d(ints(r, wi.shape))
        assert np.array_equal(ops.conv2d_grad_x(xi, wi, gz, *a, gx0), oracle_port.conv2d_grad_x(xi, wi, gz, *a, gx0))
        assert np.array_equal(ops.conv2d_grad_y(xi, wi, gz, *a, gw0), oracle_port.conv2d_grad_y(xi, wi, gz, *a, gw0))
        assert np.array_equal(ops.conv2d_grad_x(xi, wi, gz, *a, gx0 - 500, overwrite=True), oracle_port.conv2d_grad_x(xi, wi, gz, *a))
        assert np.array_equal(ops.conv2d_grad_y(xi, wi, gz, *a, gw0 - 500, overwrite=True), oracle_port.conv2d_grad_y(xi, wi, gz, *a))
        g = r.standard_normal(want.shape)
        assert rel_fro(ops.conv2d(x, w, *a), oracle_port.conv2d(x, w, *a)) <= F64_TOL
        assert rel_fro(ops.conv2d_grad_x(x, w, g, *a), oracle_port.conv2d_grad_x(x, w, g, *a)) <= F64_TOL
        assert rel_fro(ops.conv2d_grad_y(x, w, g, *a), oracle_port.conv2d_grad_y(x, w, g, *a)) <= F64_TOL


@pytest.mark.parametrize("cfg", DECONV)
def test_deconv2d_f64(oracle, oracle_port, cfg):
    from deep8_amd import ops
    B, IH, IW, IC, OC, FH, FW = cfg[:7]
    a = cfg[7:]
    r = rng(B + IH + OC + 4)
    xi, wi = d(ints(r, (B, IH, IW, IC), 10)), d(ints(r, (OC, FH, FW, IC), 10))
    x, w = r.standard_normal(xi.shape), r.standard_normal(wi.shape)
    with oracle.float64():
        want = oracle_port.deconv2d(xi, wi, *a)
        got = ops.deconv2d(xi, wi, *a)
        assert got.dtype == np.float64 and got.shape == want.shape and np.array_equal(got, want)
        gz = d(ints(r, want.shape, 10))
        gx0, gw0 = d(ints(r, xi.shape)), d(ints(r, wi.shape))
        assert np.array_equal(ops.deconv2d_grad_x(xi, wi, gz, *a, gx0), oracle_port.deconv2d_grad_x(xi, wi, gz, *a, gx0))
        assert np.array_equal(ops.deconv2d_grad_y(xi, wi, gz, *a, gw0), oracle_port.deconv2d_grad_y(xi, wi, gz, *a, gw0))
        assert np.array_equal(ops.deconv2d_grad_x(xi, wi, gz, *a, gx0 - 500, overwrite=True), oracle_port.deconv2d_grad_x(xi, wi, gz, *a))
        assert np.array_equal(ops.deconv2d_grad_y(xi, wi, gz, *a, gw0 - 500, overwrite=True), oracle_port.deconv2d_grad_y(xi, wi, gz, *a))
        g = r.standard_normal(want.shape)
        assert rel_fro(ops.deconv2d(x, w, *a), oracle_port.deconv2d(x, w, *a)) <= F64_TOL
        assert rel_fro(ops.deconv2d_grad_x(x, w, g, *a), oracle_port.deconv2d_grad_x(x, w, g, *a)) <= F64_TOL
        assert rel_fro(ops.deconv2d_grad_y(x, w, g, *a), oracle_port.deconv2d_grad_y(x, w, g, *a)) <= F64_TOL


@pytest.mark.parametrize("cfg", CONV + CONV_WIDE)
def test_conv2d_f64_stages_nothing_and_the_staged_route_agrees(oracle, oracle_port, monkeypatch, cfg):
    """Float64 convolutions read their patch matrix from the image inside the GEMM (every shape: the fp64 kernel
    moves single elements), so they ask for less scratch than the im2col matrix -- except the gradient of x under
    128 input channels, which stays staged; the staged route, forced through the same entry points, still gives
    the oracle's result."""
    from deep8_amd import capi, ops
    lib = capi.init()
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx, dy, dx = cfg
    a = cfg[7:]
    OH, OW, _, _ = ops.conv2d_geometry(IH, IW, FH, FW, *a)
    col = B * OH * OW * FH * FW * IC * 8
    for which in range(3):
        q = lambda: lib.d8_conv2d_scratch_bytes(capi.FLOAT64, which, B, IH, IW, IC, OC, FH, FW, int(cov), sy, sx, dy, dx)
        staged = which == 1 and (IC < 128 or sy * sx > 16 or IH < sy or IW < sx)
        assert (q() < col) == (not staged), (which, q(), col)
        monkeypatch.setenv("D8_CONV_EXPLICIT", "1")
        assert q() >= col
        monkeypatch.delenv("D8_CONV_EXPLICIT")
    r = rng(B + IH + OC + 31)
    xi, wi = d(ints(r, (B, IH, IW, IC))), d(ints(r, (OC, FH, FW, IC)))
    gz = d(ints(r, (B, OH, OW, OC), 10))
    monkeypatch.setenv("D8_CONV_EXPLICIT", "1")
    with oracle.float64():
        assert np.array_equal(ops.conv2d(xi, wi, *a), oracle_port.conv2d(xi, wi, *a))
        assert np.array_equal(ops.conv2d_grad_x(xi, wi, gz, *a, xi), oracle_port.conv2d_grad_x(xi, wi, gz, *a, xi))
        assert np.array_equal(ops.conv2d_grad_y(xi, wi, gz, *a, wi), oracle_port.conv2d_grad_y(xi, wi, gz, *a, wi))


@pytest.mark.parametrize("cfg", DECONV)
def test_deconv2d_f64_stages_nothing_and_the_staged_route_agrees(oracle, oracle_port, monkeypatch, cfg):
    from deep8_amd import capi, ops
    lib = capi.init()
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx = cfg
    a = cfg[7:]
    OH, OW, _, _ = ops.deconv2d_geometry(IH, IW, FH, FW, *a)
    interim = B * IH * IW * FH * FW * OC * 8
    for which in range(3):
        q = lambda: lib.d8_deconv2d_scratch_bytes(capi.FLOAT64, which, B, IH, IW, IC, OC, FH, FW, int(cov), sy, sx)
        staged = which == 0 and (OH < sy or OW < sx or sy * sx > 16)
        assert (q() < interim) == (not staged), (which, q(), interim)
        monkeypatch.setenv("D8_CONV_EXPLICIT", "1")
        assert q() >= interim
        monkeypatch.delenv("D8_CONV_EXPLICIT")
    r = rng(B + IH + OC + 32)
    xi, wi = d(ints(r, (B, IH, IW, IC), 10)), d(ints(r, (OC, FH, FW, IC), 10))
    gz = d(ints(r, (B, OH, OW, OC), 10))
    monkeypatch.setenv("D8_CONV_EXPLICIT", "1")
    with oracle.float64():
        assert np.array_equal(ops.deconv2d(xi, wi, *a), oracle_port.deconv2d(xi, wi, *a))
        assert np.array_equal(ops.deconv2d_grad_x(xi, wi, gz, *a, xi), oracle_port.deconv2d_grad_x(xi, wi, gz, *a, xi))
        assert np.array_equal(ops.deconv2d_grad_y(xi, wi, gz, *a, wi), oracle_port.deconv2d_grad_y(xi, wi, gz, *a, wi))


def test_f64_convolutions_on_the_large_tiles(oracle, oracle_port):
    """Shapes whose products fill the chip with 128 x 128 tiles: Conv2d forward (patch rows as A) and DeConv2d
    forward (four classes of output pixels), integers bit for bit and reals to 1e-12."""
    from deep8_amd import ops
    r = rng(4242)
    with oracle.float64():
        xi, wi = d(ints(r, (8, 28, 28, 256), 4)), d(ints(r, (512, 3, 3, 256), 4))
        a = (True, 1, 1, 1, 1)
        assert np.array_equal(ops.conv2d(xi, wi, *a), oracle_port.conv2d(xi, wi, *a))
        x, w = r.standard_normal(xi.shape), r.standard_normal(wi.shape)
        assert rel_fro(ops.conv2d(x, w, *a), oracle_port.conv2d(x, w, *a)) <= F64_TOL
        xi, wi = d(ints(r, (8, 14, 14, 256), 4)), d(ints(r, (512, 4, 4, 256), 4))
        a = (True, 2, 2)
        assert np.array_equal(ops.deconv2d(xi, wi, *a), oracle_port.deconv2d(xi, wi, *a))
        x, w = r.standard_normal(xi.shape), r.standard_normal(wi.shape)
        assert rel_fro(ops.deconv2d(x, w, *a), oracle_port.deconv2d(x, w, *a)) <= F64_TOL


@pytest.mark.parametrize("cfg", CONV[:5])
def test_gather_maps_f64(oracle_port, cfg):
    """im2col is a copy and col2im an ordered sum: on values that float holds exactly (and whose sums it holds
    exactly) the double kernels must reproduce the float oracle's result."""
    from deep8_amd import ops
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx, dy, dx = cfg
    OH, OW, pt, pl = oracle_port.conv2d_geometry(IH, IW, FH, FW, cov, sy, sx, dy, dx)
    r = rng(B + IH + FH + 6)
    im = ints(r, (B, IH, IW, IC), 1000)
    g = (OH, OW, FH, FW, sy, sx, dy, dx, pt, pl)
    want = oracle_port.im2col(im, *g)
    got = ops.im2col(d(im), *g)
    assert got.dtype == np.float64 and np.array_equal(got, d(want))
    col, im0 = ints(r, want.shape, 100), ints(r, im.shape, 100)
    assert np.array_equal(ops.col2im(d(col), d(im0), *g), d(oracle_port.col2im(col, im0, *g)))


def test_float64_outside_the_contraction_path_is_rejected():
    from deep8_amd import capi, ops
    x = np.ones((2, 8), np.float64)
    with pytest.raises(capi.Deep8HipError):
        ops.relu(x)
    with pytest.raises(capi.Deep8HipError):
        ops.add(x, x)
