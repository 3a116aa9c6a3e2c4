"""MatrixMultiply forward / GradX / GradY through the C ABI against the oracle: the three shape
cases of deep8/src/math/MatrixMultiply.cpp:94-116 (collapsed batch, vector-by-batch, batched with
broadcast), the reference's own test shapes (test/MatrixMultiplyTest.h), and benchmark configurations."""
import numpy as np
import pytest

from util import FP16_TOL, FP32_TOL, f, h, ints, nrm, rel_fro, rng, uni

pytestmark = pytest.mark.gpu

# (x shape, y shape): first axis is the batch
CASES = [
    ((10, 400, 200), (1, 200, 300)),   # forwardCPU / GPU1: y.batch == 1 (F1/X1/Y1)
    ((1, 300, 100), (10, 100)),        # forwardCPU2 / GPU2: x.batch == 1, y is a batch of vectors (F2/X2/Y2)
    ((6, 40, 30), (6, 30, 50)),        # batched both (F3/X3/Y3)
    ((1, 40, 30), (6, 30, 50)),        # x broadcast: dX sums over the batch
    ((6, 40, 30), (6, 30)),            # batched matrix-vector (1-D y, both batched)
    ((1, 64, 128), (1, 128, 256)),     # benchmark configuration 1
    ((3, 17), (1, 1, 9)),              # 1-D x (column vector) times a row: outer products
]


@pytest.mark.parametrize("xs,ys", CASES)
def test_matmul_integer_exact(oracle_port, xs, ys):
    from deep8_amd import ops
    r = rng(sum(xs) + sum(ys))
    x, y = ints(r, xs), ints(r, ys)
    z = ops.matmul(x, y)
    want = oracle_port.matmul(x, y)
    assert z.shape == want.shape and np.array_equal(z, want)
    dz = ints(r, z.shape)
    dx0, dy0 = ints(r, xs), ints(r, ys)
    assert np.array_equal(ops.matmul_grad_x(x, y, dz, dx0), oracle_port.matmul_grad_x(x, y, dz, dx0))
    assert np.array_equal(ops.matmul_grad_y(x, y, dz, dy0), oracle_port.matmul_grad_y(x, y, dz, dy0))


@pytest.mark.parametrize("xs,ys", CASES + [((1, 512, 512), (1, 512, 512)), ((32, 128, 64), (1, 64, 128)), ((1, 4096, 64), (1, 64, 512))])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_matmul_gradients_overwrite_form(oracle_port, xs, ys, dtype):
    """d8_matmul_grad_{x,y}_overwrite leave what "zero, then accumulate" leaves, whatever the
    destination held before (split and summed reductions included)."""
    from deep8_amd import ops
    r = rng(sum(xs) + 2 * sum(ys))
    c = (lambda a: h(a)) if dtype == np.float16 else (lambda a: a)
    hi = 2 if dtype == np.float16 else 20
    x, y = ints(r, xs, hi), ints(r, ys, hi)
    if dtype == np.float16:
        x, y = x * (r.random(xs) < 0.3), y * (r.random(ys) < 0.3)
    dz = ints(r, oracle_port.matmul(x, y).shape, hi)
    junk_x, junk_y = ints(r, xs, 1000) - 500, ints(r, ys, 1000) - 500
    want_dx, want_dy = oracle_port.matmul_grad_x(x, y, dz), oracle_port.matmul_grad_y(x, y, dz)
    assert dtype == np.float32 or max(np.abs(want_dx).max(), np.abs(want_dy).max()) < 2048
    assert np.array_equal(f(ops.matmul_grad_x(c(x), c(y), c(dz), c(junk_x), overwrite=True)), want_dx)
    assert np.array_equal(f(ops.matmul_grad_y(c(x), c(y), c(dz), c(junk_y), overwrite=True)), want_dy)


@pytest.mark.parametrize("xs,ys", CASES)
def test_matmul_half_integer_exact(oracle_port, xs, ys):
    from deep8_amd import ops
    r = rng(sum(xs) + sum(ys) + 1)
    x, y = ints(r, xs, 2), ints(r, ys, 2)
    z = ops.matmul(h(x), h(y))
    assert z.dtype == np.float16 and np.array_equal(f(z), oracle_port.matmul(x, y))
    dz = ints(r, z.shape, 2)
    want_dx, want_dy = oracle_port.matmul_grad_x(x, y, dz), oracle_port.matmul_grad_y(x, y, dz)
    assert max(want_dx.max(), want_dy.max()) < 2048
    assert np.array_equal(f(ops.matmul_grad_x(h(x), h(y), h(dz))), want_dx)
    assert np.array_equal(f(ops.matmul_grad_y(h(x), h(y), h(dz))), want_dy)


@pytest.mark.parametrize("xs,ys", CASES)
def test_matmul_real_tolerance(oracle_port, xs, ys):
    from deep8_amd import ops
    r = rng(sum(xs) + sum(ys) + 2)
    x, y = uni(r, xs), uni(r, ys)
    want = oracle_port.matmul(x, y)
    assert rel_fro(ops.matmul(x, y), want) <= FP32_TOL
    dz = uni(r, want.shape)
    assert rel_fro(ops.matmul_grad_x(x, y, dz), oracle_port.matmul_grad_x(x, y, dz)) <= FP32_TOL
    assert rel_fro(ops.matmul_grad_y(x, y, dz), oracle_port.matmul_grad_y(x, y, dz)) <= FP32_TOL
    xh, yh, dzh = h(x), h(y), h(dz)
    assert rel_fro(f(ops.matmul(xh, yh)), oracle_port.matmul(f(xh), f(yh))) <= FP16_TOL
    assert rel_fro(f(ops.matmul_grad_x(xh, yh, dzh)), oracle_port.matmul_grad_x(f(xh), f(yh), f(dzh))) <= FP16_TOL
    assert rel_fro(f(ops.matmul_grad_y(xh, yh, dzh)), oracle_port.matmul_grad_y(f(xh), f(yh), f(dzh))) <= FP16_TOL


def test_grad_accumulates_running_twice_doubles(oracle_port):
    """Every Grad routine adds into its destination (MatrixMultiply.cpp:147, MatrixMultiply.cu:203)."""
    from deep8_amd import ops
    r = rng(3)
    x, y = ints(r, (4, 20, 10)), ints(r, (1, 10, 30))
    dz = ints(r, (4, 20, 30))
    once = ops.matmul_grad_y(x, y, dz)
    twice = ops.matmul_grad_y(x, y, dz, once)
    assert np.array_equal(twice, 2 * once)
    once = ops.matmul_grad_x(x, y, dz)
    assert np.array_equal(ops.matmul_grad_x(x, y, dz, once), 2 * once)


@pytest.mark.parametrize("xs,ys", CASES)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_matmul_both_gradients_from_one_call(oracle_port, xs, ys, dtype):
    """d8_matmul_grad_xy leaves what d8_matmul_grad_x followed by d8_matmul_grad_y leave, in its accumulating and in
    its overwriting form, for every shape case (small shapes: the two products run one after the other)."""
    from deep8_amd import ops
    r = rng(sum(xs) + 3 * sum(ys))
    c = (lambda a: h(a)) if dtype == np.float16 else (lambda a: a)
    hi = 2 if dtype == np.float16 else 20
    x, y = ints(r, xs, hi), ints(r, ys, hi)
    dz = ints(r, oracle_port.matmul(x, y).shape, hi)
    dx0, dy0 = ints(r, xs, 3), ints(r, ys, 3)
    want_dx, want_dy = oracle_port.matmul_grad_x(x, y, dz), oracle_port.matmul_grad_y(x, y, dz)
    assert dtype == np.float32 or max(np.abs(want_dx).max(), np.abs(want_dy).max()) < 2040
    gx, gy = ops.matmul_grad_xy(c(x), c(y), c(dz), c(dx0), c(dy0))
    assert np.array_equal(f(gx), want_dx + dx0) and np.array_equal(f(gy), want_dy + dy0)
    gx, gy = ops.matmul_grad_xy(c(x), c(y), c(dz), c(dx0 - 500), c(dy0 + 500), overwrite_x=True, overwrite_y=True)
    assert np.array_equal(f(gx), want_dx) and np.array_equal(f(gy), want_dy)
    gx, gy = ops.matmul_grad_xy(c(x), c(y), c(dz), c(dx0), c(dy0 + 500), overwrite_y=True)
    assert np.array_equal(f(gx), want_dx + dx0) and np.array_equal(f(gy), want_dy)


# (xr, xc, yc): both products large enough for the 256 x 256-tile kernel, so the call is ONE launch whose workgroups
# walk tiles of dX, then tiles of dY
PAIRS = [
    (4096, 4096, 4096),   # configuration 3: 256 + 256 tiles on 256 compute units
    (4096, 4360, 4096),   # tiles that stick out of C (moved back inside) in both products, 288 + 288 tiles
    (3072, 4104, 4160),   # neither tile count divisible by eight: no XCD-contiguous runs
    (4096, 3072, 8192),   # 192 + 384 tiles, reductions of 8192 and 4096
]


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("xs,ys,shared", [((1, 64, 128), (1, 128, 256), (True, True)),    # benchmark configuration 1
                                          ((1, 33, 70), (1, 70, 50), (True, True)),       # ragged 32 x 32 tiles
                                          ((3, 40, 64), (3, 64, 72), (True, True)),       # a batch of three small products
                                          # a fully connected layer: the tiled kernels, both products split along their reductions
                                          ((1, 64, 1024), (1, 1024, 256), (True, True)),
                                          ((1, 256, 1024), (1, 1024, 1024), (True, True)),
                                          ((4, 128, 256), (1, 256, 384), (True, True)),   # the second input shared by a batch: its gradient sums over it
                                          ((1, 200, 264), (1, 264, 136), (False, False)),  # a reduction that is not a multiple of the K step
                                          # more workgroups than the chip holds at once (and too few 256 x 256 tiles in dX for the large-output kernel's pair)
                                          ((1, 4096, 2048), (1, 2048, 4096), (False, False))])
def test_small_and_mid_size_matmul_gradients_share_a_launch(oracle_port, xs, ys, shared, dtype):
    """d8_matmul_grad_xy runs two small products as one launch of the small-product kernel and two mid-size ones as
    one launch of the tiled kernel (shared: whether in fp32, in half); integers bit for bit against the oracle, and
    the bits of the two separate calls"""
    shared = shared[0] if dtype == np.float32 else shared[1]
    from deep8_amd import capi, ops
    lib = capi.init()
    r = rng(sum(xs) + sum(ys) + 3)
    c = (lambda v: h(v)) if dtype == np.float16 else (lambda v: v)
    hi = 2 if dtype == np.float16 else 20
    x, y = ints(r, xs, hi), ints(r, ys, hi)
    dz = ints(r, (max(xs[0], ys[0]), xs[1], ys[2]), hi)
    dx0, dy0 = ints(r, xs, hi), ints(r, ys, hi)
    if dtype == np.float16:  # thinned so that every sum stays exact in half
        keep = min(1.0, 24.0 / np.sqrt(max(xs[1] * max(xs[0], ys[0]), xs[2], ys[2])))
        x, dz = x * (r.random(x.shape) < keep), dz * (r.random(dz.shape) < keep)
    before = lib.d8_matmul_grad_pair_launches()
    gx, gy = ops.matmul_grad_xy(c(x), c(y), c(dz), c(dx0), c(dy0), False, True)
    assert lib.d8_matmul_grad_pair_launches() - before == (1 if shared else 0)
    wx, wy = oracle_port.matmul_grad_x(x, y, dz, dx0), oracle_port.matmul_grad_y(x, y, dz)
    assert dtype == np.float32 or max(np.abs(wx).max(), np.abs(wy).max()) < 2048
    assert np.array_equal(f(gx), wx) and np.array_equal(f(gy), wy)
    xr_, yr_, dzr = c(nrm(r, xs)), c(nrm(r, ys, 1 / 32.0)), c(nrm(r, dz.shape))
    gx, gy = ops.matmul_grad_xy(xr_, yr_, dzr, overwrite_x=True, overwrite_y=True)
    bits = np.uint16 if dtype == np.float16 else np.uint32
    assert np.array_equal(gx.view(bits), ops.matmul_grad_x(xr_, yr_, dzr, overwrite=True).view(bits))
    assert np.array_equal(gy.view(bits), ops.matmul_grad_y(xr_, yr_, dzr, overwrite=True).view(bits))


@pytest.mark.parametrize("xr,xc,yc", PAIRS)
@pytest.mark.parametrize("overwrite", [True, False])
def test_matmul_both_gradients_as_one_launch(xr, xc, yc, overwrite):
    """integers, sparse enough that every sum stays below 2048: bit for bit against numpy in float32"""
    from deep8_amd import ops
    r = rng(xr + xc + yc)
    keep = 300.0 / max(xr, xc, yc)
    x = h(ints(r, (1, xr, xc), 3) * (r.random((1, xr, xc)) < keep))
    y = h(ints(r, (1, xc, yc), 3))
    dz = h(ints(r, (1, xr, yc), 3) * (r.random((1, xr, yc)) < keep))
    dx0, dy0 = h(ints(r, x.shape, 3)), h(ints(r, y.shape, 3))
    gx, gy = ops.matmul_grad_xy(x, y, dz, dx0, dy0, overwrite, overwrite)
    wx = f(dz[0]) @ f(y[0]).T + (0 if overwrite else f(dx0[0]))
    wy = f(x[0]).T @ f(dz[0]) + (0 if overwrite else f(dy0[0]))
    assert wx.max() < 2048 and wy.max() < 2048
    assert np.array_equal(f(gx[0]), wx) and np.array_equal(f(gy[0]), wy)
    # and the two separate calls give the same bits
    sx = ops.matmul_grad_x(x, y, dz, dx0, overwrite=overwrite)
    sy = ops.matmul_grad_y(x, y, dz, dy0, overwrite=overwrite)
    assert np.array_equal(gx.view(np.uint16), sx.view(np.uint16)) and np.array_equal(gy.view(np.uint16), sy.view(np.uint16))


def test_matmul_both_gradients_as_one_launch_on_reals(oracle_port):
    """configuration 3's data: the one-launch form against the two calls, bit for bit, and sampled rows against the oracle"""
    from deep8_amd import ops
    r = rng(77)
    n = 4096
    A, B, dC = h(nrm(r, (1, n, n), 1 / 64.0)), h(nrm(r, (1, n, n), 1 / 64.0)), h(nrm(r, (1, n, n), 1.0))
    gx, gy = ops.matmul_grad_xy(A, B, dC, overwrite_x=True, overwrite_y=True)
    assert np.array_equal(gx.view(np.uint16), ops.matmul_grad_x(A, B, dC, overwrite=True).view(np.uint16))
    assert np.array_equal(gy.view(np.uint16), ops.matmul_grad_y(A, B, dC, overwrite=True).view(np.uint16))
    rows = r.choice(n, 16, replace=False)
    assert rel_fro(f(gx[0][rows]), oracle_port.gemm(0, 1, f(dC[0])[rows], f(B[0]))) <= FP16_TOL
    assert rel_fro(f(gy[0][rows]), oracle_port.gemm(1, 0, np.ascontiguousarray(f(A[0])[:, rows]), f(dC[0]))) <= FP16_TOL


def _against_reference_or_port(oracle_port, name, *args):
    import oracle
    src = oracle.ref if oracle.ref is not None else oracle_port
    return getattr(src, name)(*args)


@pytest.mark.parametrize("yb", [32, 1])
def test_config2_batched_fp32(oracle_port, yb):
    """benchmark configuration 2: batch 32 of 512x512x512 (and the shared-weight broadcast case), uniform(-1,1)."""
    from deep8_amd import ops
    r = rng(2024)
    x, y, dz = uni(r, (32, 512, 512)), uni(r, (yb, 512, 512)), uni(r, (32, 512, 512))
    assert rel_fro(ops.matmul(x, y), _against_reference_or_port(oracle_port, "matmul", x, y)) <= FP32_TOL
    assert rel_fro(ops.matmul_grad_x(x, y, dz),
                   _against_reference_or_port(oracle_port, "matmul_grad_x", x, y, dz)) <= FP32_TOL
    assert rel_fro(ops.matmul_grad_y(x, y, dz),
                   _against_reference_or_port(oracle_port, "matmul_grad_y", x, y, dz)) <= FP32_TOL


def test_config3_large_half_properties(oracle_port):
    """benchmark configuration 3 (4096^3 half) at full size, checked through size-independent properties:
    sampled rows/columns against the oracle's GEMM on the half-rounded inputs, and linearity."""
    from deep8_amd import ops
    r = rng(4096)
    n = 4096
    A, B = h(nrm(r, (1, n, n), 1 / 64.0)), h(nrm(r, (1, n, n), 1 / 64.0))
    dC = h(nrm(r, (1, n, n), 1.0))
    C = ops.matmul(A, B)
    dA = ops.matmul_grad_x(A, B, dC)
    dB = ops.matmul_grad_y(A, B, dC)
    rows = r.choice(n, 24, replace=False)
    Af, Bf, dCf = f(A[0]), f(B[0]), f(dC[0])
    want = oracle_port.gemm(0, 0, Af[rows], Bf)
    assert rel_fro(f(C[0][rows]), want) <= FP16_TOL
    want = oracle_port.gemm(0, 1, dCf[rows], Bf)            # dA = dC B^T
    assert rel_fro(f(dA[0][rows]), want) <= FP16_TOL
    want = oracle_port.gemm(1, 0, np.ascontiguousarray(Af[:, rows]), dCf)   # dB = A^T dC, sampled rows of dB
    assert rel_fro(f(dB[0][rows]), want) <= FP16_TOL
    # <C, dC> == <A, dA> == <B, dB> (adjoint identity of the three products), in double
    ip = lambda u, v: float(np.sum(u.astype(np.float64) * v.astype(np.float64)))
    t = ip(f(C), f(dC))
    assert abs(ip(f(A), f(dA)) - t) <= 2e-3 * abs(t) + 1.0
    assert abs(ip(f(B), f(dB)) - t) <= 2e-3 * abs(t) + 1.0


def test_matmul_step_replayed_from_a_hip_graph(oracle_port):
    """The entry points only launch kernels on the stream they are given, so a caller can capture a step into a
    HIP graph (d8_graph_begin / d8_graph_end): three replays, with eager work and synchronisations between
    them, must each reproduce the eager result (benchmark configuration 1's shapes, integer inputs: bit-exact)."""
    import ctypes
    from deep8_amd import capi
    from deep8_amd.capi import DeviceArray, check
    lib = capi.init()
    r = rng(2024)
    xs, ys = (1, 64, 128), (1, 128, 256)
    x, y = ints(r, xs), ints(r, ys)
    dz = ints(r, (1, 64, 256))
    want = (oracle_port.matmul(x, y), oracle_port.matmul_grad_x(x, y, dz), oracle_port.matmul_grad_y(x, y, dz))
    dx_, dy_, ddz = DeviceArray.from_numpy(x), DeviceArray.from_numpy(y), DeviceArray.from_numpy(dz)
    z_, gx_, gy_ = DeviceArray((1, 64, 256), np.float32), DeviceArray(xs, np.float32), DeviceArray(ys, np.float32)
    nb = max(lib.d8_matmul_scratch_bytes(capi.FLOAT32, w, *xs, *ys) for w in range(3))
    ws = DeviceArray((max(nb, 16),), np.uint8)

    def step(stream):
        check(lib.d8_matmul(capi.FLOAT32, dx_.ptr, *xs, dy_.ptr, *ys, z_.ptr, ws.ptr, nb, stream))
        gx_.zero_(stream)  # the fill is a kernel, not a memset node
        check(lib.d8_matmul_grad_x(capi.FLOAT32, gx_.ptr, *xs, dy_.ptr, *ys, ddz.ptr, ws.ptr, nb, stream))
        check(lib.d8_matmul_grad_y_overwrite(capi.FLOAT32, dx_.ptr, *xs, gy_.ptr, *ys, ddz.ptr, ws.ptr, nb, stream))

    side, graph = ctypes.c_void_p(), ctypes.c_void_p()
    check(lib.d8_stream_create(ctypes.byref(side)))
    assert lib.d8_graph_begin(None) == 10001  # not on the default stream
    step(side)
    capi.sync(side)
    check(lib.d8_graph_begin(side))
    step(side)
    check(lib.d8_graph_end(side, ctypes.byref(graph)))
    for replay in range(3):
        for out in (z_, gx_, gy_):
            out.copy_from(np.full(out.shape, -7.0, np.float32))
        check(lib.d8_graph_launch(graph, side))
        capi.sync(side)
        got = (z_.numpy(), gx_.numpy(), gy_.numpy())
        for g_, w_ in zip(got, want):
            assert np.array_equal(g_, w_), replay
        step(None)  # eager work between the replays
        capi.sync()
    check(lib.d8_graph_destroy(graph))
    check(lib.d8_stream_destroy(side))


def test_half_step_with_both_gradients_in_one_launch_replayed_from_a_hip_graph():
    """The same for the large half products: forward on the 256 x 256-tile kernel, d8_matmul_grad_xy as one launch of
    workgroups that walk several tiles -- captured once, replayed three times with eager calls in between, every
    replay bit for bit the eager result (3072 x 4104 x 4160: tile counts that fill neither the chip nor the XCDs
    evenly)."""
    import ctypes
    from deep8_amd import capi
    from deep8_amd.capi import DeviceArray, check
    lib = capi.init()
    r = rng(31)
    xs, ys, zs = (1, 3072, 4104), (1, 4104, 4160), (1, 3072, 4160)
    x, y, dz = h(nrm(r, xs, 1 / 64.0)), h(nrm(r, ys, 1 / 64.0)), h(nrm(r, zs, 1.0))
    dx_, dy_, ddz = DeviceArray.from_numpy(x), DeviceArray.from_numpy(y), DeviceArray.from_numpy(dz)
    z_, gx_, gy_ = DeviceArray(zs, np.float16), DeviceArray(xs, np.float16), DeviceArray(ys, np.float16)
    nb = max(lib.d8_matmul_scratch_bytes(capi.FLOAT16, w, *xs, *ys) for w in range(3))
    ws = DeviceArray((max(nb, 16),), np.uint8)

    def step(stream):
        check(lib.d8_matmul(capi.FLOAT16, dx_.ptr, *xs, dy_.ptr, *ys, z_.ptr, ws.ptr, nb, stream))
        gy_.zero_(stream)  # dY accumulates into a zeroed gradient, dX is written by the overwrite form
        check(lib.d8_matmul_grad_xy(capi.FLOAT16, dx_.ptr, gx_.ptr, *xs, dy_.ptr, gy_.ptr, *ys, ddz.ptr, 1, ws.ptr, nb, stream))

    step(None)
    capi.sync()
    want = [a.numpy().view(np.uint16).copy() for a in (z_, gx_, gy_)]
    assert all(w_.any() for w_ in want)
    side, graph = ctypes.c_void_p(), ctypes.c_void_p()
    check(lib.d8_stream_create(ctypes.byref(side)))
    check(lib.d8_graph_begin(side))
    step(side)
    check(lib.d8_graph_end(side, ctypes.byref(graph)))
    for replay in range(3):
        for out in (z_, gx_, gy_):
            out.copy_from(np.full(out.shape, -7.0, np.float16))
        check(lib.d8_graph_launch(graph, side))
        capi.sync(side)
        for out, w_ in zip((z_, gx_, gy_), want):
            assert np.array_equal(out.numpy().view(np.uint16), w_), replay
        step(None)  # eager work between the replays
        capi.sync()
    check(lib.d8_graph_destroy(graph))
    check(lib.d8_stream_destroy(side))


# Batches longer than one launch's third grid axis takes: cublas*gemmStridedBatched has no such limit
# (deep8/src/math/MatrixMultiply.cu:115-134), so neither may d8_gemm.  600 and 1000 are walked in slices.
LONG_BATCH = [
    ((600, 24, 16), (600, 16, 40)),     # F3/X3/Y3: both batched, any-shape kernel
    ((1000, 128, 32), (1000, 32, 128)),  # the same on the tiled kernel (128 x 128 outputs)
    ((1, 24, 16), (600, 16, 40)),       # x broadcast: dX is summed over the 600 products
    ((600, 24, 16), (1, 16, 40)),       # collapsed batch (one product of 14 400 rows)
]


@pytest.mark.parametrize("xs,ys", LONG_BATCH)
@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.float64])
def test_matmul_batch_beyond_one_launch(oracle, oracle_port, xs, ys, dtype):
    from deep8_amd import ops
    r = rng(sum(xs) + sum(ys) + 5)
    hi = 2 if dtype == np.float16 else 10
    x, y = ints(r, xs, hi), ints(r, ys, hi)
    if dtype == np.float16:  # keep every sum below 2048
        x, y = x * (r.random(xs) < 0.1), y * (r.random(ys) < 0.1)
    dz = ints(r, oracle_port.matmul(x, y).shape, hi)
    dx0, dy0 = ints(r, xs, hi), ints(r, ys, hi)
    c = lambda a: a.astype(dtype)
    want = (oracle_port.matmul(x, y), oracle_port.matmul_grad_x(x, y, dz, dx0), oracle_port.matmul_grad_y(x, y, dz, dy0))
    assert dtype != np.float16 or max(np.abs(w).max() for w in want) < 2048
    assert np.array_equal(f(ops.matmul(c(x), c(y))), want[0])
    assert np.array_equal(f(ops.matmul_grad_x(c(x), c(y), c(dz), c(dx0))), want[1])
    assert np.array_equal(f(ops.matmul_grad_y(c(x), c(y), c(dz), c(dy0))), want[2])
