"""Bias and ReLu folded into the contraction (d8_matmul_bias_relu, d8_conv2d_bias_relu, d8_bias_relu_grad)
against the unfused HIP sequence (d8_matmul / d8_conv2d, d8_add, d8_relu; d8_relu_grad, d8_add_grad) and the oracle.

Integers: bit for bit in both precisions.  Float32 reals: bit for bit against the unfused sequence wherever the
product itself runs the same way, and within 1e-5 of the oracle.  Float16 reals: the fused store rounds once
where the sequence rounds three times, so they are compared with the oracle within 2e-3."""
import numpy as np
import pytest

from util import FP16_TOL, FP32_TOL, f, h, ints, nrm, rel_fro, rng, uni

pytestmark = pytest.mark.gpu

MM = [
    ((10, 400, 200), (1, 200, 304)),   # collapsed batch on the tiled kernel (store in the tile epilogue)
    ((1, 300, 100), (10, 100)),        # batch of vectors: the any-shape kernel, then the one-pass fallback
    ((6, 40, 30), (6, 30, 50)),        # batched both, small: fallback
    ((1, 64, 128), (1, 128, 256)),     # configuration 1: the small-product kernel, fallback
    ((4, 128, 96), (4, 96, 256)),      # batched on the tiled kernel
    ((1, 1024, 512), (1, 512, 512)),   # 32 tiles over K = 512: split reduction, store in the reduce kernel
    ((1, 2048, 256), (1, 256, 2048)),  # 256 x 256 tiles (fp16: the large-output kernel)
    ((32, 8, 4096), (1, 4096, 200)),   # few rows against a wide layer
    ((5, 40, 64), (1, 64)),            # a shared vector: z is [5][40], the bias runs along x's rows (40 values)
    ((5, 40, 64), (5, 64)),            # a vector per batch element, x batched as well: likewise
    ((1, 300, 128), (1, 128)),         # one matrix times one vector
]


def _ref_forward(oracle_port, z, bias, relu):
    z = z if bias is None else oracle_port.add(z, bias.reshape((1,) * 1 + bias.shape))
    return oracle_port.relu(z) if relu else z


@pytest.mark.parametrize("xs,ys", MM)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("relu,with_bias", [(True, True), (False, True), (True, False)])
def test_matmul_bias_relu(oracle_port, xs, ys, dtype, relu, with_bias):
    from deep8_amd import ops
    r = rng(sum(xs) + sum(ys) + 7)
    c = (lambda a: h(a)) if dtype == np.float16 else (lambda a: a)
    hi = 3 if dtype == np.float16 else 10
    x, y = ints(r, xs, hi) - (hi // 2), ints(r, ys, hi) - (hi // 2)  # signed, so ReLu has something to cut
    if dtype == np.float16:
        keep = 200.0 / max(xs[-1], 200)
        x = x * (r.random(xs) < keep)
    z0 = oracle_port.matmul(x, y)
    n = z0.shape[-1]
    bias = (ints(r, (n,), 7) - 3) if with_bias else None
    want = z0 if bias is None else z0 + bias
    want = np.maximum(want, 0) if relu else want
    assert dtype == np.float32 or np.abs(want).max() < 2048
    got = ops.matmul_bias_relu(c(x), c(y), None if bias is None else c(bias), relu)
    assert got.shape == want.shape and np.array_equal(f(got), want)
    # the unfused HIP sequence gives the same
    seq = ops.matmul(c(x), c(y))
    if bias is not None:
        seq = ops.add(seq, c(bias).reshape(1, n))
    if relu:
        seq = ops.relu(seq)
    assert np.array_equal(got, seq.reshape(got.shape))
    # reals
    xr, yr = c(uni(r, xs)), c(uni(r, ys))
    br = None if bias is None else c(uni(r, (n,)))
    wr = oracle_port.matmul(f(xr), f(yr))
    wr = wr if br is None else wr + f(br)
    wr = np.maximum(wr, 0) if relu else wr
    assert rel_fro(ops.matmul_bias_relu(xr, yr, br, relu), wr) <= (FP16_TOL if dtype == np.float16 else FP32_TOL)


CONV = [
    # B, IH, IW, IC, OC, FH, FW, covered, sy, sx, dy, dx
    (2, 12, 12, 64, 64, 3, 3, True, 1, 1, 1, 1),    # patch rows read by the tile loader, 64-wide tiles
    (4, 28, 28, 32, 128, 3, 3, True, 1, 1, 1, 1),   # 128-wide tiles (fp16: 32 channels -> the im2col route)
    (2, 9, 9, 3, 4, 3, 3, True, 1, 1, 1, 1),        # first layer: im2col route, fallback pass
    (1, 12, 12, 2, 3, 4, 4, False, 2, 2, 1, 1),
    (3, 16, 16, 64, 8, 3, 3, True, 2, 2, 1, 1),     # few output channels
    (32, 56, 56, 64, 64, 3, 3, True, 1, 1, 1, 1),   # configuration 4: whole rounds + split remainder band
]


@pytest.mark.parametrize("cfg", CONV)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_conv2d_bias_relu(oracle_port, cfg, dtype):
    from deep8_amd import ops
    B, IH, IW, IC, OC, FH, FW, cov, sy, sx, dy, dx = cfg
    a = (cov, sy, sx, dy, dx)
    r = rng(sum(cfg[:7]) + 11)
    c = (lambda v: h(v)) if dtype == np.float16 else (lambda v: v)
    hi = 3 if dtype == np.float16 else 6
    x, w = ints(r, (B, IH, IW, IC), hi) - (hi // 2), ints(r, (OC, FH, FW, IC), hi) - (hi // 2)
    bias = ints(r, (OC,), 9) - 4
    # the unfused HIP sequence on the same inputs (itself checked against the oracle elsewhere); at configuration 4's
    # size the oracle's direct loops would take too long for a unit test
    seq = ops.relu(ops.add(ops.conv2d(c(x), c(w), *a), c(bias).reshape(1, OC)))
    got = ops.conv2d_bias_relu(c(x), c(w), c(bias), True, *a)
    assert got.shape == seq.shape and np.array_equal(got, seq)
    assert (f(got) == 0).any() and (f(got) > 0).any()
    if B * IH * IW * IC <= 1 << 16:
        want = np.maximum(oracle_port.conv2d(x, w, *a) + bias, 0)
        assert dtype == np.float32 or np.abs(want).max() < 2048
        assert np.array_equal(f(got), want)
        xr, wr, br = c(nrm(r, x.shape)), c(nrm(r, w.shape, 0.1)), c(nrm(r, (OC,)))
        wantr = np.maximum(oracle_port.conv2d(f(xr), f(wr), *a) + f(br), 0)
        assert rel_fro(ops.conv2d_bias_relu(xr, wr, br, True, *a), wantr) <= (FP16_TOL if dtype == np.float16 else FP32_TOL)
        # bias alone, ReLu alone
        assert np.array_equal(f(ops.conv2d_bias_relu(c(x), c(w), c(bias), False, *a)), oracle_port.conv2d(x, w, *a) + bias)
        assert np.array_equal(f(ops.conv2d_bias_relu(c(x), c(w), None, True, *a)), np.maximum(oracle_port.conv2d(x, w, *a), 0))


def test_conv2d_bias_relu_float32_reals_bit_for_bit_with_the_sequence():
    """Float32: adding the bias and cutting at zero in the store rounds exactly as the separate passes do."""
    from deep8_amd import ops
    r = rng(5)
    x, w, b = nrm(r, (4, 20, 20, 64)), nrm(r, (64, 3, 3, 64), 0.1), nrm(r, (64,))
    seq = ops.relu(ops.add(ops.conv2d(x, w), b.reshape(1, 64)))
    assert np.array_equal(ops.conv2d_bias_relu(x, w, b, True), seq)


GRAD = [(1, 7), (5, 1), (33, 12), (1000, 64), (100352, 64), (4096, 200), (3, 5000), (777, 3)]


@pytest.mark.parametrize("rows,cols", GRAD)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_bias_relu_grad(oracle_port, rows, cols, dtype):
    from deep8_amd import ops
    r = rng(rows + cols)
    c = (lambda v: h(v)) if dtype == np.float16 else (lambda v: v)
    pre = nrm(r, (rows, cols))
    z = np.maximum(pre, 0)
    hi = 3 if dtype == np.float16 else 40
    dz = ints(r, (rows, cols), hi) - 1
    if dtype == np.float16 and rows > 600:
        dz = dz * (r.random(dz.shape) < 600.0 / rows)
    db0 = ints(r, (cols,), 5)
    want_dpre = oracle_port.relu_grad(pre, dz)
    want_db = oracle_port.add_grad(db0.reshape(1, cols), want_dpre, db0.reshape(1, cols)).reshape(cols)
    assert dtype == np.float32 or np.abs(want_db).max() < 2048
    for use_scratch in (True, False):
        dpre, db = ops.bias_relu_grad(c(z), c(dz), c(db0), use_scratch)
        assert np.array_equal(f(dpre), want_dpre) and np.array_equal(f(db), want_db), use_scratch
        dpre, db = ops.bias_relu_grad(c(z), c(dz), None, use_scratch, in_place=True)   # dbias written over NaN, dpre = dz
        assert np.array_equal(f(dpre), want_dpre) and np.array_equal(f(db), want_db - db0), use_scratch
    # reals: the sums are those of d8_add_grad on dpre, bit for bit
    dzr = c(nrm(r, (rows, cols)))
    dpre, db = ops.bias_relu_grad(c(z), dzr, np.zeros(cols, dtype))
    seq_dpre = ops.relu_grad(c(z), dzr, overwrite=True)
    assert np.array_equal(dpre, seq_dpre)
    seq_db = ops.add_grad(np.zeros((1, cols), dtype), seq_dpre.reshape(1, rows, cols) if rows > 1 else seq_dpre.reshape(1, cols))
    assert np.array_equal(db, seq_db.reshape(cols))
    assert rel_fro(db, f(seq_dpre).astype(np.float64).sum(axis=0)) <= (FP16_TOL if dtype == np.float16 else FP32_TOL)


def test_fused_entry_points_reject_what_they_do_not_take():
    from deep8_amd import capi
    lib = capi.init()
    a = capi.DeviceArray((64,), np.float32, zero=True)
    assert lib.d8_matmul_bias_relu(capi.FLOAT64, a.ptr, 1, 2, 2, a.ptr, 1, 2, 2, a.ptr, 1, a.ptr, None, 0, None) == 10002
    assert lib.d8_matmul_bias_relu(capi.FLOAT32, a.ptr, 1, 2, 3, a.ptr, 1, 2, 2, a.ptr, 1, a.ptr, None, 0, None) == 10001
    assert lib.d8_bias_relu_grad(capi.FLOAT32, a.ptr, a.ptr, a.ptr, None, 4, 4, 0, None, 0, None) == 10001
    assert lib.d8_bias_relu_grad(capi.FLOAT64, a.ptr, a.ptr, a.ptr, a.ptr, 4, 4, 0, None, 0, None) == 10002
