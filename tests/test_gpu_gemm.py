"""d8_gemm against the oracle's GEMM: integer inputs must match bit for bit (every partial sum is
an exactly representable integer, so summation order cannot matter -- the reference tests' own
trick, test/MatrixMultiplyTest.h:25-41); seeded real inputs must match within the tolerance."""
import numpy as np
import pytest

from util import FP16_TOL, FP32_TOL, f, h, ints, rel_fro, rng, uni

pytestmark = pytest.mark.gpu

SHAPES = [(64, 256, 128), (128, 128, 32), (1, 1, 1), (7, 5, 3), (130, 70, 33), (257, 129, 65), (33, 300, 17),
          (300, 1, 100), (1, 300, 100), (512, 512, 512)]
TRANS = [(0, 0), (0, 1), (1, 0)]


def _ab(r, ta, tb, M, N, K, gen):
    A = gen(r, (K, M) if ta else (M, K))
    B = gen(r, (N, K) if tb else (K, N))
    return A, B


@pytest.mark.parametrize("ta,tb", TRANS)
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_gemm_f32_integer_exact(oracle_port, ta, tb, M, N, K):
    from deep8_amd import ops
    r = rng(M * 7 + N * 3 + K)
    A, B = _ab(r, ta, tb, M, N, K, lambda r, s: ints(r, s, 50))
    C0 = ints(r, (M, N), 50)
    for beta, C in ((0.0, None), (1.0, C0)):
        want = oracle_port.gemm(ta, tb, A, B, C, beta)
        got = ops.gemm(ta, tb, A, B, C, beta)
        assert np.array_equal(got, want), (ta, tb, M, N, K, beta)


@pytest.mark.parametrize("ta,tb", TRANS)
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_gemm_f16_integer_exact(oracle_port, ta, tb, M, N, K):
    from deep8_amd import ops
    r = rng(M * 7 + N * 3 + K + 1)
    hi = 4 if K <= 128 else 2  # keep every result below 2048 so fp16 holds it exactly
    A, B = _ab(r, ta, tb, M, N, K, lambda r, s: ints(r, s, hi))
    C0 = ints(r, (M, N), 4)
    for beta, C in ((0.0, None), (1.0, C0)):
        want = oracle_port.gemm(ta, tb, A, B, C, beta)
        assert want.max() < 2048
        got = ops.gemm(ta, tb, h(A), h(B), None if C is None else h(C), beta)
        assert got.dtype == np.float16
        assert np.array_equal(f(got), want), (ta, tb, M, N, K, beta)


@pytest.mark.parametrize("ta,tb", TRANS)
@pytest.mark.parametrize("M,N,K", [(300, 264, 128), (136, 130, 64), (512, 520, 256), (1000, 392, 192), (304, 261, 128),
                                   (256, 256, 64), (768, 1280, 448), (1000, 64, 192), (64, 520, 256), (300, 72, 128),
                                   (96, 264, 64), (128, 64, 64), (64, 128, 128), (2000, 120, 576),
                                   # fewer rows or columns than any tile against a wide other side
                                   (32, 520, 256), (1, 256, 128), (8, 136, 64), (300, 16, 128), (48, 1000, 192), (200, 24, 64),
                                   (16, 4096, 512), (640, 8, 256)])
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_gemm_tiled_kernels_edge_tiles(oracle_port, ta, tb, M, N, K, dtype):
    """Shapes that take the tiled kernels (K a multiple of 64, rows movable in 16-byte pieces) with
    ragged last tiles in M and N: edge tiles are shifted inwards and must not double-accumulate."""
    from deep8_amd import ops
    r = rng(M + 3 * N + 7 * K)
    hi = 3 if dtype == np.float16 else 50
    A, B = _ab(r, ta, tb, M, N, K, lambda r, s: ints(r, s, hi))
    C0 = ints(r, (M, N), hi)
    c = (lambda a: h(a)) if dtype == np.float16 else (lambda a: a)
    for beta, C in ((0.0, None), (1.0, C0)):
        want = oracle_port.gemm(ta, tb, A, B, C, beta)
        assert want.max() < 2048 or dtype == np.float32
        got = ops.gemm(ta, tb, c(A), c(B), None if C is None else c(C), beta)
        assert np.array_equal(f(got), want), (ta, tb, M, N, K, beta)


@pytest.mark.parametrize("ta,tb", TRANS)
@pytest.mark.parametrize("M,N,K", [(64, 256, 128), (257, 129, 65), (512, 512, 512), (96, 80, 4099)])
def test_gemm_real_tolerance(oracle_port, ta, tb, M, N, K):
    from deep8_amd import ops
    r = rng(11 + M + N + K)
    A, B = _ab(r, ta, tb, M, N, K, uni)
    C0 = uni(r, (M, N))
    want = oracle_port.gemm(ta, tb, A, B, C0, 1.0)
    assert rel_fro(ops.gemm(ta, tb, A, B, C0, 1.0), want) <= FP32_TOL
    Ah, Bh, Ch = h(A), h(B), h(C0)
    want_h = oracle_port.gemm(ta, tb, f(Ah), f(Bh), f(Ch), 1.0)
    assert rel_fro(f(ops.gemm(ta, tb, Ah, Bh, Ch, 1.0)), want_h) <= FP16_TOL


@pytest.mark.parametrize("ta,tb", TRANS)
def test_gemm_batched_and_broadcast(oracle_port, ta, tb):
    from deep8_amd import ops
    r = rng(5)
    M, N, K, nb = 70, 45, 50, 5
    for abatch, bbatch in ((nb, nb), (1, nb), (nb, 1)):
        A = ints(r, (abatch,) + ((K, M) if ta else (M, K)))
        B = ints(r, (bbatch,) + ((N, K) if tb else (K, N)))
        C0 = ints(r, (nb, M, N))
        got = ops.gemm(ta, tb, A, B, C0, 1.0)
        for b in range(nb):
            want = oracle_port.gemm(ta, tb, A[b % abatch], B[b % bbatch], C0[b], 1.0)
            assert np.array_equal(got[b], want)


@pytest.mark.parametrize("ta,tb", TRANS)
@pytest.mark.parametrize("use_ws", [True, False])
def test_gemm_batch_summed_into_one_output(oracle_port, ta, tb, use_ws):
    """strideC == 0: all batch products accumulate into the single C (gradient of a batch-1 operand)."""
    from deep8_amd import ops
    r = rng(6)
    M, N, K, nb = 40, 33, 70, 6
    A = ints(r, (nb,) + ((K, M) if ta else (M, K)), 20)
    B = ints(r, (nb,) + ((N, K) if tb else (K, N)), 20)
    C0 = ints(r, (M, N))
    want = C0.copy()
    for b in range(nb):
        want = oracle_port.gemm(ta, tb, A[b], B[b], want, 1.0)
    got = ops.gemm(ta, tb, A, B, C0, 1.0, use_workspace=use_ws)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("use_ws", [True, False])
def test_gemm_long_reduction_split(oracle_port, use_ws):
    """Skinny output, long K: the split path (with workspace) and the single-pass path agree with the oracle."""
    from deep8_amd import ops
    r = rng(7)
    M, N, K = 64, 96, 20000
    A, B = ints(r, (K, M), 8), ints(r, (K, N), 8)
    C0 = ints(r, (M, N))
    want = oracle_port.gemm(1, 0, A, B, C0, 1.0)
    assert np.array_equal(ops.gemm(1, 0, A, B, C0, 1.0, use_workspace=use_ws), want)
    Ar, Br = uni(r, (K, M)), uni(r, (K, N))
    want = oracle_port.gemm(1, 0, Ar, Br, C0, 1.0)
    assert rel_fro(ops.gemm(1, 0, Ar, Br, C0, 1.0, use_workspace=use_ws), want) <= FP32_TOL


@pytest.mark.parametrize("ta,tb", TRANS)
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("M,N,K,nb", [(256, 384, 8192, 1), (130, 264, 4096, 1), (256, 136, 192, 7), (512, 512, 64, 12),
                                      (128, 128, 2048, 3), (64, 576, 8192, 1), (264, 64, 4096, 1), (96, 192, 128, 9)])
def test_gemm_tiled_split_and_summed(oracle_port, ta, tb, dtype, M, N, K, nb):
    """Shapes the tiled kernels take whose output has too few tiles for the chip: the reduction (all
    nb summed products of it) is cut into pieces that meet again in the fp32 workspace."""
    from deep8_amd import ops
    r = rng(M + N + K + nb)
    hi = 2 if dtype == np.float16 else 20
    c = (lambda a: h(a)) if dtype == np.float16 else (lambda a: a)
    lead = (nb,) if nb > 1 else ()
    A = ints(r, lead + ((K, M) if ta else (M, K)), hi)
    B = ints(r, lead + ((N, K) if tb else (K, N)), hi)
    if dtype == np.float16:  # thin the operands so every sum stays an exact fp16 integer
        A = A * (r.random(A.shape) < 0.15)
        B = B * (r.random(B.shape) < 0.15)
    C0 = ints(r, (M, N), 3)
    want = C0.copy()
    for b in range(nb):
        want = oracle_port.gemm(ta, tb, A[b] if nb > 1 else A, B[b] if nb > 1 else B, want, 1.0)
    assert dtype == np.float32 or np.abs(want).max() < 2048
    for use_ws in (True, False):
        got = ops.gemm(ta, tb, c(A), c(B), c(C0), 1.0, use_workspace=use_ws)
        assert np.array_equal(f(got), want), (ta, tb, M, N, K, nb, use_ws)


@pytest.mark.parametrize("ta,tb", TRANS)
@pytest.mark.parametrize("M,N,K,nb,shared_b", [(4096, 4096, 64, 1, False), (3600, 3848, 128, 1, False),
                                               (2048, 2056, 192, 4, False), (1024, 1280, 448, 16, True)])
def test_gemm_wide_f16_kernel(oracle_port, ta, tb, M, N, K, nb, shared_b):
    """fp16 outputs large enough for the 256 x 256-tile kernel (16x16x32 MFMA, loads straight into
    LDS with an exclusive-or swizzle): ragged edge tiles, beta 0 and 1, strided and shared-operand
    batches.  Integer operands, so the result is exact; numpy gives the full expected matrix and the
    oracle's GEMM confirms a band of its rows."""
    from deep8_amd import ops
    r = rng(M + 5 * N + 11 * K + nb)
    lead = (nb,) if nb > 1 else ()
    A = ints(r, lead + ((K, M) if ta else (M, K)), 3) * (r.random(lead + ((K, M) if ta else (M, K))) < 0.5)
    B = ints(r, (() if shared_b else lead) + ((N, K) if tb else (K, N)), 3)
    C0 = ints(r, lead + (M, N), 3)
    A3, B3 = (A if nb > 1 else A[None]), (B if (nb > 1 and not shared_b) else B[None])
    opA = np.swapaxes(A3, 1, 2) if ta else A3
    opB = np.swapaxes(B3, 1, 2) if tb else B3
    prod = np.matmul(opA.astype(np.float32), opB.astype(np.float32))
    assert np.abs(prod).max() + 3 < 2048
    band = slice(M - 300, M - 236)  # crosses the last, shifted tile row
    for beta in (0.0, 1.0):
        want = prod + beta * (C0 if nb > 1 else C0[None])
        got = ops.gemm(ta, tb, h(A), h(B3 if shared_b else B), h(C0), beta)
        got3 = f(got) if nb > 1 else f(got)[None]
        assert np.array_equal(got3, want), (ta, tb, M, N, K, nb, beta)
        a_band = (A3[-1][:, band] if ta else A3[-1][band]).copy()
        chk = oracle_port.gemm(ta, tb, a_band, B3[-1], (C0 if nb > 1 else C0[None])[-1][band].copy(), beta)
        assert np.array_equal(got3[-1][band], chk)


def test_gemm_argument_errors():
    from deep8_amd import capi
    lib = capi.init()
    a = capi.DeviceArray((16, 16), np.float32, zero=True)
    rc = lib.d8_gemm(capi.FLOAT32, 1, 1, 16, 16, 16, a.ptr, 16, 0, a.ptr, 16, 0, 0.0, a.ptr, 16, 0, 1, None, 0, None)
    assert rc == 10001 and b"transA" in lib.d8_last_error()
    rc = lib.d8_gemm(9, 0, 0, 16, 16, 16, a.ptr, 16, 0, a.ptr, 16, 0, 0.0, a.ptr, 16, 0, 1, None, 0, None)
    assert rc == 10002
    rc = lib.d8_gemm(capi.FLOAT32, 0, 0, 16, 16, 16, a.ptr, 8, 0, a.ptr, 16, 0, 0.0, a.ptr, 16, 0, 1, None, 0, None)
    assert rc == 10001 and b"lda" in lib.d8_last_error()
    rc = lib.d8_gemm(capi.FLOAT32, 0, 0, 16, 16, 16, a.ptr, 16, 0, a.ptr, 16, 0, 0.5, a.ptr, 16, 0, 1, None, 0, None)
    assert rc == 10001 and b"beta" in lib.d8_last_error()


def test_gemm_operand_beyond_2_gib():
    """An operand whose byte offsets do not fit 32 bits (2.15 GB) is outside what the tiled kernels' buffer
    descriptors address: the product must take the any-shape kernel's 64-bit addressing and still be exact
    (integer inputs, every partial sum below 2^24)."""
    from deep8_amd import ops
    r = rng(31)
    M, K, N = 16400, 32800, 64
    A = r.integers(0, 4, size=(M, K), dtype=np.int8).astype(np.float32)
    B = r.integers(0, 4, size=(K, N), dtype=np.int8).astype(np.float32)
    assert A.nbytes > 2**31
    got = ops.gemm(0, 0, A, B)
    assert np.array_equal(got[0] if got.ndim == 3 else got, A @ B)
    # and as the transposed operand of a TN product (rows of the result come from columns of A)
    At = A[:4100].T.copy()                      # [K x 4100]: 538 MB, fits; the 2 GiB case again through B
    Bbig = np.ascontiguousarray(A.T[:, :16384])  # [K x 16384] fp32 = 2.15 GB
    got = ops.gemm(1, 0, np.ascontiguousarray(At[:, :128]), Bbig)
    want = At[:, :128].T @ Bbig
    assert np.array_equal(got[0] if got.ndim == 3 else got, want)


@pytest.mark.parametrize("ta,tb", TRANS)
@pytest.mark.parametrize("M,N,K", [(256, 1000, 784), (300, 264, 100), (136, 130, 72), (128, 128, 40), (512, 256, 1000),
                                   (2000, 64, 200), (64, 520, 328), (1024, 1024, 4000), (32, 520, 200), (304, 16, 72), (8, 256, 1000),
                                   (300, 264, 32), (2000, 64, 8), (136, 130, 16), (64, 520, 24)])
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_gemm_reduction_not_a_multiple_of_the_k_step(ta, tb, M, N, K, dtype):
    """K ends inside a K step of the tiled kernels: what lies past K must count as zero whatever the memory there
    holds.  Operands stored along K are given a leading dimension of K + 8 with NaN in the padding, operands stored
    K-row-major are followed by rows of NaN; two products are summed into one C as well (strideC = 0), where the
    rows past K of the first are the second's."""
    from deep8_amd import capi
    lib = capi.init()
    r = rng(M + 3 * N + 7 * K)
    hi = 2 if dtype == np.float16 else 30
    dt = capi.dtype_id(np.dtype(dtype))
    for batch in (1, 2):
        A = r.integers(0, hi, size=(batch, K, M) if ta else (batch, M, K)).astype(np.float64)
        B = r.integers(0, hi, size=(batch, N, K) if tb else (batch, K, N)).astype(np.float64)
        if dtype == np.float16:  # thin the operands so that every sum stays below 2048
            A *= r.random(A.shape) < 0.3
            B *= r.random(B.shape) < 0.3
        want = np.einsum("bmk,bkn->mn", A.transpose(0, 2, 1) if ta else A, B.transpose(0, 2, 1) if tb else B)
        assert dtype == np.float32 or want.max() < 2048

        def padded(X, along_k):
            b, rows, cols = X.shape
            P = np.full((b, rows + (0 if along_k else 8), cols + (8 if along_k else 0)), np.nan)
            P[:, :rows, :cols] = X
            return P.astype(dtype)
        Ap, Bp = padded(A, not ta), padded(B, bool(tb))
        dA, dB = capi.DeviceArray.from_numpy(Ap), capi.DeviceArray.from_numpy(Bp)
        dC = capi.DeviceArray.from_numpy(np.full((M, N), np.nan, dtype))
        wsb = lib.d8_gemm_workspace_bytes(dt, ta, tb, M, N, K, batch, 0)
        ws = capi.DeviceArray((max(wsb, 16),), np.uint8)
        capi.check(lib.d8_gemm(dt, ta, tb, M, N, K, dA.ptr, Ap.shape[2], Ap.shape[1] * Ap.shape[2], dB.ptr, Bp.shape[2],
                               Bp.shape[1] * Bp.shape[2], 0.0, dC.ptr, N, 0, batch, ws.ptr, wsb, None))
        assert np.array_equal(dC.numpy().astype(np.float64), want), (ta, tb, M, N, K, batch)


@pytest.mark.parametrize("ta,tb,M,N,K", [
    (0, 0, 99304, 64, 96),     # 776 tiles of 128 rows on 256 CUs: 768 in whole rounds, a ragged band of 1000 rows
    (0, 1, 98304 + 128, 64, 64),  # a band of exactly one tile
    (0, 1, 98304 + 100, 96, 64),  # a band shorter than a tile: runs as a product of its own
    (0, 0, 131072 + 2048, 64, 32),
    (0, 1, 100352, 64, 576),   # 16 band tiles over 18 (fp32) / 9 (fp16) K steps: nine / five pieces per tile ride along
])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_gemm_tall_product_with_a_remainder_band(ta, tb, M, N, K, dtype, monkeypatch):
    """A tall product whose tile count is not a multiple of the chip's rounds: the remainder band's split pieces
    ride in the main launch (or, forced, run as a second launch); both forms, beta 0 and 1, against numpy on
    integers (exact)."""
    from deep8_amd import ops
    r = rng(M + N + K)
    c = (lambda a: h(a)) if dtype == np.float16 else (lambda a: a)
    A, B = _ab(r, ta, tb, M, N, K, lambda r, s: ints(r, s, 3))
    C0 = ints(r, (M, N), 3)
    prod = (A.T if ta else A) @ (B.T if tb else B)
    assert prod.max() < 2048
    for band_launch in (False, True):
        if band_launch:
            monkeypatch.setenv("D8_GEMM_BAND_LAUNCH", "1")  # (read at every call) the band as a second launch of its own
        for beta, C in ((0.0, None), (1.0, C0)):
            got = ops.gemm(ta, tb, c(A), c(B), None if C is None else c(C), beta)
            assert np.array_equal(f(got), prod + (0 if C is None else C)), (band_launch, beta)


@pytest.mark.gpu
def test_gemm_phase_record_of_the_tiled_kernels():
    """d8_gemm_phase_record: a tiled launch leaves one record per workgroup (clock values in order, band pieces
    marked), the product is the same with and without it, a buffer that is too small stays untouched, and null
    switches the records off."""
    from deep8_amd import capi, ops
    lib = capi.init()
    r = rng(77)
    M, N, K = 98304 + 2048, 64, 256
    A, B = ints(r, (M, K), 3), ints(r, (K, N), 3)
    want = A @ B
    nrec = 1024
    rec = capi.DeviceArray((nrec * 8,), np.uint64, zero=True)
    try:
        capi.check(lib.d8_gemm_phase_record(rec.ptr, nrec * 64))
        got = ops.gemm(0, 0, A, B)
        v = rec.numpy().astype(np.int64).reshape(nrec, 8)
        done = v[v[:, 3] != 0]
        band = done[:, 7] == 1
        assert len(done) == 768 + band.sum() and band.sum() >= 32, (len(done), band.sum())
        assert (done[:, 0] <= done[:, 1]).all() and (done[:, 1] <= done[:, 2]).all() and (done[:, 2] <= done[:, 3]).all()
        assert (done[:, 5] > done[:, 4]).all()
        assert np.array_equal(got, want)
        small = capi.DeviceArray((64,), np.uint64, zero=True)
        capi.check(lib.d8_gemm_phase_record(small.ptr, 64 * 8))  # 8 records: the launch has more workgroups
        assert np.array_equal(ops.gemm(0, 0, A, B), want)
        assert not small.numpy().any()
    finally:
        capi.check(lib.d8_gemm_phase_record(None, 0))
    rec.zero_()
    assert np.array_equal(ops.gemm(0, 0, A, B), want)
    assert not rec.numpy().any()
