// Row-major fp64 GEMM for gfx950 on v_mfma_f64_16x16x4_f64: C_b = op(A_b) op(B_b) + beta C_b,
// NN / NT / TN, any size and leading dimension, strided batch with broadcast operands, optional
// summation of the whole batch into one C.  A long reduction over a small output (a filter
// gradient) is cut into pieces that write double partial sums to the caller's workspace, added up
// in a fixed order by a second kernel.
//
// One operand may be the patch matrix of a convolution read straight from its image (GemmArgs::virt, as in the
// tiled fp16 / fp32 kernels): the loads are element-wise here, so a patch element is just another address, or a
// zero outside the image.
//
// Replaces the cublasDgemm call sites of deep8/src/math/MatrixMultiply.cu, Conv2d.cu and
// DeConv2d.cu (the `double` twins of the calls listed in include/deep8_hip.h).
//
// Operand layout of the instruction (wave64): lane l supplies A[row l%16][k = l/16] and
// B[k = l/16][col l%16]; accumulator element r (0..3) of lane l is C[4*r + l/16][l%16].
#include "gemm_args.h"

namespace d8 {

typedef double f64x4 __attribute__((ext_vector_type(4)));

// BM x BN tile (64 x 64 or 128 x 128), 4 waves in a 2 x 2 arrangement, each wave WT x WT instruction
// blocks (WT = 2 or 4), K step 16.  Both LDS tiles are [row][k] with an odd row pitch, so the 16 rows
// one operand read touches fall into different banks.  Tile loads are element-wise and
// bounds-checked.  Everything that is not a matrix instruction is issued under one: the next K
// step's elements are fetched into registers before the current step is multiplied (a step is
// 4 * WT * WT matrix instructions of 64 cycles per wave, which covers the fetch) and written to the
// other half of the double-buffered LDS tiles half-way through it, and the operand fragments of
// the next group of four k are read from LDS before the current group is multiplied.  One barrier
// per K step.  The 128 x 128 tile halves the operand traffic per flop; it keeps 64 accumulator
// doubles per lane, one wave per SIMD.
template <bool TA, bool TB, int WT, int VIRT = VIRT_NONE>
__global__ __launch_bounds__(256) void gemm_f64_kernel(GemmArgs g) {
    constexpr int BM = 32 * WT, BN = 32 * WT, BK = 16, LD = 17;
    constexpr int NA = BM * BK / 256, NB = BN * BK / 256;  // elements a thread moves per K step
    constexpr bool VA = VIRT == VIRT_A_ROWS || VIRT == VIRT_A_CLASSES;  // A's rows are patch rows
    static_assert(!VA || !TA, "patch rows are rows of A");
    static_assert(VIRT != VIRT_B_KROWS || !TB, "patch k-rows are rows of B");
    __shared__ double As[2][BM * LD];
    __shared__ double Bs[2][BN * LD];

    // a class of a transposed convolution (blockIdx.z) brings its own row count, patch grid and taps
    PatchGeom pg = g.pg;
    int M = g.M, red = g.red;
    long b_cls = 0;
    int c_plane = 0, c_ow = 1, c_py = 0, c_px = 0;
    if constexpr (VIRT == VIRT_A_CLASSES) {
        const OutClass &c = g.cls[blockIdx.z];
        M = c.M, red = c.red, b_cls = c.b_off;
        pg.OH = c.OH, pg.OW = c.OW, pg.FW = c.taps_w, pg.pt = c.pt, pg.pl = c.pl;
        c_plane = c.OH * c.OW, c_ow = c.OW, c_py = c.py, c_px = c.px;
    }

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    // Which tile: workgroups are dispatched x-fastest and ids congruent mod 8 share an XCD (and its L2).  Each XCD
    // takes a contiguous run of tiles laid out in bands of 4 tile rows walked column by column, so the A and B
    // panels it re-reads are few (2048^2: 4 + 8 panels per XCD instead of 2 + 16).
    const int tilesM = gridDim.x, tilesN = gridDim.y, total = tilesM * tilesN;
    int id = blockIdx.x + tilesM * blockIdx.y;
    if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    constexpr int GM = 4;
    const int band = id / (GM * tilesN), first = band * GM;
    const int rows_in_band = min(GM, tilesM - first);
    const int in_band = id - band * GM * tilesN;
    const int m0 = (first + in_band % rows_in_band) * BM, n0 = (in_band / rows_in_band) * BN;
    if (m0 >= M) return;  // (classes: the grid is sized for the largest one)
    const int b = VIRT == VIRT_A_CLASSES ? 0 : blockIdx.z / g.splits;
    const int piece = VIRT == VIRT_A_CLASSES ? 0 : blockIdx.z - b * g.splits;

    const int ktiles = (g.K + BK - 1) / BK;
    // this workgroup's share of the extended reduction (products x K steps); a class walks all its taps
    const int t0 = piece * g.tiles_per_split;
    const int t1 = VIRT == VIRT_A_CLASSES ? red * ktiles : min(red * ktiles, t0 + g.tiles_per_split);

    f64x4 acc[WT][WT];
#pragma unroll
    for (int i = 0; i < WT; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j) acc[i][j] = f64x4{0., 0., 0., 0.};

    // element u of this thread: A (m, k) and B (n, k) inside the tile, the same for every K step
    int am[NA], ak[NA], bn[NB], bk[NB];
#pragma unroll
    for (int u = 0; u < NA; ++u) {
        const int i = tid + 256 * u;
        am[u] = TA ? i % BM : i / BK;
        ak[u] = TA ? i / BM : i % BK;
    }
#pragma unroll
    for (int u = 0; u < NB; ++u) {
        const int i = tid + 256 * u;
        bn[u] = TB ? i / BK : i % BN;
        bk[u] = TB ? i % BK : i / BN;
    }
    // patch rows as A: this thread's rows never change, a step selects the tap (product r = tap r)
    int va_iy[NA], va_ix[NA];
    long va_base[NA];
    if constexpr (VA) {
        const int plane = pg.OH * pg.OW;
#pragma unroll
        for (int u = 0; u < NA; ++u) {
            const int m = g.m_base + m0 + am[u], img = m / plane, rem = m - img * plane;
            const int oy = rem / pg.OW, ox = rem - oy * pg.OW;
            va_iy[u] = oy * pg.sy - pg.pt;
            va_ix[u] = ox * pg.sx - pg.pl;
            va_base[u] = (((long)img * pg.H + va_iy[u]) * pg.W + va_ix[u]) * pg.C;
        }
    }
    // patch k-rows as B: this thread's tap and channel never change, a step selects the patch rows
    int vb_dy[NB], vb_dx[NB], vb_c[NB];
    if constexpr (VIRT == VIRT_B_KROWS) {
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int n = n0 + bn[u], t = n / pg.C, fy = t / pg.FW, fx = t - fy * pg.FW;
            vb_c[u] = n - t * pg.C;
            vb_dy[u] = fy * pg.dy - pg.pt;
            vb_dx[u] = fx * pg.dx - pg.pl;
        }
    }
    double pa[NA], pb[NB];
    auto fetch = [&](int t) {
        const int r = t / ktiles, k0 = (t - r * ktiles) * BK;
        const double *Ap = (const double *)g.A + (VA ? 0L : (long)(b + r) * g.sA);
        const double *Bp = (const double *)g.B + (VIRT == VIRT_B_KROWS ? 0L : (long)(b + r) * g.sB);
        int tdy = 0, tdx = 0;
        long toff = 0;
        if constexpr (VA) {
            const int fy = r / pg.FW, fx = r - fy * pg.FW;
            tdy = fy * pg.dy, tdx = fx * pg.dx;
            toff = ((long)tdy * pg.W + tdx) * pg.C;
            if constexpr (VIRT == VIRT_A_CLASSES) Bp = (const double *)g.B + b_cls + fy * g.sB_row + fx * g.sB;
        }
#pragma unroll
        for (int u = 0; u < NA; ++u) {
            const int gm = m0 + am[u], gk = k0 + ak[u];
            pa[u] = 0.;
            if constexpr (VA) {
                const bool inside = (unsigned)(va_iy[u] + tdy) < (unsigned)pg.H && (unsigned)(va_ix[u] + tdx) < (unsigned)pg.W;
                if (gm < M && gk < g.K && inside) pa[u] = Ap[va_base[u] + toff + gk];
            } else {
                if (gm < M && gk < g.K) pa[u] = TA ? Ap[(long)gk * g.lda + gm] : Ap[(long)gm * g.lda + gk];
            }
        }
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int gn = n0 + bn[u], gk = k0 + bk[u];
            pb[u] = 0.;
            if constexpr (VIRT == VIRT_B_KROWS) {
                const unsigned plane = pg.OH * pg.OW, m = (unsigned)gk;
                unsigned img = __umulhi(m, pg.mg_plane), rem = m - img * plane;
                if (rem >= plane) ++img, rem -= plane;
                unsigned oy = __umulhi(rem, pg.mg_ow), ox = rem - oy * pg.OW;
                if (ox >= (unsigned)pg.OW) ++oy, ox -= pg.OW;
                const int iy = (int)oy * pg.sy + vb_dy[u], ix = (int)ox * pg.sx + vb_dx[u];
                const bool inside = (unsigned)iy < (unsigned)pg.H && (unsigned)ix < (unsigned)pg.W;
                if (gn < g.N && gk < g.K && inside) pb[u] = Bp[(((long)img * pg.H + iy) * pg.W + ix) * pg.C + vb_c[u]];
            } else {
                if (gn < g.N && gk < g.K) pb[u] = TB ? Bp[(long)gn * g.ldb + gk] : Bp[(long)gk * g.ldb + gn];
            }
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int u = 0; u < NA; ++u) As[buf][am[u] * LD + ak[u]] = pa[u];
#pragma unroll
        for (int u = 0; u < NB; ++u) Bs[buf][bn[u] * LD + bk[u]] = pb[u];
    };

    const int l16 = lane & 15, kq = lane >> 4;
    const int a_row = (wm * 16 * WT + l16) * LD + kq, b_row = (wn * 16 * WT + l16) * LD + kq;
    if (t0 < t1) {
        fetch(t0);
        stage(0);
    }
    __syncthreads();
    for (int t = t0; t < t1; ++t) {
        const bool more = t + 1 < t1;
        const int cur = (t - t0) & 1;
        if (more) fetch(t + 1);
        double fa[2][WT], fb[2][WT];
#pragma unroll
        for (int i = 0; i < WT; ++i) fa[0][i] = As[cur][a_row + i * 16 * LD];
#pragma unroll
        for (int j = 0; j < WT; ++j) fb[0][j] = Bs[cur][b_row + j * 16 * LD];
#pragma unroll
        for (int s = 0; s < BK / 4; ++s) {
            if (s + 1 < BK / 4) {
#pragma unroll
                for (int i = 0; i < WT; ++i) fa[(s + 1) & 1][i] = As[cur][a_row + i * 16 * LD + 4 * (s + 1)];
#pragma unroll
                for (int j = 0; j < WT; ++j) fb[(s + 1) & 1][j] = Bs[cur][b_row + j * 16 * LD + 4 * (s + 1)];
            }
#pragma unroll
            for (int i = 0; i < WT; ++i)
#pragma unroll
                for (int j = 0; j < WT; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[s & 1][i], fb[s & 1][j], acc[i][j], 0, 0, 0);
            if (s == 1 && more) stage(cur ^ 1);  // the other half: nobody reads it before the barrier below
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < WT; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j) {
            const int n = n0 + wn * 16 * WT + j * 16 + l16;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + wm * 16 * WT + i * 16 + 4 * r + kq;
                if (m < M && n < g.N) {
                    if (VIRT != VIRT_A_CLASSES && g.splits > 1) {  // partial sums [piece][b][M][N]
                        ((double *)g.ws)[((long)piece * g.batch + b) * g.M * g.N + (long)m * g.N + n] = acc[i][j][r];
                        continue;
                    }
                    long at = (long)m * g.ldc + n;
                    if constexpr (VIRT == VIRT_A_CLASSES) {  // row (b, y', x') of the class is an output pixel
                        const int img = m / c_plane, rem = m - img * c_plane, y = rem / c_ow, x = rem - y * c_ow;
                        at = (((long)img * g.out_H + g.out_sy * y + c_py) * g.out_W + g.out_sx * x + c_px) * g.ldc + n;
                    } else if constexpr (VIRT == VIRT_B_KROWS) {
                        if (g.perm_OC) {  // stored transposed per tap (GemmArgs::perm_OC)
                            const int t = n / g.perm_OC, oc = n - t * g.perm_OC;
                            at = ((long)oc * g.perm_T + t) * g.ldc + m;
                        }
                    }
                    double *c = (double *)g.C + (long)b * g.sC + at;
                    double v = acc[i][j][r];
                    if (g.beta != 0.f) v += *c;
                    *c = v;
                }
            }
        }
}

// C = beta C + the pieces' partial sums, piece 0 first.
__global__ __launch_bounds__(256) void gemm_f64_reduce_kernel(GemmArgs g) {
    const long mn = (long)g.M * g.N, total = mn * g.batch;
    for (long idx = (long)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (long)gridDim.x * 256) {
        const long b = idx / mn, e = idx - b * mn;
        const int m = (int)(e / g.N), n = (int)(e - (long)m * g.N);
        const double *p = (const double *)g.ws + idx;
        double v = 0.;
        for (int s = 0; s < g.splits; ++s) v += p[(long)s * total];
        long at = (long)m * g.ldc + n;
        if (g.perm_OC) {
            const int t = n / g.perm_OC, oc = n - t * g.perm_OC;
            at = ((long)oc * g.perm_T + t) * g.ldc + m;
        }
        double *c = (double *)g.C + b * g.sC + at;
        if (g.beta != 0.f) v += *c;
        *c = v;
    }
}

// Pieces for the fp64 kernel: only when 64 x 64 tiles leave most CUs idle, at least 16 K steps (256 k) per
// piece, no more than the workspace holds.
int gemm_f64_splits(int M, int N, int K, int batch, int red, size_t workspace_bytes, int *tiles_per_split) {
    const long tiles = (long)ceil_div(M, 64) * ceil_div(N, 64) * batch, cus = cu_count();
    const long total = (long)red * ceil_div(K, 16);
    long splits = tiles * 2 <= cus ? 2 * cus / tiles : 1;
    if (splits > total / 16) splits = total / 16;
    if (splits > 256) splits = 256;
    const size_t per = (size_t)batch * M * N * sizeof(double);
    if (per && splits > (long)(workspace_bytes / per)) splits = (long)(workspace_bytes / per);
    if (splits < 2) splits = 1;
    const long tps = (total + splits - 1) / splits;
    *tiles_per_split = (int)(tps < 1 ? 1 : tps);
    return tps > 0 ? (int)((total + tps - 1) / tps) : 1;
}

template <int WT>
static void launch_f64(const GemmArgs &g, int transA, int transB, hipStream_t stream) {
    dim3 grid(ceil_div(g.M, 32 * WT), ceil_div(g.N, 32 * WT), g.virt == VIRT_A_CLASSES ? g.ncls : g.batch * g.splits);
    if (g.virt == VIRT_A_ROWS && transB)
        hipLaunchKernelGGL((gemm_f64_kernel<false, true, WT, VIRT_A_ROWS>), grid, dim3(256), 0, stream, g);
    else if (g.virt == VIRT_A_ROWS)
        hipLaunchKernelGGL((gemm_f64_kernel<false, false, WT, VIRT_A_ROWS>), grid, dim3(256), 0, stream, g);
    else if (g.virt == VIRT_A_CLASSES && transB)
        hipLaunchKernelGGL((gemm_f64_kernel<false, true, WT, VIRT_A_CLASSES>), grid, dim3(256), 0, stream, g);
    else if (g.virt == VIRT_A_CLASSES)
        hipLaunchKernelGGL((gemm_f64_kernel<false, false, WT, VIRT_A_CLASSES>), grid, dim3(256), 0, stream, g);
    else if (g.virt == VIRT_B_KROWS)
        hipLaunchKernelGGL((gemm_f64_kernel<true, false, WT, VIRT_B_KROWS>), grid, dim3(256), 0, stream, g);
    else if (!transA && !transB)
        hipLaunchKernelGGL((gemm_f64_kernel<false, false, WT>), grid, dim3(256), 0, stream, g);
    else if (!transA && transB)
        hipLaunchKernelGGL((gemm_f64_kernel<false, true, WT>), grid, dim3(256), 0, stream, g);
    else
        hipLaunchKernelGGL((gemm_f64_kernel<true, false, WT>), grid, dim3(256), 0, stream, g);
}

int gemm_f64_launch(const GemmArgs &args, int transA, int transB, hipStream_t stream) {
    GemmArgs g = args;
    const bool ws_ok = g.ws && ((size_t)g.ws & 7) == 0;
    D8_REQUIRE(g.virt == VIRT_NONE || (transA ? g.virt == VIRT_B_KROWS && !transB : g.virt != VIRT_B_KROWS),
               "fp64 GEMM: a patch matrix stands for the rows of A, or for the rows of B under a transposed A");
    if (g.virt == VIRT_A_CLASSES) {  // g.M is the largest class's row count; no class is split
        D8_REQUIRE(g.ncls >= 1 && g.ncls <= MAX_CLASSES && g.batch == 1, "fp64 GEMM: %d output classes", g.ncls);
        g.splits = 1;
    } else {
        g.splits = gemm_f64_splits(g.M, g.N, g.K, g.batch, g.red, ws_ok ? g.ws_bytes : 0, &g.tiles_per_split);
    }
    D8_REQUIRE(ceil_div(g.N, 64) < 65536 && (long)g.batch * g.splits < 65536, "d8_gemm: grid too large");
    // 128 x 128 tiles when they alone fill most of the chip
    const long big = (long)ceil_div(g.M, 128) * ceil_div(g.N, 128) * (g.virt == VIRT_A_CLASSES ? g.ncls : g.batch);
    if (big >= (long)cu_count() * 3 / 4) launch_f64<4>(g, transA, transB, stream);
    else launch_f64<2>(g, transA, transB, stream);
    D8_LAUNCH_CHECK();
    if (g.splits > 1) {
        long blocks = ((long)g.M * g.N * g.batch + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(gemm_f64_reduce_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, g);
        D8_LAUNCH_CHECK();
    }
    return 0;
}

}  // namespace d8
