// Row-major fp64 GEMM for gfx950 on v_mfma_f64_16x16x4_f64: C_b = op(A_b) op(B_b) + beta C_b,
// NN / NT / TN, any size and leading dimension, strided batch with broadcast operands, optional
// summation of the whole batch into one C.  A long reduction over a small output (a filter
// gradient) is cut into pieces that write double partial sums to the caller's workspace, added up
// in a fixed order by a second kernel.
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
template <bool TA, bool TB, int WT>
__global__ __launch_bounds__(256) void gemm_f64_kernel(GemmArgs g) {
    constexpr int BM = 32 * WT, BN = 32 * WT, BK = 16, LD = 17;
    constexpr int NA = BM * BK / 256, NB = BN * BK / 256;  // elements a thread moves per K step
    __shared__ double As[2][BM * LD];
    __shared__ double Bs[2][BN * LD];

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
    const int b = blockIdx.z / g.splits, piece = blockIdx.z - b * g.splits;

    const int ktiles = (g.K + BK - 1) / BK;
    // this workgroup's share of the extended reduction (products x K steps)
    const int t0 = piece * g.tiles_per_split, t1 = min(g.red * ktiles, t0 + g.tiles_per_split);

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
    double pa[NA], pb[NB];
    auto fetch = [&](int t) {
        const int r = t / ktiles, k0 = (t - r * ktiles) * BK;
        const double *Ap = (const double *)g.A + (long)(b + r) * g.sA;
        const double *Bp = (const double *)g.B + (long)(b + r) * g.sB;
#pragma unroll
        for (int u = 0; u < NA; ++u) {
            const int gm = m0 + am[u], gk = k0 + ak[u];
            pa[u] = 0.;
            if (gm < g.M && gk < g.K) pa[u] = TA ? Ap[(long)gk * g.lda + gm] : Ap[(long)gm * g.lda + gk];
        }
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int gn = n0 + bn[u], gk = k0 + bk[u];
            pb[u] = 0.;
            if (gn < g.N && gk < g.K) pb[u] = TB ? Bp[(long)gn * g.ldb + gk] : Bp[(long)gk * g.ldb + gn];
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
                if (m < g.M && n < g.N) {
                    if (g.splits > 1) {  // partial sums [piece][b][M][N]
                        ((double *)g.ws)[((long)piece * g.batch + b) * g.M * g.N + (long)m * g.N + n] = acc[i][j][r];
                        continue;
                    }
                    double *c = (double *)g.C + (long)b * g.sC + (long)m * g.ldc + n;
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
        double *c = (double *)g.C + b * g.sC + (long)m * g.ldc + n;
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
    dim3 grid(ceil_div(g.M, 32 * WT), ceil_div(g.N, 32 * WT), g.batch * g.splits);
    if (!transA && !transB)
        hipLaunchKernelGGL((gemm_f64_kernel<false, false, WT>), grid, dim3(256), 0, stream, g);
    else if (!transA && transB)
        hipLaunchKernelGGL((gemm_f64_kernel<false, true, WT>), grid, dim3(256), 0, stream, g);
    else
        hipLaunchKernelGGL((gemm_f64_kernel<true, false, WT>), grid, dim3(256), 0, stream, g);
}

int gemm_f64_launch(const GemmArgs &args, int transA, int transB, hipStream_t stream) {
    GemmArgs g = args;
    const bool ws_ok = g.ws && ((size_t)g.ws & 7) == 0;
    g.splits = gemm_f64_splits(g.M, g.N, g.K, g.batch, g.red, ws_ok ? g.ws_bytes : 0, &g.tiles_per_split);
    D8_REQUIRE(ceil_div(g.N, 64) < 65536 && (long)g.batch * g.splits < 65536, "d8_gemm: grid too large");
    // 128 x 128 tiles when they alone fill most of the chip
    const long big = (long)ceil_div(g.M, 128) * ceil_div(g.N, 128) * g.batch;
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
