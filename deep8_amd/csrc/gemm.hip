// Row-major GEMM for gfx950 on MFMA: C_b = op(A_b) op(B_b) + beta C_b, fp32 and fp16 (fp32
// accumulate), NN / NT / TN, strided batch with broadcast operands, optional summation of the
// whole batch into one C, and a deterministic split of the reduction through a workspace.
//
// Replaces the cuBLAS calls of deep8/src/math/MatrixMultiply.cu, Conv2d.cu and DeConv2d.cu
// (call sites listed in include/deep8_hip.h).
//
// MFMA operand layouts used throughout (wave64):
//   v_mfma_f32_32x32x16_f16 : lane l supplies A[row l%32][8 consecutive k of group l/32] and
//                             B[8 consecutive k of group l/32][col l%32]
//   v_mfma_f32_32x32x2_f32  : lane l supplies A[row l%32][k = l/32], B[k = l/32][col l%32]
//   accumulator register r of lane l is C[8*(r/4) + 4*(l/32) + r%4][l%32]
// Both LDS tiles are kept K-contiguous ([row][k]), so one 16-byte LDS read feeds an MFMA
// operand; the transposed-operand cases differ only in how the tile loader walks global memory.
#include <atomic>

#include "gemm_args.h"

namespace d8 {

template <typename T>
struct Tile;
template <>
struct Tile<f16> {
    static constexpr int BK = 32, LD = 40;
};
template <>
struct Tile<float> {
    static constexpr int BK = 16, LD = 20;
};

__device__ inline float to_f32(float v) { return v; }
__device__ inline float to_f32(f16 v) { return (float)v; }

// One wave multiplies its (TM*32) x (TN*32) sub-tile over one K tile held in LDS.
template <int TM, int TN, int LD, int BK>
__device__ inline void wave_mma(const f16 *As, const f16 *Bs, int arow, int brow, int lane,
                                f32x16 (&acc)[TM][TN]) {
    const int l32 = lane & 31, kg = (lane >> 5) * 8;
#pragma unroll
    for (int kk = 0; kk < BK; kk += 16) {
        f16x8 a[TM], b[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) a[i] = *(const f16x8 *)&As[(arow + i * 32 + l32) * LD + kk + kg];
#pragma unroll
        for (int j = 0; j < TN; ++j) b[j] = *(const f16x8 *)&Bs[(brow + j * 32 + l32) * LD + kk + kg];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
}

// fp32: an 8-wide K chunk is read as two float4 per operand row (lanes 0-31 take k 0..3,
// lanes 32-63 take k 4..7); MFMA q of the chunk then pairs k = q with k = 4 + q.  A and B use
// the same assignment, so every k is multiplied exactly once.
template <int TM, int TN, int LD, int BK>
__device__ inline void wave_mma(const float *As, const float *Bs, int arow, int brow, int lane,
                                f32x16 (&acc)[TM][TN]) {
    const int l32 = lane & 31, kg = (lane >> 5) * 4;
#pragma unroll
    for (int kk = 0; kk < BK; kk += 8) {
        f32x4 a[TM], b[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) a[i] = *(const f32x4 *)&As[(arow + i * 32 + l32) * LD + kk + kg];
#pragma unroll
        for (int j = 0; j < TN; ++j) b[j] = *(const f32x4 *)&Bs[(brow + j * 32 + l32) * LD + kk + kg];
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][q], b[j][q], acc[i][j], 0, 0, 0);
    }
}

// ------------------------------------------------------------------------------------------
// General kernel: any M, N, K, leading dimension and alignment.  128 x 128 tile, 4 waves in a
// 2 x 2 arrangement, 64 x 64 per wave; element-wise, bounds-checked tile loads.
// ------------------------------------------------------------------------------------------
template <typename T, bool TA, bool TB>
__global__ __launch_bounds__(256) void gemm_general_kernel(GemmArgs g) {
    constexpr int BM = 128, BN = 128, BK = Tile<T>::BK, LD = Tile<T>::LD;
    __shared__ __attribute__((aligned(16))) T As[2][BM * LD];
    __shared__ __attribute__((aligned(16))) T Bs[2][BN * LD];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int b = blockIdx.z / g.splits, s = blockIdx.z % g.splits;

    const int ktiles = (g.K + BK - 1) / BK;
    const int total = g.red * ktiles;
    const int t0 = s * g.tiles_per_split;
    const int t1 = min(total, t0 + g.tiles_per_split);

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // A thread moves NE elements of each operand per K step; element u is tile element tid + 256 u.  Stored
    // along K (A not transposed, B transposed): k = tid % BK for every u, row tid / BK + u * (256 / BK); stored
    // K-row-major: row or column tid % 128, k = tid / 128 + 2 u.  The next step's elements are fetched into
    // registers before the current step is multiplied and written to the other LDS half after it.
    constexpr int NE = BM * BK / 256;
    static_assert(BM == BN && 256 % BK == 0 && BM == 128, "element map");
    const int kc_k = tid % BK, kc_row = tid / BK, tr_col = tid % 128, tr_k = tid / 128;
    const bool a_in = TA ? m0 + tr_col < g.M : true, b_in = TB ? true : n0 + tr_col < g.N;
    T pa[NE], pb[NE];
    auto fetch = [&](int t) {
        const int r = t / ktiles, k0 = (t - r * ktiles) * BK;
        const T *Ap = (const T *)g.A + (long)(b + r) * g.sA;
        const T *Bp = (const T *)g.B + (long)(b + r) * g.sB;
#pragma unroll
        for (int u = 0; u < NE; ++u) {
            pa[u] = (T)0;
            if (TA) {
                const int gk = k0 + tr_k + 2 * u;
                if (a_in && gk < g.K) pa[u] = Ap[(long)gk * g.lda + m0 + tr_col];
            } else {
                const int gm = m0 + kc_row + u * (256 / BK);
                if (gm < g.M && k0 + kc_k < g.K) pa[u] = Ap[(long)gm * g.lda + k0 + kc_k];
            }
        }
#pragma unroll
        for (int u = 0; u < NE; ++u) {
            pb[u] = (T)0;
            if (TB) {
                const int gn = n0 + kc_row + u * (256 / BK);
                if (gn < g.N && k0 + kc_k < g.K) pb[u] = Bp[(long)gn * g.ldb + k0 + kc_k];
            } else {
                const int gk = k0 + tr_k + 2 * u;
                if (b_in && gk < g.K) pb[u] = Bp[(long)gk * g.ldb + n0 + tr_col];
            }
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int u = 0; u < NE; ++u) {
            if (TA) As[buf][tr_col * LD + tr_k + 2 * u] = pa[u];
            else As[buf][(kc_row + u * (256 / BK)) * LD + kc_k] = pa[u];
            if (TB) Bs[buf][(kc_row + u * (256 / BK)) * LD + kc_k] = pb[u];
            else Bs[buf][tr_col * LD + tr_k + 2 * u] = pb[u];
        }
    };

    if (t0 < t1) {
        fetch(t0);
        stage(0);
    }
    __syncthreads();
    for (int t = t0; t < t1; ++t) {
        const int cur = (t - t0) & 1;
        const bool more = t + 1 < t1;
        if (more) fetch(t + 1);
        wave_mma<2, 2, LD, BK>(As[cur], Bs[cur], wm * 64, wn * 64, lane, acc);
        if (more) stage(cur ^ 1);  // nobody reads that half before the barrier below
        __syncthreads();
    }

    const int l32 = lane & 31, lhi = lane >> 5;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int n = n0 + wn * 64 + j * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * 64 + i * 32 + (r >> 2) * 8 + lhi * 4 + (r & 3);
                if (m < g.M && n < g.N) {
                    if (g.splits == 1) {
                        T *c = (T *)g.C + (long)b * g.sC + (long)m * g.ldc + n;
                        float v = acc[i][j][r];
                        if (g.beta != 0.f) v += to_f32(*c);
                        *c = (T)v;
                    } else {
                        g.ws[((long)(b * g.splits + s) * g.M + m) * g.N + n] = acc[i][j][r];
                    }
                }
            }
        }
}

// Where element (m, n) of an output lives (GemmArgs::perm_OC: a filter gradient stored transposed per tap).
__device__ inline long c_index(const GemmArgs &g, int m, int n) {
    if (g.perm_OC) {
        const int t = n / g.perm_OC, oc = n - t * g.perm_OC;
        return ((long)oc * g.perm_T + t) * g.ldc + m;
    }
    return (long)m * g.ldc + n;
}

// ------------------------------------------------------------------------------------------
// Small products: a handful of 128 x 128 tiles would leave the chip to a few workgroups, each
// walking its whole reduction at one MFMA per 64 (fp32) cycles behind one load latency per K step.
// Here a workgroup owns a 32 x 32 tile of C and its four waves take every fourth chunk of the
// reduction each (8 k values for fp32, 16 for fp16: one MFMA operand per lane).  A lane fetches
// its operand values of ALL its chunks straight from global memory into registers before the
// first MFMA, so the whole product costs one load latency; the four partial tiles meet in LDS in
// wave order, so the result does not depend on scheduling.  Any M, N, K, leading dimension and
// alignment; element-wise, bounds-checked loads.
// ------------------------------------------------------------------------------------------
template <typename T>
struct SmallOp;
template <>
struct SmallOp<float> {
    static constexpr int PER = 4, KG = 8, MAXC = 16;  // values per lane and chunk, k per chunk, chunks per wave
    typedef f32x4 Frag;
    __device__ static void mma(const Frag &a, const Frag &b, f32x16 &acc) {
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], acc, 0, 0, 0);
    }
};
template <>
struct SmallOp<f16> {
    static constexpr int PER = 8, KG = 16, MAXC = 8;
    typedef f16x8 Frag;
    __device__ static void mma(const Frag &a, const Frag &b, f32x16 &acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc, 0, 0, 0);
    }
};

// (the work of workgroup (bx, by) of output b; part: 3 x 32 x 32 floats of LDS)
template <typename T, bool TA, bool TB>
__device__ __forceinline__ void gemm_small_body(const GemmArgs &g, const int bx, const int by, const int b, float (*part)[32 * 32]) {
    typedef SmallOp<T> OP;
    constexpr int BT = 32, PER = OP::PER, KG = OP::KG, MAXC = OP::MAXC;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lhi = lane >> 5;
    const int gm = by * BT + l32, gn = bx * BT + l32;  // this lane's row of A and column of B
    const int kchunks = (g.K + KG - 1) / KG, total = g.red * kchunks;   // total <= 4 * MAXC (gemm_is_small)

    // a K-contiguous operand whose rows can be read 16 bytes at a time gives a lane its values in one load
    const bool vec_a = !TA && g.lda % PER == 0 && g.sA % PER == 0 && g.K % PER == 0 && ((size_t)g.A & 15) == 0;
    const bool vec_b = TB && g.ldb % PER == 0 && g.sB % PER == 0 && g.K % PER == 0 && ((size_t)g.B & 15) == 0;
    typename OP::Frag fa[MAXC], fb[MAXC];
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        const int t = wave + 4 * c;
#pragma unroll
        for (int e = 0; e < PER; ++e) fa[c][e] = (T)0, fb[c][e] = (T)0;
        if (t < total) {
            const int r = t / kchunks, k0 = (t - r * kchunks) * KG + lhi * PER;
            const T *Ap = (const T *)g.A + (long)(b + r) * g.sA;
            const T *Bp = (const T *)g.B + (long)(b + r) * g.sB;
            if (vec_a) {
                if (gm < g.M && k0 < g.K) fa[c] = *(const typename OP::Frag *)(Ap + (long)gm * g.lda + k0);
            } else {
#pragma unroll
                for (int e = 0; e < PER; ++e)
                    if (gm < g.M && k0 + e < g.K) fa[c][e] = TA ? Ap[(long)(k0 + e) * g.lda + gm] : Ap[(long)gm * g.lda + k0 + e];
            }
            if (vec_b) {
                if (gn < g.N && k0 < g.K) fb[c] = *(const typename OP::Frag *)(Bp + (long)gn * g.ldb + k0);
            } else {
#pragma unroll
                for (int e = 0; e < PER; ++e)
                    if (gn < g.N && k0 + e < g.K) fb[c][e] = TB ? Bp[(long)gn * g.ldb + k0 + e] : Bp[(long)(k0 + e) * g.ldb + gn];
            }
        }
    }
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
    for (int c = 0; c < MAXC; ++c)
        if (wave + 4 * c < total) OP::mma(fa[c], fb[c], acc);

    if (wave > 0) {
#pragma unroll
        for (int r = 0; r < 16; ++r) part[wave - 1][((r >> 2) * 8 + lhi * 4 + (r & 3)) * BT + l32] = acc[r];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = (r >> 2) * 8 + lhi * 4 + (r & 3), m = by * BT + row;
            float v = acc[r];
#pragma unroll
            for (int w = 0; w < 3; ++w) v += part[w][row * BT + l32];
            if (m < g.M && gn < g.N) {
                T *c = (T *)g.C + (long)b * g.sC + (long)m * g.ldc + gn;
                if (g.beta != 0.f) v += to_f32(*c);
                *c = (T)v;
            }
        }
    }
}

template <typename T, bool TA, bool TB>
__global__ __launch_bounds__(256) void gemm_small_kernel(GemmArgs g) {
    __shared__ float part[3][32 * 32];
    gemm_small_body<T, TA, TB>(g, (int)blockIdx.x, (int)blockIdx.y, (int)blockIdx.z, part);
}

// Two small products in one launch: the first n0 = nx0 * ny0 * batch workgroups are g0's grid (NT: the gradient of
// a MatrixMultiply's first input), the rest g1's (TN: the gradient of its second).  Each of them is one load
// latency and a few matrix instructions long; what a launch of its own costs on top is most of its time.
template <typename T>
__global__ __launch_bounds__(256) void gemm_small_pair_kernel(GemmArgs g0, GemmArgs g1, int nx0, int ny0, int n0, int nx1, int ny1) {
    __shared__ float part[3][32 * 32];
    int id = (int)blockIdx.x;
    if (id < n0) {
        gemm_small_body<T, false, true>(g0, id % nx0, (id / nx0) % ny0, id / (nx0 * ny0), part);
    } else {
        id -= n0;
        gemm_small_body<T, true, false>(g1, id % nx1, (id / nx1) % ny1, id / (nx1 * ny1), part);
    }
}

// Whether a product is small in the sense above: at most four 128 x 128 tiles of output and a reduction of
// at most 512 (summed products included) in at most 64 chunks of 8.
static bool gemm_is_small(int M, int N, int K, int batch, int red) {
    return (long)ceil_div(M, 128) * ceil_div(N, 128) * batch <= 4 && (long)K * red <= 512 && (long)red * ceil_div(K, 8) <= 64 &&
           batch * 1L < 65536;
}

// C[b][m][n] = beta * C + sum_s ws[b][s][m][n].  A workgroup covers 32 groups of 4 consecutive
// outputs; its 8 thread rows each add every 8th partial (16-byte loads), and the 8 sums meet in
// LDS in a fixed order, so the result does not depend on scheduling.
template <typename T>
__device__ __forceinline__ void gemm_split_reduce_body(const GemmArgs &g, const long block, f32x4 (*part)[32]) {
    const long mn = (long)g.M * g.N;
    const int lane = threadIdx.x & 31, row = threadIdx.x >> 5;
    const long e = (block * 32 + lane) * 4;  // first of this thread's 4 outputs (N % 4 == 0)
    const bool live = e < mn * g.batch;
    const int b = live ? (int)(e / mn) : 0;
    const long r = e - (long)b * mn;
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (live) {
        const float *p = g.ws + (long)b * g.splits * mn + r;
        for (int s = row; s < g.splits; s += 8) v += *(const f32x4 *)(p + (long)s * mn);
    }
    part[row][lane] = v;
    __syncthreads();
    if (row == 0 && live) {
#pragma unroll
        for (int k = 1; k < 8; ++k) v += part[k][lane];
        const int m = (int)(r / g.N), n = (int)(r - (long)m * g.N);
        T *c0 = (T *)g.C + (long)b * g.sC;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            T *c = c0 + c_index(g, m, n + k);
            float o = v[k];
            if (g.beta != 0.f) o += to_f32(*c);
            if (g.bias) o += to_f32(((const T *)g.bias)[n + k]);
            *c = (T)(g.relu && !(o > 0.f) ? 0.f : o);
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void gemm_split_reduce_kernel(GemmArgs g) {
    __shared__ f32x4 part[8][32];
    gemm_split_reduce_body<T>(g, (long)blockIdx.x, part);
}

// The reductions of two products in one launch: the first blocks0 workgroups are g0's, the rest g1's.
template <typename T>
__global__ __launch_bounds__(256) void gemm_split_reduce_pair_kernel(GemmArgs g0, GemmArgs g1, unsigned blocks0) {
    __shared__ f32x4 part[8][32];
    if (blockIdx.x < blocks0) gemm_split_reduce_body<T>(g0, (long)blockIdx.x, part);
    else gemm_split_reduce_body<T>(g1, (long)(blockIdx.x - blocks0), part);
}

// The same for N not a multiple of 4: a workgroup covers 32 outputs; its 8 thread rows each add every 8th
// partial (four loads in flight) and the 8 sums meet in LDS in a fixed order.
template <typename T>
__global__ __launch_bounds__(256) void gemm_split_reduce_scalar_kernel(GemmArgs g) {
    __shared__ float part[8][32];
    const long mn = (long)g.M * g.N;
    const int lane = threadIdx.x & 31, row = threadIdx.x >> 5;
    const long i = (long)blockIdx.x * 32 + lane;
    const bool live = i < mn * g.batch;
    const int b = live ? (int)(i / mn) : 0;
    const long e = i - (long)b * mn;
    float v = 0.f;
    if (live) {
        const float *p = g.ws + (long)b * g.splits * mn + e;
        int s = row;
        for (; s + 24 < g.splits; s += 32) {
            float t[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) t[u] = p[(long)(s + 8 * u) * mn];
#pragma unroll
            for (int u = 0; u < 4; ++u) v += t[u];
        }
        for (; s < g.splits; s += 8) v += p[(long)s * mn];
    }
    part[row][lane] = v;
    __syncthreads();
    if (row == 0 && live) {
#pragma unroll
        for (int k = 1; k < 8; ++k) v += part[k][lane];
        const int m = (int)(e / g.N), n = (int)(e - (long)m * g.N);
        T *c = (T *)g.C + (long)b * g.sC + c_index(g, m, n);
        if (g.beta != 0.f) v += to_f32(*c);
        if (g.bias) v += to_f32(((const T *)g.bias)[n]);
        *c = (T)(g.relu && !(v > 0.f) ? 0.f : v);
    }
}

// ---- planning a product whose 128 x 128 tiles are fewer than the CUs -----------------------------------------
// Three ways to spread it: cut the reduction into s pieces per tile (a second pass adds them up), run it whole on
// 64 x 128 tiles (twice as many workgroups, no second pass), or leave it.  Rules of thumb give a first choice --
// a workgroup or two per CU, pieces of at least 8 K steps -- and a count of steps per CU decides among the
// admitted alternatives, because how the workgroups fall into rounds matters as much as how many there are: a
// CU's share is ceil(workgroups / CUs) pieces of ceil(total / s) steps plus a prologue and an epilogue each, a
// workgroup alone on its CU walks its steps about a tenth slower than two that share one, a half tile's step is
// half a step (0.65 in half precision), and the second pass costs a launch plus the s partial sums read back (at
// some 4 TB/s).  In units of a K step (about 2 us of a CU's time in fp32, 0.5 us in half): prologue + epilogue
// 2.5 / 7, second pass 2 / 14.
// Measured against it: Conv2d 14 x 14 x 256 fp32, 98 tiles over 72 steps, 36 / 48 / 36 / 30 / 36 steps per CU for
// s = 2 .. 6, ran 83.9 / 103.3 / 82.9 / 72.8 / 86.9 us; 7 x 7 x 512, 52 tiles over 144 steps, 146 / 102 / 80.7 / 116 /
// 100 us for s = 2 .. 6; 1024 x 2048 x 2048 fp32 64.9 us on half tiles against 77.4 in two pieces, 1024 x 1024 x 2048
// 63.4 us on (128) half tiles against 43.9 in four pieces.
struct FewTiles {
    long splits;         // pieces per tile (1: unsplit)
    bool half;           // unsplit on 64 x 128 tiles
    bool half_if_whole;  // were it to run unsplit (no workspace for the pieces, say): on 64 x 128 tiles rather than 128 x 128
};

static long piece_limit(long tiles, long total, int cus) {
    // Every piece costs a tile's prologue, a tile of fp32 partial sums written and read back: at least 8 K steps
    // per piece, or 4 where 8 would leave more than half of the CUs without a workgroup.
    long most = total / 8;
    if (most * tiles < cus / 2) most = total / 4;
    if (most > 512) most = 512;
    return most < 1 ? 1 : most;
}

static FewTiles plan_few_tiles(int BK, int M, int N, int batch, long total) {
    const long tiles = (long)ceil_div(M, 128) * ceil_div(N, 128) * batch, cus = cu_count();
    // the rules' choice: at most two workgroups per CU (a third one would run alone, after the rest) ...
    long rule = 2L * cus / tiles;
    // ... one per CU where its pieces are then still 32 K steps or longer: as fast, and half the partial sums (C2b's
    // dY, 512 x 512 over 16 384: 72.8 -> 70.6 us)
    if (M >= 128 && N >= 128 && total / (cus / tiles) >= 32) rule = cus / tiles;
    // (never more than two pieces per CU in all: a long reduction would otherwise be cut ever finer for an ever
    // smaller gain, and the partial sums -- at most 2 x CUs tiles of fp32, 32 MiB -- would grow with it)
    long most = piece_limit(tiles, total, (int)cus);
    if (most > 2 * cus / tiles) most = 2 * cus / tiles;
    if (rule > most) rule = most;
    if (rule < 1) rule = 1;
    const bool half_elems = BK == 64;
    const double ends = half_elems ? 7.0 : 2.5, second = half_elems ? 14.0 : 2.0;
    const double per_split = (double)M * N * batch / (half_elems ? 0.5e6 : 2e6);
    auto cost = [&](long s) {
        const long rounds = (tiles * s + cus - 1) / cus, len = (total + s - 1) / s;
        return rounds * (len * (rounds == 1 ? 1.1 : 1.0) + ends) + (s > 1 ? second + s * per_split : 0.0);
    };
    FewTiles best = {rule, false, false};
    double best_cost = cost(rule) * 0.97;  // the rules' own choice on a tie
    for (long c = 1; c <= most; ++c)
        if (cost(c) < best_cost) best.splits = c, best_cost = cost(c);
    // half tiles: a short reduction over an output that they spread over most of the chip saves the fp32 partial
    // sums, their round trip through memory and the second launch (C5's dX, 98 tiles over 16 steps: 16.8 + 10.9 us
    // in four pieces, 11.3 us whole on 196 half tiles)
    if (M >= 128 && N >= 128 && 4 * tiles >= cus) {
        const long rounds = (2 * tiles + cus - 1) / cus;
        // (a 64 x 128 tile's step against a 128 x 128 tile's: half the MFMAs; 0.65 in half, where the rest of the step weighs more)
        const double c = rounds * ((half_elems ? 0.65 : 0.5) * total * (rounds == 1 ? 1.1 : 1.0) + ends);
        best.half_if_whole = c < cost(1);
        if (c < best_cost) best.splits = 1, best.half = true;
    }
    return best;
}

bool gemm_tiled_half_tiles(int M, int N, int batch, long k_steps, int BK) {
    if (M < 128 || N < 128) return false;
    const long tiles = (long)ceil_div(M, 128) * ceil_div(N, 128) * batch;
    return tiles < cu_count() && plan_few_tiles(BK, M, N, batch, k_steps).half_if_whole;  // (asked of an unsplit product)
}

// How many pieces to cut the reduction into, for a kernel whose K step is BK.  Splitting is only
// worth a second pass when the output alone gives the 256 CUs too few tiles; the long reductions
// this catches are also the ones whose single fp32 accumulation chain would be longest.
static int plan_splits(int BK, int M, int N, int K, int batch, int red, size_t workspace_bytes, int *tiles_per_split, int virt = VIRT_NONE) {
    const bool t64 = gemm_tiled_krows_64(virt, M, N);  // 64 x 64 tiles, 37 KB of LDS each
    const long tiles = t64 ? (long)ceil_div(M, 64) * ceil_div(N, 64) * batch : (long)ceil_div(M, 128) * ceil_div(N, 128) * batch;
    const long total = (long)red * ceil_div(K, BK);
    if (gemm_is_small(M, N, K, batch, red)) {  // runs whole on gemm_small_kernel
        *tiles_per_split = (int)total;
        return 1;
    }
    const int cus = cu_count();
    long splits = 1;
    if (tiles < cus) {
        if (t64) {
            // three of the small tiles per CU (56 / 85 / 113 / 140 pieces on C4's dW: 75.6 / 73.8 / 75.0 / 78.5 us)
            splits = 3L * cus / tiles;
            const long most = piece_limit(tiles, total, cus);
            if (splits > most) splits = most;
        } else {
            const FewTiles plan = plan_few_tiles(BK, M, N, batch, total);
            splits = plan.half ? 1 : plan.splits;  // (half: the tiled kernel asks gemm_tiled_half_tiles itself)
        }
        static const char *force = getenv("D8_GEMM_SPLITS");  // tuning aid
        if (force && splits > 1) splits = atoi(force);
    }
    // no more pieces than the caller's workspace holds
    const size_t per_split = (size_t)batch * M * N * sizeof(float);
    const long fit = (long)(workspace_bytes / per_split);
    if (splits > fit) splits = fit;
    if (splits < 2) splits = 1;
    const long tps = (total + splits - 1) / splits;
    *tiles_per_split = (int)tps;
    return tps > 0 ? (int)((total + tps - 1) / tps) : 1;
}

// C = beta * C + the g.splits partial sums in g.ws (+ bias, ReLu)
template <typename T>
static int launch_reduce(const GemmArgs &g, hipStream_t stream) {
    const long total = (long)g.M * g.N * g.batch;
    if (g.N % 4 == 0 && ((size_t)g.ws & 15) == 0) {
        hipLaunchKernelGGL((gemm_split_reduce_kernel<T>), dim3((unsigned)((total / 4 + 31) / 32)), dim3(256), 0, stream, g);
    } else {
        hipLaunchKernelGGL((gemm_split_reduce_scalar_kernel<T>), dim3((unsigned)((total + 31) / 32)), dim3(256), 0, stream, g);
    }
    D8_LAUNCH_CHECK();
    return 0;
}

// The reductions that follow a launch of two products (either may be unsplit): one launch for both where both take
// the 16-byte form.
static int launch_reduce_pair(int dtype, const GemmArgs &g0, const GemmArgs &g1, hipStream_t stream) {
    const bool r0 = g0.splits > 1, r1 = g1.splits > 1;
    auto vec = [](const GemmArgs &g) { return g.N % 4 == 0 && ((size_t)g.ws & 15) == 0; };
    if (r0 && r1 && vec(g0) && vec(g1)) {
        const long b0 = ((long)g0.M * g0.N * g0.batch / 4 + 31) / 32, b1 = ((long)g1.M * g1.N * g1.batch / 4 + 31) / 32;
        if (b0 + b1 < 0x7fffffffL) {
            if (dtype == D8_FLOAT16)
                hipLaunchKernelGGL((gemm_split_reduce_pair_kernel<f16>), dim3((unsigned)(b0 + b1)), dim3(256), 0, stream, g0, g1, (unsigned)b0);
            else
                hipLaunchKernelGGL((gemm_split_reduce_pair_kernel<float>), dim3((unsigned)(b0 + b1)), dim3(256), 0, stream, g0, g1, (unsigned)b0);
            D8_LAUNCH_CHECK();
            return 0;
        }
    }
    if (r0)
        if (int rc = dtype == D8_FLOAT16 ? launch_reduce<f16>(g0, stream) : launch_reduce<float>(g0, stream)) return rc;
    if (r1)
        if (int rc = dtype == D8_FLOAT16 ? launch_reduce<f16>(g1, stream) : launch_reduce<float>(g1, stream)) return rc;
    return 0;
}

template <typename T>
static int launch(GemmArgs &g, int transA, int transB, bool tiled, hipStream_t stream) {
    if (g.virt == VIRT_NONE && g.splits == 1 && gemm_is_small(g.M, g.N, g.K, g.batch, g.red)) {
        dim3 grid(ceil_div(g.N, 32), ceil_div(g.M, 32), g.batch);
        if (!transA && !transB)
            hipLaunchKernelGGL((gemm_small_kernel<T, false, false>), grid, dim3(256), 0, stream, g);
        else if (!transA && transB)
            hipLaunchKernelGGL((gemm_small_kernel<T, false, true>), grid, dim3(256), 0, stream, g);
        else
            hipLaunchKernelGGL((gemm_small_kernel<T, true, false>), grid, dim3(256), 0, stream, g);
        D8_LAUNCH_CHECK();
        return 0;
    }
    if (tiled) {
        if (int rc = gemm_tiled_launch(sizeof(T) == 2 ? D8_FLOAT16 : D8_FLOAT32, g, transA, transB, stream)) return rc;
    } else {
        dim3 grid(ceil_div(g.N, 128), ceil_div(g.M, 128), g.batch * g.splits);
        if (!transA && !transB)
            hipLaunchKernelGGL((gemm_general_kernel<T, false, false>), grid, dim3(256), 0, stream, g);
        else if (!transA && transB)
            hipLaunchKernelGGL((gemm_general_kernel<T, false, true>), grid, dim3(256), 0, stream, g);
        else
            hipLaunchKernelGGL((gemm_general_kernel<T, true, false>), grid, dim3(256), 0, stream, g);
        D8_LAUNCH_CHECK();
    }
    return g.splits > 1 ? launch_reduce<T>(g, stream) : 0;
}

// A tall product whose output is one column of 128-row tiles (a convolution with up to 127 output
// channels: M = images x pixels) rarely gives every CU the same number of tiles: 784 tiles on 256
// CUs run as long as 1024 would.  Such a product is cut in two along M: the rows that fill whole
// rounds of the chip run unsplit, the remaining band of rows runs as a second product whose
// reduction is split so that it, too, occupies the whole chip for a fraction of a tile's time.
// Returns the rows of the first part (0: do not cut).
static int balanced_rows(const GemmArgs &g) {
    if (g.batch != 1 || g.N >= 128 || g.M < 128 || g.virt == VIRT_B_KROWS) return 0;
    const long tiles = ceil_div(g.M, 128), cus = cu_count();
    const long rest = tiles % cus;
    if (tiles < cus || rest == 0 || rest * 2 > cus) return 0;
    return (int)((tiles - rest) * 128);
}

// Pieces of a remainder band whose workgroups ride in the launch of the rows before it: they start as that launch's
// first tiles retire and cost neither a launch nor a tile's prologue on an idle chip, so they may be short -- about one
// piece per CU, two K steps at least (C4's band of 16 tiles over 18 steps: 4 / 6 / 9 pieces per tile gave
// 0.2105 / 0.2065 / 0.2060 ms per Conv2d step, 18 pieces 0.2147).  0: the band does not ride along.
static int plan_band_pieces(int BK, int rows, int N, int K, int red, size_t workspace_bytes, int *tiles_per_split) {
    if (rows < 128) return 0;
    const long total = (long)red * ceil_div(K, BK), tiles = (long)ceil_div(rows, 128) * ceil_div(N, 128);
    long tps = ceil_div(total, (long)ceil_div((long)cu_count(), tiles));
    if (tps < 2) tps = 2;
    long splits = ceil_div(total, tps);
    const long fit = (long)(workspace_bytes / ((size_t)rows * N * sizeof(float)));
    if (splits > fit) splits = fit;
    if (splits < 2) return 0;
    tps = ceil_div(total, splits);
    *tiles_per_split = (int)tps;
    return (int)ceil_div(total, tps);
}

size_t gemm_tiled_workspace(int dtype, int M, int N, int K, int red, int virt) {
    int tps = 0;
    GemmArgs probe;
    memset(&probe, 0, sizeof(probe));
    probe.M = M, probe.N = N, probe.K = K, probe.batch = 1, probe.red = red;
    const int head = balanced_rows(probe);
    const int rows = head ? M - head : M;  // with a cut, only the second part is split
    int splits = plan_splits(gemm_tiled_k_step(dtype), rows, N, K, 1, red, (size_t)-1, &tps, virt);
    if (head) {  // (the band may run either way: as pieces of the first part's launch or as a launch of its own)
        const int riding = plan_band_pieces(gemm_tiled_k_step(dtype), rows, N, K, red, (size_t)-1, &tps);
        if (riding > splits) splits = riding;
    }
    return splits > 1 ? (size_t)splits * rows * N * sizeof(float) : 0;
}

static int gemm_tiled_run_whole(int dtype, GemmArgs &g, int transA, int transB, void *workspace, size_t workspace_bytes,
                                hipStream_t stream) {
    g.ws = (float *)workspace;
    g.splits = plan_splits(gemm_tiled_k_step(dtype), g.M, g.N, g.K, g.batch, g.red, (workspace && ((size_t)workspace & 15) == 0) ? workspace_bytes : 0,
                           &g.tiles_per_split, g.virt);
    return dtype == D8_FLOAT16 ? launch<f16>(g, transA, transB, true, stream) : launch<float>(g, transA, transB, true, stream);
}

int gemm_tiled_run(int dtype, GemmArgs &g, int transA, int transB, void *workspace, size_t workspace_bytes,
                   hipStream_t stream) {
    static const bool no_cut = getenv("D8_GEMM_NO_ROW_CUT") != nullptr;  // tuning and test aid
    const int head = (no_cut || transA) ? 0 : balanced_rows(g);
    if (!head) return gemm_tiled_run_whole(dtype, g, transA, transB, workspace, workspace_bytes, stream);
    const size_t es = dtype_bytes(dtype);
    GemmArgs first = g, second = g;
    first.M = head;
    second.M = g.M - head;
    second.C = (char *)g.C + (size_t)head * g.ldc * es;
    if (g.virt == VIRT_A_ROWS) second.m_base = g.m_base + head;
    else second.A = (const char *)g.A + (size_t)head * g.lda * es;
    if (!gemm_tiled_eligible(dtype, second, transA, transB))
        return gemm_tiled_run_whole(dtype, g, transA, transB, workspace, workspace_bytes, stream);
    // The band's pieces ride in the first part's launch (GemmArgs::tail_m0) when it is split at all and is at least
    // one tile high; only its reduction is a launch of its own.
    const bool two_launches = getenv("D8_GEMM_BAND_LAUNCH") != nullptr;  // tuning and test aid (read at every call)
    second.ws = (float *)workspace;
    second.splits = (two_launches || g.splits != 1 || g.perm_OC != 0) ? 0
                    : plan_band_pieces(gemm_tiled_k_step(dtype), second.M, second.N, second.K, second.red,
                                       (workspace && ((size_t)workspace & 15) == 0) ? workspace_bytes : 0, &second.tiles_per_split);
    if (second.splits > 1) {
        GemmArgs both = g;
        both.ws = second.ws;
        both.splits = 1;
        both.tiles_per_split = g.red * ceil_div(g.K, gemm_tiled_k_step(dtype));
        both.tail_m0 = head, both.tail_splits = second.splits, both.tail_tps = second.tiles_per_split;
        if (int rc = gemm_tiled_launch(dtype, both, transA, transB, stream)) return rc;
        return dtype == D8_FLOAT16 ? launch_reduce<f16>(second, stream) : launch_reduce<float>(second, stream);
    }
    if (int rc = gemm_tiled_run_whole(dtype, first, transA, transB, nullptr, 0, stream)) return rc;
    return gemm_tiled_run_whole(dtype, second, transA, transB, workspace, workspace_bytes, stream);
}

// The two gradients of a small MatrixMultiply (g0 = dZ . Y^T, NT; g1 = X^T . dZ, TN; both small in the sense of
// gemm_is_small, neither Float64) as one launch.  False, with nothing launched, when they do not qualify.
bool gemm_small_pair_run(int dtype, const GemmArgs &g0, int ta0, int tb0, const GemmArgs &g1, int ta1, int tb1, hipStream_t stream, int *rc) {
    if (dtype == D8_FLOAT64 || ta0 || !tb0 || !ta1 || tb1) return false;
    if (g0.virt != VIRT_NONE || g1.virt != VIRT_NONE || g0.K < 1 || g1.K < 1) return false;
    if (!gemm_is_small(g0.M, g0.N, g0.K, g0.batch, g0.red) || !gemm_is_small(g1.M, g1.N, g1.K, g1.batch, g1.red)) return false;
    const int nx0 = ceil_div(g0.N, 32), ny0 = ceil_div(g0.M, 32), nx1 = ceil_div(g1.N, 32), ny1 = ceil_div(g1.M, 32);
    const long n0 = (long)nx0 * ny0 * g0.batch, n1 = (long)nx1 * ny1 * g1.batch;
    if (n0 + n1 > 0x7fffffffL) return false;
    GemmArgs a = g0, b = g1;
    a.splits = b.splits = 1;
    if (dtype == D8_FLOAT16)
        hipLaunchKernelGGL((gemm_small_pair_kernel<f16>), dim3((unsigned)(n0 + n1)), dim3(256), 0, stream, a, b, nx0, ny0, (int)n0, nx1, ny1);
    else
        hipLaunchKernelGGL((gemm_small_pair_kernel<float>), dim3((unsigned)(n0 + n1)), dim3(256), 0, stream, a, b, nx0, ny0, (int)n0, nx1, ny1);
    const hipError_t e = hipGetLastError();
    *rc = e == hipSuccess ? 0 : fail((int)e, "kernel launch: %s", hipGetErrorString(e));
    return true;
}

static std::atomic<unsigned long> pair_launches{0};  // d8_conv_grad_pair_launches

// Both gradients of a convolution as one launch (gemm_tiled_pair_launch) when that fills compute units the two
// products would each leave idle: gx is not cut into a band and not split, the workgroups of both fit the chip
// side by side (two per compute unit).  gy's reduction is split as it would be alone and reduced afterwards.
// Returns false, with nothing launched, when the pair does not qualify; *rc is the launches' status otherwise.
bool gemm_tiled_run_pair(int dtype, GemmArgs &gx, GemmArgs &gy, void *workspace, size_t workspace_bytes, hipStream_t stream, int *rc) {
    const bool off = getenv("D8_CONV_GRADS_APART") != nullptr;  // tuning and test aid (read at every call)
    if (off || dtype == D8_FLOAT64) return false;
    if (gx.virt != VIRT_A_ROWS || gy.virt != VIRT_B_KROWS || gx.batch != 1 || gy.batch != 1) return false;
    if (!gemm_tiled_eligible(dtype, gx, 0, 0) || !gemm_tiled_eligible(dtype, gy, 1, 0)) return false;
    // More workgroups than the chip holds at once (two per compute unit): in half the shared launch still gains
    // (3x3 Conv2d, B32: 56x56x64 49.9 -> 47.0 us, 14x14x256 46.0 -> 34.9, 56x56x64->128 74.2 -> 65.0; DeConv2d 4x4 s2
    // B64 14x14x256 60.7 -> 47.9), gx's remainder band riding along as it does alone.  In fp32, bound by the matrix
    // pipe, it gains 2-4 % where gx's output is narrow (fewer than 128 input channels: three workgroups of either
    // product fit a compute unit; B32 56x56x64 135.4 -> 129.7 us) and loses 8-21 % on 3x3 layers of 128 channels at
    // 28x28 (128 x 128 tiles in both products): there only a gx with a remainder band, i.e. a narrow one, pairs.
    const int head = balanced_rows(gx);
    const bool big = dtype == D8_FLOAT16 || head != 0;
    const size_t usable = (workspace && ((size_t)workspace & 15) == 0) ? workspace_bytes : 0;
    const int BK = gemm_tiled_k_step(dtype);
    int tps = 0;
    // Alone, a gx of few tiles would be cut into pieces to fill the chip; beside gy's workgroups it runs whole when
    // its reduction is short: up to 40 K steps in half, where a step waits longer than it multiplies (B16 14x14x256
    // 4x4 s2 DeConv2d: 43.3 -> 30.1 us, 3x3 Conv2d of 256 channels at B16 14x14: 45.5 -> 37.4 us); never in fp32,
    // whose steps are bound by the matrix pipe (36 steps whole: 49 -> 80 us).
    const char *lim = getenv("D8_CONV_PAIR_STEPS");  // tuning and test aid (read at every call)
    const long whole_steps = lim ? atol(lim) : (dtype == D8_FLOAT16 ? 40 : 0);
    if (plan_splits(BK, gx.M, gx.N, gx.K, 1, gx.red, usable, &tps, gx.virt) != 1 && (long)gx.red * ceil_div(gx.K, BK) > whole_steps) return false;
    gx.splits = 1, gx.tiles_per_split = gx.red * ceil_div(gx.K, BK);
    gx.ws = nullptr, gx.tail_splits = 0;
    gy.ws = (float *)workspace, gy.tail_splits = 0;
    gy.splits = plan_splits(BK, gy.M, gy.N, gy.K, 1, gy.red, usable, &gy.tiles_per_split, gy.virt);
    GemmArgs band = gx;
    if (head) {  // the band's pieces behind gy's partial sums in the workspace (the scratch query's which = 3 has room for both)
        const size_t gy_bytes = gy.splits > 1 ? ((size_t)gy.splits * gy.M * gy.N * sizeof(float) + 255) & ~(size_t)255 : 0;
        if (usable <= gy_bytes) return false;
        band.M = gx.M - head;
        band.C = (char *)gx.C + (size_t)head * gx.ldc * dtype_bytes(dtype);
        band.m_base = gx.m_base + head;
        band.ws = (float *)((char *)workspace + gy_bytes);
        band.splits = plan_band_pieces(BK, band.M, band.N, band.K, band.red, usable - gy_bytes, &band.tiles_per_split);
        if (band.splits < 2) return false;
        gx.ws = band.ws;
        gx.tail_m0 = head, gx.tail_splits = band.splits, gx.tail_tps = band.tiles_per_split;
    }
    const long wgs = gemm_tiled_pair_workgroups(dtype, gx, gy);
    if (wgs <= 0 || (wgs > 2L * cu_count() && !big)) return false;
    ++pair_launches;
    *rc = gemm_tiled_pair_launch(dtype, gx, gy, stream);
    if (!head) band.splits = 1;  // (no band: nothing of gx's to reduce)
    if (*rc == 0) *rc = launch_reduce_pair(dtype, band, gy, stream);
    return true;
}

bool gemm_tiled_run_plain_pair(int dtype, GemmArgs &g0, int ta0, int tb0, GemmArgs &g1, int ta1, int tb1, void *workspace,
                               size_t workspace_bytes, hipStream_t stream, int *rc) {
    const bool off = getenv("D8_MATMUL_GRADS_APART") != nullptr;  // tuning and test aid (read at every call)
    if (off || dtype == D8_FLOAT64 || ta0 || !tb0 || !ta1 || tb1) return false;
    if (g0.virt != VIRT_NONE || g1.virt != VIRT_NONE || g0.K < 1 || g1.K < 1) return false;
    if (!gemm_tiled_eligible(dtype, g0, ta0, tb0) || !gemm_tiled_eligible(dtype, g1, ta1, tb1)) return false;
    if (gemm_is_small(g0.M, g0.N, g0.K, g0.batch, g0.red) || gemm_is_small(g1.M, g1.N, g1.K, g1.batch, g1.red)) return false;
    if (balanced_rows(g0) || balanced_rows(g1)) return false;
    const size_t usable = (workspace && ((size_t)workspace & 15) == 0) ? workspace_bytes : 0;
    const int BK = gemm_tiled_k_step(dtype);
    // each split as it would be alone, the partial sums of the two side by side in the workspace
    g0.splits = plan_splits(BK, g0.M, g0.N, g0.K, g0.batch, g0.red, usable, &g0.tiles_per_split);
    g1.splits = plan_splits(BK, g1.M, g1.N, g1.K, g1.batch, g1.red, usable, &g1.tiles_per_split);
    const size_t need0 = g0.splits > 1 ? ((size_t)g0.splits * g0.batch * g0.M * g0.N * sizeof(float) + 255) & ~(size_t)255 : 0;
    const size_t need1 = g1.splits > 1 ? (size_t)g1.splits * g1.batch * g1.M * g1.N * sizeof(float) : 0;
    if (need0 + need1 > usable) return false;
    g0.ws = (float *)workspace, g1.ws = (float *)((char *)workspace + need0);
    g0.tail_splits = g1.tail_splits = 0;
    const long wgs = gemm_tiled_plain_pair_workgroups(dtype, g0, g1);
    if (wgs <= 0 || wgs > 2L * cu_count()) return false;
    *rc = gemm_tiled_plain_pair_launch(dtype, g0, g1, stream);
    if (*rc == 0) *rc = launch_reduce_pair(dtype, g0, g1, stream);
    return true;
}

bool gemm_fuses_store(int dtype, const GemmArgs &g, int transA, int transB) {
    // (a product beyond one launch's limits -- more than 448 outputs, more than 65535 * 128 rows -- is cut into several
    // by d8_gemm; the fused store stays out of that: the caller runs the product and one pass over its result)
    if (dtype == D8_FLOAT64 || g.K < 1 || g.beta != 0.f || g.red != 1 || g.batch > 448 || g.M > 65535 * 128) return false;
    if (g.virt == VIRT_NONE && gemm_is_small(g.M, g.N, g.K, g.batch, g.red)) return false;  // gemm_small_kernel has no fused store
    return gemm_tiled_eligible(dtype, g, transA, transB);
}

int gemm_run_fused(int dtype, GemmArgs &g, int transA, int transB, void *workspace, size_t workspace_bytes, hipStream_t stream) {
    return gemm_tiled_run(dtype, g, transA, transB, workspace, workspace_bytes, stream);
}

}  // namespace d8

using namespace d8;

extern "C" {

size_t d8_gemm_workspace_bytes(int dtype, int transA, int transB, int M, int N, int K,
                               int batch, long strideC) {
    (void)transA;
    (void)transB;
    if (M <= 0 || N <= 0 || K <= 0 || batch <= 0) return 0;
    const int red = (strideC == 0 && batch > 1) ? batch : 1;
    const int outs = red > 1 ? 1 : batch;
    if (dtype == D8_FLOAT64) {
        int tps64 = 0;
        const int pieces = gemm_f64_splits(M, N, K, outs, red, (size_t)-1, &tps64);
        return pieces > 1 ? (size_t)pieces * outs * M * N * sizeof(double) : 0;
    }
    // whichever kernel ends up running, the larger of the two plans fits
    int tps = 0;
    const int a = plan_splits(gemm_tiled_k_step(dtype), M, N, K, outs, red, (size_t)-1, &tps);
    const int b = plan_splits(dtype == D8_FLOAT16 ? Tile<f16>::BK : Tile<float>::BK, M, N, K, outs, red, (size_t)-1, &tps);
    const int splits = a > b ? a : b;
    const size_t whole = splits > 1 ? (size_t)splits * outs * M * N * sizeof(float) : 0;
    const size_t band = outs == 1 ? gemm_tiled_workspace(dtype, M, N, K, red) : 0;  // a tall product's remainder band, split
    return whole > band ? whole : band;
}

// One product whose grid fits the launch limits (at most MAX_BATCH independent outputs, at most MAX_ROWS rows).
static int gemm_one(int dtype, int transA, int transB, int M, int N, int K,
                    const void *A, int lda, long strideA, const void *B, int ldb, long strideB,
                    float beta, void *C, int ldc, long strideC, int batch,
                    void *workspace, size_t workspace_bytes, void *stream) {
    GemmArgs g;
    memset(&g, 0, sizeof(g));
    g.A = A;
    g.B = B;
    g.C = C;
    g.ws = (float *)workspace;
    g.ws_bytes = workspace_bytes;
    g.M = M;
    g.N = N;
    g.K = K;
    g.lda = lda;
    g.ldb = ldb;
    g.ldc = ldc;
    g.sA = strideA;
    g.sB = strideB;
    g.sC = strideC;
    g.beta = beta;
    g.red = (strideC == 0 && batch > 1) ? batch : 1;
    g.batch = g.red > 1 ? 1 : batch;
    g.splits = 1;
    g.tiles_per_split = 0;
    g.virt = VIRT_NONE;
    g.m_base = 0;
    memset(&g.pg, 0, sizeof(g.pg));
    if (dtype == D8_FLOAT64) return gemm_f64_launch(g, transA, transB, as_stream(stream));
    const bool tiled = K > 0 && gemm_tiled_eligible(dtype, g, transA, transB);
    // the tiled kernels' own driver plans the split and cuts a tall product's remainder band
    if (tiled && !gemm_is_small(M, N, K, g.batch, g.red)) return gemm_tiled_run(dtype, g, transA, transB, workspace, workspace_bytes, as_stream(stream));
    if (K > 0) {  // K == 0 is the empty reduction: C = beta * C
        const int BK = tiled ? gemm_tiled_k_step(dtype) : (dtype == D8_FLOAT16 ? Tile<f16>::BK : Tile<float>::BK);
        g.splits = plan_splits(BK, M, N, K, g.batch, g.red, (workspace && ((size_t)workspace & 15) == 0) ? workspace_bytes : 0, &g.tiles_per_split);
    }
    return dtype == D8_FLOAT16 ? launch<f16>(g, transA, transB, tiled, as_stream(stream))
                               : launch<float>(g, transA, transB, tiled, as_stream(stream));
}

unsigned long d8_conv_grad_pair_launches(void) { return pair_launches.load(); }

int d8_gemm_phase_record(void *records, size_t bytes) {
    D8_REQUIRE(((size_t)records & 7) == 0, "d8_gemm_phase_record: the record buffer is not 8-byte aligned");
    gemm_tiled_phase_record(records, bytes);
    return 0;
}

int d8_gemm(int dtype, int transA, int transB, int M, int N, int K,
            const void *A, int lda, long strideA,
            const void *B, int ldb, long strideB,
            float beta, void *C, int ldc, long strideC, int batch,
            void *workspace, size_t workspace_bytes, void *stream) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32 && dtype != D8_FLOAT64)
        return fail(D8_ERR_DTYPE, "d8_gemm: element type %d is not supported", dtype);
    D8_REQUIRE(!(transA && transB), "d8_gemm: transA and transB together are not supported");
    D8_REQUIRE(M >= 0 && N >= 0 && K >= 0 && batch >= 0, "d8_gemm: negative size");
    D8_REQUIRE(beta == 0.f || beta == 1.f, "d8_gemm: beta must be 0 or 1");
    if (M == 0 || N == 0 || batch == 0) return 0;
    D8_REQUIRE(A && B && C, "d8_gemm: null operand");
    D8_REQUIRE(lda >= (transA ? M : K), "d8_gemm: lda %d too small", lda);
    D8_REQUIRE(ldb >= (transB ? K : N), "d8_gemm: ldb %d too small", ldb);
    D8_REQUIRE(ldc >= N, "d8_gemm: ldc %d too small", ldc);
    D8_REQUIRE(strideA >= 0 && strideB >= 0 && strideC >= 0, "d8_gemm: negative stride");
    D8_REQUIRE(dtype != D8_FLOAT64 || (long)ceil_div(N, 64) < 65536, "d8_gemm: N = %d is beyond the %d columns a Float64 launch covers", N, 65535 * 64);

    // A launch covers at most 65535 workgroups along its second and third axes.  A longer batch of independent
    // products and a taller matrix are walked in slices, each an ordinary product on advanced pointers (the
    // slices run one after the other on the stream, so they may share the workspace).
    constexpr int MAX_BATCH = 448;            // independent outputs per launch (the tiled kernels take fewer than 512)
    constexpr int MAX_ROWS = 65535 * 128;     // rows of C per launch
    const size_t es = dtype_bytes(dtype);
    const bool summed = strideC == 0 && batch > 1;
    const int nb = summed ? 1 : ceil_div(batch, MAX_BATCH), per_b = summed ? batch : ceil_div(batch, nb);
    const int nm = ceil_div(M, MAX_ROWS);
    const int per_m = nm > 1 ? (ceil_div(ceil_div(M, nm), 128) * 128) : M;
    for (int b0 = 0; b0 < batch; b0 += per_b) {
        const int bn = batch - b0 < per_b ? batch - b0 : per_b;
        for (int m0 = 0; m0 < M; m0 += per_m) {
            const int mn = M - m0 < per_m ? M - m0 : per_m;
            const char *a = (const char *)A + ((size_t)b0 * strideA + (transA ? (size_t)m0 : (size_t)m0 * lda)) * es;
            const char *b = (const char *)B + (size_t)b0 * strideB * es;
            char *c = (char *)C + ((size_t)b0 * strideC + (size_t)m0 * ldc) * es;
            if (int rc = gemm_one(dtype, transA, transB, mn, N, K, a, lda, strideA, b, ldb, strideB, beta, c, ldc, strideC, bn,
                                  workspace, workspace_bytes, stream))
                return rc;
        }
    }
    return 0;
}

}  // extern "C"
