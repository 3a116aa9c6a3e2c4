// Row-major fp64 GEMM for gfx950 on v_mfma_f64_16x16x4_f64: C_b = op(A_b) op(B_b) + beta C_b,
// NN / NT / TN, any size and leading dimension, strided batch with broadcast operands, optional
// summation of the whole batch into one C.  The reduction is never split (no workspace).
//
// Replaces the cublasDgemm call sites of deep8/src/math/MatrixMultiply.cu, Conv2d.cu and
// DeConv2d.cu (the `double` twins of the calls listed in include/deep8_hip.h).
//
// Operand layout of the instruction (wave64): lane l supplies A[row l%16][k = l/16] and
// B[k = l/16][col l%16]; accumulator element r (0..3) of lane l is C[4*r + l/16][l%16].
#include "gemm_args.h"

namespace d8 {

typedef double f64x4 __attribute__((ext_vector_type(4)));

// 64 x 64 tile, 4 waves in a 2 x 2 arrangement, 32 x 32 per wave (2 x 2 instruction blocks),
// K step 16.  Both LDS tiles are [row][k] with an odd row pitch, so the 16 rows one operand read
// touches fall into different banks.  Tile loads are element-wise and bounds-checked.
template <bool TA, bool TB>
__global__ __launch_bounds__(256) void gemm_f64_kernel(GemmArgs g) {
    constexpr int BM = 64, BN = 64, BK = 16, LD = 17;
    __shared__ double As[BM * LD];
    __shared__ double Bs[BN * LD];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.x * BM, n0 = blockIdx.y * BN;
    const int b = blockIdx.z;

    const int ktiles = (g.K + BK - 1) / BK;
    const int total = g.red * ktiles;

    f64x4 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = f64x4{0., 0., 0., 0.};

    const int l16 = lane & 15, kq = lane >> 4;
    for (int t = 0; t < total; ++t) {
        const int r = t / ktiles, k0 = (t - r * ktiles) * BK;
        const double *Ap = (const double *)g.A + (long)(b + r) * g.sA;
        const double *Bp = (const double *)g.B + (long)(b + r) * g.sB;

        for (int i = tid; i < BM * BK; i += 256) {
            int m, k;
            if (!TA) {
                m = i / BK;
                k = i % BK;
            } else {
                k = i / BM;
                m = i % BM;
            }
            const int gm = m0 + m, gk = k0 + k;
            double v = 0.;
            if (gm < g.M && gk < g.K) v = TA ? Ap[(long)gk * g.lda + gm] : Ap[(long)gm * g.lda + gk];
            As[m * LD + k] = v;
        }
        for (int i = tid; i < BN * BK; i += 256) {
            int n, k;
            if (TB) {
                n = i / BK;
                k = i % BK;
            } else {
                k = i / BN;
                n = i % BN;
            }
            const int gn = n0 + n, gk = k0 + k;
            double v = 0.;
            if (gn < g.N && gk < g.K) v = TB ? Bp[(long)gn * g.ldb + gk] : Bp[(long)gk * g.ldb + gn];
            Bs[n * LD + k] = v;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; kk += 4) {
            double a[2], bb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) a[i] = As[(wm * 32 + i * 16 + l16) * LD + kk + kq];
#pragma unroll
            for (int j = 0; j < 2; ++j) bb[j] = Bs[(wn * 32 + j * 16 + l16) * LD + kk + kq];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[i], bb[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int n = n0 + wn * 32 + j * 16 + l16;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + wm * 32 + i * 16 + 4 * r + kq;
                if (m < g.M && n < g.N) {
                    double *c = (double *)g.C + (long)b * g.sC + (long)m * g.ldc + n;
                    double v = acc[i][j][r];
                    if (g.beta != 0.f) v += *c;
                    *c = v;
                }
            }
        }
}

int gemm_f64_launch(const GemmArgs &g, int transA, int transB, hipStream_t stream) {
    D8_REQUIRE(ceil_div(g.N, 64) < 65536 && g.batch < 65536, "d8_gemm: grid too large");
    dim3 grid(ceil_div(g.M, 64), ceil_div(g.N, 64), g.batch);
    if (!transA && !transB)
        hipLaunchKernelGGL((gemm_f64_kernel<false, false>), grid, dim3(256), 0, stream, g);
    else if (!transA && transB)
        hipLaunchKernelGGL((gemm_f64_kernel<false, true>), grid, dim3(256), 0, stream, g);
    else
        hipLaunchKernelGGL((gemm_f64_kernel<true, false>), grid, dim3(256), 0, stream, g);
    D8_LAUNCH_CHECK();
    return 0;
}

}  // namespace d8
