// Measurement aid: the rate the matrix pipe sustains on given operand bits when nothing else
// runs -- no LDS, no global loads in the loop.  The GEMM kernels' MFMA instruction
// (v_mfma_f32_16x16x32_f16 as an 8 x 8 block per wave, one wave per SIMD, accumulators in AGPRs,
// like the fp16 kernel for large outputs; v_mfma_f32_32x32x2_f32 as 2 x 4, two waves per SIMD,
// like the fp32 tiles; v_mfma_f64_16x16x4_f64 as 2 x 2, four waves per SIMD) is issued back to back on operands held in registers, on every CU.  The achievable clock
// under matrix load depends on how many operand bits toggle, so this gives the ceiling any GEMM
// kernel has on that data (it is well below the nominal peak for real-valued operands).
#include "common.h"

namespace d8 {

// A wave keeps 2 A and 4 B fragments per set and cycles through SETS sets, so that the operand
// registers differ from one MFMA to the next as they do in a GEMM.
template <typename E>
struct StreamOp;
template <>
struct StreamOp<float> {
    typedef float Frag;
    static constexpr double FLOPS = 2.0 * 32 * 32 * 2;
    __device__ static f32x16 mfma(Frag a, Frag b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }
};

template <typename E, int SETS>
__global__ __launch_bounds__(256) void mfma_stream_kernel(const typename StreamOp<E>::Frag *data, unsigned nfrag,
                                                          float *out, int iters) {
    typedef StreamOp<E> Op;
    const unsigned t = blockIdx.x * 256 + threadIdx.x;
    typename Op::Frag a[SETS][2], b[SETS][4];
#pragma unroll
    for (int s = 0; s < SETS; ++s) {
#pragma unroll
        for (int i = 0; i < 2; ++i) a[s][i] = data[(t * 6 * SETS + s * 6 + i) % nfrag];
#pragma unroll
        for (int j = 0; j < 4; ++j) b[s][j] = data[(t * 6 * SETS + s * 6 + 2 + j) % nfrag];
    }
    f32x16 acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int s = 0; s < SETS; ++s)
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = Op::mfma(a[s][i], b[s][j], acc[i][j]);
    }
    float v = 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) v += acc[i][j][r];
    out[t] = v;
}

// fp16: 8 A and 8 B fragments, 64 accumulator blocks pinned to AGPRs and updated in place.
__global__ __launch_bounds__(256) void mfma_stream_f16_kernel(const f16x8 *data, unsigned nfrag, float *out, int iters) {
    const unsigned t = blockIdx.x * 256 + threadIdx.x;
    f16x8 a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = data[(t * 16 + i) % nfrag];
        b[i] = data[(t * 16 + 8 + i) % nfrag];
    }
    f32x4 acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
            asm volatile("" : "+a"(acc[i][j]));
        }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j)
                asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(a[i]), "v"(b[j]));
    }
    float v = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) v += acc[i][j][r];
    out[t] = v;
}

// fp64: 2 A and 2 B fragments, 4 accumulator blocks per wave, four waves per SIMD: the arrangement
// that issues v_mfma_f64_16x16x4_f64 fastest (a single wave per SIMD with 4 x 4 blocks, the
// 128 x 128 tile's shape, streams a quarter slower: consecutive fp64 matrix instructions of one
// wave do not issue back to back).
typedef double f64x4s __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void mfma_stream_f64_kernel(const double *data, unsigned nfrag, float *out, int iters) {
    const unsigned t = blockIdx.x * 256 + threadIdx.x;
    double a[2], b[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        a[i] = data[(t * 4 + i) % nfrag];
        b[i] = data[(t * 4 + 2 + i) % nfrag];
    }
    f64x4s acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = f64x4s{0., 0., 0., 0.};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    double v = 0.;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) v += acc[i][j][r];
    out[t] = (float)v;
}

}  // namespace d8

using namespace d8;

extern "C" {

size_t d8_mfma_stream_out_bytes(void) { return (size_t)cu_count() * 4 * 256 * sizeof(float); }  // the fp64 stream: 4 blocks per CU

int d8_mfma_stream(int dtype, const void *operands, size_t operand_bytes, void *out, int iters, double *flops, void *stream) {
    D8_REQUIRE(dtype == D8_FLOAT16 || dtype == D8_FLOAT32 || dtype == D8_FLOAT64, "dtype %d not supported", dtype);
    D8_REQUIRE(operands && out && flops, "null argument");
    D8_REQUIRE(((size_t)operands & 15) == 0 && operand_bytes >= 16, "operands must be 16-byte aligned and hold 16 bytes or more");
    D8_REQUIRE(iters > 0, "iters must be positive");
    constexpr int SETS = 4;
    const int blocks = cu_count() * 2;
    const size_t frag = dtype == D8_FLOAT16 ? 16 : dtype == D8_FLOAT64 ? 8 : 4;
    const size_t nfrag = operand_bytes / frag;
    D8_REQUIRE(nfrag < (1ull << 32), "at most 2^32 fragments");
    if (dtype == D8_FLOAT16) {
        hipLaunchKernelGGL(mfma_stream_f16_kernel, dim3(blocks / 2), dim3(256), 0, as_stream(stream), (const f16x8 *)operands,
                           (unsigned)nfrag, (float *)out, iters);
        *flops = 2.0 * 16 * 16 * 32 * 64 * iters * 4.0 * (blocks / 2);
    } else if (dtype == D8_FLOAT64) {
        hipLaunchKernelGGL(mfma_stream_f64_kernel, dim3(blocks * 2), dim3(256), 0, as_stream(stream), (const double *)operands,
                           (unsigned)nfrag, (float *)out, iters);
        *flops = 2.0 * 16 * 16 * 4 * 4 * iters * 4.0 * (blocks * 2);
    } else {
        hipLaunchKernelGGL((mfma_stream_kernel<float, SETS>), dim3(blocks), dim3(256), 0, as_stream(stream), (const float *)operands,
                           (unsigned)nfrag, (float *)out, iters);
        *flops = StreamOp<float>::FLOPS * 8 * SETS * iters * 4.0 * blocks;
    }
    D8_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
