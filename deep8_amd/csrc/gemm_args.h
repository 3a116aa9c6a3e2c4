// Argument block shared by the GEMM kernels and their host-side dispatcher.
#ifndef DEEP8_AMD_GEMM_ARGS_H
#define DEEP8_AMD_GEMM_ARGS_H

#include "common.h"

namespace d8 {

struct GemmArgs {
    const void *A;
    const void *B;
    void *C;
    float *ws;
    int M, N, K;
    int lda, ldb, ldc;
    long sA, sB, sC;
    int batch;            // independent outputs
    int red;              // products summed into each output (1 unless strideC == 0)
    int splits;           // pieces the extended reduction (red x K tiles) is cut into
    int tiles_per_split;  // K tiles per piece
    float beta;
};

// Tiled kernels (fp16 and fp32) for shapes whose operands can be moved in 16-byte pieces.
int gemm_tiled_k_step(int dtype);  // K elements per step: 64 (fp16) or 32 (fp32)
// Whether the shape qualifies (g.splits / g.tiles_per_split need not be set yet).
bool gemm_tiled_eligible(int dtype, const GemmArgs &g, int transA, int transB);
// Launch; with g.splits > 1 the fp32 partial sums go to g.ws for the caller to reduce.
int gemm_tiled_launch(int dtype, const GemmArgs &g, int transA, int transB, hipStream_t stream);

}  // namespace d8

#endif
