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

// Tiled fp16 kernels for shapes whose operands can be moved in 16-byte pieces.  Returns false
// when the shape does not qualify (the caller then uses the general kernel); otherwise launches
// and stores the launch status in *rc.
bool gemm_f16_tiled(const GemmArgs &g, int transA, int transB, hipStream_t stream, int *rc);
bool gemm_f32_tiled(const GemmArgs &g, int transA, int transB, hipStream_t stream, int *rc);

}  // namespace d8

#endif
