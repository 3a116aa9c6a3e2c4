// Argument block shared by the GEMM kernels and their host-side dispatcher.
#ifndef DEEP8_AMD_GEMM_ARGS_H
#define DEEP8_AMD_GEMM_ARGS_H

#include "common.h"

namespace d8 {

// A patch matrix that is never written out: row m = (b, oy, ox) enumerates an OH x OW grid per
// image, column (t, c) is channel c of filter tap t = fy * FW + fx, and the element is
//   image[b][oy * sy + fy * dy - pt][ox * sx + fx * dx - pl][c]      (0 outside the image).
// dy, dx, pt, pl may be negative, which expresses the gradient-side gather of a stride-1
// convolution (source row = iy + pt - fy * dy) with the same formula.
struct PatchGeom {
    int H, W, C;    // the image [B][H][W][C] the patches are cut from
    int OH, OW;     // the grid the rows enumerate
    int FW;         // taps per filter row
    int sy, sx, dy, dx, pt, pl;
    unsigned mg_plane, mg_ow;  // floor(2^32 / (OH * OW)), floor(2^32 / OW): division by multiplication
    unsigned bytes;            // size of the image
};

enum { VIRT_NONE = 0, VIRT_A_ROWS = 1, VIRT_B_KROWS = 2, VIRT_A_CLASSES = 3 };

// A strided transposed convolution, output pixel by output pixel: the output pixels whose
// coordinates have one residue (py, px) modulo the stride form a class; a class is an ordinary
// stride-1 patch product over the taps fy = f0y + sy * j, fx = f0x + sx * i that reach it:
//   z[b][sy * y' + py][sx * x' + px][:] = sum over (j, i) of x[b][y' + j - pt][x' + i - pl][:] . w[:][fy][fx][:]
// VIRT_A_CLASSES runs all classes in one launch (blockIdx.z = class): the patch grid, the taps, the
// filter slice and the rows of C a class writes come from its OutClass, everything else from GemmArgs.
struct OutClass {
    int M;             // rows (b, y', x') of the class
    int OH, OW;        // its grid of (y', x')
    int taps_w, red;   // taps per filter row that reach it, and in all
    int pt, pl;        // patch origin (may be negative)
    int py, px;        // residue: output pixel = (sy * y' + py, sx * x' + px)
    unsigned b_off;    // element offset of the filter slice of its first tap (f0y, f0x)
};
enum { MAX_CLASSES = 16 };

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
    // Implicit convolution: one operand is a patch matrix read straight from the image.
    //   VIRT_A_ROWS   A is the image; product r of the `red` summed products is filter tap r, its
    //                 A[m][k] = channel k of tap r of patch row m (K = channels per tap)
    //   VIRT_B_KROWS  B is the image; B[k][n] = column n of patch row k (N = taps x channels)
    int virt;
    PatchGeom pg;
    int m_base;  // VIRT_A_ROWS: row 0 of this product is patch row m_base (a product over a band of rows)
    // VIRT_A_CLASSES: product (j, i) of a class reads B at b_off + j * sB_row + i * sB; row (b, y', x') of
    // the class is row ((b * out_H + out_sy * y' + py) * out_W + out_sx * x' + px) of C
    long sB_row;
    int out_H, out_W, out_sy, out_sx;
    int ncls;
    OutClass cls[MAX_CLASSES];
    // perm_OC > 0: the result is stored transposed per filter tap: element (m, n = t * perm_OC + oc) of the
    // product goes to C[(oc * perm_T + t) * ldc + m] (a filter gradient [OC][taps][IC] computed as [IC][taps x OC])
    int perm_T, perm_OC;
    // measurement aid (gemm_wide only, set by its launcher when the environment asks for it and a workspace
    // is given): every workgroup records when its prologue, K loop and epilogue ended into ws
    int stamps;
    size_t ws_bytes;  // size of ws as d8_gemm received it (0 where a planner filled the block in)
    // Fused store (the tiled kernels, the large-output fp16 kernel and the split reduction): after the product
    // (and beta * C), column n of the result gets bias[n] added (bias: N elements of C's type, may be null),
    // then negative values become 0 when relu is set.  What Add (a per-column bias broadcast over the rows) and
    // ReLu do as separate passes over C in the reference (deep8/src/math/Add.cu:21-52, ReLu.cu:20-59).
    const void *bias;
    int relu;
    // Remainder band in the same launch (tail_splits > 0; unsplit, unbatched products only): rows tail_m0 .. M - 1
    // are not tiled by the launch's first tiles(tail_m0) x tiles(N) workgroups but by further ones, tail_splits per
    // tile, each walking tail_tps K steps and writing fp32 partial sums to ws[piece][row - tail_m0][n].  They start
    // as the first workgroups retire, so the band costs a fraction of a tile's time instead of a launch of its own.
    int tail_m0, tail_splits, tail_tps;
    // measurement aid of the tiled kernels (d8_gemm_phase_record): when set, every workgroup writes eight 64-bit words
    // at index blockIdx.x + gridDim.x * blockIdx.z -- the chip's 100 MHz wall clock at its start, after its prologue,
    // after its K loop and after its last store was acknowledged, the shader clock at both ends of the loop, its
    // placement (XCC_ID << 32 | HW_ID) and, in the last word, whether it worked on the remainder band (bit 0) and which
    // product of a launch of two it belongs to (bit 1: gemm_tiled_pair_launch's gx)
    unsigned long long *phase_rec;
};

// Whether a product with these arguments would run on a kernel that applies GemmArgs::bias / relu in its store
// (else the caller runs the plain product and launch_bias_relu).
bool gemm_fuses_store(int dtype, const GemmArgs &g, int transA, int transB);
// The product of d8_gemm (beta = 0, no summed batch) with the fused store; the shape must pass gemm_fuses_store.
int gemm_run_fused(int dtype, GemmArgs &g, int transA, int transB, void *workspace, size_t workspace_bytes, hipStream_t stream);
// z[r][c] = relu?(z[r][c] + bias[c]) in place, one pass (bias may be null): the fallback for shapes the fused store does not take.
int launch_bias_relu(int dtype, void *z, const void *bias, long rows, int cols, int relu, hipStream_t stream);

// Tiled kernels (fp16 and fp32) for shapes whose operands can be moved in 16-byte pieces.
int gemm_tiled_k_step(int dtype);  // K elements per step: 64 (fp16) or 32 (fp32)
// Whether the shape qualifies (g.splits / g.tiles_per_split need not be set yet).
bool gemm_tiled_eligible(int dtype, const GemmArgs &g, int transA, int transB);
// Launch; with g.splits > 1 the fp32 partial sums go to g.ws for the caller to reduce.
int gemm_tiled_launch(int dtype, const GemmArgs &g, int transA, int transB, hipStream_t stream);
// Two patch-matrix products as ONE launch: gx with patch rows as A (NN: a convolution's gradient of its input), gy with
// patch k-rows as B (TN: its filter gradient; g.splits / tiles_per_split set, the caller reduces).  Workgroups of
// both are resident side by side.  gemm_tiled_pair_workgroups: how many workgroups the launch would have, 0 when the
// pair cannot run this way (the tiles the two products would choose have no common kernel, or one is cut into a band).
long gemm_tiled_pair_workgroups(int dtype, const GemmArgs &gx, const GemmArgs &gy);
int gemm_tiled_pair_launch(int dtype, const GemmArgs &gx, const GemmArgs &gy, hipStream_t stream);
// The same for two real products: g0 NT, g1 TN (the two gradients of a MatrixMultiply), each batched or split as planned
// (g.splits / tiles_per_split / ws set; the caller reduces).
long gemm_tiled_plain_pair_workgroups(int dtype, const GemmArgs &g0, const GemmArgs &g1);
int gemm_tiled_plain_pair_launch(int dtype, const GemmArgs &g0, const GemmArgs &g1, hipStream_t stream);
// Where the next launches write their per-workgroup phase records (GemmArgs::phase_rec); null switches them off.
void gemm_tiled_phase_record(void *records, size_t bytes);

// fp16 kernel for large outputs (256 x 256 tiles, v_mfma_f32_16x16x32_f16, loads straight into
// LDS): unsplit, unsummed products of real matrices with M, N >= 256 and K a multiple of 64.
bool gemm_wide_eligible(const GemmArgs &g, int transA, int transB);
int gemm_wide_launch(const GemmArgs &g, int transA, int transB, hipStream_t stream);
// Two such products (each eligible) as ONE launch: a workgroup that has finished a tile of the first goes on to a
// tile of the second without the kernel boundary in between (the end of one launch -- the write of the whole of
// C, the wait for its acknowledgement, the gap -- and the start of the next, whose first operand bytes come from
// memory).  Built for the two gradients of a MatrixMultiply, which are independent of each other.
int gemm_wide_pair_launch(const GemmArgs &g0, int transA0, int transB0, const GemmArgs &g1, int transA1, int transB1,
                          hipStream_t stream);

// The two gradients of a small MatrixMultiply (NT then TN, both on the small-product kernel) as ONE launch; false, with
// nothing launched, when they do not qualify.
bool gemm_small_pair_run(int dtype, const GemmArgs &g0, int ta0, int tb0, const GemmArgs &g1, int ta1, int tb1, hipStream_t stream, int *rc);

// fp64 kernel (64 x 64 or 128 x 128 tiles, v_mfma_f64_16x16x4_f64): any shape; plans its own split of the
// reduction from g.ws / g.ws_bytes (double partial sums) and reduces.
int gemm_f64_launch(const GemmArgs &g, int transA, int transB, hipStream_t stream);
// Pieces it would cut the reduction into given that much workspace.
int gemm_f64_splits(int M, int N, int K, int batch, int red, size_t workspace_bytes, int *tiles_per_split);

// Whether an unsplit product of this shape should run on 64 x 128 tiles: too few 128 x 128 tiles
// for the chip, enough half-height ones, and a reduction (k_steps K steps in all) too short to
// be worth splitting.
bool gemm_tiled_half_tiles(int M, int N, int batch, long k_steps, int BK);

// Plan the split of the reduction, launch the tiled kernel (which must be eligible) and reduce.
int gemm_tiled_run(int dtype, GemmArgs &g, int transA, int transB, void *workspace, size_t workspace_bytes,
                   hipStream_t stream);
// The two gradients of a convolution (gx: patch rows as A, NN, into the input's gradient; gy: patch k-rows as B, TN,
// into the filter's) as one launch where that pays; false, with nothing launched, where it does not (the caller then
// runs them one after the other).  The workspace is gy's.
bool gemm_tiled_run_pair(int dtype, GemmArgs &gx, GemmArgs &gy, void *workspace, size_t workspace_bytes, hipStream_t stream, int *rc);
// The two gradients of a mid-size MatrixMultiply (g0 = dZ . Y^T, NT; g1 = X^T . dZ, TN; both on the tiled kernels, all their
// workgroups resident at once) as one launch plus their split reductions; false, with nothing launched, otherwise.
// The workspace holds both products' partial sums side by side.
bool gemm_tiled_run_plain_pair(int dtype, GemmArgs &g0, int ta0, int tb0, GemmArgs &g1, int ta1, int tb1, void *workspace,
                               size_t workspace_bytes, hipStream_t stream, int *rc);
// Workspace gemm_tiled_run may use for this shape.
size_t gemm_tiled_workspace(int dtype, int M, int N, int K, int red, int virt = VIRT_NONE);
// Whether a product whose B is a patch matrix (VIRT_B_KROWS) runs on 64 x 64 tiles: fewer than 128 rows, and the last
// 128-column tile would be half empty or emptier (a 3 x 3 x 64 filter gradient: N = 576 = 4.5 x 128).
inline bool gemm_tiled_krows_64(int virt, int M, int N) { return virt == VIRT_B_KROWS && M < 128 && N % 128 != 0 && N % 128 <= 64; }

}  // namespace d8

#endif
