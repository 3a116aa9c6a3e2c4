/*
 * deep8_hip.h -- C ABI of libdeep8_hip.so: the MI355X (gfx950) kernels behind Deep8's
 * MatrixMultiply / Conv2d / DeConv2d GPU entry points.
 *
 * Plain pointers and integers only.  Every function returns 0 on success or a non-zero code
 * (a hipError_t value, or D8_ERR_* below); d8_last_error() gives the text.  Nothing throws
 * across this boundary; the C++ host layer turns a non-zero code into the same
 * std::runtime_error Deep8's CUDA_CHECK raises (deep8/include/basic/GPUException.h:15-24).
 *
 * All matrices are row-major (deep8/src/model/Shape.cpp:86-96).  Device pointers unless said
 * otherwise.  `stream` is a hipStream_t passed as void* (NULL = the default stream, which is
 * what Deep8 uses everywhere).  All launches are asynchronous.
 */
#ifndef DEEP8_HIP_H
#define DEEP8_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types: the ids of Deep8's DType (deep8/include/model/ElementType.h:8-22) */
#define D8_FLOAT16 10
#define D8_FLOAT32 11
#define D8_FLOAT64 12 /* the contraction path only: d8_fill, d8_gemm, the four gather maps, d8_matmul*, d8_conv2d*, d8_deconv2d* */

#define D8_ERR_ARGUMENT 10001 /* bad shape / leading dimension / null pointer */
#define D8_ERR_DTYPE    10002 /* element type not supported by this build     */
#define D8_ERR_ARCH     10003 /* the device is not gfx950                      */

const char *d8_last_error(void);

/* ---- device plumbing -------------------------------------------------------------------
 * Replaces what GPUDevice / GPUMemoryAllocator do through the CUDA runtime
 * (deep8/src/model/GPUDevice.cu:10-12, deep8/src/model/GPUMemoryAllocator.cu:17-56).      */
int d8_device_init(int device_id);                /* hipSetDevice + arch check (gfx950)    */
int d8_device_count(int *count);
int d8_device_info(int *cu_count, int *clock_khz, size_t *hbm_bytes, char *name, int name_len);
int d8_mem_info(size_t *free_bytes, size_t *total_bytes); /* device memory free / in all (no counterpart in
                                                     the reference; lets a caller see that a call allocated nothing) */
int d8_malloc(void **ptr, size_t bytes);          /* cudaMalloc      GPUMemoryAllocator.cu:17 */
int d8_free(void *ptr);                           /* cudaFree        GPUMemoryAllocator.cu:27 */
int d8_host_malloc(void **ptr, size_t bytes);     /* pinned host memory                    */
int d8_host_free(void *ptr);
int d8_memset(void *ptr, int value, size_t bytes, void *stream);   /* cudaMemset  :34      */
int d8_memcpy_h2d(void *dst, const void *src, size_t bytes);       /* cudaMemcpy  :46      */
int d8_memcpy_d2h(void *dst, const void *src, size_t bytes);       /* cudaMemcpy  :50      */
int d8_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream);  /* :40,:54     */
/* value[i] = scalar for n elements.  Replaces ConstantKernel (deep8/src/math/Constant.cu:10-44),
 * which Variable::zeroGradient / oneGradient use (deep8/src/nodes/Variable.cpp:119-130).   */
int d8_fill(int dtype, void *ptr, size_t n, float scalar, void *stream);
int d8_stream_create(void **stream);
int d8_stream_destroy(void *stream);
int d8_stream_sync(void *stream);
/* Every entry point of this header only launches kernels on the stream it is given (no allocation, no
 * synchronisation, no memset node), so a sequence of calls can be captured once and replayed: for products
 * so small that the launches cost more than the arithmetic.  d8_graph_begin starts capturing on `stream`
 * (not the default stream); the calls that follow, given the same stream, are recorded instead of run;
 * d8_graph_end returns the instantiated graph; d8_graph_launch replays it on a stream.  No counterpart in
 * the reference (hipStreamBeginCapture / hipStreamEndCapture / hipGraphInstantiate / hipGraphLaunch). */
int d8_graph_begin(void *stream);
int d8_graph_end(void *stream, void **graph);
int d8_graph_launch(void *graph, void *stream);
int d8_graph_destroy(void *graph);
int d8_event_create(void **event);
int d8_event_destroy(void *event);
int d8_event_record(void *event, void *stream);
int d8_event_elapsed_ms(void *start, void *stop, float *ms);  /* synchronises on `stop` */

/* ---- GEMM ------------------------------------------------------------------------------
 * C_b = op(A_b) * op(B_b) + beta * C_b,   b = 0 .. batch-1,  beta in {0, 1}
 *
 * op(A) is M x K, op(B) is K x N.  transA != 0: A is stored K x M (lda >= M); otherwise M x K
 * (lda >= K).  transB != 0: B is stored N x K (ldb >= K); otherwise K x N (ldb >= N).
 * transA and transB both set is rejected (Deep8 never issues it).  Strides are in elements;
 * strideA/strideB 0 broadcasts that operand over the batch.  strideC == 0 with batch > 1
 * sums all batch products into the one C (Deep8's gradient of a batch-1 operand).
 * fp16 operands accumulate in fp32 and are rounded once; beta = 1 adds the old C in fp32.
 * D8_FLOAT64 operands accumulate in fp64 (the cublasDgemm twins of the call sites below); a split
 * reduction keeps its partial sums in fp64 too.
 *
 * Sizes: any batch and any M (a batch of more than 448 independent products and a matrix of more than
 * 8 388 480 rows are run as several launches on slices); Float64 takes at most 4 194 240 columns.
 *
 * `workspace` (may be NULL) lets the kernel split the reduction (long K / summed batch, small
 * M x N) over more workgroups; d8_gemm_workspace_bytes says how much it can use.  It must be
 * 16-byte aligned (a misaligned workspace is ignored).
 *
 * Replaces the 27 cublas{S,H}gemm call sites in deep8/src/math/MatrixMultiply.cu:36-55,
 * 75-94,115-134 (forward), :211-230,253-272,296-315 (GradX), :399-418,441-460,484-503
 * (GradY) and the 18 in deep8/src/math/Conv2d.cu:195,473,801 / DeConv2d.cu:109,428,699
 * (+ their half twins).                                                                    */
size_t d8_gemm_workspace_bytes(int dtype, int transA, int transB, int M, int N, int K,
                               int batch, long strideC);
int d8_gemm(int dtype, int transA, int transB, int M, int N, int K,
            const void *A, int lda, long strideA,
            const void *B, int ldb, long strideB,
            float beta, void *C, int ldc, long strideC, int batch,
            void *workspace, size_t workspace_bytes, void *stream);

/* ---- Conv2d gather / scatter -------------------------------------------------------------
 * Geometry is explicit; padTop/padLeft >= 0 count the zero rows/columns before the image
 * (Deep8 passes the same numbers negated, deep8/src/math/Conv2d.cu:335-336).
 *
 * d8_im2col:  col[(b,oy,ox)][(fy,fx,c)] = im[b, oy*sy + fy*dy - padTop, ox*sx + fx*dx - padLeft, c]
 *             or +0 outside.  col is [B*OH*OW, FH*FW*C].   Replaces Conv2dIm2ColKernel
 *             (deep8/src/math/Conv2d.cu:10-61, launched :170,:776).
 * d8_col2im:  im += transpose of that map applied to col; taps added in (fy,fx) ascending
 *             order.  Replaces Conv2dCol2ImKernel (Conv2d.cu:64-118, launched :475).       */
int d8_im2col(int dtype, const void *im, void *col,
              int B, int IH, int IW, int C, int OH, int OW, int FH, int FW,
              int sy, int sx, int dy, int dx, int padTop, int padLeft, void *stream);
int d8_col2im(int dtype, const void *col, void *im,
              int B, int IH, int IW, int C, int OH, int OW, int FH, int FW,
              int sy, int sx, int dy, int dx, int padTop, int padLeft, void *stream);

/* ---- DeConv2d gather maps ------------------------------------------------------------------
 * zmat / dzmat are [B*IH*IW, OC*FH*FW] with column index oc*FH*FW + fy*FW + fx.
 *
 * d8_deconv_col2im: z[b,oy,ox,oc] = sum over taps (fy,fx) with iy*sy == oy - padTop + fy,
 *             ix*sx == ox - padLeft + fx inside the input, of zmat[(b,iy,ix)][oc,fy,fx];
 *             overwrites z.  Replaces DeConv2dCol2ImKernel (deep8/src/math/DeConv2d.cu:11-58,
 *             launched :115).
 * d8_deconv_im2col: dzmat[(b,iy,ix)][oc,fy,fx] = dz[b, iy*sy + padTop - fy, ix*sx + padLeft - fx, oc]
 *             or +0 outside.  Replaces DeConv2dIm2ColKernel (DeConv2d.cu:310-351, launched
 *             :405,:675).                                                                   */
int d8_deconv_col2im(int dtype, const void *zmat, void *z,
                     int B, int IH, int IW, int OH, int OW, int OC, int FH, int FW,
                     int sy, int sx, int padTop, int padLeft, void *stream);
int d8_deconv_im2col(int dtype, const void *dz, void *dzmat,
                     int B, int IH, int IW, int OH, int OW, int OC, int FH, int FW,
                     int sy, int sx, int padTop, int padLeft, void *stream);

/* ---- whole-operator entry points -----------------------------------------------------------
 * What Math::*GPU call (deep8/include/math/MatrixMultiply.h:17,26,35, Conv2d.h:23,33,45,
 * DeConv2d.h:18,28,38): shape cases, pad formulas, scratch use and accumulate-vs-overwrite
 * semantics are Deep8's.  A matrix operand is (batch, rows, cols) with cols = 1 for a 1-D
 * tensor.  `scratch` is the interim buffer the node allocates (size from the *_scratch_bytes
 * function, which already includes any split-reduction workspace).  Where that function
 * returns 0 the operator stages nothing (its patch matrix is read by the GEMM's tile loader)
 * and `scratch` may be NULL; a scratch smaller than asked for is an error only when the
 * operator has to stage.  The size functions assume tensors that are 16-byte aligned (every
 * allocation of d8_malloc and of Deep8's pools is): a Conv2d / DeConv2d tensor at an address that
 * is not can only take the staged route, whose interim matrix is sizeof(T)*B*OH*OW*FH*FW*IC
 * (Conv2d) or sizeof(T)*B*IH*IW*OC*FH*FW (DeConv2d) bytes plus d8_gemm_workspace_bytes; with
 * less the call fails with D8_ERR_ARGUMENT and says so.                                       */
size_t d8_matmul_scratch_bytes(int dtype, int which /*0 fwd, 1 gradX, 2 gradY, 3 both gradients from one call*/,
                               int xb, int xr, int xc, int yb, int yr, int yc);
int d8_matmul(int dtype, const void *x, int xb, int xr, int xc,
              const void *y, int yb, int yr, int yc, void *z,
              void *scratch, size_t scratch_bytes, void *stream);
int d8_matmul_grad_x(int dtype, void *dx, int xb, int xr, int xc,
                     const void *y, int yb, int yr, int yc, const void *dz,
                     void *scratch, size_t scratch_bytes, void *stream);
int d8_matmul_grad_y(int dtype, const void *x, int xb, int xr, int xc,
                     void *dy, int yb, int yr, int yc, const void *dz,
                     void *scratch, size_t scratch_bytes, void *stream);
/* The same two products written over their destination instead of added to it: what the pair
 * "zero the gradient, then accumulate" (deep8/src/model/EagerExecutor.cpp:51-65 followed by
 * Math::MatrixMultiplyGradX/YGPU) leaves behind, without the fill and without reading the zeros
 * back.  For callers that know the destination holds zeros (or nothing yet).                    */
int d8_matmul_grad_x_overwrite(int dtype, void *dx, int xb, int xr, int xc,
                               const void *y, int yb, int yr, int yc, const void *dz,
                               void *scratch, size_t scratch_bytes, void *stream);
int d8_matmul_grad_y_overwrite(int dtype, const void *x, int xb, int xr, int xc,
                               void *dy, int yb, int yr, int yc, const void *dz,
                               void *scratch, size_t scratch_bytes, void *stream);
/* Both gradients of one MatrixMultiply from one call: what Function::backward leaves after it has run for
 * index 0 and for index 1 (deep8/src/nodes/MatrixMultiply.cpp:31-52 -> Math::MatrixMultiplyGradX, then
 * Math::MatrixMultiplyGradY; deep8/src/math/MatrixMultiply.cu:193-363,381-551).  The two products are independent
 * of each other, so large Float16 ones run as ONE launch in which a workgroup goes from a tile of dx straight on
 * to a tile of dy; everything else is d8_matmul_grad_x followed by d8_matmul_grad_y.  The results are bit for bit
 * those of the two calls.  overwrite: bit 0 -- dx is written instead of added to, bit 1 -- dy likewise (the
 * _overwrite forms above).  scratch: d8_matmul_scratch_bytes(which = 3), room for both gradients' scratch side by
 * side; with less, but at least the larger of which = 1 and which = 2, the call still works (mid-size products
 * then run as two launches).  Two small products (each at most four 128 x 128 tiles over a reduction of at most
 * 512) share a launch as well, and so do two mid-size ones whose workgroups all fit the chip at once.          */
int d8_matmul_grad_xy(int dtype, const void *x, void *dx, int xb, int xr, int xc,
                      const void *y, void *dy, int yb, int yr, int yc, const void *dz, int overwrite,
                      void *scratch, size_t scratch_bytes, void *stream);

/* d8_matmul_grad_y for callers that cannot allocate and have no scratch to pass.  No counterpart in the
 * reference: it is for code under HIP graph capture, tight serving loops and harnesses that forbid
 * hipMalloc.  Same arguments, checks and result (bit for bit) as d8_matmul_grad_y given a scratch of
 * d8_matmul_scratch_bytes(dtype, 2, ...) bytes, but the split reduction's partial sums go to a device
 * array of D8_STATIC_SCRATCH_BYTES that lives in the library (each GPU the library runs on holds one
 * until the process ends).  A shape that would need more is refused with D8_ERR_ARGUMENT.  The call
 * allocates and frees nothing.  All calls on one GPU share that GPU's array: calls that overlap in time
 * on one GPU (different streams or host threads) race.                                                  */
#define D8_STATIC_SCRATCH_BYTES (32u << 20)
int d8_matmul_grad_y_static(int dtype, const void *x, int xb, int xr, int xc,
                            void *dy, int yb, int yr, int yc, const void *dz, void *stream);

/* out[0..3] = OH, OW, padTop, padLeft (deep8/src/math/Conv2d.cpp:20-32, Conv2d.cu:332-336;
 * deep8/src/math/DeConv2d.cpp:23-29, DeConv2d.cu:99-100) */
int d8_conv2d_geometry(int IH, int IW, int FH, int FW, int covered,
                       int sy, int sx, int dy, int dx, int *out);
int d8_deconv2d_geometry(int IH, int IW, int FH, int FW, int covered, int sy, int sx, int *out);

/* which: 0 forward, 1 gradient of x, 2 gradient of the filter, 3 both gradients from one call (the _grad_xy entry
 * points; the same for the DeConv2d queries) */
size_t d8_conv2d_scratch_bytes(int dtype, int which, int B, int IH, int IW, int IC,
                               int OC, int FH, int FW, int covered, int sy, int sx, int dy, int dx);
int d8_conv2d(int dtype, const void *x, int B, int IH, int IW, int IC,
              const void *w, int OC, int FH, int FW, void *z,
              int covered, int sy, int sx, int dy, int dx,
              void *scratch, size_t scratch_bytes, void *stream);
int d8_conv2d_grad_x(int dtype, void *gx, int B, int IH, int IW, int IC,
                     const void *w, int OC, int FH, int FW, const void *gz,
                     int covered, int sy, int sx, int dy, int dx,
                     void *scratch, size_t scratch_bytes, void *stream);
int d8_conv2d_grad_y(int dtype, const void *x, int B, int IH, int IW, int IC,
                     void *gw, int OC, int FH, int FW, const void *gz,
                     int covered, int sy, int sx, int dy, int dx,
                     void *scratch, size_t scratch_bytes, void *stream);

size_t d8_deconv2d_scratch_bytes(int dtype, int which, int B, int IH, int IW, int IC,
                                 int OC, int FH, int FW, int covered, int sy, int sx);
int d8_deconv2d(int dtype, const void *x, int B, int IH, int IW, int IC,
                const void *w, int OC, int FH, int FW, void *z,
                int covered, int sy, int sx,
                void *scratch, size_t scratch_bytes, void *stream);
int d8_deconv2d_grad_x(int dtype, void *gx, int B, int IH, int IW, int IC,
                       const void *w, int OC, int FH, int FW, const void *gz,
                       int covered, int sy, int sx,
                       void *scratch, size_t scratch_bytes, void *stream);
int d8_deconv2d_grad_y(int dtype, const void *x, int B, int IH, int IW, int IC,
                       void *gw, int OC, int FH, int FW, const void *gz,
                       int covered, int sy, int sx,
                       void *scratch, size_t scratch_bytes, void *stream);

/* DeConv2d with the geometry given outright instead of derived from `covered`: the output is OH x OW and
 * z[b,oy,ox,:] sums the taps (fy,fx) with iy*sy == oy - padTop + fy, ix*sx == ox - padLeft + fx inside the input
 * (padTop, padLeft >= 0: the pads of the stride-1 correlation over the zero-inflated input, as returned by
 * d8_deconv2d_geometry).  Math::DeConv2d admits only two output sizes per input (deep8/src/nodes/DeConv2d.cpp:36-52,
 * pads deep8/src/math/DeConv2d.cpp:295-301); these entry points run the same kernels on any other, e.g. PyTorch's
 * ConvTranspose2d(k, s, p) = OH (IH-1)*s + k - 2p, padTop = k - 1 - p.  The gradients accumulate unless
 * overwrite != 0.  scratch from d8_deconv2d_scratch_bytes_ex.                                                  */
size_t d8_deconv2d_scratch_bytes_ex(int dtype, int which, int B, int IH, int IW, int IC,
                                    int OC, int FH, int FW, int OH, int OW, int padTop, int padLeft, int sy, int sx);
int d8_deconv2d_ex(int dtype, const void *x, int B, int IH, int IW, int IC,
                   const void *w, int OC, int FH, int FW, void *z,
                   int OH, int OW, int padTop, int padLeft, int sy, int sx,
                   void *scratch, size_t scratch_bytes, void *stream);
int d8_deconv2d_grad_x_ex(int dtype, void *gx, int B, int IH, int IW, int IC,
                          const void *w, int OC, int FH, int FW, const void *gz,
                          int OH, int OW, int padTop, int padLeft, int sy, int sx, int overwrite,
                          void *scratch, size_t scratch_bytes, void *stream);
int d8_deconv2d_grad_y_ex(int dtype, const void *x, int B, int IH, int IW, int IC,
                          void *gw, int OC, int FH, int FW, const void *gz,
                          int OH, int OW, int padTop, int padLeft, int sy, int sx, int overwrite,
                          void *scratch, size_t scratch_bytes, void *stream);

/* Overwrite forms of the four convolution gradients: the destination's old contents are ignored
 * (what "zero the gradient, then accumulate" leaves, without the fill and the read-back).      */
int d8_conv2d_grad_x_overwrite(int dtype, void *gx, int B, int IH, int IW, int IC,
                               const void *w, int OC, int FH, int FW, const void *gz,
                               int covered, int sy, int sx, int dy, int dx,
                               void *scratch, size_t scratch_bytes, void *stream);
int d8_conv2d_grad_y_overwrite(int dtype, const void *x, int B, int IH, int IW, int IC,
                               void *gw, int OC, int FH, int FW, const void *gz,
                               int covered, int sy, int sx, int dy, int dx,
                               void *scratch, size_t scratch_bytes, void *stream);
int d8_deconv2d_grad_x_overwrite(int dtype, void *gx, int B, int IH, int IW, int IC,
                                 const void *w, int OC, int FH, int FW, const void *gz,
                                 int covered, int sy, int sx,
                                 void *scratch, size_t scratch_bytes, void *stream);
int d8_deconv2d_grad_y_overwrite(int dtype, const void *x, int B, int IH, int IW, int IC,
                                 void *gw, int OC, int FH, int FW, const void *gz,
                                 int covered, int sy, int sx,
                                 void *scratch, size_t scratch_bytes, void *stream);

/* Both gradients of a convolution from one call: what the _grad_x call followed by the _grad_y call of the same
 * operator leave (Conv2d::backward / DeConv2d::backward run once per input, deep8/src/nodes/Conv2d.cpp:85-151,
 * deep8/src/nodes/DeConv2d.cpp:74-126, each a cublasSgemm / cublasHgemm sequence of its own:
 * deep8/src/math/Conv2d.cu:440-492 and :750-802, deep8/src/math/DeConv2d.cu:371-429 and :642-700).  The two are
 * independent of each other; on a layer whose products each leave compute units idle they run as ONE launch, the
 * workgroups of both side by side.  gw is bit for bit what the _grad_y call leaves; so is gx, except on small half
 * layers where the product behind gx, cut into pieces when it runs alone, runs whole beside the other's workgroups:
 * the same sums added in another order (equal within half rounding).  overwrite: bit 0 -- gx is
 * written instead of added to, bit 1 -- gw likewise.  scratch: the scratch query with which = 3 (room for both
 * gradients' scratch side by side); with less, but at least the larger of which = 1 and which = 2, the call still
 * works and large layers run as two launches.                                                                     */
int d8_conv2d_grad_xy(int dtype, const void *x, void *gx, int B, int IH, int IW, int IC,
                      const void *w, void *gw, int OC, int FH, int FW, const void *gz,
                      int covered, int sy, int sx, int dy, int dx, int overwrite,
                      void *scratch, size_t scratch_bytes, void *stream);
int d8_deconv2d_grad_xy(int dtype, const void *x, void *gx, int B, int IH, int IW, int IC,
                        const void *w, void *gw, int OC, int FH, int FW, const void *gz,
                        int covered, int sy, int sx, int overwrite,
                        void *scratch, size_t scratch_bytes, void *stream);
int d8_deconv2d_grad_xy_ex(int dtype, const void *x, void *gx, int B, int IH, int IW, int IC,
                           const void *w, void *gw, int OC, int FH, int FW, const void *gz,
                           int OH, int OW, int padTop, int padLeft, int sy, int sx, int overwrite,
                           void *scratch, size_t scratch_bytes, void *stream);

/* Test and measurement aid: how many of the _grad_xy calls above have run as one launch since the library was
 * loaded (no counterpart in the reference).                                                                       */
unsigned long d8_conv_grad_pair_launches(void);
unsigned long d8_matmul_grad_pair_launches(void);  /* ... and of the d8_matmul_grad_xy calls */

/* ---- Add (broadcasting) and ReLu -----------------------------------------------------------
 * The element-wise steps that follow MatrixMultiply / Conv2d in a network (bias, activation).
 * Shapes are Deep8's 5-entry enlarged form [batch, d0, d1, d2, d3]: dims right-aligned, padded
 * with 1 (deep8/include/utils/ShapeUtils.h:41-56); an operand axis equals z's or is 1.
 *
 * d8_add       z = x + y with broadcasting.  Replaces Math::AddGPU (deep8/include/math/Add.h:20,
 *              deep8/src/math/Add.cu:21-52).
 * d8_add_grad  g += dz summed over the axes where g has extent 1 and dz does not; this one map
 *              is both Math::AddGradXGPU and Math::AddGradYGPU (Add.h:31,42; Add.cu:64-133:
 *              the gradient op returns dz).  `scratch` (may be NULL; size from
 *              d8_add_grad_scratch_bytes, 16-byte aligned) lets the reduction run in two passes.
 * d8_relu      y = x > 0 ? x : 0.   Replaces Math::ReLuGPU (deep8/include/math/ReLu.h:19,
 *              deep8/src/math/ReLu.cu:20-59).
 * d8_relu_grad dx += x > 0 ? dy : 0.  Replaces Math::ReLuGradGPU (ReLu.h:30, ReLu.cu:61-116).     */
int d8_add(int dtype, const void *x, const int *xdims, const void *y, const int *ydims,
           void *z, const int *zdims, void *stream);
size_t d8_add_grad_scratch_bytes(int dtype, const int *gdims, const int *zdims);
int d8_add_grad(int dtype, void *g, const int *gdims, const void *dz, const int *zdims,
                void *scratch, size_t scratch_bytes, void *stream);
int d8_relu(int dtype, const void *x, void *y, long n, void *stream);
int d8_relu_grad(int dtype, const void *x, void *dx, const void *dy, long n, void *stream);
/* Overwrite forms of the two gradients: the destination's old contents are not read (what "zero the
 * gradient, then accumulate" leaves, deep8/src/model/EagerExecutor.cpp:51-65, without the fill and
 * the read-back).                                                                                   */
int d8_add_grad_overwrite(int dtype, void *g, const int *gdims, const void *dz, const int *zdims,
                          void *scratch, size_t scratch_bytes, void *stream);
int d8_relu_grad_overwrite(int dtype, const void *x, void *dx, const void *dy, long n, void *stream);

/* ---- bias and activation folded into the contraction --------------------------------------------------
 * In a network Add (a per-channel bias broadcast over the rows) and ReLu follow every MatrixMultiply / Conv2d as
 * passes of their own over the result (Math::AddGPU, deep8/src/math/Add.cu:21-52; Math::ReLuGPU,
 * deep8/src/math/ReLu.cu:20-59).  These entry points give the result of the three-call sequence from one call:
 *
 * d8_matmul_bias_relu   z = relu?(x * y + bias): d8_matmul, then bias[n] added along z's last axis (bias: that many
 *                       elements of the tensors' type, or NULL), then ReLu when relu != 0.  z's last axis has yc
 *                       elements when yc > 1; when y is a vector or a batch of vectors (yc == 1) z is [batch][xr]
 *                       (deep8/src/nodes/MatrixMultiply.cpp:23-27) and the bias has xr elements.
 * d8_conv2d_bias_relu   the same after d8_conv2d (bias: OC elements).
 *     Both apply bias and ReLu in the store of the product's kernel (before the one rounding to the element type)
 *     wherever that kernel is one of the tiled ones, and otherwise run the product followed by ONE in-place pass.
 *     Float32: bit for bit the result of d8_matmul / d8_conv2d, d8_add, d8_relu.  Float16: the fused store rounds
 *     once instead of three times.  scratch as for d8_matmul / d8_conv2d.  Float64 is rejected.
 * d8_bias_relu_grad     the way back in one pass over the [rows][cols] gradient of z: dpre = z > 0 ? dz : 0 is
 *                       written (dpre may be dz), and dbias (cols elements) receives its column sums, added to
 *                       what it holds when accumulate_bias != 0, else written.  z is the layer's output (it is
 *                       positive exactly where the pre-activation was).  Replaces Math::ReLuGradGPU
 *                       (ReLu.cu:61-116) + Math::AddGradYGPU (Add.cu:99-133); the sums are bit for bit those of
 *                       d8_add_grad on dpre.  scratch (may be NULL): d8_bias_relu_grad_scratch_bytes, 16-byte aligned.
 *                       dpre then feeds d8_matmul_grad_* / d8_conv2d_grad_* as dz.                                  */
int d8_matmul_bias_relu(int dtype, const void *x, int xb, int xr, int xc,
                        const void *y, int yb, int yr, int yc, const void *bias, int relu, void *z,
                        void *scratch, size_t scratch_bytes, void *stream);
int d8_conv2d_bias_relu(int dtype, const void *x, int B, int IH, int IW, int IC,
                        const void *w, int OC, int FH, int FW, const void *bias, int relu, void *z,
                        int covered, int sy, int sx, int dy, int dx,
                        void *scratch, size_t scratch_bytes, void *stream);
size_t d8_bias_relu_grad_scratch_bytes(int dtype, long rows, int cols);
int d8_bias_relu_grad(int dtype, const void *z, const void *dz, void *dpre, void *dbias, long rows, int cols,
                      int accumulate_bias, void *scratch, size_t scratch_bytes, void *stream);

/* ---- Minus, L1Norm / L2Norm, ReduceMean, AXPBY ------------------------------------------------
 * What a loss and a trainer step need on top of the operators above.  Shapes as for d8_add.
 * Reductions take an optional two-pass `scratch` (16-byte aligned; size from
 * d8_add_grad_scratch_bytes(dtype, shape of the reduced tensor, shape of the full tensor)).
 *
 * d8_minus            z = x - y with broadcasting.  Math::MinusGPU (deep8/include/math/Minus.h:16,
 *                     deep8/src/math/Minus.cu:21-52).  Math::MinusGradXGPU (Minus.h:27) is d8_add_grad.
 * d8_minus_grad_y     g -= dz summed over the axes where g has extent 1.  Math::MinusGradYGPU
 *                     (Minus.h:38, Minus.cu:103-147).
 * d8_l1norm           y[b] = sum_i |x[b][i]|.  Math::L1NormGPU (deep8/include/math/L1Norm.h,
 *                     deep8/src/math/L1Norm.cu:27-75).
 * d8_l1norm_grad      dx[b][i] += dy[b] * sign(x[b][i]) (sign(0) = 0).  Math::L1NormGradGPU
 *                     (L1Norm.cu:77-136).
 * d8_l2norm           y[b] = sqrt(sum_i x[b][i]^2).  Math::L2NormGPU (deep8/src/math/L2Norm.cu).
 * d8_l2norm_grad      dx[b][i] += dy[b] / y[b] * x[b][i].  Math::L2NormGradGPU.
 * d8_reduce_mean      y = mean of x over the axes where ydims is 1 and xdims is not (ydims is the
 *                     keepDims form of the output shape; dropping the axes does not move data).
 *                     Math::ReduceMeanGPU (deep8/include/math/ReduceMean.h, deep8/src/math/ReduceMean.cu:30-110).
 * d8_reduce_mean_grad dx += dy / count, dy broadcast over the reduced axes.  Math::ReduceMeanGradGPU
 *                     (ReduceMean.cu:112-203).
 * d8_axpby            z = alpha * x + beta * y (z may be x or y).  Math::AXPBYGPU
 *                     (deep8/include/math/AXPBY.h, deep8/src/math/AXPBY.cu:9-47): the SGD update.       */
int d8_minus(int dtype, const void *x, const int *xdims, const void *y, const int *ydims,
             void *z, const int *zdims, void *stream);
int d8_minus_grad_y(int dtype, void *g, const int *gdims, const void *dz, const int *zdims,
                    void *scratch, size_t scratch_bytes, void *stream);
int d8_l1norm(int dtype, const void *x, void *y, int batch, long size,
              void *scratch, size_t scratch_bytes, void *stream);
int d8_l1norm_grad(int dtype, const void *x, void *dx, const void *dy, int batch, long size, void *stream);
int d8_l2norm(int dtype, const void *x, void *y, int batch, long size,
              void *scratch, size_t scratch_bytes, void *stream);
int d8_l2norm_grad(int dtype, const void *x, void *dx, const void *y, const void *dy, int batch, long size,
                   void *stream);
int d8_reduce_mean(int dtype, const void *x, const int *xdims, void *y, const int *ydims,
                   void *scratch, size_t scratch_bytes, void *stream);
int d8_reduce_mean_grad(int dtype, void *dx, const int *xdims, const void *dy, const int *ydims, void *stream);
int d8_axpby(int dtype, const void *x, float alpha, const void *y, float beta, void *z, long n, void *stream);
/* d8_adam_update: gradient += weight_decay * value; m = beta1 m + (1 - beta1) gradient;
 * v = beta2 v + (1 - beta2) gradient^2; value -= ratio * m / (sqrt(v) + epsilon) with
 * ratio = learning_rate * sqrt(1 - beta2^steps) / (1 - beta1^steps), steps < 1 taken as 1.
 * Math::AdamUpdateGPU (deep8/include/math/AdamUpdate.h, deep8/src/math/AdamUpdate.cu:9-47).      */
int d8_adam_update(int dtype, void *value, void *gradient, void *m, void *v, float beta1, float beta2,
                   float epsilon, float learning_rate, float weight_decay, long steps, long n, void *stream);

/* ---- MaxPooling2d / AvgPooling2d --------------------------------------------------------------
 * x [B][IH][IW][C], y [B][OH][OW][C]; (OH, OW, padTop, padLeft) = d8_conv2d_geometry(IH, IW, FH, FW,
 * covered, sy, sx, 1, 1).  Semantics are those of Deep8's CPU path: the forward window is cut from
 * the zero-padded image (zeros take part in the maximum and in the mean, which divides by FH * FW);
 * the max gradient goes to the first maximum of the window clipped to the image; gradients are
 * added into dx.
 * d8_maxpool2d / _grad  Math::MaxPooling2dGPU / MaxPooling2dGradGPU (deep8/include/math/MaxPooling2d.h,
 *                       deep8/src/math/MaxPooling2d.cu:41-147 -- a cuDNN call there; checks and CPU
 *                       semantics deep8/src/math/MaxPooling2d.cpp:6-251)
 * d8_avgpool2d / _grad  Math::AvgPooling2dGPU / AvgPooling2dGradGPU (deep8/include/math/AvgPooling2d.h,
 *                       deep8/src/math/AvgPooling2d.cu; CPU semantics AvgPooling2d.cpp:99-245)          */
int d8_maxpool2d(int dtype, const void *x, void *y, int B, int IH, int IW, int C,
                 int FH, int FW, int covered, int sy, int sx, void *stream);
int d8_maxpool2d_grad(int dtype, const void *x, void *dx, const void *dy, int B, int IH, int IW, int C,
                      int FH, int FW, int covered, int sy, int sx, void *stream);
int d8_avgpool2d(int dtype, const void *x, void *y, int B, int IH, int IW, int C,
                 int FH, int FW, int covered, int sy, int sx, void *stream);
int d8_avgpool2d_grad(int dtype, void *dx, const void *dy, int B, int IH, int IW, int C,
                      int FH, int FW, int covered, int sy, int sx, void *stream);
/* The two pooling gradients written over dx instead of added to it (see d8_relu_grad_overwrite). */
int d8_maxpool2d_grad_overwrite(int dtype, const void *x, void *dx, const void *dy, int B, int IH, int IW, int C,
                                int FH, int FW, int covered, int sy, int sx, void *stream);
int d8_avgpool2d_grad_overwrite(int dtype, void *dx, const void *dy, int B, int IH, int IW, int C,
                                int FH, int FW, int covered, int sy, int sx, void *stream);

/* ---- measurement aid (no counterpart in the reference) ---------------------------------------
 * d8_mfma_stream issues the GEMM kernels' MFMA instruction for `dtype` (D8_FLOAT16, D8_FLOAT32 or
 * D8_FLOAT64) back to back on operands taken from `operands` (any device buffer; 16-byte aligned)
 * and held in registers, on every CU, no LDS or global traffic in the loop.  Timing one launch gives the rate the matrix
 * pipe sustains on those operand bits, i.e. the ceiling a GEMM has on that data.  `out` takes
 * d8_mfma_stream_out_bytes() bytes; *flops receives the flops one launch performs.             */
/* A second aid needs no entry point: with D8_GEMM_STAMPS set in the environment before the first launch, a
 * d8_gemm call that runs the large-output fp16 kernel and is given an 8-byte aligned workspace of at least
 * 48 bytes per 256 x 256 tile of C leaves there, per tile, six 64-bit values: the chip's 100 MHz wall
 * clock when its workgroup turned to the tile, when its K loop began and ended and when its epilogue was through
 * (its stores acknowledged, for the workgroup's last tile), and the shader clock before and after the loop.
 * d8_matmul_grad_xy does the same with its scratch when the two products run as one launch (the first product's
 * tiles, then the second's).                                                                            */
/* A third one, for the tiled kernels (fp16 / fp32 products and the convolutions they carry): after
 * d8_gemm_phase_record(records, bytes) every tiled launch whose records fit leaves 64 bytes per workgroup in
 * `records` (a device buffer, 8-byte aligned; index = workgroup id x + grid size x * id z): the same four wall
 * clock values and two shader clock values, then (XCC_ID << 32 | HW_ID) of the wave that wrote them and 1 if the
 * workgroup worked on a remainder band.  Each launch writes from index 0, so read the buffer between launches.
 * records = null switches the records off again.  Process-wide and not thread-safe: a tool for one measuring thread. */
int d8_gemm_phase_record(void *records, size_t bytes);
size_t d8_mfma_stream_out_bytes(void);
int d8_mfma_stream(int dtype, const void *operands, size_t operand_bytes, void *out, int iters,
                   double *flops, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DEEP8_HIP_H */
