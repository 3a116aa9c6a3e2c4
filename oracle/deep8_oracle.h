/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement (plain C) of Deep8's dense-contraction hot path.
 * Only tests, the smoke check and the benchmark's cpu_baseline leg may load this library; the
 * product path (the HIP library) never does.
 *
 * Conventions: every matrix is row-major; images are [B,H,W,C]; filters are [OC,FH,FW,IC].
 * All sums are carried in double and rounded to float once, so for integer-valued inputs the
 * results are exact and for real inputs they are at least as accurate as the reference's Eigen
 * float accumulation (the parity tests compare against both).
 *
 * Pin status (which independent check fixes each function) is recorded in deep8_oracle.c.
 */
#ifndef DEEP8_ORACLE_H
#define DEEP8_ORACLE_H

#ifdef __cplusplus
extern "C" {
#endif

/* ---- MatrixMultiply: x (xb,[xr,xc]), y (yb,[yr,yc]), z (max(xb,yb),[xr,yc]) -------------- */
void orc_matmul(const float *x, int xb, int xr, int xc,
                const float *y, int yb, int yr, int yc, float *z);
void orc_matmul_grad_x(float *dx, int xb, int xr, int xc,
                       const float *y, int yb, int yr, int yc, const float *dz);
void orc_matmul_grad_y(const float *x, int xb, int xr, int xc,
                       float *dy, int yb, int yr, int yc, const float *dz);

/* ---- generic row-major GEMM, C = op(A) op(B) + beta*C, beta in {0,1} ---------------------- */
void orc_gemm(int transA, int transB, int M, int N, int K,
              const float *A, int lda, const float *B, int ldb, float beta, float *C, int ldc);

/* ---- Deep8 geometry ------------------------------------------------------------------------ */
/* out[0..3] = OH, OW, padTop, padLeft (pads >= 0, rows/cols of zeros before the image) */
void orc_conv2d_geometry(int IH, int IW, int FH, int FW, int covered,
                         int sy, int sx, int dy, int dx, int *out);
void orc_deconv2d_geometry(int IH, int IW, int FH, int FW, int covered,
                           int sy, int sx, int *out);

/* ---- Conv2d, direct loops ------------------------------------------------------------------- */
void orc_conv2d(const float *x, int B, int IH, int IW, int IC,
                const float *w, int OC, int FH, int FW, float *z,
                int covered, int sy, int sx, int dy, int dx);
void orc_conv2d_grad_x(float *gx, int B, int IH, int IW, int IC,
                       const float *w, int OC, int FH, int FW, const float *gz,
                       int covered, int sy, int sx, int dy, int dx);
void orc_conv2d_grad_y(const float *x, int B, int IH, int IW, int IC,
                       float *gw, int OC, int FH, int FW, const float *gz,
                       int covered, int sy, int sx, int dy, int dx);

/* ---- DeConv2d, direct loops ----------------------------------------------------------------- */
void orc_deconv2d(const float *x, int B, int IH, int IW, int IC,
                  const float *w, int OC, int FH, int FW, float *z,
                  int covered, int sy, int sx);
void orc_deconv2d_grad_x(float *gx, int B, int IH, int IW, int IC,
                         const float *w, int OC, int FH, int FW, const float *gz,
                         int covered, int sy, int sx);
void orc_deconv2d_grad_y(const float *x, int B, int IH, int IW, int IC,
                         float *gw, int OC, int FH, int FW, const float *gz,
                         int covered, int sy, int sx);

/* ---- the same contraction path on double operands (the reference's Float64 cases) ----------- */
void orc_matmul_f64(const double *x, int xb, int xr, int xc,
                const double *y, int yb, int yr, int yc, double *z);
void orc_matmul_grad_x_f64(double *dx, int xb, int xr, int xc,
                       const double *y, int yb, int yr, int yc, const double *dz);
void orc_matmul_grad_y_f64(const double *x, int xb, int xr, int xc,
                       double *dy, int yb, int yr, int yc, const double *dz);

void orc_gemm_f64(int transA, int transB, int M, int N, int K,
              const double *A, int lda, const double *B, int ldb, float beta, double *C, int ldc);

void orc_conv2d_f64(const double *x, int B, int IH, int IW, int IC,
                const double *w, int OC, int FH, int FW, double *z,
                int covered, int sy, int sx, int dy, int dx);
void orc_conv2d_grad_x_f64(double *gx, int B, int IH, int IW, int IC,
                       const double *w, int OC, int FH, int FW, const double *gz,
                       int covered, int sy, int sx, int dy, int dx);
void orc_conv2d_grad_y_f64(const double *x, int B, int IH, int IW, int IC,
                       double *gw, int OC, int FH, int FW, const double *gz,
                       int covered, int sy, int sx, int dy, int dx);

void orc_deconv2d_f64(const double *x, int B, int IH, int IW, int IC,
                  const double *w, int OC, int FH, int FW, double *z,
                  int covered, int sy, int sx);
void orc_deconv2d_grad_x_f64(double *gx, int B, int IH, int IW, int IC,
                         const double *w, int OC, int FH, int FW, const double *gz,
                         int covered, int sy, int sx);
void orc_deconv2d_grad_y_f64(const double *x, int B, int IH, int IW, int IC,
                         double *gw, int OC, int FH, int FW, const double *gz,
                         int covered, int sy, int sx);


/* ---- the four gather/scatter maps, explicit geometry ---------------------------------------- */
/* col[(b,oy,ox)][(fy,fx,c)] = im[b, oy*sy + fy*dy - padTop, ox*sx + fx*dx - padLeft, c] or +0 */
void orc_im2col(const float *im, float *col, int B, int IH, int IW, int C, int OH, int OW,
                int FH, int FW, int sy, int sx, int dy, int dx, int padTop, int padLeft);
/* im[...] += the same map transposed */
void orc_col2im(const float *col, float *im, int B, int IH, int IW, int C, int OH, int OW,
                int FH, int FW, int sy, int sx, int dy, int dx, int padTop, int padLeft);
/* z[b,oy,ox,oc] = sum_{fy,fx : (oy-padTop+fy) = iy*sy, ...} zmat[(b,iy,ix)][oc*FH*FW+fy*FW+fx] */
void orc_deconv_col2im(const float *zmat, float *z, int B, int IH, int IW, int OH, int OW, int OC,
                       int FH, int FW, int sy, int sx, int padTop, int padLeft);
/* dzmat[(b,iy,ix)][oc*FH*FW+fy*FW+fx] = dz[b, iy*sy+padTop-fy, ix*sx+padLeft-fx, oc] or +0 */
void orc_deconv_im2col(const float *dz, float *dzmat, int B, int IH, int IW, int OH, int OW, int OC,
                       int FH, int FW, int sy, int sx, int padTop, int padLeft);

/* ---- Add (broadcasting) and ReLu ------------------------------------------------------------
 * Shapes are the 5-entry enlarged form [batch, d0, d1, d2, d3], dims right-aligned and padded
 * with 1 (deep8/include/utils/ShapeUtils.h:41-56); an operand axis is either equal to z's or 1. */
void orc_add(const float *x, const int *xd, const float *y, const int *yd, float *z, const int *zd);
/* dxy += dz summed over the axes where dxy has extent 1 and dz does not (AddGradX == AddGradY) */
void orc_add_grad(float *dxy, const int *d, const float *dz, const int *zd);
void orc_relu(const float *x, float *y, long n);
/* dx += x > 0 ? dy : 0 */
void orc_relu_grad(const float *x, float *dx, const float *dy, long n);

/* ---- Minus, L1Norm / L2Norm, ReduceMean, AXPBY (shapes as above; yd of the mean is the keepDims
 * form of its output shape) */
void orc_minus(const float *x, const int *xd, const float *y, const int *yd, float *z, const int *zd);
void orc_minus_grad_y(float *dy, const int *d, const float *dz, const int *zd);
void orc_l1norm(const float *x, float *y, int batch, long size);
void orc_l1norm_grad(const float *x, float *dx, const float *dy, int batch, long size);
void orc_l2norm(const float *x, float *y, int batch, long size);
void orc_l2norm_grad(const float *x, float *dx, const float *y, const float *dy, int batch, long size);
void orc_reduce_mean(const float *x, const int *xd, float *y, const int *yd);
void orc_reduce_mean_grad(float *dx, const int *xd, const float *dy, const int *yd);
void orc_axpby(const float *x, float alpha, const float *y, float beta, float *z, long n);
/* MaxPooling2d (is_max) / AvgPooling2d on NHWC images; gradients are added into dx */
void orc_pool2d(int is_max, const float *x, float *y, int B, int IH, int IW, int C, int FH, int FW, int covered, int sy, int sx);
void orc_pool2d_grad(int is_max, const float *x, float *dx, const float *dy, int B, int IH, int IW, int C, int FH, int FW,
                     int covered, int sy, int sx);
void orc_adam_update(float *value, float *gradient, float *m, float *v, float beta1, float beta2, float epsilon,
                     float learning_rate, float weight_decay, long steps, long n);

int orc_threads(void);

#ifdef __cplusplus
}
#endif
#endif
