/*
 * TEST INFRASTRUCTURE ONLY -- see deep8_oracle.h.  CPU restatement of Deep8's
 * MatrixMultiply / Conv2d / DeConv2d forward and backward, in plain C.
 *
 * What each function follows in the reference, and what pins it (tests/test_oracle_*.py):
 *
 *   orc_matmul, _grad_x, _grad_y   deep8/src/math/MatrixMultiply.cpp:94-116,134-163,181-210
 *        (three shape cases each).  Pinned by: the reference's own library on seeded inputs
 *        (golden fixtures + live when oracle/_ref is built), numpy matmul per case,
 *        K=1 outer product, identity operand, "grad twice doubles".
 *   orc_conv2d, _grad_x, _grad_y   deep8/src/math/Conv2d.cpp:293-357,396-466,541-604, pads
 *        :341-350; loops as in test/Conv2dTest.h:63-89.  Pinned by: the reference library,
 *        torch.nn.functional.conv2d + autograd on CPU, 1x1 filter == GEMM, adjoint identity.
 *   orc_deconv2d, _grad_x, _grad_y deep8/src/math/DeConv2d.cpp:246-307,344-415,463-529, pads
 *        :295-301; loops as in test/DeConv2dTest.h:56-92.  Pinned by: the reference library,
 *        torch conv_transpose2d with flipped kernel, adjoint identity with orc_conv-like maps.
 *   orc_im2col        index map of deep8/src/math/Conv2d.cu:27-60 and Eigen's patch layout
 *        (TensorImagePatch.h:298-322).  Pinned bit-exactly by the reference's materialised
 *        extract_image_patches expression and by brute-force numpy indexing.
 *   orc_col2im        deep8/src/math/Conv2d.cu:82-117.  Pinned by adjointness with orc_im2col
 *        (exact on integers) and by "no overlap when stride >= filter" copies.
 *   orc_deconv_col2im deep8/src/math/DeConv2d.cu:27-57; orc_deconv_im2col :327-350.  Pinned by
 *        adjointness with each other, by the permutation identity against the reference's
 *        DeConv2dGradX patches, and through orc_deconv2d == GEMM + col2im compositions.
 *
 * No function here is "parity unpinned".  The half (fp16) results the HIP path produces have
 * no CPU twin in the reference (MatrixMultiply.cpp:119-131 supports float/double only); tests
 * feed this fp32 oracle the half-rounded inputs.
 */
#include "deep8_oracle.h"

#include <math.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ---- Add / ReLu -------------------------------------------------------------------------------
 * orc_add       deep8/src/math/Add.cpp:110-142 (reshape to 5 axes, broadcast the size-1 axes, add)
 * orc_add_grad  deep8/src/math/Add.cpp:163-184 (dxy += dz.sum(axes that differ)); the sum is carried
 *               in double here
 * orc_relu      deep8/src/math/ReLu.cpp:38-44 (cwiseMax(0));  orc_relu_grad  ReLu.cpp:62-77
 * Pins: numpy broadcasting / np.sum over the same axes, the live reference build and the golden
 * fixtures (tests/test_oracle_pins.py). */
static long stride5(const int *d, int axis) {
    long s = 1;
    for (int i = 4; i > axis; --i) s *= d[i];
    return s;
}

void orc_add(const float *x, const int *xd, const float *y, const int *yd, float *z, const int *zd) {
    long n = 1;
    for (int i = 0; i < 5; ++i) n *= zd[i];
    for (long e = 0; e < n; ++e) {
        long rem = e, xi = 0, yi = 0;
        for (int a = 0; a < 5; ++a) {
            const long zs = stride5(zd, a), idx = rem / zs;
            rem -= idx * zs;
            if (xd[a] != 1) xi += idx * stride5(xd, a);
            if (yd[a] != 1) yi += idx * stride5(yd, a);
        }
        z[e] = x[xi] + y[yi];
    }
}

void orc_add_grad(float *dxy, const int *d, const float *dz, const int *zd) {
    long n = 1, nz = 1;
    for (int i = 0; i < 5; ++i) n *= d[i], nz *= zd[i];
    double *acc = (double *)calloc((size_t)n, sizeof(double));
    for (long e = 0; e < nz; ++e) {
        long rem = e, o = 0;
        for (int a = 0; a < 5; ++a) {
            const long zs = stride5(zd, a), idx = rem / zs;
            rem -= idx * zs;
            if (d[a] != 1) o += idx * stride5(d, a);
        }
        acc[o] += (double)dz[e];
    }
    for (long o = 0; o < n; ++o) dxy[o] += (float)acc[o];
    free(acc);
}

void orc_relu(const float *x, float *y, long n) {
    for (long i = 0; i < n; ++i) y[i] = x[i] > 0.f ? x[i] : 0.f;
}

void orc_relu_grad(const float *x, float *dx, const float *dy, long n) {
    for (long i = 0; i < n; ++i) dx[i] += x[i] > 0.f ? dy[i] : 0.f;
}

/* ---- Minus, L1Norm / L2Norm, ReduceMean, AXPBY ------------------------------------------------
 * orc_minus            deep8/src/math/Minus.cpp:109-143 (z = x - y, size-1 axes broadcast)
 * orc_minus_grad_y     deep8/src/math/Minus.cpp:268-294 (dy -= dz.sum(axes that differ)); MinusGradX
 *                      (Minus.cpp:163-189) is orc_add_grad
 * orc_l1norm           deep8/src/math/L1Norm.cpp:42-54   (y[b] = sum |x[b][:]|)
 * orc_l1norm_grad      deep8/src/math/L1Norm.cpp:72-99   (dx += dy[b] * sign(x), sign(0) = 0)
 * orc_l2norm           deep8/src/math/L2Norm.cpp:45-57   (y[b] = sqrt(sum x^2))
 * orc_l2norm_grad      deep8/src/math/L2Norm.cpp:77-90   (dx += dy[b] / y[b] * x)
 * orc_reduce_mean      deep8/src/math/ReduceMean.cpp:124-157 (mean over the axes where yd is 1)
 * orc_reduce_mean_grad deep8/src/math/ReduceMean.cpp:285-320 (dx += dy broadcast / ratio)
 * orc_axpby            deep8/src/math/AXPBY.cpp:23-31    (z = x * alpha + y * beta)
 * Sums are carried in double.  Pins: numpy expressions of the same formulas, the live reference
 * build and the golden fixtures (tests/test_oracle_pins.py). */
void orc_minus(const float *x, const int *xd, const float *y, const int *yd, float *z, const int *zd) {
    long n = 1;
    for (int i = 0; i < 5; ++i) n *= zd[i];
    for (long e = 0; e < n; ++e) {
        long rem = e, xi = 0, yi = 0;
        for (int a = 0; a < 5; ++a) {
            const long zs = stride5(zd, a), idx = rem / zs;
            rem -= idx * zs;
            if (xd[a] != 1) xi += idx * stride5(xd, a);
            if (yd[a] != 1) yi += idx * stride5(yd, a);
        }
        z[e] = x[xi] - y[yi];
    }
}

/* out[o] = sum of scale-free dz over the axes where d is 1 and zd is not, in double */
static double *sum_to(const int *d, const float *dz, const int *zd, long *n_out) {
    long n = 1, nz = 1;
    for (int i = 0; i < 5; ++i) n *= d[i], nz *= zd[i];
    double *acc = (double *)calloc((size_t)n, sizeof(double));
    for (long e = 0; e < nz; ++e) {
        long rem = e, o = 0;
        for (int a = 0; a < 5; ++a) {
            const long zs = stride5(zd, a), idx = rem / zs;
            rem -= idx * zs;
            if (d[a] != 1) o += idx * stride5(d, a);
        }
        acc[o] += (double)dz[e];
    }
    *n_out = n;
    return acc;
}

void orc_minus_grad_y(float *dy, const int *d, const float *dz, const int *zd) {
    long n;
    double *acc = sum_to(d, dz, zd, &n);
    for (long o = 0; o < n; ++o) dy[o] -= (float)acc[o];
    free(acc);
}

void orc_l1norm(const float *x, float *y, int batch, long size) {
    for (int b = 0; b < batch; ++b) {
        double acc = 0;
        for (long i = 0; i < size; ++i) acc += fabs((double)x[b * size + i]);
        y[b] = (float)acc;
    }
}

void orc_l1norm_grad(const float *x, float *dx, const float *dy, int batch, long size) {
    for (int b = 0; b < batch; ++b)
        for (long i = 0; i < size; ++i) {
            const float v = x[b * size + i];
            dx[b * size + i] += v > 0.f ? dy[b] : (v == 0.f ? 0.f : -dy[b]);
        }
}

void orc_l2norm(const float *x, float *y, int batch, long size) {
    for (int b = 0; b < batch; ++b) {
        double acc = 0;
        for (long i = 0; i < size; ++i) acc += (double)x[b * size + i] * (double)x[b * size + i];
        y[b] = (float)sqrt(acc);
    }
}

void orc_l2norm_grad(const float *x, float *dx, const float *y, const float *dy, int batch, long size) {
    for (int b = 0; b < batch; ++b)
        for (long i = 0; i < size; ++i) dx[b * size + i] += dy[b] / y[b] * x[b * size + i];
}

void orc_reduce_mean(const float *x, const int *xd, float *y, const int *yd) {
    long n, nx = 1;
    for (int i = 0; i < 5; ++i) nx *= xd[i];
    double *acc = sum_to(yd, x, xd, &n);
    const double count = (double)nx / (double)n;
    for (long o = 0; o < n; ++o) y[o] = (float)(acc[o] / count);
    free(acc);
}

void orc_reduce_mean_grad(float *dx, const int *xd, const float *dy, const int *yd) {
    long nx = 1, ny = 1;
    for (int i = 0; i < 5; ++i) nx *= xd[i], ny *= yd[i];
    const float ratio = (float)(nx / ny);
    for (long e = 0; e < nx; ++e) {
        long rem = e, o = 0;
        for (int a = 0; a < 5; ++a) {
            const long zs = stride5(xd, a), idx = rem / zs;
            rem -= idx * zs;
            if (yd[a] != 1) o += idx * stride5(yd, a);
        }
        dx[e] += dy[o] / ratio;
    }
}

void orc_axpby(const float *x, float alpha, const float *y, float beta, float *z, long n) {
    for (long i = 0; i < n; ++i) z[i] = x[i] * alpha + y[i] * beta;
}

/* deep8/src/math/AdamUpdate.cpp:25-41: the four Eigen statements in their order, float arithmetic
 * as there (T = float); ratio computed in float from float pow / sqrt.  Pins: the live reference
 * build, the golden fixtures and a textbook bias-corrected Adam step in numpy. */
void orc_adam_update(float *value, float *gradient, float *m, float *v, float beta1, float beta2, float epsilon,
                     float learning_rate, float weight_decay, long steps, long n) {
    if (steps <= 0) steps = 1;
    const float ratio = learning_rate * sqrtf(1.0f - powf(beta2, (float)steps)) / (1.0f - powf(beta1, (float)steps));
    for (long i = 0; i < n; ++i) {
        gradient[i] += value[i] * weight_decay;
        m[i] = m[i] * beta1 + gradient[i] * (1.0f - beta1);
        v[i] = v[i] * beta2 + gradient[i] * gradient[i] * (1.0f - beta2);
        value[i] -= m[i] / (sqrtf(v[i]) + epsilon) * ratio;
    }
}

/* ---- MaxPooling2d / AvgPooling2d ----------------------------------------------------------------
 * Forward: deep8/src/math/MaxPooling2d.cpp:99-142 and AvgPooling2d.cpp:99-142 -- patches of the image
 * padded with zeros (pad = max(0, (O-1)s + F - I), top = pad / 2), reduced with maximum / mean over
 * the FH x FW positions.  Gradients: MaxPooling2d.cpp:199-251 (first maximum of the window clipped
 * to the image, strict >) and AvgPooling2d.cpp:199-245 (ratio = 1 / (FH FW) to every in-image
 * element).  Pins: torch max_pool2d / avg_pool2d (+ autograd) for windows inside the image, a
 * zero-padded copy for the others, the live reference build and the golden fixtures. */
static void pool_geo(int IH, int IW, int FH, int FW, int covered, int sy, int sx, int *OH, int *OW, int *pt, int *pl) {
    if (!covered) {
        *OH = (IH - FH) / sy + 1;
        *OW = (IW - FW) / sx + 1;
    } else {
        *OH = (IH - 1) / sy + 1;
        *OW = (IW - 1) / sx + 1;
    }
    int py = (*OH - 1) * sy + FH - IH, px = (*OW - 1) * sx + FW - IW;
    *pt = (py > 0 ? py : 0) / 2;
    *pl = (px > 0 ? px : 0) / 2;
}

void orc_pool2d(int is_max, const float *x, float *y, int B, int IH, int IW, int C, int FH, int FW, int covered, int sy, int sx) {
    int OH, OW, pt, pl;
    pool_geo(IH, IW, FH, FW, covered, sy, sx, &OH, &OW, &pt, &pl);
    for (int b = 0; b < B; ++b)
        for (int oh = 0; oh < OH; ++oh)
            for (int ow = 0; ow < OW; ++ow)
                for (int c = 0; c < C; ++c) {
                    double acc = 0;
                    float mx = 0;
                    int first = 1;
                    for (int fh = 0; fh < FH; ++fh)
                        for (int fw = 0; fw < FW; ++fw) {
                            const int ih = oh * sy + fh - pt, iw = ow * sx + fw - pl;
                            const float v = (ih >= 0 && ih < IH && iw >= 0 && iw < IW) ? x[(((size_t)b * IH + ih) * IW + iw) * C + c] : 0.f;
                            acc += v;
                            if (first || v > mx) mx = v;
                            first = 0;
                        }
                    y[(((size_t)b * OH + oh) * OW + ow) * C + c] = is_max ? mx : (float)(acc / ((double)FH * FW));
                }
}

void orc_pool2d_grad(int is_max, const float *x, float *dx, const float *dy, int B, int IH, int IW, int C, int FH, int FW,
                     int covered, int sy, int sx) {
    int OH, OW, pt, pl;
    pool_geo(IH, IW, FH, FW, covered, sy, sx, &OH, &OW, &pt, &pl);
    const float ratio = 1.0f / ((float)FH * (float)FW);
    for (int b = 0; b < B; ++b)
        for (int c = 0; c < C; ++c)
            for (int oh = 0; oh < OH; ++oh)
                for (int ow = 0; ow < OW; ++ow) {
                    int h0 = oh * sy - pt, h1 = h0 + FH, w0 = ow * sx - pl, w1 = w0 + FW;
                    if (h0 < 0) h0 = 0;
                    if (h1 > IH) h1 = IH;
                    if (w0 < 0) w0 = 0;
                    if (w1 > IW) w1 = IW;
                    if (h0 >= h1 || w0 >= w1) continue;
                    const float g = dy[(((size_t)b * OH + oh) * OW + ow) * C + c];
                    if (!is_max) {
                        for (int h = h0; h < h1; ++h)
                            for (int w = w0; w < w1; ++w) dx[(((size_t)b * IH + h) * IW + w) * C + c] += ratio * g;
                        continue;
                    }
                    int mh = h0, mw = w0;
                    float mv = x[(((size_t)b * IH + h0) * IW + w0) * C + c];
                    for (int h = h0; h < h1; ++h)
                        for (int w = w0; w < w1; ++w) {
                            const float v = x[(((size_t)b * IH + h) * IW + w) * C + c];
                            if (v > mv) mv = v, mh = h, mw = w;
                        }
                    dx[(((size_t)b * IH + mh) * IW + mw) * C + c] += g;
                }
}

int orc_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

static int imax(int a, int b) { return a > b ? a : b; }

/* ---------------------------------------------------------------------------------------- */
/* deep8/src/math/Conv2d.cpp:20-32 (output size), :341-350 (padding) */
void orc_conv2d_geometry(int IH, int IW, int FH, int FW, int covered,
                         int sy, int sx, int dy, int dx, int *out) {
    int rfh = FH + (FH - 1) * (dy - 1);
    int rfw = FW + (FW - 1) * (dx - 1);
    int OH, OW;
    if (!covered) {
        OH = (IH - rfh) / sy + 1;
        OW = (IW - rfw) / sx + 1;
    } else {
        OH = (IH - 1) / sy + 1;
        OW = (IW - 1) / sx + 1;
    }
    out[0] = OH;
    out[1] = OW;
    out[2] = imax(0, (OH - 1) * sy + rfh - IH) / 2;
    out[3] = imax(0, (OW - 1) * sx + rfw - IW) / 2;
}

/* deep8/src/math/DeConv2d.cpp:23-29 (output size), :295-301 (padding) */
void orc_deconv2d_geometry(int IH, int IW, int FH, int FW, int covered,
                           int sy, int sx, int *out) {
    int OH, OW;
    if (!covered) {
        OH = (IH - 1) * sy + FH;
        OW = (IW - 1) * sx + FW;
    } else {
        OH = (IH - 1) * sy + 1;
        OW = (IW - 1) * sx + 1;
    }
    out[0] = OH;
    out[1] = OW;
    out[2] = imax(0, OH + FH - (IH - 1) * sy - 2) / 2;
    out[3] = imax(0, OW + FW - (IW - 1) * sx - 2) / 2;
}

/* the contraction path, once per element type */
#define REAL float
#define ORC(name) orc_##name
#include "deep8_oracle_path.inc"
#undef REAL
#undef ORC
#define REAL double
#define ORC(name) orc_##name##_f64
#include "deep8_oracle_path.inc"
#undef REAL
#undef ORC

/* ---------------------------------------------------------------------------------------- */
/* deep8/src/math/Conv2d.cu:27-60 (padTop there is stored negated) */
void orc_im2col(const float *im, float *col, int B, int IH, int IW, int C, int OH, int OW,
                int FH, int FW, int sy, int sx, int dy, int dx, int padTop, int padLeft) {
    size_t K = (size_t)FH * FW * C;
#pragma omp parallel for schedule(static)
    for (long r = 0; r < (long)B * OH * OW; ++r) {
        int b = (int)(r / ((long)OH * OW));
        int oy = (int)((r / OW) % OH);
        int ox = (int)(r % OW);
        for (int fy = 0; fy < FH; ++fy)
            for (int fx = 0; fx < FW; ++fx) {
                float *dst = col + (size_t)r * K + ((size_t)fy * FW + fx) * C;
                int iy = oy * sy + fy * dy - padTop;
                int ix = ox * sx + fx * dx - padLeft;
                if (iy < 0 || iy >= IH || ix < 0 || ix >= IW) {
                    for (int c = 0; c < C; ++c) dst[c] = 0.f;
                } else {
                    memcpy(dst, im + (((size_t)b * IH + iy) * IW + ix) * C, sizeof(float) * C);
                }
            }
    }
}

/* deep8/src/math/Conv2d.cu:82-117: gather form, one image pixel at a time, filter taps in
 * (fy, fx) ascending order, each tap added to the running float value -- the same order of
 * float additions as the reference kernel, so results are comparable bit for bit. */
void orc_col2im(const float *col, float *im, int B, int IH, int IW, int C, int OH, int OW,
                int FH, int FW, int sy, int sx, int dy, int dx, int padTop, int padLeft) {
    size_t K = (size_t)FH * FW * C;
#pragma omp parallel for schedule(static)
    for (long p = 0; p < (long)B * IH * IW; ++p) {
        int b = (int)(p / ((long)IH * IW));
        int iy = (int)((p / IW) % IH);
        int ix = (int)(p % IW);
        float *dst = im + (size_t)p * C;
        for (int fy = 0; fy < FH; ++fy) {
            int ty = iy + padTop - fy * dy;
            if (ty < 0 || ty % sy) continue;
            int oy = ty / sy;
            if (oy >= OH) continue;
            for (int fx = 0; fx < FW; ++fx) {
                int tx = ix + padLeft - fx * dx;
                if (tx < 0 || tx % sx) continue;
                int ox = tx / sx;
                if (ox >= OW) continue;
                const float *src = col + (((size_t)b * OH + oy) * OW + ox) * K + ((size_t)fy * FW + fx) * C;
                for (int c = 0; c < C; ++c) dst[c] += src[c];
            }
        }
    }
}

/* deep8/src/math/DeConv2d.cu:27-57 (padTop there is stored negated); overwrites z */
void orc_deconv_col2im(const float *zmat, float *z, int B, int IH, int IW, int OH, int OW, int OC,
                       int FH, int FW, int sy, int sx, int padTop, int padLeft) {
    size_t N = (size_t)OC * FH * FW;
#pragma omp parallel for schedule(static)
    for (long p = 0; p < (long)B * OH * OW; ++p) {
        int b = (int)(p / ((long)OH * OW));
        int oy = (int)((p / OW) % OH);
        int ox = (int)(p % OW);
        for (int oc = 0; oc < OC; ++oc) {
            float acc = 0.f;
            for (int fy = 0; fy < FH; ++fy) {
                int ty = oy - padTop + fy;
                if (ty < 0 || ty % sy) continue;
                int iy = ty / sy;
                if (iy >= IH) continue;
                for (int fx = 0; fx < FW; ++fx) {
                    int tx = ox - padLeft + fx;
                    if (tx < 0 || tx % sx) continue;
                    int ix = tx / sx;
                    if (ix >= IW) continue;
                    acc += zmat[(((size_t)b * IH + iy) * IW + ix) * N + ((size_t)oc * FH + fy) * FW + fx];
                }
            }
            z[(size_t)p * OC + oc] = acc;
        }
    }
}

/* deep8/src/math/DeConv2d.cu:327-350 */
void orc_deconv_im2col(const float *dz, float *dzmat, int B, int IH, int IW, int OH, int OW, int OC,
                       int FH, int FW, int sy, int sx, int padTop, int padLeft) {
    size_t N = (size_t)OC * FH * FW;
#pragma omp parallel for schedule(static)
    for (long r = 0; r < (long)B * IH * IW; ++r) {
        int b = (int)(r / ((long)IH * IW));
        int iy = (int)((r / IW) % IH);
        int ix = (int)(r % IW);
        for (int oc = 0; oc < OC; ++oc)
            for (int fy = 0; fy < FH; ++fy)
                for (int fx = 0; fx < FW; ++fx) {
                    int oy = iy * sy + padTop - fy;
                    int ox = ix * sx + padLeft - fx;
                    float v = 0.f;
                    if (oy >= 0 && oy < OH && ox >= 0 && ox < OW)
                        v = dz[(((size_t)b * OH + oy) * OW + ox) * OC + oc];
                    dzmat[(size_t)r * N + ((size_t)oc * FH + fy) * FW + fx] = v;
                }
    }
}
