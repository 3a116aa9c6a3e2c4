/*
 * TEST INFRASTRUCTURE ONLY.  Runs every contraction-path function of deep8_oracle.c once or twice on small,
 * awkward geometries with buffers of exactly the documented sizes, so that a build with
 * -fsanitize=address,undefined (make -C oracle asan) reports any access outside them and any undefined arithmetic.
 * It checks no values: the parity tests do that.
 */
#include <stdio.h>
#include <stdlib.h>

#include "deep8_oracle.h"

static float *buf(long n) {
    float *p = (float *)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
    for (long i = 0; i < n; ++i) p[i] = (float)((i * 7 + 3) % 11) - 5.f;
    return p;
}

static void matmul_case(int xb, int xr, int xc, int yb, int yc) {
    const int zb = xb > yb ? xb : yb;
    float *x = buf((long)xb * xr * xc), *y = buf((long)yb * xc * yc), *z = buf((long)zb * xr * yc);
    orc_matmul(x, xb, xr, xc, y, yb, xc, yc, z);
    orc_matmul_grad_x(x, xb, xr, xc, y, yb, xc, yc, z);
    orc_matmul_grad_y(x, xb, xr, xc, y, yb, xc, yc, z);
    free(x), free(y), free(z);
}

static void conv_case(int B, int IH, int IW, int IC, int OC, int FH, int FW, int cov, int sy, int sx, int dy, int dx) {
    int g[4];
    orc_conv2d_geometry(IH, IW, FH, FW, cov, sy, sx, dy, dx, g);
    const long nx = (long)B * IH * IW * IC, nw = (long)OC * FH * FW * IC, nz = (long)B * g[0] * g[1] * OC;
    const long ncol = (long)B * g[0] * g[1] * FH * FW * IC;
    float *x = buf(nx), *w = buf(nw), *z = buf(nz), *col = buf(ncol);
    orc_conv2d(x, B, IH, IW, IC, w, OC, FH, FW, z, cov, sy, sx, dy, dx);
    orc_conv2d_grad_x(x, B, IH, IW, IC, w, OC, FH, FW, z, cov, sy, sx, dy, dx);
    orc_conv2d_grad_y(x, B, IH, IW, IC, w, OC, FH, FW, z, cov, sy, sx, dy, dx);
    orc_im2col(x, col, B, IH, IW, IC, g[0], g[1], FH, FW, sy, sx, dy, dx, g[2], g[3]);
    orc_col2im(col, x, B, IH, IW, IC, g[0], g[1], FH, FW, sy, sx, dy, dx, g[2], g[3]);
    free(x), free(w), free(z), free(col);
}

static void deconv_case(int B, int IH, int IW, int IC, int OC, int FH, int FW, int cov, int sy, int sx) {
    int g[4];
    orc_deconv2d_geometry(IH, IW, FH, FW, cov, sy, sx, g);
    const long nx = (long)B * IH * IW * IC, nw = (long)OC * FH * FW * IC, nz = (long)B * g[0] * g[1] * OC;
    const long nmat = (long)B * IH * IW * OC * FH * FW;
    float *x = buf(nx), *w = buf(nw), *z = buf(nz), *mat = buf(nmat);
    orc_deconv2d(x, B, IH, IW, IC, w, OC, FH, FW, z, cov, sy, sx);
    orc_deconv2d_grad_x(x, B, IH, IW, IC, w, OC, FH, FW, z, cov, sy, sx);
    orc_deconv2d_grad_y(x, B, IH, IW, IC, w, OC, FH, FW, z, cov, sy, sx);
    orc_deconv_im2col(z, mat, B, IH, IW, g[0], g[1], OC, FH, FW, sy, sx, g[2], g[3]);
    orc_deconv_col2im(mat, z, B, IH, IW, g[0], g[1], OC, FH, FW, sy, sx, g[2], g[3]);
    free(x), free(w), free(z), free(mat);
}

int main(void) {
    matmul_case(3, 5, 7, 1, 4);   /* collapsed batch */
    matmul_case(1, 6, 5, 4, 1);   /* batch of vectors */
    matmul_case(3, 4, 5, 3, 2);   /* batched both */
    matmul_case(1, 4, 5, 3, 2);   /* x broadcast */
    matmul_case(1, 1, 1, 1, 1);
    {
        float *a = buf(6 * 9), *b = buf(9 * 5), *c = buf(6 * 8);
        orc_gemm(0, 0, 6, 5, 7, a, 9, b, 5, 0.f, c, 8);
        orc_gemm(0, 1, 6, 5, 7, a, 9, b, 9, 1.f, c, 8);
        orc_gemm(1, 0, 6, 5, 7, a, 6, b, 5, 1.f, c, 8);
        free(a), free(b), free(c);
    }
    conv_case(2, 9, 7, 3, 4, 3, 3, 1, 1, 1, 1, 1);
    conv_case(1, 8, 8, 2, 3, 4, 4, 1, 2, 2, 2, 2);
    conv_case(2, 7, 9, 2, 2, 3, 2, 0, 2, 1, 1, 2);
    conv_case(1, 5, 5, 1, 1, 2, 2, 1, 3, 3, 1, 1);  /* stride larger than the filter */
    conv_case(1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1);
    deconv_case(2, 4, 5, 3, 2, 4, 4, 0, 2, 2);
    deconv_case(1, 5, 4, 2, 3, 4, 4, 1, 3, 3);
    deconv_case(1, 3, 3, 2, 2, 2, 2, 0, 3, 3);      /* stride larger than the filter */
    deconv_case(2, 4, 4, 1, 1, 3, 2, 1, 1, 2);
    printf("oracle self-test under the sanitizers: no report\n");
    return 0;
}
