/*
 * TEST INFRASTRUCTURE ONLY -- never linked into or called from the product path.
 *
 * C-ABI shim around the *unmodified* Deep8 CPU (Eigen) implementation.  The reference sources
 * are compiled where they lie (see oracle/Makefile); this file only wraps caller memory in
 * Deep8 Tensors and calls the reference's public dispatchers:
 *
 *   Math::MatrixMultiply / GradX / GradY      deep8/src/math/MatrixMultiply.cpp:7-91
 *   Math::Conv2d / GradX / GradY              deep8/src/math/Conv2d.cpp:46-96,140-193,237-290
 *   Math::DeConv2d / GradX / GradY            deep8/src/math/DeConv2d.cpp:43-82,122-162,203-243
 *   Math::Add / AddGradX / AddGradY           deep8/src/math/Add.cpp:7-107
 *   Math::ReLu / ReLuGrad                     deep8/src/math/ReLu.cpp:6-36
 *
 * plus one materialisation of the patch expression the CPU Conv2d contracts over
 * (deep8/src/math/Conv2d.cpp:352-356), which is the "CPU Eigen im2col" the HIP im2col must
 * equal bit for bit, and the two DeConv2d patch expressions (DeConv2d.cpp:303-306,411-414).
 *
 * Every function returns 0 on success, 1 for std::invalid_argument, 2 for any other
 * exception; ref_last_error() returns the message.
 */
#include "model/Device.h"
#include "model/Tensor.h"
#include "math/MatrixMultiply.h"
#include "math/Conv2d.h"
#include "math/DeConv2d.h"
#include "math/Add.h"
#include "math/ReLu.h"

#include <chrono>
#include <cstring>
#include <memory>
#include <string>

using namespace Deep8;

namespace {

std::string g_error;

CPUDevice *cpu() {
    static CPUDevice *device = new CPUDevice();
    return device;
}

/* Wrap caller memory without copying.  The storage's reference count lives in `ref` and is
 * bumped once more so that it never reaches zero: the pool must never try to free memory it
 * does not own. */
struct Wrapped {
    size_t ref;
    std::unique_ptr<Tensor> t;
};

void wrap(Wrapped &w, const float *ptr, size_t batch, std::vector<size_t> dims) {
    Shape shape(batch, dims);
    TensorStorage storage((void *)ptr, &w.ref, sizeof(float) * shape.size(), cpu());
    w.ref += 1;
    w.t.reset(new Tensor(storage, 0, shape, ElementType::from<float>()));
}

std::vector<size_t> mdims(int nd, int r, int c) {
    if (1 == nd) return {(size_t)r};
    return {(size_t)r, (size_t)c};
}

template <typename F>
int guarded(F f) {
    try {
        f();
        return 0;
    } catch (const std::invalid_argument &e) {
        g_error = e.what();
        return 1;
    } catch (const std::exception &e) {
        g_error = e.what();
        return 2;
    }
}

struct MM {
    Wrapped x, y, z, dx, dy, dz;
};

}  // namespace

extern "C" {

const char *ref_last_error() { return g_error.c_str(); }

/* thread count the reference's CPUDevice gives Eigen (deep8/src/model/Device.cpp:67-85) */
int ref_threads() { return cpu()->getDeviceThreadNum(); }

/* A matrix operand is (batch, nDims in {1,2}, rows, cols).  z has batch max(xb,yb), rows xr and
 * is 1-D when y has one column (deep8/src/nodes/MatrixMultiply.cpp:23-27). */
int ref_matmul(const float *x, int xb, int xnd, int xr, int xc,
               const float *y, int yb, int ynd, int yr, int yc,
               float *z, int zb, int znd, int zr, int zc) {
    return guarded([&] {
        MM m;
        wrap(m.x, x, xb, mdims(xnd, xr, xc));
        wrap(m.y, y, yb, mdims(ynd, yr, yc));
        wrap(m.z, z, zb, mdims(znd, zr, zc));
        Math::MatrixMultiply(*m.x.t, *m.y.t, *m.z.t);
    });
}

int ref_matmul_grad_x(const float *x, float *dx, int xb, int xnd, int xr, int xc,
                      const float *y, int yb, int ynd, int yr, int yc,
                      const float *z, const float *dz, int zb, int znd, int zr, int zc) {
    return guarded([&] {
        MM m;
        wrap(m.x, x, xb, mdims(xnd, xr, xc));
        wrap(m.dx, dx, xb, mdims(xnd, xr, xc));
        wrap(m.y, y, yb, mdims(ynd, yr, yc));
        wrap(m.z, z, zb, mdims(znd, zr, zc));
        wrap(m.dz, dz, zb, mdims(znd, zr, zc));
        Math::MatrixMultiplyGradX(*m.x.t, *m.dx.t, *m.y.t, *m.z.t, *m.dz.t);
    });
}

int ref_matmul_grad_y(const float *x, int xb, int xnd, int xr, int xc,
                      const float *y, float *dy, int yb, int ynd, int yr, int yc,
                      const float *z, const float *dz, int zb, int znd, int zr, int zc) {
    return guarded([&] {
        MM m;
        wrap(m.x, x, xb, mdims(xnd, xr, xc));
        wrap(m.y, y, yb, mdims(ynd, yr, yc));
        wrap(m.dy, dy, yb, mdims(ynd, yr, yc));
        wrap(m.z, z, zb, mdims(znd, zr, zc));
        wrap(m.dz, dz, zb, mdims(znd, zr, zc));
        Math::MatrixMultiplyGradY(*m.x.t, *m.y.t, *m.dy.t, *m.z.t, *m.dz.t);
    });
}

/* x [B,IH,IW,IC], w [OC,FH,FW,IC] (batch 1), z [B,OH,OW,OC] */
int ref_conv2d(const float *x, int B, int IH, int IW, int IC,
               const float *w, int OC, int FH, int FW,
               float *z, int OH, int OW,
               int covered, int sy, int sx, int dy, int dx) {
    return guarded([&] {
        Wrapped X, W, Z;
        wrap(X, x, B, {(size_t)IH, (size_t)IW, (size_t)IC});
        wrap(W, w, 1, {(size_t)OC, (size_t)FH, (size_t)FW, (size_t)IC});
        wrap(Z, z, B, {(size_t)OH, (size_t)OW, (size_t)OC});
        Math::Conv2d(*X.t, *W.t, *Z.t, covered != 0, sy, sx, dy, dx, nullptr);
    });
}

int ref_conv2d_grad_x(const float *x, float *gx, int B, int IH, int IW, int IC,
                      const float *w, int OC, int FH, int FW,
                      const float *z, const float *gz, int OH, int OW,
                      int covered, int sy, int sx, int dy, int dx) {
    return guarded([&] {
        Wrapped X, GX, W, Z, GZ;
        wrap(X, x, B, {(size_t)IH, (size_t)IW, (size_t)IC});
        wrap(GX, gx, B, {(size_t)IH, (size_t)IW, (size_t)IC});
        wrap(W, w, 1, {(size_t)OC, (size_t)FH, (size_t)FW, (size_t)IC});
        wrap(Z, z, B, {(size_t)OH, (size_t)OW, (size_t)OC});
        wrap(GZ, gz, B, {(size_t)OH, (size_t)OW, (size_t)OC});
        Math::Conv2dGradX(*X.t, *GX.t, *W.t, *Z.t, *GZ.t, covered != 0, sy, sx, dy, dx, nullptr);
    });
}

int ref_conv2d_grad_y(const float *x, int B, int IH, int IW, int IC,
                      const float *w, float *gw, int OC, int FH, int FW,
                      const float *z, const float *gz, int OH, int OW,
                      int covered, int sy, int sx, int dy, int dx) {
    return guarded([&] {
        Wrapped X, W, GW, Z, GZ;
        wrap(X, x, B, {(size_t)IH, (size_t)IW, (size_t)IC});
        wrap(W, w, 1, {(size_t)OC, (size_t)FH, (size_t)FW, (size_t)IC});
        wrap(GW, gw, 1, {(size_t)OC, (size_t)FH, (size_t)FW, (size_t)IC});
        wrap(Z, z, B, {(size_t)OH, (size_t)OW, (size_t)OC});
        wrap(GZ, gz, B, {(size_t)OH, (size_t)OW, (size_t)OC});
        Math::Conv2dGradY(*X.t, *W.t, *GW.t, *Z.t, *GZ.t, covered != 0, sy, sx, dy, dx, nullptr);
    });
}

int ref_deconv2d(const float *x, int B, int IH, int IW, int IC,
                 const float *w, int OC, int FH, int FW,
                 float *z, int OH, int OW, int covered, int sy, int sx) {
    return guarded([&] {
        Wrapped X, W, Z;
        wrap(X, x, B, {(size_t)IH, (size_t)IW, (size_t)IC});
        wrap(W, w, 1, {(size_t)OC, (size_t)FH, (size_t)FW, (size_t)IC});
        wrap(Z, z, B, {(size_t)OH, (size_t)OW, (size_t)OC});
        Math::DeConv2d(*X.t, *W.t, *Z.t, covered != 0, sy, sx, nullptr);
    });
}

int ref_deconv2d_grad_x(const float *x, float *gx, int B, int IH, int IW, int IC,
                        const float *w, int OC, int FH, int FW,
                        const float *z, const float *gz, int OH, int OW,
                        int covered, int sy, int sx) {
    return guarded([&] {
        Wrapped X, GX, W, Z, GZ;
        wrap(X, x, B, {(size_t)IH, (size_t)IW, (size_t)IC});
        wrap(GX, gx, B, {(size_t)IH, (size_t)IW, (size_t)IC});
        wrap(W, w, 1, {(size_t)OC, (size_t)FH, (size_t)FW, (size_t)IC});
        wrap(Z, z, B, {(size_t)OH, (size_t)OW, (size_t)OC});
        wrap(GZ, gz, B, {(size_t)OH, (size_t)OW, (size_t)OC});
        Math::DeConv2dGradX(*X.t, *GX.t, *W.t, *Z.t, *GZ.t, covered != 0, sy, sx, nullptr);
    });
}

int ref_deconv2d_grad_y(const float *x, int B, int IH, int IW, int IC,
                        const float *w, float *gw, int OC, int FH, int FW,
                        const float *z, const float *gz, int OH, int OW,
                        int covered, int sy, int sx) {
    return guarded([&] {
        Wrapped X, W, GW, Z, GZ;
        wrap(X, x, B, {(size_t)IH, (size_t)IW, (size_t)IC});
        wrap(W, w, 1, {(size_t)OC, (size_t)FH, (size_t)FW, (size_t)IC});
        wrap(GW, gw, 1, {(size_t)OC, (size_t)FH, (size_t)FW, (size_t)IC});
        wrap(Z, z, B, {(size_t)OH, (size_t)OW, (size_t)OC});
        wrap(GZ, gz, B, {(size_t)OH, (size_t)OW, (size_t)OC});
        Math::DeConv2dGradY(*X.t, *W.t, *GW.t, *Z.t, *GZ.t, covered != 0, sy, sx, nullptr);
    });
}

/*
 * The patch matrix the CPU path contracts over, materialised:
 *   im.extract_image_patches(FW, FH, strideX, strideY, dilX, dilY, inflateX, inflateY,
 *                            padTop, padBottom, padLeft, padRight, 0).reshape([B*OH*OW, FH*FW*C])
 * with the argument order of deep8/src/math/Conv2d.cpp:352-353 (inflate 1) and
 * deep8/src/math/DeConv2d.cpp:303 (stride 1, inflate = deconv stride).  `out` holds
 * B*OH*OW*FH*FW*C floats; the caller supplies OH/OW (they follow from the geometry).
 */
int ref_image_patches(const float *im, int B, int H, int W, int C,
                      int FH, int FW, int sy, int sx, int dy, int dx, int iy, int ix,
                      int padTop, int padBottom, int padLeft, int padRight,
                      int OH, int OW, float *out) {
    return guarded([&] {
        Eigen::TensorMap<Eigen::Tensor<float, 4, Eigen::RowMajor>> t((float *)im, B, H, W, C);
        Eigen::TensorMap<Eigen::Tensor<float, 2, Eigen::RowMajor>> o(out, B * OH * OW, FH * FW * C);
        Eigen::DSizes<int, 2> pre;
        pre[0] = B * OH * OW;
        pre[1] = FH * FW * C;
        o.device(*cpu()->eigenDevice) =
            t.extract_image_patches(FW, FH, sx, sy, dx, dy, ix, iy, padTop, padBottom, padLeft, padRight, 0.f)
                .reshape(pre);
    });
}

/* Add / ReLu.  A tensor is (batch, nd in 1..4, dims[nd]). */
static std::vector<size_t> vdims(int nd, const int *d) { return std::vector<size_t>(d, d + nd); }

int ref_add(const float *x, int xb, int xnd, const int *xd, const float *y, int yb, int ynd, const int *yd,
            float *z, int zb, int znd, const int *zd) {
    return guarded([&] {
        Wrapped X, Y, Z;
        wrap(X, x, xb, vdims(xnd, xd));
        wrap(Y, y, yb, vdims(ynd, yd));
        wrap(Z, z, zb, vdims(znd, zd));
        Math::Add(*X.t, *Y.t, *Z.t);
    });
}

/* which = 0: AddGradX (g plays dx), 1: AddGradY (g plays dy) */
int ref_add_grad(int which, const float *x, int xb, int xnd, const int *xd, const float *y, int yb, int ynd,
                 const int *yd, float *g, const float *z, const float *dz, int zb, int znd, const int *zd) {
    return guarded([&] {
        Wrapped X, Y, Z, G, DZ;
        wrap(X, x, xb, vdims(xnd, xd));
        wrap(Y, y, yb, vdims(ynd, yd));
        wrap(Z, z, zb, vdims(znd, zd));
        wrap(DZ, dz, zb, vdims(znd, zd));
        if (0 == which) {
            wrap(G, g, xb, vdims(xnd, xd));
            Math::AddGradX(*X.t, *G.t, *Y.t, *Z.t, *DZ.t);
        } else {
            wrap(G, g, yb, vdims(ynd, yd));
            Math::AddGradY(*X.t, *Y.t, *G.t, *Z.t, *DZ.t);
        }
    });
}

int ref_relu(const float *x, float *y, int b, int nd, const int *d) {
    return guarded([&] {
        Wrapped X, Y;
        wrap(X, x, b, vdims(nd, d));
        wrap(Y, y, b, vdims(nd, d));
        Math::ReLu(*X.t, *Y.t);
    });
}

int ref_relu_grad(const float *x, float *dx, const float *y, const float *dy, int b, int nd, const int *d) {
    return guarded([&] {
        Wrapped X, DX, Y, DY;
        wrap(X, x, b, vdims(nd, d));
        wrap(DX, dx, b, vdims(nd, d));
        wrap(Y, y, b, vdims(nd, d));
        wrap(DY, dy, b, vdims(nd, d));
        Math::ReLuGrad(*X.t, *DX.t, *Y.t, *DY.t);
    });
}

}  // extern "C"
