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
 *   Math::Minus / MinusGradX / MinusGradY     deep8/src/math/Minus.cpp:7-107
 *   Math::L1Norm / L1NormGrad                 deep8/src/math/L1Norm.cpp:6-39
 *   Math::L2Norm / L2NormGrad                 deep8/src/math/L2Norm.cpp:6-42
 *   Math::ReduceMean / ReduceMeanGrad         deep8/src/math/ReduceMean.cpp:7-121
 *   Math::AXPBY                               deep8/src/math/AXPBY.cpp:6-20
 *   Math::AdamUpdate                          deep8/src/math/AdamUpdate.cpp:6-23
 *   Math::MaxPooling2d / MaxPooling2dGrad     deep8/src/math/MaxPooling2d.cpp:6-96
 *   Math::AvgPooling2d / AvgPooling2dGrad     deep8/src/math/AvgPooling2d.cpp
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
#include "math/Minus.h"
#include "math/L1Norm.h"
#include "math/L2Norm.h"
#include "math/ReduceMean.h"
#include "math/AXPBY.h"
#include "math/AdamUpdate.h"
#include "math/MaxPooling2d.h"
#include "math/AvgPooling2d.h"

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

/* Element type of every tensor wrapped from now on: float, or double after ref_set_double(1)
 * (the pointers then address doubles whatever the prototypes below say). */
bool g_double = false;

void wrap(Wrapped &w, const float *ptr, size_t batch, std::vector<size_t> dims) {
    Shape shape(batch, dims);
    TensorStorage storage((void *)ptr, &w.ref, (g_double ? sizeof(double) : sizeof(float)) * shape.size(), cpu());
    w.ref += 1;
    w.t.reset(new Tensor(storage, 0, shape, g_double ? ElementType::from<double>() : ElementType::from<float>()));
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

/* Selects the reference's Float64 path for the calls that follow (used for MatrixMultiply, Conv2d
 * and DeConv2d only). */
void ref_set_double(int on) { g_double = on != 0; }

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

int ref_minus(const float *x, int xb, int xnd, const int *xd, const float *y, int yb, int ynd, const int *yd,
              float *z, int zb, int znd, const int *zd) {
    return guarded([&] {
        Wrapped X, Y, Z;
        wrap(X, x, xb, vdims(xnd, xd));
        wrap(Y, y, yb, vdims(ynd, yd));
        wrap(Z, z, zb, vdims(znd, zd));
        Math::Minus(*X.t, *Y.t, *Z.t);
    });
}

/* which = 0: MinusGradX (g plays dx), 1: MinusGradY (g plays dy) */
int ref_minus_grad(int which, const float *x, int xb, int xnd, const int *xd, const float *y, int yb, int ynd,
                   const int *yd, float *g, const float *z, const float *dz, int zb, int znd, const int *zd) {
    return guarded([&] {
        Wrapped X, Y, Z, G, DZ;
        wrap(X, x, xb, vdims(xnd, xd));
        wrap(Y, y, yb, vdims(ynd, yd));
        wrap(Z, z, zb, vdims(znd, zd));
        wrap(DZ, dz, zb, vdims(znd, zd));
        if (0 == which) {
            wrap(G, g, xb, vdims(xnd, xd));
            Math::MinusGradX(*X.t, *G.t, *Y.t, *Z.t, *DZ.t);
        } else {
            wrap(G, g, yb, vdims(ynd, yd));
            Math::MinusGradY(*X.t, *Y.t, *G.t, *Z.t, *DZ.t);
        }
    });
}

/* which = 1: L1Norm, 2: L2Norm; y is (batch, {1}) */
int ref_norm(int which, const float *x, int b, int nd, const int *d, float *y) {
    return guarded([&] {
        Wrapped X, Y;
        wrap(X, x, b, vdims(nd, d));
        wrap(Y, y, b, std::vector<size_t>{1});
        if (1 == which) Math::L1Norm(*X.t, *Y.t);
        else Math::L2Norm(*X.t, *Y.t);
    });
}

int ref_norm_grad(int which, const float *x, float *dx, int b, int nd, const int *d, const float *y, const float *dy) {
    return guarded([&] {
        Wrapped X, DX, Y, DY;
        wrap(X, x, b, vdims(nd, d));
        wrap(DX, dx, b, vdims(nd, d));
        wrap(Y, y, b, std::vector<size_t>{1});
        wrap(DY, dy, b, std::vector<size_t>{1});
        if (1 == which) Math::L1NormGrad(*X.t, *DX.t, *Y.t, *DY.t);
        else Math::L2NormGrad(*X.t, *DX.t, *Y.t, *DY.t);
    });
}

/* the output shape is derived as the reference's ReduceMean::checkShape does (deep8/src/nodes/ReduceMean.cpp:11-57) */
static void mean_shape(int b, int nd, const int *d, const std::vector<int> &axis, bool keep, size_t &yb, std::vector<size_t> &yl) {
    const int rank = nd + 1;
    std::vector<bool> red(rank, axis.empty());
    for (int a : axis) red[(a + rank) % rank] = true;
    yb = red[0] ? 1 : (size_t)b;
    for (int i = 1; i < rank; ++i) {
        if (red[i]) {
            if (keep) yl.push_back(1);
        } else {
            yl.push_back((size_t)d[i - 1]);
        }
    }
    if (yl.empty()) yl.push_back(1);
}

int ref_reduce_mean(const float *x, int b, int nd, const int *d, float *y, const int *axis, int naxis, int keep) {
    return guarded([&] {
        std::vector<int> ax(axis, axis + naxis);
        size_t yb;
        std::vector<size_t> yl;
        mean_shape(b, nd, d, ax, keep != 0, yb, yl);
        Wrapped X, Y;
        wrap(X, x, b, vdims(nd, d));
        wrap(Y, y, (int)yb, yl);
        Math::ReduceMean(*X.t, *Y.t, ax, keep != 0);
    });
}

int ref_reduce_mean_grad(const float *x, float *dx, int b, int nd, const int *d, const float *y, const float *dy,
                         const int *axis, int naxis, int keep) {
    return guarded([&] {
        std::vector<int> ax(axis, axis + naxis);
        size_t yb;
        std::vector<size_t> yl;
        mean_shape(b, nd, d, ax, keep != 0, yb, yl);
        Wrapped X, DX, Y, DY;
        wrap(X, x, b, vdims(nd, d));
        wrap(DX, dx, b, vdims(nd, d));
        wrap(Y, y, (int)yb, yl);
        wrap(DY, dy, (int)yb, yl);
        Math::ReduceMeanGrad(*X.t, *DX.t, *Y.t, *DY.t, ax, keep != 0);
    });
}

int ref_axpby(const float *x, float alpha, const float *y, float beta, float *z, int b, int nd, const int *d) {
    return guarded([&] {
        Wrapped X, Y, Z;
        wrap(X, x, b, vdims(nd, d));
        wrap(Y, y, b, vdims(nd, d));
        wrap(Z, z, b, vdims(nd, d));
        Math::AXPBY(*X.t, alpha, *Y.t, beta, *Z.t);
    });
}

int ref_adam_update(float *value, float *gradient, float *m, float *v, float beta1, float beta2, float epsilon,
                    float learningRate, float weightDecay, long steps, int b, int nd, const int *d) {
    return guarded([&] {
        Wrapped X, G, M, V;
        wrap(X, value, b, vdims(nd, d));
        wrap(G, gradient, b, vdims(nd, d));
        wrap(M, m, b, vdims(nd, d));
        wrap(V, v, b, vdims(nd, d));
        Math::AdamUpdate(*X.t, *G.t, *M.t, *V.t, beta1, beta2, epsilon, learningRate, weightDecay, (int64_t)steps);
    });
}

int ref_pool2d(int is_max, const float *x, float *y, int B, int IH, int IW, int C, int OH, int OW, int FH, int FW,
               int covered, int sy, int sx) {
    return guarded([&] {
        Wrapped X, Y;
        wrap(X, x, B, {(size_t)IH, (size_t)IW, (size_t)C});
        wrap(Y, y, B, {(size_t)OH, (size_t)OW, (size_t)C});
        if (is_max) Math::MaxPooling2d(*X.t, *Y.t, covered != 0, FH, FW, sy, sx);
        else Math::AvgPooling2d(*X.t, *Y.t, covered != 0, FH, FW, sy, sx);
    });
}

int ref_pool2d_grad(int is_max, const float *x, float *dx, const float *y, const float *dy, int B, int IH, int IW, int C,
                    int OH, int OW, int FH, int FW, int covered, int sy, int sx) {
    return guarded([&] {
        Wrapped X, DX, Y, DY;
        wrap(X, x, B, {(size_t)IH, (size_t)IW, (size_t)C});
        wrap(DX, dx, B, {(size_t)IH, (size_t)IW, (size_t)C});
        wrap(Y, y, B, {(size_t)OH, (size_t)OW, (size_t)C});
        wrap(DY, dy, B, {(size_t)OH, (size_t)OW, (size_t)C});
        if (is_max) Math::MaxPooling2dGrad(*X.t, *DX.t, *Y.t, *DY.t, covered != 0, FH, FW, sy, sx);
        else Math::AvgPooling2dGrad(*X.t, *DX.t, *Y.t, *DY.t, covered != 0, FH, FW, sy, sx);
    });
}

}  // extern "C"
