// Math:: dispatchers (argument checks as in the reference) and their GPU bodies, which hand the
// raw pointers and sizes to libdeep8_hip.so.  See deep8/Math.h for the reference line numbers.
#include <algorithm>
#include "deep8/Math.h"

#include "deep8_hip.h"

namespace Deep8 {
namespace Math {

namespace {

int dtypeOf(const Tensor &t) {
    switch (t.elementType.id) {
    case DType::Float64: return D8_FLOAT64;  // MatrixMultiply, Conv2d, DeConv2d and Constant only
    case DType::Float32: return D8_FLOAT32;
    case DType::Float16: return D8_FLOAT16;
    default: DEEP8_RUNTIME_ERROR("type " << t.elementType.name << " is not support");
    }
}

void requireGPU(const Tensor &t) {
    if (DeviceType::GPU != t.deviceType())
        DEEP8_RUNTIME_ERROR("this build carries the GPU path only: CPU tensors are not supported");
}

// Device scratch taken from the tensor's pool for the duration of one call.  Freed as soon as
// the launches are queued: the pool never returns memory to the driver while it lives and all
// work runs on the one default stream, the same rule Deep8's nodes rely on for their interim
// buffers (deep8/src/nodes/Conv2d.cpp:77-82).
struct PoolScratch {
    Device *device;
    void *ptr;
    size_t bytes;
    PoolScratch(Device *d, size_t n) : device(d), ptr(n ? d->malloc(n) : nullptr), bytes(n) {}
    ~PoolScratch() {
        if (ptr) device->free(ptr);
    }
};

struct MM {
    int xb, xr, xc, yb, yr, yc;
};

MM mmDims(const Tensor &x, const Tensor &y) {
    return MM{(int)x.batch(), (int)x.row(), (int)x.col(), (int)y.batch(), (int)y.row(), (int)y.col()};
}

void checkMatrixMultiplyShapes(const Tensor &x, const Tensor &y, const Tensor &z) {
    const Shape &xs = x.shape, &ys = y.shape, &zs = z.shape;
    DEEP8_ARGUMENT_CHECK(1 == xs.batch || xs.batch == zs.batch, "the shape is error");
    DEEP8_ARGUMENT_CHECK(1 == ys.batch || ys.batch == zs.batch, "the shape is error");
    DEEP8_ARGUMENT_CHECK((1 == xs.nDims || 2 == xs.nDims) && (1 == ys.nDims || 2 == ys.nDims) &&
                             (1 == zs.nDims || 2 == zs.nDims),
                         "the shape is error");
    DEEP8_ARGUMENT_CHECK(xs.row() == zs.row() && ys.col() == zs.col() && xs.col() == ys.row(), "the shape is error");
}

struct ConvDims {
    int B, IH, IW, IC, OC, FH, FW, OH, OW;
};

ConvDims convDims(const Tensor &x, const Tensor &y, const Tensor &z) {
    return ConvDims{(int)x.batch(), (int)x.dim(0), (int)x.dim(1), (int)x.dim(2), (int)y.dim(0),
                    (int)y.dim(1),  (int)y.dim(2), (int)z.dim(0), (int)z.dim(1)};
}

// shared by Conv2d / GradX / GradY and their InterimSize twins (deep8/src/math/Conv2d.cpp:6-38)
ConvDims checkConv(const Tensor &x, const Tensor &y, const Tensor &z, bool covered, int strideY, int strideX,
                   int dilationY, int dilationX) {
    DEEP8_ARGUMENT_CHECK(strideY >= 1 && strideX >= 1 && dilationY >= 1 && dilationX >= 1,
                         "the stride and dilation must >= 1");
    DEEP8_ARGUMENT_CHECK(3 == x.nDims() && 4 == y.nDims() && 3 == z.nDims(), "the shape is error");
    ConvDims d = convDims(x, y, z);
    int g[4];
    const int rc = d8_conv2d_geometry(d.IH, d.IW, d.FH, d.FW, covered, strideY, strideX, dilationY, dilationX, g);
    DEEP8_ARGUMENT_CHECK(0 == rc, "the shape is error: " << d8_last_error());
    DEEP8_ARGUMENT_CHECK(d.B == (int)z.batch() && g[0] == d.OH && g[1] == d.OW && d.OC == (int)z.dim(2),
                         "the z shape is error");
    DEEP8_ARGUMENT_CHECK(1 == y.batch() && d.IC == (int)y.dim(3), "the filter shape is error");
    return d;
}

// deep8/src/math/DeConv2d.cpp:6-35
ConvDims checkDeConv(const Tensor &x, const Tensor &y, const Tensor &z, bool covered, int strideY, int strideX) {
    DEEP8_ARGUMENT_CHECK(strideY >= 1 && strideX >= 1, "the stride must >= 1");
    DEEP8_ARGUMENT_CHECK(3 == x.nDims() && 4 == y.nDims() && 3 == z.nDims(), "the shape is error");
    ConvDims d = convDims(x, y, z);
    int g[4];
    const int rc = d8_deconv2d_geometry(d.IH, d.IW, d.FH, d.FW, covered, strideY, strideX, g);
    DEEP8_ARGUMENT_CHECK(0 == rc, "the shape is error: " << d8_last_error());
    DEEP8_ARGUMENT_CHECK(d.B == (int)z.batch() && g[0] == d.OH && g[1] == d.OW && d.OC == (int)z.dim(2),
                         "the z shape is error");
    DEEP8_ARGUMENT_CHECK(1 == y.batch() && d.IC == (int)y.dim(3), "the filter shape is error");
    return d;
}

}  // namespace

// ---- Constant ---------------------------------------------------------------------------------------------
void Constant(Tensor &x, float scalar) {
    requireGPU(x);
    ConstantGPU(x, scalar);
}

void ConstantGPU(Tensor &x, float scalar) {
    x.takeZero();  // every element is written: a deferred zero fill is moot
    D8_CHECK(d8_fill(dtypeOf(x), x.raw(), x.size(), scalar, nullptr));
}

// ---- MatrixMultiply -------------------------------------------------------------------------------------------
void MatrixMultiply(const Tensor &x, const Tensor &y, Tensor &z) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == y.deviceType() && x.deviceType() == z.deviceType(), "the device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType && x.elementType == z.elementType, "the data type must be same");
    checkMatrixMultiplyShapes(x, y, z);
    requireGPU(x);
    MatrixMultiplyGPU(x, y, z);
}

void MatrixMultiplyGPU(const Tensor &x, const Tensor &y, Tensor &z) {
    const MM d = mmDims(x, y);
    const int dt = dtypeOf(x);
    PoolScratch ws(x.device(), d8_matmul_scratch_bytes(dt, 0, d.xb, d.xr, d.xc, d.yb, d.yr, d.yc));
    D8_CHECK(d8_matmul(dt, x.raw(), d.xb, d.xr, d.xc, y.raw(), d.yb, d.yr, d.yc, z.raw(), ws.ptr, ws.bytes, nullptr));
}

void MatrixMultiplyGradX(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == dx.deviceType() && x.deviceType() == y.deviceType() &&
                             x.deviceType() == z.deviceType() && x.deviceType() == dz.deviceType(),
                         "the device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == dx.elementType && x.elementType == y.elementType &&
                             x.elementType == z.elementType && x.elementType == dz.elementType,
                         "the data type must be same");
    DEEP8_ARGUMENT_CHECK(x.shape == dx.shape && z.shape == dz.shape, "the shape is error");
    checkMatrixMultiplyShapes(x, y, z);
    requireGPU(x);
    MatrixMultiplyGradXGPU(x, dx, y, z, dz);
}

void MatrixMultiplyGradXGPU(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &, const Tensor &dz) {
    const MM d = mmDims(x, y);
    const int dt = dtypeOf(x);
    PoolScratch ws(x.device(), d8_matmul_scratch_bytes(dt, 1, d.xb, d.xr, d.xc, d.yb, d.yr, d.yc));
    // a gradient whose zero fill is still deferred is written, not added to
    const bool fresh = dx.takeZero();
    D8_CHECK((fresh ? d8_matmul_grad_x_overwrite : d8_matmul_grad_x)(dt, dx.raw(), d.xb, d.xr, d.xc, y.raw(), d.yb, d.yr, d.yc,
                                                                    dz.raw(), ws.ptr, ws.bytes, nullptr));
}

void MatrixMultiplyGradY(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == y.deviceType() && x.deviceType() == dy.deviceType() &&
                             x.deviceType() == z.deviceType() && x.deviceType() == dz.deviceType(),
                         "the device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType && x.elementType == dy.elementType &&
                             x.elementType == z.elementType && x.elementType == dz.elementType,
                         "the data type must be same");
    DEEP8_ARGUMENT_CHECK(y.shape == dy.shape && z.shape == dz.shape, "the shape is error");
    checkMatrixMultiplyShapes(x, y, z);
    requireGPU(x);
    MatrixMultiplyGradYGPU(x, y, dy, z, dz);
}

void MatrixMultiplyGradYGPU(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &, const Tensor &dz) {
    const MM d = mmDims(x, y);
    const int dt = dtypeOf(x);
    PoolScratch ws(x.device(), d8_matmul_scratch_bytes(dt, 2, d.xb, d.xr, d.xc, d.yb, d.yr, d.yc));
    const bool fresh = dy.takeZero();
    D8_CHECK((fresh ? d8_matmul_grad_y_overwrite : d8_matmul_grad_y)(dt, x.raw(), d.xb, d.xr, d.xc, dy.raw(), d.yb, d.yr, d.yc,
                                                                    dz.raw(), ws.ptr, ws.bytes, nullptr));
}

// Both gradients from one call (no counterpart in the reference, whose Function::backward runs once per input:
// deep8/src/nodes/MatrixMultiply.cpp:31-52).  The two products are independent, so the library may run them as
// one launch (d8_matmul_grad_xy); the results are those of MatrixMultiplyGradX followed by MatrixMultiplyGradY.
void MatrixMultiplyGradXY(const Tensor &x, Tensor &dx, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == dx.deviceType() && x.deviceType() == y.deviceType() && x.deviceType() == dy.deviceType() &&
                             x.deviceType() == z.deviceType() && x.deviceType() == dz.deviceType(),
                         "the device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == dx.elementType && x.elementType == y.elementType && x.elementType == dy.elementType &&
                             x.elementType == z.elementType && x.elementType == dz.elementType,
                         "the data type must be same");
    DEEP8_ARGUMENT_CHECK(x.shape == dx.shape && y.shape == dy.shape && z.shape == dz.shape, "the shape is error");
    checkMatrixMultiplyShapes(x, y, z);
    requireGPU(x);
    MatrixMultiplyGradXYGPU(x, dx, y, dy, z, dz);
}

void MatrixMultiplyGradXYGPU(const Tensor &x, Tensor &dx, const Tensor &y, Tensor &dy, const Tensor &, const Tensor &dz) {
    const MM d = mmDims(x, y);
    const int dt = dtypeOf(x);
    const size_t need = d8_matmul_scratch_bytes(dt, 3, d.xb, d.xr, d.xc, d.yb, d.yr, d.yc);  // both gradients' scratch
    PoolScratch ws(x.device(), need);
    // a gradient whose zero fill is still deferred is written, not added to
    const int overwrite = (dx.takeZero() ? 1 : 0) | (dy.takeZero() ? 2 : 0);
    D8_CHECK(d8_matmul_grad_xy(dt, x.raw(), dx.raw(), d.xb, d.xr, d.xc, y.raw(), dy.raw(), d.yb, d.yr, d.yc, dz.raw(), overwrite,
                               ws.ptr, ws.bytes, nullptr));
}

// ---- Conv2d -------------------------------------------------------------------------------------------------------
#define CONV_ARGS covered, strideY, strideX, dilationY, dilationX

size_t Conv2dInterimSize(const Tensor &x, const Tensor &y, Tensor &z, bool covered, int strideY, int strideX, int dilationY, int dilationX) {
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType && x.elementType == z.elementType, "the data type must be same");
    const ConvDims d = checkConv(x, y, z, CONV_ARGS);
    requireGPU(x);
    return d8_conv2d_scratch_bytes(dtypeOf(x), 0, d.B, d.IH, d.IW, d.IC, d.OC, d.FH, d.FW, CONV_ARGS);
}

void Conv2d(const Tensor &x, const Tensor &y, Tensor &z, bool covered, int strideY, int strideX, int dilationY, int dilationX, void *interimPtr) {
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType && x.elementType == z.elementType, "the data type must be same");
    checkConv(x, y, z, CONV_ARGS);
    requireGPU(x);
    Conv2dGPU(x, y, z, CONV_ARGS, interimPtr);
}

void Conv2dGPU(const Tensor &x, const Tensor &y, Tensor &z, bool covered, int strideY, int strideX, int dilationY, int dilationX, void *xcol) {
    const ConvDims d = convDims(x, y, z);
    const int dt = dtypeOf(x);
    const size_t bytes = d8_conv2d_scratch_bytes(dt, 0, d.B, d.IH, d.IW, d.IC, d.OC, d.FH, d.FW, CONV_ARGS);
    D8_CHECK(d8_conv2d(dt, x.raw(), d.B, d.IH, d.IW, d.IC, y.raw(), d.OC, d.FH, d.FW, z.raw(), CONV_ARGS, xcol, bytes, nullptr));
}

size_t Conv2dGradXInterimSize(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, int dilationY, int dilationX) {
    DEEP8_ARGUMENT_CHECK(x.elementType == dx.elementType && x.elementType == y.elementType && x.elementType == z.elementType && x.elementType == dz.elementType, "the data type must be same");
    DEEP8_ARGUMENT_CHECK(x.shape == dx.shape && z.shape == dz.shape, "the shape is error");
    const ConvDims d = checkConv(x, y, z, CONV_ARGS);
    requireGPU(x);
    return d8_conv2d_scratch_bytes(dtypeOf(x), 1, d.B, d.IH, d.IW, d.IC, d.OC, d.FH, d.FW, CONV_ARGS);
}

void Conv2dGradX(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, int dilationY, int dilationX, void *interimPtr) {
    DEEP8_ARGUMENT_CHECK(x.elementType == dx.elementType && x.elementType == y.elementType && x.elementType == z.elementType && x.elementType == dz.elementType, "the data type must be same");
    DEEP8_ARGUMENT_CHECK(x.shape == dx.shape && z.shape == dz.shape, "the shape is error");
    checkConv(x, y, z, CONV_ARGS);
    requireGPU(x);
    Conv2dGradXGPU(x, dx, y, z, dz, CONV_ARGS, interimPtr);
}

void Conv2dGradXGPU(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, int dilationY, int dilationX, void *dxcol) {
    const ConvDims d = convDims(x, y, z);
    const int dt = dtypeOf(x);
    const size_t bytes = d8_conv2d_scratch_bytes(dt, 1, d.B, d.IH, d.IW, d.IC, d.OC, d.FH, d.FW, CONV_ARGS);
    const bool fresh = dx.takeZero();  // deferred zero fill: write instead of add
    D8_CHECK((fresh ? d8_conv2d_grad_x_overwrite : d8_conv2d_grad_x)(dt, dx.raw(), d.B, d.IH, d.IW, d.IC, y.raw(), d.OC, d.FH, d.FW, dz.raw(), CONV_ARGS, dxcol, bytes, nullptr));
}

size_t Conv2dGradYInterimSize(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, int dilationY, int dilationX) {
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType && x.elementType == dy.elementType && x.elementType == z.elementType && x.elementType == dz.elementType, "the data type must be same");
    DEEP8_ARGUMENT_CHECK(y.shape == dy.shape && z.shape == dz.shape, "the shape is error");
    const ConvDims d = checkConv(x, y, z, CONV_ARGS);
    requireGPU(x);
    return d8_conv2d_scratch_bytes(dtypeOf(x), 2, d.B, d.IH, d.IW, d.IC, d.OC, d.FH, d.FW, CONV_ARGS);
}

void Conv2dGradY(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, int dilationY, int dilationX, void *interimPtr) {
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType && x.elementType == dy.elementType && x.elementType == z.elementType && x.elementType == dz.elementType, "the data type must be same");
    DEEP8_ARGUMENT_CHECK(y.shape == dy.shape && z.shape == dz.shape, "the shape is error");
    checkConv(x, y, z, CONV_ARGS);
    requireGPU(x);
    Conv2dGradYGPU(x, y, dy, z, dz, CONV_ARGS, interimPtr);
}

void Conv2dGradYGPU(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, int dilationY, int dilationX, void *xcol) {
    const ConvDims d = convDims(x, y, z);
    const int dt = dtypeOf(x);
    const size_t bytes = d8_conv2d_scratch_bytes(dt, 2, d.B, d.IH, d.IW, d.IC, d.OC, d.FH, d.FW, CONV_ARGS);
    const bool fresh = dy.takeZero();  // deferred zero fill: write instead of add
    D8_CHECK((fresh ? d8_conv2d_grad_y_overwrite : d8_conv2d_grad_y)(dt, x.raw(), d.B, d.IH, d.IW, d.IC, dy.raw(), d.OC, d.FH, d.FW, dz.raw(), CONV_ARGS, xcol, bytes, nullptr));
}

// Both gradients from one call (no counterpart in the reference, whose Conv2d::backward runs once per input:
// deep8/src/nodes/Conv2d.cpp:85-151).  The products are independent; on a small layer the library runs them as one
// launch (d8_conv2d_grad_xy).  The results are those of Conv2dGradX followed by Conv2dGradY.
void Conv2dGradXY(const Tensor &x, Tensor &dx, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz, bool covered, int strideY,
                  int strideX, int dilationY, int dilationX) {
    DEEP8_ARGUMENT_CHECK(x.elementType == dx.elementType && x.elementType == y.elementType && x.elementType == dy.elementType &&
                             x.elementType == z.elementType && x.elementType == dz.elementType,
                         "the data type must be same");
    DEEP8_ARGUMENT_CHECK(x.shape == dx.shape && y.shape == dy.shape && z.shape == dz.shape, "the shape is error");
    const ConvDims d = checkConv(x, y, z, CONV_ARGS);
    requireGPU(x);
    const int dt = dtypeOf(x);
    const size_t need = d8_conv2d_scratch_bytes(dt, 3, d.B, d.IH, d.IW, d.IC, d.OC, d.FH, d.FW, CONV_ARGS);  // both gradients' scratch
    PoolScratch ws(x.device(), need);
    const int overwrite = (dx.takeZero() ? 1 : 0) | (dy.takeZero() ? 2 : 0);  // deferred zero fills: write instead of add
    D8_CHECK(d8_conv2d_grad_xy(dt, x.raw(), dx.raw(), d.B, d.IH, d.IW, d.IC, y.raw(), dy.raw(), d.OC, d.FH, d.FW, dz.raw(), CONV_ARGS,
                               overwrite, ws.ptr, ws.bytes, nullptr));
}

#undef CONV_ARGS

// ---- DeConv2d -------------------------------------------------------------------------------------------------------
#define DECONV_ARGS covered, strideY, strideX

size_t DeConv2dInterimSize(const Tensor &x, const Tensor &y, Tensor &z, bool covered, int strideY, int strideX) {
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType && x.elementType == z.elementType, "the data type must be same");
    const ConvDims d = checkDeConv(x, y, z, DECONV_ARGS);
    requireGPU(x);
    return d8_deconv2d_scratch_bytes(dtypeOf(x), 0, d.B, d.IH, d.IW, d.IC, d.OC, d.FH, d.FW, DECONV_ARGS);
}

void DeConv2d(const Tensor &x, const Tensor &y, Tensor &z, bool covered, int strideY, int strideX, void *interimPtr) {
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType && x.elementType == z.elementType, "the data type must be same");
    checkDeConv(x, y, z, DECONV_ARGS);
    requireGPU(x);
    DeConv2dGPU(x, y, z, DECONV_ARGS, interimPtr);
}

void DeConv2dGPU(const Tensor &x, const Tensor &y, Tensor &z, bool covered, int strideY, int strideX, void *interimPtr) {
    const ConvDims d = convDims(x, y, z);
    const int dt = dtypeOf(x);
    const size_t bytes = d8_deconv2d_scratch_bytes(dt, 0, d.B, d.IH, d.IW, d.IC, d.OC, d.FH, d.FW, DECONV_ARGS);
    D8_CHECK(d8_deconv2d(dt, x.raw(), d.B, d.IH, d.IW, d.IC, y.raw(), d.OC, d.FH, d.FW, z.raw(), DECONV_ARGS, interimPtr, bytes, nullptr));
}

size_t DeConv2dGradXInterimSize(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX) {
    DEEP8_ARGUMENT_CHECK(x.elementType == dx.elementType && x.elementType == y.elementType && x.elementType == z.elementType && x.elementType == dz.elementType, "the data type must be same");
    DEEP8_ARGUMENT_CHECK(x.shape == dx.shape && z.shape == dz.shape, "the shape is error");
    const ConvDims d = checkDeConv(x, y, z, DECONV_ARGS);
    requireGPU(x);
    return d8_deconv2d_scratch_bytes(dtypeOf(x), 1, d.B, d.IH, d.IW, d.IC, d.OC, d.FH, d.FW, DECONV_ARGS);
}

void DeConv2dGradX(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, void *interimPtr) {
    DEEP8_ARGUMENT_CHECK(x.elementType == dx.elementType && x.elementType == y.elementType && x.elementType == z.elementType && x.elementType == dz.elementType, "the data type must be same");
    DEEP8_ARGUMENT_CHECK(x.shape == dx.shape && z.shape == dz.shape, "the shape is error");
    checkDeConv(x, y, z, DECONV_ARGS);
    requireGPU(x);
    DeConv2dGradXGPU(x, dx, y, z, dz, DECONV_ARGS, interimPtr);
}

void DeConv2dGradXGPU(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, void *interimPtr) {
    const ConvDims d = convDims(x, y, z);
    const int dt = dtypeOf(x);
    const size_t bytes = d8_deconv2d_scratch_bytes(dt, 1, d.B, d.IH, d.IW, d.IC, d.OC, d.FH, d.FW, DECONV_ARGS);
    const bool fresh = dx.takeZero();  // deferred zero fill: write instead of add
    D8_CHECK((fresh ? d8_deconv2d_grad_x_overwrite : d8_deconv2d_grad_x)(dt, dx.raw(), d.B, d.IH, d.IW, d.IC, y.raw(), d.OC, d.FH, d.FW, dz.raw(), DECONV_ARGS, interimPtr, bytes, nullptr));
}

size_t DeConv2dGradYInterimSize(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX) {
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType && x.elementType == dy.elementType && x.elementType == z.elementType && x.elementType == dz.elementType, "the data type must be same");
    DEEP8_ARGUMENT_CHECK(y.shape == dy.shape && z.shape == dz.shape, "the shape is error");
    const ConvDims d = checkDeConv(x, y, z, DECONV_ARGS);
    requireGPU(x);
    return d8_deconv2d_scratch_bytes(dtypeOf(x), 2, d.B, d.IH, d.IW, d.IC, d.OC, d.FH, d.FW, DECONV_ARGS);
}

void DeConv2dGradY(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, void *interimPtr) {
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType && x.elementType == dy.elementType && x.elementType == z.elementType && x.elementType == dz.elementType, "the data type must be same");
    DEEP8_ARGUMENT_CHECK(y.shape == dy.shape && z.shape == dz.shape, "the shape is error");
    checkDeConv(x, y, z, DECONV_ARGS);
    requireGPU(x);
    DeConv2dGradYGPU(x, y, dy, z, dz, DECONV_ARGS, interimPtr);
}

void DeConv2dGradYGPU(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, void *interimPtr) {
    const ConvDims d = convDims(x, y, z);
    const int dt = dtypeOf(x);
    const size_t bytes = d8_deconv2d_scratch_bytes(dt, 2, d.B, d.IH, d.IW, d.IC, d.OC, d.FH, d.FW, DECONV_ARGS);
    const bool fresh = dy.takeZero();  // deferred zero fill: write instead of add
    D8_CHECK((fresh ? d8_deconv2d_grad_y_overwrite : d8_deconv2d_grad_y)(dt, x.raw(), d.B, d.IH, d.IW, d.IC, dy.raw(), d.OC, d.FH, d.FW, dz.raw(), DECONV_ARGS, interimPtr, bytes, nullptr));
}

// Both gradients from one call, as Conv2dGradXY (deep8/src/nodes/DeConv2d.cpp:74-126 runs them one per input).
void DeConv2dGradXY(const Tensor &x, Tensor &dx, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz, bool covered, int strideY,
                    int strideX) {
    DEEP8_ARGUMENT_CHECK(x.elementType == dx.elementType && x.elementType == y.elementType && x.elementType == dy.elementType &&
                             x.elementType == z.elementType && x.elementType == dz.elementType,
                         "the data type must be same");
    DEEP8_ARGUMENT_CHECK(x.shape == dx.shape && y.shape == dy.shape && z.shape == dz.shape, "the shape is error");
    const ConvDims d = checkDeConv(x, y, z, DECONV_ARGS);
    requireGPU(x);
    const int dt = dtypeOf(x);
    const size_t need = d8_deconv2d_scratch_bytes(dt, 3, d.B, d.IH, d.IW, d.IC, d.OC, d.FH, d.FW, DECONV_ARGS);
    PoolScratch ws(x.device(), need);
    const int overwrite = (dx.takeZero() ? 1 : 0) | (dy.takeZero() ? 2 : 0);
    D8_CHECK(d8_deconv2d_grad_xy(dt, x.raw(), dx.raw(), d.B, d.IH, d.IW, d.IC, y.raw(), dy.raw(), d.OC, d.FH, d.FW, dz.raw(), DECONV_ARGS,
                                 overwrite, ws.ptr, ws.bytes, nullptr));
}

#undef DECONV_ARGS

// ---- Add / ReLu -------------------------------------------------------------------------------------------------
namespace {

// [batch, d0..d3] with the dims right-aligned and padded with 1 (deep8/include/utils/ShapeUtils.h:41-56)
struct Dims5 {
    int d[5];
};

Dims5 enlargeShapeToMaxDim(const Shape &shape) {
    DEEP8_ARGUMENT_CHECK(MAX_TENSOR_DIMS >= shape.nDims && shape.nDims >= 1, "the dim is error");
    Dims5 r;
    r.d[0] = (int)shape.batch;
    for (int i = MAX_TENSOR_DIMS, j = (int)shape.nDims - 1; i > 0; --i, --j) r.d[i] = j >= 0 ? (int)shape.dim(j) : 1;
    return r;
}

void checkBroadcast(const Tensor &x, const Tensor &y, const Tensor &z) {
    const Dims5 xa = enlargeShapeToMaxDim(x.shape), ya = enlargeShapeToMaxDim(y.shape), za = enlargeShapeToMaxDim(z.shape);
    for (int i = 0; i <= MAX_TENSOR_DIMS; ++i) {
        DEEP8_ARGUMENT_CHECK(1 == xa.d[i] || xa.d[i] == za.d[i], "the shape is error");
        DEEP8_ARGUMENT_CHECK(1 == ya.d[i] || ya.d[i] == za.d[i], "the shape is error");
        DEEP8_ARGUMENT_CHECK(za.d[i] == (xa.d[i] > ya.d[i] ? xa.d[i] : ya.d[i]), "the shape is error");
    }
}

void addGradGPU(Tensor &g, const Tensor &dz) {
    const Dims5 ga = enlargeShapeToMaxDim(g.shape), za = enlargeShapeToMaxDim(dz.shape);
    const int dt = dtypeOf(g);
    PoolScratch ws(g.device(), d8_add_grad_scratch_bytes(dt, ga.d, za.d));
    const bool fresh = g.takeZero();  // deferred zero fill: write instead of add
    D8_CHECK((fresh ? d8_add_grad_overwrite : d8_add_grad)(dt, g.raw(), ga.d, dz.raw(), za.d, ws.ptr, ws.bytes, nullptr));
}

}  // namespace

void Add(const Tensor &x, const Tensor &y, Tensor &z) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == y.deviceType() && x.deviceType() == z.deviceType(), "the param device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType && x.elementType == z.elementType, "the param data type must be same");
    checkBroadcast(x, y, z);
    requireGPU(x);
    AddGPU(x, y, z);
}

void AddGPU(const Tensor &x, const Tensor &y, Tensor &z) {
    const Dims5 xa = enlargeShapeToMaxDim(x.shape), ya = enlargeShapeToMaxDim(y.shape), za = enlargeShapeToMaxDim(z.shape);
    D8_CHECK(d8_add(dtypeOf(x), x.raw(), xa.d, y.raw(), ya.d, z.raw(), za.d, nullptr));
}

void AddGradX(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == dx.deviceType() && x.deviceType() == y.deviceType() &&
                             x.deviceType() == z.deviceType() && x.deviceType() == dz.deviceType(),
                         "the param device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == dx.elementType && x.elementType == y.elementType &&
                             x.elementType == z.elementType && x.elementType == dz.elementType,
                         "the param data type must be same");
    DEEP8_ARGUMENT_CHECK(x.shape == dx.shape, "the x shape is error");
    DEEP8_ARGUMENT_CHECK(z.shape == dz.shape, "the z shape is error");
    checkBroadcast(x, y, z);
    requireGPU(x);
    AddGradXGPU(x, dx, y, z, dz);
}

void AddGradXGPU(const Tensor &, Tensor &dx, const Tensor &, const Tensor &, const Tensor &dz) { addGradGPU(dx, dz); }

void AddGradY(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == y.deviceType() && x.deviceType() == dy.deviceType() &&
                             x.deviceType() == z.deviceType() && x.deviceType() == dz.deviceType(),
                         "the param device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType && x.elementType == dy.elementType &&
                             x.elementType == z.elementType && x.elementType == dz.elementType,
                         "the param data type must be same");
    DEEP8_ARGUMENT_CHECK(y.shape == dy.shape, "the y shape is error");
    DEEP8_ARGUMENT_CHECK(z.shape == dz.shape, "the z shape is error");
    checkBroadcast(x, y, z);
    requireGPU(x);
    AddGradYGPU(x, y, dy, z, dz);
}

void AddGradYGPU(const Tensor &, const Tensor &, Tensor &dy, const Tensor &, const Tensor &dz) { addGradGPU(dy, dz); }

void ReLu(const Tensor &x, Tensor &y) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == y.deviceType(), "the param device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType, "the param data type must be same");
    DEEP8_ARGUMENT_CHECK(x.shape == y.shape, "the param shape must be same");
    requireGPU(x);
    ReLuGPU(x, y);
}

void ReLuGPU(const Tensor &x, Tensor &y) { D8_CHECK(d8_relu(dtypeOf(x), x.raw(), y.raw(), (long)x.shape.size(), nullptr)); }

void ReLuGrad(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == dx.deviceType() && x.deviceType() == y.deviceType() && x.deviceType() == dy.deviceType(),
                         "the param device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == dx.elementType && x.elementType == y.elementType && x.elementType == dy.elementType,
                         "the param data type must be same");
    DEEP8_ARGUMENT_CHECK(x.shape == dx.shape && x.shape == y.shape && x.shape == dy.shape, "the param shape must be same");
    requireGPU(x);
    ReLuGradGPU(x, dx, y, dy);
}

void ReLuGradGPU(const Tensor &x, Tensor &dx, const Tensor &, const Tensor &dy) {
    const bool fresh = dx.takeZero();  // deferred zero fill: write instead of add
    D8_CHECK((fresh ? d8_relu_grad_overwrite : d8_relu_grad)(dtypeOf(x), x.raw(), dx.raw(), dy.raw(), (long)x.shape.size(), nullptr));
}

// ---- Minus / L1Norm / L2Norm / ReduceMean / AXPBY ---------------------------------------------------------------
namespace {

void checkBinaryGrad(const Tensor &x, const Tensor &y, const Tensor &z, const Tensor &g, const Tensor &dz) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == g.deviceType() && x.deviceType() == y.deviceType() &&
                             x.deviceType() == z.deviceType() && x.deviceType() == dz.deviceType(),
                         "the param device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == g.elementType && x.elementType == y.elementType &&
                             x.elementType == z.elementType && x.elementType == dz.elementType,
                         "the param data type must be same");
    DEEP8_ARGUMENT_CHECK(z.shape == dz.shape, "the z shape is error");
    checkBroadcast(x, y, z);
    requireGPU(x);
}

void checkNorm(const Tensor &x, const Tensor &y) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == y.deviceType(), "the param device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType, "the param data type must be same");
    DEEP8_ARGUMENT_CHECK(x.batch() == y.batch(), "the shape is error");
    DEEP8_ARGUMENT_CHECK(1 == y.batchSize(), "the shape is error");
    requireGPU(x);
}

void checkNormGrad(const Tensor &x, const Tensor &dx, const Tensor &y, const Tensor &dy) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == dx.deviceType() && x.deviceType() == y.deviceType() && x.deviceType() == dy.deviceType(),
                         "the param device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == dx.elementType && x.elementType == y.elementType && x.elementType == dy.elementType,
                         "the param data type must be same");
    DEEP8_ARGUMENT_CHECK(x.shape == dx.shape && y.shape == dy.shape, "the param shape error");
    DEEP8_ARGUMENT_CHECK(x.batch() == y.batch(), "the shape is error");
    DEEP8_ARGUMENT_CHECK(1 == y.batchSize(), "the shape is error");
    requireGPU(x);
}

// [batch, dims..] of x and the same with 1 at every reduced axis, both in the enlarged 5-entry form
void meanDims(const Shape &x, const std::vector<int> &axis, Dims5 &xa, Dims5 &ya) {
    const int rank = (int)x.nDims + 1;
    std::vector<bool> reduce(rank, axis.empty());
    for (size_t i = 0; i < axis.size(); ++i) {
        DEEP8_ARGUMENT_CHECK(-rank <= axis[i] && axis[i] < rank, "the reduce dim is error");
        reduce[(axis[i] + rank) % rank] = true;
    }
    xa = enlargeShapeToMaxDim(x);
    ya = xa;
    if (reduce[0]) ya.d[0] = 1;
    // dim i (1-based over [batch, dims..]) sits at enlarged position MAX_TENSOR_DIMS - nDims + i
    for (int i = 1; i < rank; ++i)
        if (reduce[i]) ya.d[MAX_TENSOR_DIMS - (int)x.nDims + i] = 1;
}

}  // namespace

void Minus(const Tensor &x, const Tensor &y, Tensor &z) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == y.deviceType() && x.deviceType() == z.deviceType(), "the param device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType && x.elementType == z.elementType, "the param data type must be same");
    checkBroadcast(x, y, z);
    requireGPU(x);
    MinusGPU(x, y, z);
}

void MinusGPU(const Tensor &x, const Tensor &y, Tensor &z) {
    const Dims5 xa = enlargeShapeToMaxDim(x.shape), ya = enlargeShapeToMaxDim(y.shape), za = enlargeShapeToMaxDim(z.shape);
    D8_CHECK(d8_minus(dtypeOf(x), x.raw(), xa.d, y.raw(), ya.d, z.raw(), za.d, nullptr));
}

void MinusGradX(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz) {
    DEEP8_ARGUMENT_CHECK(x.shape == dx.shape, "the x shape is error");
    checkBinaryGrad(x, y, z, dx, dz);
    MinusGradXGPU(x, dx, y, z, dz);
}

void MinusGradXGPU(const Tensor &, Tensor &dx, const Tensor &, const Tensor &, const Tensor &dz) { addGradGPU(dx, dz); }

void MinusGradY(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz) {
    DEEP8_ARGUMENT_CHECK(y.shape == dy.shape, "the y shape is error");
    checkBinaryGrad(x, y, z, dy, dz);
    MinusGradYGPU(x, y, dy, z, dz);
}

void MinusGradYGPU(const Tensor &, const Tensor &, Tensor &dy, const Tensor &, const Tensor &dz) {
    const Dims5 ga = enlargeShapeToMaxDim(dy.shape), za = enlargeShapeToMaxDim(dz.shape);
    const int dt = dtypeOf(dy);
    PoolScratch ws(dy.device(), d8_add_grad_scratch_bytes(dt, ga.d, za.d));
    D8_CHECK(d8_minus_grad_y(dt, dy.raw(), ga.d, dz.raw(), za.d, ws.ptr, ws.bytes, nullptr));
}

namespace {
typedef int (*NormFn)(int, const void *, void *, int, long, void *, size_t, void *);
void normGPU(NormFn fn, const Tensor &x, Tensor &y) {
    const int dt = dtypeOf(x), batch = (int)x.batch();
    const long size = (long)x.batchSize();
    const int yd[5] = {batch, 1, 1, 1, 1}, xd[5] = {batch, 1, 1, 1, (int)size};
    PoolScratch ws(x.device(), d8_add_grad_scratch_bytes(dt, yd, xd));
    D8_CHECK(fn(dt, x.raw(), y.raw(), batch, size, ws.ptr, ws.bytes, nullptr));
}
}  // namespace

void L1Norm(const Tensor &x, Tensor &y) {
    checkNorm(x, y);
    L1NormGPU(x, y);
}
void L1NormGPU(const Tensor &x, Tensor &y) { normGPU(d8_l1norm, x, y); }

void L1NormGrad(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy) {
    checkNormGrad(x, dx, y, dy);
    L1NormGradGPU(x, dx, y, dy);
}
void L1NormGradGPU(const Tensor &x, Tensor &dx, const Tensor &, const Tensor &dy) {
    D8_CHECK(d8_l1norm_grad(dtypeOf(x), x.raw(), dx.raw(), dy.raw(), (int)x.batch(), (long)x.batchSize(), nullptr));
}

void L2Norm(const Tensor &x, Tensor &y) {
    checkNorm(x, y);
    L2NormGPU(x, y);
}
void L2NormGPU(const Tensor &x, Tensor &y) { normGPU(d8_l2norm, x, y); }

void L2NormGrad(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy) {
    checkNormGrad(x, dx, y, dy);
    L2NormGradGPU(x, dx, y, dy);
}
void L2NormGradGPU(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy) {
    D8_CHECK(d8_l2norm_grad(dtypeOf(x), x.raw(), dx.raw(), y.raw(), dy.raw(), (int)x.batch(), (long)x.batchSize(), nullptr));
}

Shape ReduceMeanShape(const Shape &x, const std::vector<int> &axis, bool keepDims) {
    const int rank = (int)x.nDims + 1;
    std::vector<bool> reduce(rank, axis.empty());
    for (size_t i = 0; i < axis.size(); ++i) {
        DEEP8_ARGUMENT_CHECK(-rank <= axis[i] && axis[i] < rank, "the reduce dim is error");
        reduce[(axis[i] + rank) % rank] = true;
    }
    DEEP8_ARGUMENT_CHECK(rank >= 2, "the shape is error");
    const size_t batch = reduce[0] ? 1 : x.batch;
    std::vector<size_t> list;
    for (int i = 1; i < rank; ++i) {
        if (reduce[i]) {
            if (keepDims) list.emplace_back(1);
        } else {
            list.emplace_back(x.dim(i - 1));
        }
    }
    if (list.empty()) list.emplace_back(1);
    return Shape(batch, list);
}

void ReduceMean(const Tensor &x, Tensor &y, const std::vector<int> &axis, bool keepDims) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == y.deviceType(), "the param device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType, "the param data type must be same");
    DEEP8_ARGUMENT_CHECK(ReduceMeanShape(x.shape, axis, keepDims) == y.shape, "the y shape is error");
    requireGPU(x);
    ReduceMeanGPU(x, y, axis, keepDims);
}

void ReduceMeanGPU(const Tensor &x, Tensor &y, const std::vector<int> &axis, bool) {
    Dims5 xa, ya;
    meanDims(x.shape, axis, xa, ya);
    const int dt = dtypeOf(x);
    PoolScratch ws(x.device(), d8_add_grad_scratch_bytes(dt, ya.d, xa.d));
    D8_CHECK(d8_reduce_mean(dt, x.raw(), xa.d, y.raw(), ya.d, ws.ptr, ws.bytes, nullptr));
}

void ReduceMeanGrad(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy, const std::vector<int> &axis, bool keepDims) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == dx.deviceType() && x.deviceType() == y.deviceType() && x.deviceType() == dy.deviceType(),
                         "the param device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == dx.elementType && x.elementType == y.elementType && x.elementType == dy.elementType,
                         "the param data type must be same");
    DEEP8_ARGUMENT_CHECK(x.shape == dx.shape && y.shape == dy.shape, "the x/dx or y/dy shape must be same");
    DEEP8_ARGUMENT_CHECK(ReduceMeanShape(x.shape, axis, keepDims) == y.shape, "the y shape is error");
    requireGPU(x);
    ReduceMeanGradGPU(x, dx, y, dy, axis, keepDims);
}

void ReduceMeanGradGPU(const Tensor &x, Tensor &dx, const Tensor &, const Tensor &dy, const std::vector<int> &axis, bool) {
    Dims5 xa, ya;
    meanDims(x.shape, axis, xa, ya);
    D8_CHECK(d8_reduce_mean_grad(dtypeOf(x), dx.raw(), xa.d, dy.raw(), ya.d, nullptr));
}

void AXPBY(const Tensor &x, float alpha, const Tensor &y, float beta, Tensor &z) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == y.deviceType() && x.deviceType() == z.deviceType(), "the param device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType && x.elementType == z.elementType, "the param data type must be same");
    DEEP8_ARGUMENT_CHECK(x.shape.size() == y.shape.size() && x.shape.size() == z.shape.size(), "the param shape size must be same");
    requireGPU(x);
    AXPBYGPU(x, alpha, y, beta, z);
}

void AXPBYGPU(const Tensor &x, float alpha, const Tensor &y, float beta, Tensor &z) {
    D8_CHECK(d8_axpby(dtypeOf(x), x.raw(), alpha, y.raw(), beta, z.raw(), (long)x.shape.size(), nullptr));
}

// ---- MaxPooling2d / AvgPooling2d --------------------------------------------------------------------------------
#define POOL_ARGS covered, filterHeight, filterWidth, strideY, strideX

Shape Pooling2dShape(const Shape &x, bool covered, int filterHeight, int filterWidth, int strideY, int strideX) {
    DEEP8_ARGUMENT_CHECK(3 == x.nDims, "the tensor dim must be 3");
    DEEP8_ARGUMENT_CHECK(filterHeight >= 1 && filterWidth >= 1 && strideY >= 1 && strideX >= 1, "the params is error");
    const int IH = (int)x.dim(0), IW = (int)x.dim(1);
    int OH, OW;
    if (!covered) {
        OH = (IH - filterHeight) / strideY + 1;
        OW = (IW - filterWidth) / strideX + 1;
    } else {
        OH = (IH - 1) / strideY + 1;
        OW = (IW - 1) / strideX + 1;
    }
    DEEP8_ARGUMENT_CHECK(OH >= 1 && OW >= 1 && IH >= (covered ? 1 : filterHeight) && IW >= (covered ? 1 : filterWidth), "the shape is error");
    return Shape(x.batch, {(size_t)OH, (size_t)OW, x.dim(2)});
}

namespace {
void checkPool(const Tensor &x, const Tensor &y, bool covered, int filterHeight, int filterWidth, int strideY, int strideX) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == y.deviceType(), "the param device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType, "the data type must be same");
    DEEP8_ARGUMENT_CHECK(3 == x.nDims() && 3 == y.nDims(), "the tensor dim must be 3");
    DEEP8_ARGUMENT_CHECK(Pooling2dShape(x.shape, POOL_ARGS) == y.shape, "the shape is error");
    requireGPU(x);
}
void checkPoolGrad(const Tensor &x, const Tensor &dx, const Tensor &y, const Tensor &dy, bool covered, int filterHeight, int filterWidth,
                   int strideY, int strideX) {
    DEEP8_ARGUMENT_CHECK(x.shape == dx.shape, "the x and dx shape must be same");
    DEEP8_ARGUMENT_CHECK(y.shape == dy.shape, "the y and dy shape must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == dx.elementType && x.elementType == y.elementType && x.elementType == dy.elementType, "the type must be same");
    DEEP8_ARGUMENT_CHECK(x.deviceType() == dx.deviceType() && x.deviceType() == y.deviceType() && x.deviceType() == dy.deviceType(),
                         "the device type must be same");
    checkPool(x, y, POOL_ARGS);
}
#define POOL_DIMS(t) (int)(t).batch(), (int)(t).dim(0), (int)(t).dim(1), (int)(t).dim(2)
}  // namespace

void MaxPooling2d(const Tensor &x, Tensor &y, bool covered, int filterHeight, int filterWidth, int strideY, int strideX) {
    checkPool(x, y, POOL_ARGS);
    MaxPooling2dGPU(x, y, POOL_ARGS);
}
void MaxPooling2dGPU(const Tensor &x, Tensor &y, bool covered, int filterHeight, int filterWidth, int strideY, int strideX) {
    D8_CHECK(d8_maxpool2d(dtypeOf(x), x.raw(), y.raw(), POOL_DIMS(x), filterHeight, filterWidth, covered, strideY, strideX, nullptr));
}
void MaxPooling2dGrad(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy, bool covered, int filterHeight, int filterWidth, int strideY, int strideX) {
    checkPoolGrad(x, dx, y, dy, POOL_ARGS);
    MaxPooling2dGradGPU(x, dx, y, dy, POOL_ARGS);
}
void MaxPooling2dGradGPU(const Tensor &x, Tensor &dx, const Tensor &, const Tensor &dy, bool covered, int filterHeight, int filterWidth, int strideY, int strideX) {
    const bool fresh = dx.takeZero();  // deferred zero fill: write instead of add
    D8_CHECK((fresh ? d8_maxpool2d_grad_overwrite : d8_maxpool2d_grad)(dtypeOf(x), x.raw(), dx.raw(), dy.raw(), POOL_DIMS(x), filterHeight, filterWidth,
                                                                      covered, strideY, strideX, nullptr));
}
void AvgPooling2d(const Tensor &x, Tensor &y, bool covered, int filterHeight, int filterWidth, int strideY, int strideX) {
    checkPool(x, y, POOL_ARGS);
    AvgPooling2dGPU(x, y, POOL_ARGS);
}
void AvgPooling2dGPU(const Tensor &x, Tensor &y, bool covered, int filterHeight, int filterWidth, int strideY, int strideX) {
    D8_CHECK(d8_avgpool2d(dtypeOf(x), x.raw(), y.raw(), POOL_DIMS(x), filterHeight, filterWidth, covered, strideY, strideX, nullptr));
}
void AvgPooling2dGrad(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy, bool covered, int filterHeight, int filterWidth, int strideY, int strideX) {
    checkPoolGrad(x, dx, y, dy, POOL_ARGS);
    AvgPooling2dGradGPU(x, dx, y, dy, POOL_ARGS);
}
void AvgPooling2dGradGPU(const Tensor &x, Tensor &dx, const Tensor &, const Tensor &dy, bool covered, int filterHeight, int filterWidth, int strideY, int strideX) {
    const bool fresh = dx.takeZero();  // deferred zero fill: write instead of add
    D8_CHECK((fresh ? d8_avgpool2d_grad_overwrite : d8_avgpool2d_grad)(dtypeOf(x), dx.raw(), dy.raw(), POOL_DIMS(x), filterHeight, filterWidth, covered,
                                                                      strideY, strideX, nullptr));
}
#undef POOL_ARGS
#undef POOL_DIMS

void AdamUpdate(Tensor &value, Tensor &gradient, Tensor &m, Tensor &v, float beta1, float beta2, float epsilon, float learningRate, float weightDecay, int64_t steps) {
    DEEP8_ARGUMENT_CHECK(value.deviceType() == gradient.deviceType() && value.deviceType() == m.deviceType() && value.deviceType() == v.deviceType(),
                         "the param device type must be same");
    DEEP8_ARGUMENT_CHECK(value.elementType == gradient.elementType && value.elementType == m.elementType && value.elementType == v.elementType,
                         "the param data type must be same");
    DEEP8_ARGUMENT_CHECK(value.shape.size() == gradient.shape.size() && value.shape.size() == m.shape.size() && value.shape.size() == v.shape.size(),
                         "the param shape size must be same");
    if (steps <= 0) steps = 1;  // avoid divide by 0
    requireGPU(value);
    AdamUpdateGPU(value, gradient, m, v, beta1, beta2, epsilon, learningRate, weightDecay, steps);
}

void AdamUpdateGPU(Tensor &value, Tensor &gradient, Tensor &m, Tensor &v, float beta1, float beta2, float epsilon, float learningRate, float weightDecay, int64_t steps) {
    D8_CHECK(d8_adam_update(dtypeOf(value), value.raw(), gradient.raw(), m.raw(), v.raw(), beta1, beta2, epsilon, learningRate, weightDecay,
                            (long)steps, (long)value.shape.size(), nullptr));
}

// ---- bias and ReLu folded into the contraction ----------------------------------------------------------------------------
namespace {
void checkBias(const Tensor &bias, const Tensor &z) {
    DEEP8_ARGUMENT_CHECK(bias.deviceType() == z.deviceType(), "the device type must be same");
    DEEP8_ARGUMENT_CHECK(bias.elementType == z.elementType, "the data type must be same");
    DEEP8_ARGUMENT_CHECK(1 == bias.shape.batch && 1 == bias.shape.nDims && bias.shape.dim(0) == z.shape.dim(z.shape.nDims - 1),
                         "the bias must have one value per element of the output's last dimension");
}
}  // namespace

void MatrixMultiplyBiasReLu(const Tensor &x, const Tensor &y, const Tensor &bias, Tensor &z, bool relu) {
    DEEP8_ARGUMENT_CHECK(x.deviceType() == y.deviceType() && x.deviceType() == z.deviceType(), "the device type must be same");
    DEEP8_ARGUMENT_CHECK(x.elementType == y.elementType && x.elementType == z.elementType, "the data type must be same");
    checkMatrixMultiplyShapes(x, y, z);
    checkBias(bias, z);
    requireGPU(x);
    const MM d = mmDims(x, y);
    const int dt = dtypeOf(x);
    PoolScratch ws(x.device(), d8_matmul_scratch_bytes(dt, 0, d.xb, d.xr, d.xc, d.yb, d.yr, d.yc));
    D8_CHECK(d8_matmul_bias_relu(dt, x.raw(), d.xb, d.xr, d.xc, y.raw(), d.yb, d.yr, d.yc, bias.raw(), relu ? 1 : 0, z.raw(),
                                 ws.ptr, ws.bytes, nullptr));
}

void Conv2dBiasReLu(const Tensor &x, const Tensor &y, const Tensor &bias, Tensor &z, bool covered, int strideY, int strideX,
                    int dilationY, int dilationX, void *interimPtr, bool relu) {
    const ConvDims d = checkConv(x, y, z, covered, strideY, strideX, dilationY, dilationX);
    checkBias(bias, z);
    requireGPU(x);
    const int dt = dtypeOf(x);
    const size_t bytes = d8_conv2d_scratch_bytes(dt, 0, d.B, d.IH, d.IW, d.IC, d.OC, d.FH, d.FW, covered, strideY, strideX, dilationY, dilationX);
    D8_CHECK(d8_conv2d_bias_relu(dt, x.raw(), d.B, d.IH, d.IW, d.IC, y.raw(), d.OC, d.FH, d.FW, bias.raw(), relu ? 1 : 0, z.raw(),
                                 covered, strideY, strideX, dilationY, dilationX, interimPtr, bytes, nullptr));
}

void BiasReLuGrad(const Tensor &z, const Tensor &dz, Tensor &dpre, Tensor &dbias) {
    DEEP8_ARGUMENT_CHECK(z.deviceType() == dz.deviceType() && z.deviceType() == dpre.deviceType(), "the device type must be same");
    DEEP8_ARGUMENT_CHECK(z.elementType == dz.elementType && z.elementType == dpre.elementType, "the data type must be same");
    DEEP8_ARGUMENT_CHECK(z.shape == dz.shape && z.shape == dpre.shape, "the shape must be same");
    checkBias(dbias, z);
    requireGPU(z);
    const int dt = dtypeOf(z), cols = (int)dbias.shape.dim(0);
    const long rows = (long)(z.shape.size() / (size_t)cols);
    PoolScratch ws(z.device(), d8_bias_relu_grad_scratch_bytes(dt, rows, cols));
    const bool fresh = dbias.takeZero();  // deferred zero fill: write instead of add
    D8_CHECK(d8_bias_relu_grad(dt, z.raw(), dz.raw(), dpre.raw(), dbias.raw(), rows, cols, fresh ? 0 : 1, ws.ptr, ws.bytes, nullptr));
}

}  // namespace Math
}  // namespace Deep8
