// Math:: dispatchers and their GPU implementations for the dense-contraction path, with the
// reference's signatures:
//   MatrixMultiply   deep8/include/math/MatrixMultiply.h:12-36, checks deep8/src/math/MatrixMultiply.cpp:7-91
//   Conv2d           deep8/include/math/Conv2d.h:17-47,         checks deep8/src/math/Conv2d.cpp:6-290
//   DeConv2d         deep8/include/math/DeConv2d.h:11-40,       checks deep8/src/math/DeConv2d.cpp:6-243
//   Constant         deep8/include/math/Constant.h (zeroGradient / oneGradient)
// Forward routines overwrite their output; every Grad routine adds into its destination.
// The *GPU functions call libdeep8_hip.so through its C ABI (include/deep8_hip.h).  Tensors on
// DeviceType::CPU are refused with std::runtime_error: there is no CPU path in this build.
#ifndef DEEP8_HOST_MATH_H
#define DEEP8_HOST_MATH_H

#include "deep8/Model.h"

namespace Deep8 {
namespace Math {

void Constant(Tensor &x, float scalar);
void ConstantGPU(Tensor &x, float scalar);

/** z = x * y */
void MatrixMultiply(const Tensor &x, const Tensor &y, Tensor &z);
void MatrixMultiplyGPU(const Tensor &x, const Tensor &y, Tensor &z);
/** dx += dz * y^T */
void MatrixMultiplyGradX(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz);
void MatrixMultiplyGradXGPU(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz);
/** dy += x^T * dz */
void MatrixMultiplyGradY(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz);
void MatrixMultiplyGradYGPU(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz);
// both at once (this build's addition: the executor calls it when both inputs take a gradient)
void MatrixMultiplyGradXY(const Tensor &x, Tensor &dx, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz);
void MatrixMultiplyGradXYGPU(const Tensor &x, Tensor &dx, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz);

/** x [B,IH,IW,IC], y [OC,FH,FW,IC] (batch 1), z [B,OH,OW,OC]; the *InterimSize functions give
 *  the bytes of device scratch the caller must pass as the last argument. */
size_t Conv2dInterimSize(const Tensor &x, const Tensor &y, Tensor &z, bool covered, int strideY, int strideX, int dilationY, int dilationX);
void Conv2d(const Tensor &x, const Tensor &y, Tensor &z, bool covered, int strideY, int strideX, int dilationY, int dilationX, void *interimPtr);
void Conv2dGPU(const Tensor &x, const Tensor &y, Tensor &z, bool covered, int strideY, int strideX, int dilationY, int dilationX, void *xcol);

size_t Conv2dGradXInterimSize(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, int dilationY, int dilationX);
void Conv2dGradX(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, int dilationY, int dilationX, void *interimPtr);
void Conv2dGradXGPU(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, int dilationY, int dilationX, void *dxcol);

size_t Conv2dGradYInterimSize(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, int dilationY, int dilationX);
void Conv2dGradY(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, int dilationY, int dilationX, void *interimPtr);
void Conv2dGradYGPU(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, int dilationY, int dilationX, void *xcol);
// both gradients from one call; takes its scratch from the device pool itself
void Conv2dGradXY(const Tensor &x, Tensor &dx, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, int dilationY, int dilationX);

size_t DeConv2dInterimSize(const Tensor &x, const Tensor &y, Tensor &z, bool covered, int strideY, int strideX);
void DeConv2d(const Tensor &x, const Tensor &y, Tensor &z, bool covered, int strideY, int strideX, void *interimPtr);
void DeConv2dGPU(const Tensor &x, const Tensor &y, Tensor &z, bool covered, int strideY, int strideX, void *interimPtr);

size_t DeConv2dGradXInterimSize(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX);
void DeConv2dGradX(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, void *interimPtr);
void DeConv2dGradXGPU(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, void *interimPtr);

size_t DeConv2dGradYInterimSize(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX);
void DeConv2dGradY(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, void *interimPtr);
void DeConv2dGradYGPU(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX, void *interimPtr);
void DeConv2dGradXY(const Tensor &x, Tensor &dx, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz, bool covered, int strideY, int strideX);

// Add (broadcasting) and ReLu: deep8/include/math/Add.h:15-42 (checks deep8/src/math/Add.cpp:7-107),
// deep8/include/math/ReLu.h:14-30 (checks deep8/src/math/ReLu.cpp:6-36).  Unlike the reference, whose
// shape loop tests only the batch axis (Add.cpp:16-19), every axis is checked.
void Add(const Tensor &x, const Tensor &y, Tensor &z);
void AddGPU(const Tensor &x, const Tensor &y, Tensor &z);
void AddGradX(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz);
void AddGradXGPU(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz);
void AddGradY(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz);
void AddGradYGPU(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz);
void ReLu(const Tensor &x, Tensor &y);
void ReLuGPU(const Tensor &x, Tensor &y);
void ReLuGrad(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy);
void ReLuGradGPU(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy);

// Minus (broadcasting), L1Norm, L2Norm, ReduceMean and AXPBY: a loss and a trainer step on top of the
// operators above.  deep8/include/math/Minus.h:14-42 (checks deep8/src/math/Minus.cpp:7-107),
// L1Norm.h / L2Norm.h (checks deep8/src/math/L1Norm.cpp:6-39, L2Norm.cpp:6-42), ReduceMean.h (checks
// and output shape deep8/src/math/ReduceMean.cpp:7-121), AXPBY.h (deep8/src/math/AXPBY.cpp:6-20).
void Minus(const Tensor &x, const Tensor &y, Tensor &z);
void MinusGPU(const Tensor &x, const Tensor &y, Tensor &z);
void MinusGradX(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz);
void MinusGradXGPU(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &z, const Tensor &dz);
void MinusGradY(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz);
void MinusGradYGPU(const Tensor &x, const Tensor &y, Tensor &dy, const Tensor &z, const Tensor &dz);
/** y[b] = sum |x[b]|,  y is [batch, {1}] */
void L1Norm(const Tensor &x, Tensor &y);
void L1NormGPU(const Tensor &x, Tensor &y);
void L1NormGrad(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy);
void L1NormGradGPU(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy);
/** y[b] = sqrt(sum x[b]^2) */
void L2Norm(const Tensor &x, Tensor &y);
void L2NormGPU(const Tensor &x, Tensor &y);
void L2NormGrad(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy);
void L2NormGradGPU(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy);
/** mean over `axis` (0 is the batch; empty = every axis) */
void ReduceMean(const Tensor &x, Tensor &y, const std::vector<int> &axis = {-1}, bool keepDims = true);
void ReduceMeanGPU(const Tensor &x, Tensor &y, const std::vector<int> &axis, bool keepDims);
void ReduceMeanGrad(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy, const std::vector<int> &axis = {-1}, bool keepDims = true);
void ReduceMeanGradGPU(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy, const std::vector<int> &axis, bool keepDims);
/** the output shape of ReduceMean (shared with the node's checkShape) */
Shape ReduceMeanShape(const Shape &x, const std::vector<int> &axis, bool keepDims);
/** z = alpha * x + beta * y */
void AXPBY(const Tensor &x, float alpha, const Tensor &y, float beta, Tensor &z);
void AXPBYGPU(const Tensor &x, float alpha, const Tensor &y, float beta, Tensor &z);
/** x [B,IH,IW,C] -> y [B,OH,OW,C]; checks and output size deep8/src/math/MaxPooling2d.cpp:6-96, AvgPooling2d.cpp */
void MaxPooling2d(const Tensor &x, Tensor &y, bool covered = false, int filterHeight = 1, int filterWidth = 1, int strideY = 1, int strideX = 1);
void MaxPooling2dGPU(const Tensor &x, Tensor &y, bool covered, int filterHeight, int filterWidth, int strideY, int strideX);
void MaxPooling2dGrad(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy, bool covered = false, int filterHeight = 1, int filterWidth = 1, int strideY = 1, int strideX = 1);
void MaxPooling2dGradGPU(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy, bool covered, int filterHeight, int filterWidth, int strideY, int strideX);
void AvgPooling2d(const Tensor &x, Tensor &y, bool covered = false, int filterHeight = 1, int filterWidth = 1, int strideY = 1, int strideX = 1);
void AvgPooling2dGPU(const Tensor &x, Tensor &y, bool covered, int filterHeight, int filterWidth, int strideY, int strideX);
void AvgPooling2dGrad(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy, bool covered = false, int filterHeight = 1, int filterWidth = 1, int strideY = 1, int strideX = 1);
void AvgPooling2dGradGPU(const Tensor &x, Tensor &dx, const Tensor &y, const Tensor &dy, bool covered, int filterHeight, int filterWidth, int strideY, int strideX);
/** [B, OH, OW, C] of a pooling over x (shared with the nodes' checkShape) */
Shape Pooling2dShape(const Shape &x, bool covered, int filterHeight, int filterWidth, int strideY, int strideX);
/** one Adam step on value / gradient / m / v (deep8/include/math/AdamUpdate.h, checks deep8/src/math/AdamUpdate.cpp:6-23) */
void AdamUpdate(Tensor &value, Tensor &gradient, Tensor &m, Tensor &v, float beta1, float beta2, float epsilon, float learningRate, float weightDecay, int64_t steps);
void AdamUpdateGPU(Tensor &value, Tensor &gradient, Tensor &m, Tensor &v, float beta1, float beta2, float epsilon, float learningRate, float weightDecay, int64_t steps);

// Add (a bias with one value per element of the last axis) and ReLu folded into the contraction before them; no
// counterpart in the reference, which runs MatrixMultiplyGPU / Conv2dGPU, AddGPU (deep8/src/math/Add.cu:21-52) and
// ReLuGPU (deep8/src/math/ReLu.cu:20-59) one after the other.  Same checks as the operators they combine.
void MatrixMultiplyBiasReLu(const Tensor &x, const Tensor &y, const Tensor &bias, Tensor &z, bool relu = true);
void Conv2dBiasReLu(const Tensor &x, const Tensor &y, const Tensor &bias, Tensor &z, bool covered, int strideY, int strideX,
                    int dilationY, int dilationX, void *interimPtr, bool relu = true);
// The way back through ReLu and the bias in one pass: dpre = dz where z > 0, else 0 (dpre may be dz); dbias += its sums
// over every axis but the last.  Replaces ReLuGradGPU (ReLu.cu:61-116) followed by AddGradYGPU (Add.cu:99-133).
void BiasReLuGrad(const Tensor &z, const Tensor &dz, Tensor &dpre, Tensor &dbias);

}  // namespace Math
}  // namespace Deep8

#endif
