// Test driver of the C++ host layer.  Node-level tests in the style of the reference's
// test/MatrixMultiplyTest.h, test/Conv2dTest.h and test/DeConv2dTest.h: build a node over two
// placeholder Variables, call the explicit-tensor forward/backward, and compare with naive host
// loops on small non-negative integer inputs, for which float results are exact.
//
//   deep8_host_tests            run everything (needs a GPU)
//   deep8_host_tests --cpu      run only the tests that touch no device
//   deep8_host_tests --list     list test names
// Prints "PASS <name>" / "FAIL <name>: <why>" per test; exit code = number of failures.
#include <cmath>
#include <cstdio>
#include <chrono>
#include <cstring>
#include <functional>
#include <iostream>
#include <random>

#include "deep8/Deep8.h"

using namespace Deep8;

namespace {

struct Failure : std::runtime_error {
    using std::runtime_error::runtime_error;
};

#define EXPECT(cond)                                                                      \
    do {                                                                                  \
        if (!(cond)) throw Failure(std::string(#cond) + " at line " + std::to_string(__LINE__)); \
    } while (0)

template <typename E, typename F>
bool throws(F f) {
    try {
        f();
    } catch (const E &) {
        return true;
    } catch (...) {
        return false;
    }
    return false;
}

std::mt19937 rng(12345);
float randInt(int hi) { return (float)(rng() % hi); }

struct Test {
    const char *name;
    bool needsGpu;
    std::function<void()> body;
};
std::vector<Test> &tests() {
    static std::vector<Test> t;
    return t;
}
struct Reg {
    Reg(const char *n, bool gpu, std::function<void()> b) { tests().push_back({n, gpu, std::move(b)}); }
};
#define TEST_CPU(name) \
    void name();       \
    Reg reg_##name(#name, false, name); \
    void name()
#define TEST_GPU(name) \
    void name();       \
    Reg reg_##name(#name, true, name); \
    void name()

GPUDevice &gpu() {
    static GPUDevice *d = new GPUDevice();
    return *d;
}

// A device tensor plus its host mirror (float values; stored as float or half on the device).
struct HostTensor {
    Tensor t;
    std::vector<float> host;
};

Tensor makeTensor(GPUDevice &dev, ElementType type, size_t batch, std::vector<size_t> dims) {
    Shape shape(batch, dims);
    const size_t bytes = type.byteWidth * shape.size();
    void *ptr = dev.malloc(bytes);
    size_t *ref = (size_t *)dev.mallocCPU(sizeof(size_t));
    TensorStorage storage(ptr, ref, bytes, &dev);
    return Tensor(storage, 0, shape, type);
}

void upload(HostTensor &h) {
    if (h.t.elementType.id == DType::Float32) {
        h.t.device()->copyFromCPUToGPU(h.host.data(), h.t.raw(), h.t.byteCount());
    } else if (h.t.elementType.id == DType::Float64) {
        std::vector<double> tmp(h.host.begin(), h.host.end());
        h.t.device()->copyFromCPUToGPU(tmp.data(), h.t.raw(), h.t.byteCount());
    } else {
        std::vector<half> tmp(h.host.begin(), h.host.end());
        h.t.device()->copyFromCPUToGPU(tmp.data(), h.t.raw(), h.t.byteCount());
    }
}

void download(HostTensor &h) {
    if (h.t.elementType.id == DType::Float32) {
        h.t.device()->copyFromGPUToCPU(h.t.raw(), h.host.data(), h.t.byteCount());
    } else if (h.t.elementType.id == DType::Float64) {
        std::vector<double> tmp(h.host.size());
        h.t.device()->copyFromGPUToCPU(h.t.raw(), tmp.data(), h.t.byteCount());
        for (size_t i = 0; i < tmp.size(); ++i) h.host[i] = (float)tmp[i];
    } else {
        std::vector<half> tmp(h.host.size());
        h.t.device()->copyFromGPUToCPU(h.t.raw(), tmp.data(), h.t.byteCount());
        for (size_t i = 0; i < tmp.size(); ++i) h.host[i] = (float)tmp[i];
    }
}

HostTensor randomTensor(ElementType type, size_t batch, std::vector<size_t> dims, int hi) {
    HostTensor h;
    h.t = makeTensor(gpu(), type, batch, dims);
    h.host.resize(h.t.size());
    for (float &v : h.host) v = hi ? randInt(hi) : 0.f;
    upload(h);
    return h;
}

Variable placeholder(ElementType type) {
    Tensor v = makeTensor(gpu(), type, 1, {1});
    Tensor g = makeTensor(gpu(), type, 1, {1});
    return Variable(0, "", nullptr, v, g);
}

// ---------------------------------------------------------------------------------------------
TEST_CPU(half_conversion) {
    EXPECT(half(1.0f).bits == 0x3c00);
    EXPECT(half(-2.0f).bits == 0xc000);
    EXPECT(half(65504.0f).bits == 0x7bff);
    EXPECT(half(65520.0f).bits == 0x7c00);
    EXPECT(half(5.9604645e-8f).bits == 0x0001);
    EXPECT(half(2.9802322e-8f).bits == 0x0000);  // tie to even
    EXPECT(half(1.0009766f).bits == 0x3c01);
    EXPECT(half(1.00048828125f).bits == 0x3c00);  // tie to even
    EXPECT(half(1.00146484375f).bits == 0x3c02);  // tie to even, upwards
    for (uint32_t b = 0; b < 65536; ++b) {
        const uint32_t exp = (b >> 10) & 31, man = b & 1023;
        if (exp == 31 && man) continue;  // NaN
        EXPECT(half(half::toFloat((uint16_t)b)).bits == b);
    }
}

TEST_CPU(shape_basics) {
    Shape s(5, {2, 3, 4});
    EXPECT(s.batch == 5 && s.nDims == 3 && s.size() == 120 && s.batchSize() == 24);
    EXPECT(s.stride(0) == 12 && s.stride(1) == 4 && s.stride(2) == 1);
    EXPECT(s.row() == 2 && s.col() == 3);
    Shape v(3, {7});
    EXPECT(v.row() == 7 && v.col() == 1);
    EXPECT(Shape(5, {2, 3, 4}) == s && Shape(4, {2, 3, 4}) != s);
    EXPECT(s.equalExceptBatch(Shape(1, {2, 3, 4})));
    EXPECT(throws<std::invalid_argument>([] { Shape bad(1, {2, 0}); }));
    EXPECT(throws<std::invalid_argument>([] { Shape bad(1, {1, 2, 3, 4, 5}); }));
    EXPECT(throws<std::invalid_argument>([&] { s.dim(3); }));
    EXPECT(ElementType::from<float>().byteWidth == 4 && ElementType::from<half>().byteWidth == 2);
    EXPECT(ElementType::from(DType::Float16).id == DType::Float16);
}

TEST_CPU(node_shape_inference) {
    // checkShape needs no device
    std::vector<Node *> none;
    struct Probe : Variable {
        Probe() : Variable(0, "", nullptr) {}
    } a, b;
    std::vector<Node *> in = {&a, &b};
    MatrixMultiply mm(in);
    std::vector<Shape> s = {Shape(10, {400, 200}), Shape(1, {200, 300})};
    EXPECT(mm.checkShape(s) == Shape(10, {400, 300}));
    s = {Shape(1, {300, 100}), Shape(10, {100})};
    EXPECT(mm.checkShape(s) == Shape(10, {300}));
    s = {Shape(2, {3, 4}), Shape(3, {4, 5})};
    EXPECT(throws<std::invalid_argument>([&] { mm.checkShape(s); }));
    s = {Shape(1, {3, 4}), Shape(1, {5, 5})};
    EXPECT(throws<std::invalid_argument>([&] { mm.checkShape(s); }));

    Conv2d same(in, true, 1, 1, 1, 1);
    s = {Shape(32, {56, 56, 64}), Shape(1, {64, 3, 3, 64})};
    EXPECT(same.checkShape(s) == Shape(32, {56, 56, 64}));
    Conv2d strided(in, true, 2, 2, 2, 2);
    s = {Shape(2, {32, 32, 64}), Shape(1, {32, 4, 4, 64})};
    EXPECT(strided.checkShape(s) == Shape(2, {16, 16, 32}));
    Conv2d valid(in, false, 1, 1, 1, 1);
    EXPECT(valid.checkShape(s) == Shape(2, {29, 29, 32}));
    s = {Shape(2, {3, 3, 64}), Shape(1, {32, 4, 4, 64})};
    EXPECT(throws<std::invalid_argument>([&] { valid.checkShape(s); }));
    EXPECT(throws<std::invalid_argument>([&] { Conv2d bad(in, true, 0, 1, 1, 1); }));

    DeConv2d up(in, false, 2, 2), upCovered(in, true, 2, 2);
    s = {Shape(16, {28, 28, 128}), Shape(1, {64, 4, 4, 128})};
    EXPECT(up.checkShape(s) == Shape(16, {58, 58, 64}));
    EXPECT(upCovered.checkShape(s) == Shape(16, {55, 55, 64}));
    s = {Shape(16, {28, 28, 128}), Shape(1, {64, 4, 4, 100})};
    EXPECT(throws<std::invalid_argument>([&] { up.checkShape(s); }));

    // the fused nodes take a third input, one bias value per element of the output's last dimension
    Probe c;
    std::vector<Node *> in3 = {&a, &b, &c};
    Conv2dBiasReLu fusedConv(in3, true, 1, 1, 1, 1);
    s = {Shape(32, {56, 56, 64}), Shape(1, {64, 3, 3, 64}), Shape(1, {64})};
    EXPECT(fusedConv.checkShape(s) == Shape(32, {56, 56, 64}));
    s[2] = Shape(1, {63});
    EXPECT(throws<std::invalid_argument>([&] { fusedConv.checkShape(s); }));
    s[2] = Shape(2, {64});
    EXPECT(throws<std::invalid_argument>([&] { fusedConv.checkShape(s); }));
    MatrixMultiplyBiasReLu fusedMm(in3);
    s = {Shape(10, {400, 200}), Shape(1, {200, 300}), Shape(1, {300})};
    EXPECT(fusedMm.checkShape(s) == Shape(10, {400, 300}));
    s = {Shape(1, {300, 100}), Shape(10, {100}), Shape(1, {300})};  // a batch of vectors: the last dimension is x's rows
    EXPECT(fusedMm.checkShape(s) == Shape(10, {300}));
    EXPECT(throws<std::invalid_argument>([&] { Conv2dBiasReLu two(in, true, 1, 1, 1, 1); }));
    EXPECT(throws<std::invalid_argument>([&] { MatrixMultiply three(in3); }));
}

TEST_GPU(memory_pool) {
    GPUMemoryPool pool(0, size_t(1) << 24);  // 16 MiB blocks
    void *a = pool.malloc(1000);
    void *b = pool.malloc(1000);
    EXPECT(a && b && a != b);
    EXPECT(pool.blockCount() == 1 && pool.bytesInUse() == 2048);
    pool.free(a);
    void *c = pool.malloc(600);  // reuses the 1 KiB chunk just freed
    EXPECT(c == a);
    pool.free(b);
    pool.free(c);
    EXPECT(pool.bytesInUse() == 0);
    void *whole = pool.malloc(size_t(1) << 24);  // everything merged back: the whole block is free
    EXPECT(whole && pool.blockCount() == 1);
    void *more = pool.malloc(5 << 20);  // needs a second block
    EXPECT(more && pool.blockCount() == 2);
    pool.free(whole);
    pool.free(more);
    EXPECT(pool.malloc(0) == nullptr);
    EXPECT(throws<std::invalid_argument>([&] { pool.malloc((size_t(1) << 24) + 1); }));
    int onStack = 0;
    EXPECT(throws<std::runtime_error>([&] { pool.free(&onStack); }));
    void *d = pool.malloc(4096);
    pool.free(d);
    EXPECT(throws<std::runtime_error>([&] { pool.free(d); }));  // double free
    // the default pool refuses more than 512 MiB in one piece, like the reference's
    EXPECT(throws<std::invalid_argument>([&] { gpu().malloc((size_t(512) << 20) + 1); }));
}

TEST_GPU(tensor_storage_refcount) {
    const size_t before = gpu().memoryPool->bytesInUse();
    {
        Tensor t = makeTensor(gpu(), ElementType::from<float>(), 2, {8, 8});
        EXPECT(t.refCount() == 1 && t.byteCount() == 512);
        {
            Tensor u = t;
            EXPECT(t.refCount() == 2 && u.raw() == t.raw());
        }
        EXPECT(t.refCount() == 1);
        t.zero();
        std::vector<float> h(128, 1.f);
        gpu().copyFromGPUToCPU(t.raw(), h.data(), 512);
        for (float v : h) EXPECT(v == 0.f);
        EXPECT(throws<std::invalid_argument>([&] { t.data<half>(); }));
        EXPECT(t.data<float>() == t.raw());
    }
    EXPECT(gpu().memoryPool->bytesInUse() == before);
    Tensor s = makeTensor(gpu(), ElementType::from<half>(), 1, {1});
    s.one();
    half one;
    gpu().copyFromGPUToCPU(s.raw(), &one, 2);
    EXPECT(one.bits == 0x3c00);
}

// ---- MatrixMultiply ---------------------------------------------------------------------------------------
void matmulCase(ElementType type, size_t xb, std::vector<size_t> xd, size_t yb, std::vector<size_t> yd, int hi) {
    HostTensor x = randomTensor(type, xb, xd, hi), y = randomTensor(type, yb, yd, hi);
    Variable v0 = placeholder(type), v1 = placeholder(type);
    std::vector<Node *> in = {&v0, &v1};
    MatrixMultiply mm(in);
    std::vector<Shape> shapes = {x.t.shape, y.t.shape};
    Shape zs = mm.checkShape(shapes);
    HostTensor z = randomTensor(type, zs.batch, std::vector<size_t>(zs.dims, zs.dims + zs.nDims), 0);
    HostTensor dz = randomTensor(type, zs.batch, std::vector<size_t>(zs.dims, zs.dims + zs.nDims), hi);
    HostTensor dx = randomTensor(type, xb, xd, 0), dy = randomTensor(type, yb, yd, 0);

    std::vector<const Tensor *> tin = {&x.t, &y.t};
    mm.forward(tin, &z.t);
    mm.backward(tin, &z.t, &dz.t, 0, &dx.t);
    mm.backward(tin, &z.t, &dz.t, 1, &dy.t);
    download(z);
    download(dx);
    download(dy);

    const size_t M = x.t.row(), K = x.t.col(), N = y.t.col(), B = zs.batch;
    std::vector<float> wz(z.host.size(), 0.f), wdx(dx.host.size(), 0.f), wdy(dy.host.size(), 0.f);
    for (size_t b = 0; b < B; ++b) {
        const float *xp = x.host.data() + (b % xb) * M * K, *yp = y.host.data() + (b % yb) * K * N;
        const float *gp = dz.host.data() + b * M * N;
        float *zp = wz.data() + b * M * N, *dxp = wdx.data() + (b % xb) * M * K, *dyp = wdy.data() + (b % yb) * K * N;
        for (size_t m = 0; m < M; ++m)
            for (size_t n = 0; n < N; ++n) {
                float acc = 0;
                for (size_t k = 0; k < K; ++k) {
                    acc += xp[m * K + k] * yp[k * N + n];
                    dxp[m * K + k] += gp[m * N + n] * yp[k * N + n];
                    dyp[k * N + n] += xp[m * K + k] * gp[m * N + n];
                }
                zp[m * N + n] = acc;
            }
    }
    EXPECT(z.host == wz);
    EXPECT(dx.host == wdx);
    EXPECT(dy.host == wdy);
    // both gradients from one Math call, added to what the two calls left: twice the sums
    Math::MatrixMultiplyGradXY(x.t, dx.t, y.t, dy.t, z.t, dz.t);
    download(dx);
    download(dy);
    for (float &v : wdx) v *= 2;
    for (float &v : wdy) v *= 2;
    EXPECT(dx.host == wdx);
    EXPECT(dy.host == wdy);
}

TEST_GPU(matrix_multiply_float_collapsed_batch) {  // MatrixMultiplyTest GPU1_float shape, reduced
    matmulCase(ElementType::from<float>(), 10, {40, 20}, 1, {20, 30}, 50);
}
TEST_GPU(matrix_multiply_float_vector_batch) {  // GPU2_float: x batch 1, y a batch of vectors
    matmulCase(ElementType::from<float>(), 1, {30, 10}, 10, {10}, 50);
}
TEST_GPU(matrix_multiply_float_batched) {
    matmulCase(ElementType::from<float>(), 6, {33, 17}, 6, {17, 29}, 50);
    matmulCase(ElementType::from<float>(), 1, {33, 17}, 6, {17, 29}, 50);  // dX sums over the batch
}
TEST_GPU(matrix_multiply_half) {
    matmulCase(ElementType::from<half>(), 4, {24, 16}, 1, {16, 40}, 3);
    matmulCase(ElementType::from<half>(), 1, {24, 16}, 5, {16}, 3);
    matmulCase(ElementType::from<half>(), 3, {24, 16}, 3, {16, 8}, 3);
}

TEST_GPU(matrix_multiply_double) {  // the reference's Float64 branch (MatrixMultiply.cu:142-175)
    matmulCase(ElementType::from<double>(), 10, {40, 20}, 1, {20, 30}, 50);
    matmulCase(ElementType::from<double>(), 1, {30, 10}, 10, {10}, 50);
    matmulCase(ElementType::from<double>(), 6, {33, 17}, 6, {17, 29}, 50);
    matmulCase(ElementType::from<double>(), 1, {33, 17}, 6, {17, 29}, 50);
    Tensor s = makeTensor(gpu(), ElementType::from<double>(), 1, {1});
    s.one();
    double one = 0;
    gpu().copyFromGPUToCPU(s.raw(), &one, 8);
    EXPECT(one == 1.0);
}

TEST_GPU(matrix_multiply_errors) {
    ElementType f32 = ElementType::from<float>();
    HostTensor x = randomTensor(f32, 1, {4, 5}, 5), y = randomTensor(f32, 1, {5, 6}, 5);
    HostTensor z = randomTensor(f32, 1, {4, 6}, 0), bad = randomTensor(f32, 1, {4, 7}, 0);
    HostTensor zh = randomTensor(ElementType::from<half>(), 1, {4, 6}, 0);
    EXPECT(throws<std::invalid_argument>([&] { Math::MatrixMultiply(x.t, y.t, bad.t); }));
    EXPECT(throws<std::invalid_argument>([&] { Math::MatrixMultiply(x.t, y.t, zh.t); }));
    EXPECT(throws<std::invalid_argument>([&] { Math::MatrixMultiplyGradX(x.t, bad.t, y.t, z.t, z.t); }));
    Tensor d64 = makeTensor(gpu(), ElementType::from<double>(), 1, {4, 4});
    EXPECT(throws<std::runtime_error>([&] { Math::ReLu(d64, d64); }));  // Float64 exists on the contraction path only
    Variable v0 = placeholder(f32);
    std::vector<Node *> one = {&v0};
    EXPECT(throws<std::invalid_argument>([&] { MatrixMultiply mm(one); }));
    Variable v1 = placeholder(f32);
    std::vector<Node *> two = {&v0, &v1};
    MatrixMultiply mm(two);
    std::vector<const Tensor *> tin = {&x.t, &y.t};
    EXPECT(throws<std::runtime_error>([&] { mm.backward(tin, &z.t, &z.t, 2, &z.t); }));
}

// ---- Conv2d ---------------------------------------------------------------------------------------------------
void convCase(ElementType type, int B, int IH, int IW, int IC, int OC, int FH, int FW, bool covered, int sy, int sx,
              int dy, int dx, int hi) {
    HostTensor x = randomTensor(type, B, {(size_t)IH, (size_t)IW, (size_t)IC}, hi);
    HostTensor w = randomTensor(type, 1, {(size_t)OC, (size_t)FH, (size_t)FW, (size_t)IC}, hi);
    Variable v0 = placeholder(type), v1 = placeholder(type);
    std::vector<Node *> in = {&v0, &v1};
    Conv2d conv(in, covered, sy, sx, dy, dx);
    std::vector<Shape> shapes = {x.t.shape, w.t.shape};
    Shape zs = conv.checkShape(shapes);
    const int OH = (int)zs.dim(0), OW = (int)zs.dim(1);
    HostTensor z = randomTensor(type, B, {(size_t)OH, (size_t)OW, (size_t)OC}, 0);
    HostTensor gz = randomTensor(type, B, {(size_t)OH, (size_t)OW, (size_t)OC}, hi);
    HostTensor gx = randomTensor(type, B, {(size_t)IH, (size_t)IW, (size_t)IC}, 0);
    HostTensor gw = randomTensor(type, 1, {(size_t)OC, (size_t)FH, (size_t)FW, (size_t)IC}, 0);

    std::vector<const Tensor *> tin = {&x.t, &w.t};
    conv.forward(tin, &z.t);
    conv.backward(tin, &z.t, &gz.t, 0, &gx.t);
    conv.backward(tin, &z.t, &gz.t, 1, &gw.t);
    download(z);
    download(gx);
    download(gw);

    const int rfh = FH + (FH - 1) * (dy - 1), rfw = FW + (FW - 1) * (dx - 1);
    const int padTop = std::max(0, (OH - 1) * sy + rfh - IH) / 2, padLeft = std::max(0, (OW - 1) * sx + rfw - IW) / 2;
    std::vector<float> wz(z.host.size(), 0.f), wgx(gx.host.size(), 0.f), wgw(gw.host.size(), 0.f);
    for (int b = 0; b < B; ++b)
        for (int oy = 0; oy < OH; ++oy)
            for (int ox = 0; ox < OW; ++ox)
                for (int oc = 0; oc < OC; ++oc) {
                    const size_t zi = (((size_t)b * OH + oy) * OW + ox) * OC + oc;
                    for (int fy = 0; fy < FH; ++fy)
                        for (int fx = 0; fx < FW; ++fx) {
                            const int iy = oy * sy + fy * dy - padTop, ix = ox * sx + fx * dx - padLeft;
                            if (iy < 0 || iy >= IH || ix < 0 || ix >= IW) continue;
                            for (int ic = 0; ic < IC; ++ic) {
                                const size_t xi = (((size_t)b * IH + iy) * IW + ix) * IC + ic;
                                const size_t wi = (((size_t)oc * FH + fy) * FW + fx) * IC + ic;
                                wz[zi] += x.host[xi] * w.host[wi];
                                wgx[xi] += gz.host[zi] * w.host[wi];
                                wgw[wi] += gz.host[zi] * x.host[xi];
                            }
                        }
                }
    EXPECT(z.host == wz);
    EXPECT(gx.host == wgx);
    EXPECT(gw.host == wgw);
    // both gradients from one Math call, added to what the two calls left: twice the sums
    Math::Conv2dGradXY(x.t, gx.t, w.t, gw.t, z.t, gz.t, covered, sy, sx, dy, dx);
    download(gx);
    download(gw);
    for (float &v : wgx) v *= 2;
    for (float &v : wgw) v *= 2;
    EXPECT(gx.host == wgx);
    EXPECT(gw.host == wgw);
}

TEST_GPU(conv2d_float_covered_stride_dilation) {  // Conv2dTest forwardCPU_float geometry, smaller tensors
    convCase(ElementType::from<float>(), 2, 16, 16, 8, 6, 4, 4, true, 2, 2, 2, 2, 20);
}
TEST_GPU(conv2d_float_covered_5x5) { convCase(ElementType::from<float>(), 2, 12, 12, 4, 4, 5, 5, true, 1, 1, 1, 1, 20); }
TEST_GPU(conv2d_float_not_covered) { convCase(ElementType::from<float>(), 2, 13, 11, 5, 3, 3, 3, false, 1, 1, 1, 1, 20); }
TEST_GPU(conv2d_double) { convCase(ElementType::from<double>(), 2, 13, 11, 5, 3, 3, 3, true, 2, 2, 1, 1, 20); }
TEST_GPU(conv2d_half) { convCase(ElementType::from<half>(), 2, 8, 8, 8, 8, 3, 3, true, 1, 1, 1, 1, 2); }
// wide enough for the tiled kernels: in half the two gradient products of the one-call form share a launch
TEST_GPU(conv2d_half_64_channels) { convCase(ElementType::from<half>(), 2, 16, 16, 64, 64, 3, 3, true, 1, 1, 1, 1, 1); }
TEST_GPU(conv2d_float_64_channels) { convCase(ElementType::from<float>(), 2, 16, 16, 64, 64, 3, 3, true, 1, 1, 1, 1, 5); }

// ---- DeConv2d -----------------------------------------------------------------------------------------------------
void deconvCase(ElementType type, int B, int IH, int IW, int IC, int OC, int FH, int FW, bool covered, int sy, int sx, int hi) {
    HostTensor x = randomTensor(type, B, {(size_t)IH, (size_t)IW, (size_t)IC}, hi);
    HostTensor w = randomTensor(type, 1, {(size_t)OC, (size_t)FH, (size_t)FW, (size_t)IC}, hi);
    Variable v0 = placeholder(type), v1 = placeholder(type);
    std::vector<Node *> in = {&v0, &v1};
    DeConv2d deconv(in, covered, sy, sx);
    std::vector<Shape> shapes = {x.t.shape, w.t.shape};
    Shape zs = deconv.checkShape(shapes);
    const int OH = (int)zs.dim(0), OW = (int)zs.dim(1);
    HostTensor z = randomTensor(type, B, {(size_t)OH, (size_t)OW, (size_t)OC}, 0);
    HostTensor gz = randomTensor(type, B, {(size_t)OH, (size_t)OW, (size_t)OC}, hi);
    HostTensor gx = randomTensor(type, B, {(size_t)IH, (size_t)IW, (size_t)IC}, 0);
    HostTensor gw = randomTensor(type, 1, {(size_t)OC, (size_t)FH, (size_t)FW, (size_t)IC}, 0);

    std::vector<const Tensor *> tin = {&x.t, &w.t};
    deconv.forward(tin, &z.t);
    deconv.backward(tin, &z.t, &gz.t, 0, &gx.t);
    deconv.backward(tin, &z.t, &gz.t, 1, &gw.t);
    download(z);
    download(gx);
    download(gw);

    const int padTop = std::max(0, OH + FH - (IH - 1) * sy - 2) / 2, padLeft = std::max(0, OW + FW - (IW - 1) * sx - 2) / 2;
    std::vector<float> wz(z.host.size(), 0.f), wgx(gx.host.size(), 0.f), wgw(gw.host.size(), 0.f);
    for (int b = 0; b < B; ++b)
        for (int oy = 0; oy < OH; ++oy)
            for (int ox = 0; ox < OW; ++ox)
                for (int oc = 0; oc < OC; ++oc) {
                    const size_t zi = (((size_t)b * OH + oy) * OW + ox) * OC + oc;
                    for (int fy = 0; fy < FH; ++fy)
                        for (int fx = 0; fx < FW; ++fx) {
                            const int ty = oy - padTop + fy, tx = ox - padLeft + fx;
                            if (ty < 0 || tx < 0 || ty % sy || tx % sx) continue;
                            const int iy = ty / sy, ix = tx / sx;
                            if (iy >= IH || ix >= IW) continue;
                            for (int ic = 0; ic < IC; ++ic) {
                                const size_t xi = (((size_t)b * IH + iy) * IW + ix) * IC + ic;
                                const size_t wi = (((size_t)oc * FH + fy) * FW + fx) * IC + ic;
                                wz[zi] += x.host[xi] * w.host[wi];
                                wgx[xi] += gz.host[zi] * w.host[wi];
                                wgw[wi] += gz.host[zi] * x.host[xi];
                            }
                        }
                }
    EXPECT(z.host == wz);
    EXPECT(gx.host == wgx);
    EXPECT(gw.host == wgw);
    Math::DeConv2dGradXY(x.t, gx.t, w.t, gw.t, z.t, gz.t, covered, sy, sx);
    download(gx);
    download(gw);
    for (float &v : wgx) v *= 2;
    for (float &v : wgw) v *= 2;
    EXPECT(gx.host == wgx);
    EXPECT(gw.host == wgw);
}

TEST_GPU(deconv2d_float_not_covered_stride3) { deconvCase(ElementType::from<float>(), 2, 8, 8, 8, 4, 4, 4, false, 3, 3, 20); }
TEST_GPU(deconv2d_float_covered_stride3) { deconvCase(ElementType::from<float>(), 2, 8, 8, 8, 4, 4, 4, true, 3, 3, 20); }
TEST_GPU(deconv2d_float_stride2) { deconvCase(ElementType::from<float>(), 2, 7, 6, 4, 6, 4, 4, false, 2, 2, 20); }
TEST_GPU(deconv2d_double) { deconvCase(ElementType::from<double>(), 2, 7, 6, 4, 6, 4, 4, false, 2, 2, 20); }
TEST_GPU(deconv2d_half) { deconvCase(ElementType::from<half>(), 2, 6, 6, 8, 8, 4, 4, false, 2, 2, 2); }
TEST_GPU(deconv2d_half_64_channels) { deconvCase(ElementType::from<half>(), 2, 8, 8, 64, 64, 4, 4, false, 2, 2, 1); }
TEST_GPU(deconv2d_float_64_channels) { deconvCase(ElementType::from<float>(), 2, 8, 8, 64, 64, 4, 4, false, 2, 2, 5); }

TEST_GPU(conv2d_errors) {
    ElementType f32 = ElementType::from<float>();
    HostTensor x = randomTensor(f32, 2, {8, 8, 4}, 5), w = randomTensor(f32, 1, {3, 3, 3, 4}, 5);
    HostTensor z = randomTensor(f32, 2, {8, 8, 3}, 0), bad = randomTensor(f32, 2, {7, 8, 3}, 0);
    EXPECT(Math::Conv2dInterimSize(x.t, w.t, z.t, true, 1, 1, 1, 1) >= sizeof(float) * 2 * 8 * 8 * 3 * 3 * 4);
    EXPECT(throws<std::invalid_argument>([&] { Math::Conv2dInterimSize(x.t, w.t, bad.t, true, 1, 1, 1, 1); }));
    EXPECT(throws<std::invalid_argument>([&] { Math::Conv2d(x.t, w.t, z.t, true, 0, 1, 1, 1, nullptr); }));
    EXPECT(throws<std::invalid_argument>([&] { Math::DeConv2dInterimSize(x.t, w.t, z.t, false, 1, 1); }));
}

// ---- through the executor ---------------------------------------------------------------------------------------------
TEST_GPU(eager_executor_matmul_chain) {
    EagerExecutor executor(DeviceType::GPU);
    const size_t K = 48, N = 40;
    Variable &x = inputParameter(&executor, {1, K});
    Variable &W = parameter(&executor, {K, N});
    Variable &v = parameter(&executor, {N});
    std::vector<float> hx(K), hW(K * N), hv(N);
    for (float &f : hx) f = randInt(10);
    for (float &f : hW) f = randInt(10);
    for (float &f : hv) f = randInt(10);
    x.feed(hx.data());
    W.feed(hW.data());
    v.feed(hv.data());

    Variable &h = x * W;  // [1 x N]
    Variable &loss = h * v;  // scalar
    EXPECT(h.shape() == Shape(1, {1, N}) && loss.isScalar());
    float got = 0;
    loss.fetch(&got);
    std::vector<float> hh(N, 0.f);
    float want = 0;
    for (size_t n = 0; n < N; ++n) {
        for (size_t k = 0; k < K; ++k) hh[n] += hx[k] * hW[k * N + n];
        want += hh[n] * hv[n];
    }
    EXPECT(got == want);

    const std::string interimName = h.name;
    backward(loss);
    std::vector<float> gW(K * N), gv(N);
    gpu().copyFromGPUToCPU(W.gradient.raw(), gW.data(), gW.size() * 4);
    gpu().copyFromGPUToCPU(v.gradient.raw(), gv.data(), gv.size() * 4);
    for (size_t n = 0; n < N; ++n) {
        EXPECT(gv[n] == hh[n]);
        for (size_t k = 0; k < K; ++k) EXPECT(gW[k * N + n] == hx[k] * hv[n]);
    }
    EXPECT(executor.trainableParameters().size() == 2);
    EXPECT(executor.nodeByName(interimName) == nullptr);  // interim nodes are gone after backward
}

// ---- Add / ReLu: the shapes of test/AddTest.h (a batch of matrices plus one row shared by all) --------------
void addCase(ElementType type, size_t xb, std::vector<size_t> xd, size_t yb, std::vector<size_t> yd, int hi) {
    HostTensor x = randomTensor(type, xb, xd, hi), y = randomTensor(type, yb, yd, hi);
    Variable v0 = placeholder(type), v1 = placeholder(type);
    std::vector<Node *> in = {&v0, &v1};
    Add add(in);
    std::vector<Shape> shapes = {x.t.shape, y.t.shape};
    Shape zs = add.checkShape(shapes);
    std::vector<size_t> zd(zs.dims, zs.dims + zs.nDims);
    HostTensor z = randomTensor(type, zs.batch, zd, 0), dz = randomTensor(type, zs.batch, zd, hi);
    HostTensor dx = randomTensor(type, xb, xd, hi), dy = randomTensor(type, yb, yd, hi);
    std::vector<float> wdx = dx.host, wdy = dy.host;

    std::vector<const Tensor *> tin = {&x.t, &y.t};
    add.forward(tin, &z.t);
    add.backward(tin, &z.t, &dz.t, 0, &dx.t);
    add.backward(tin, &z.t, &dz.t, 1, &dy.t);
    download(z);
    download(dx);
    download(dy);

    // walk z with the five enlarged axes; an operand index ignores the axes it is broadcast along
    auto enlarge = [](const Shape &s) {
        std::vector<size_t> d(5, 1);
        d[0] = s.batch;
        for (int i = 4, j = (int)s.nDims - 1; j >= 0; --i, --j) d[i] = s.dim(j);
        return d;
    };
    const std::vector<size_t> xe = enlarge(x.t.shape), ye = enlarge(y.t.shape), ze = enlarge(zs);
    std::vector<float> wz(z.host.size());
    for (size_t e = 0; e < wz.size(); ++e) {
        size_t rem = e, xi = 0, yi = 0, idx[5];
        for (int a = 4; a >= 0; --a) idx[a] = rem % ze[a], rem /= ze[a];
        for (int a = 0; a < 5; ++a) {
            xi = xi * xe[a] + (xe[a] == 1 ? 0 : idx[a]);
            yi = yi * ye[a] + (ye[a] == 1 ? 0 : idx[a]);
        }
        wz[e] = x.host[xi] + y.host[yi];
        wdx[xi] += dz.host[e];
        wdy[yi] += dz.host[e];
    }
    EXPECT(z.host == wz);
    EXPECT(dx.host == wdx);
    EXPECT(dy.host == wdy);
}

TEST_GPU(add_float_shared_row) { addCase(ElementType::from<float>(), 10, {50, 20}, 1, {20}, 50); }
TEST_GPU(add_float_same_shape) { addCase(ElementType::from<float>(), 3, {7, 5}, 3, {7, 5}, 50); }
TEST_GPU(add_float_both_broadcast) { addCase(ElementType::from<float>(), 1, {6, 1}, 4, {1, 9}, 50); }
TEST_GPU(add_float_channel_bias) { addCase(ElementType::from<float>(), 2, {6, 6, 8}, 1, {8}, 50); }
TEST_GPU(add_half) { addCase(ElementType::from<half>(), 2, {6, 8}, 1, {8}, 4); }

TEST_GPU(relu_float_and_errors) {
    ElementType type = ElementType::from<float>();
    HostTensor x = randomTensor(type, 2, {9, 7}, 21), y = randomTensor(type, 2, {9, 7}, 0);
    for (float &f : x.host) f -= 10.f;  // integers in [-10, 10]
    upload(x);
    HostTensor dy = randomTensor(type, 2, {9, 7}, 20), dx = randomTensor(type, 2, {9, 7}, 20);
    std::vector<float> wdx = dx.host;
    Variable v0 = placeholder(type);
    std::vector<Node *> in = {&v0};
    ReLu relu(in);
    std::vector<const Tensor *> tin = {&x.t};
    relu.forward(tin, &y.t);
    relu.backward(tin, &y.t, &dy.t, 0, &dx.t);
    download(y);
    download(dx);
    for (size_t i = 0; i < x.host.size(); ++i) {
        EXPECT(y.host[i] == (x.host[i] > 0 ? x.host[i] : 0.f));
        EXPECT(dx.host[i] == wdx[i] + (x.host[i] > 0 ? dy.host[i] : 0.f));
    }
    HostTensor bad = randomTensor(type, 2, {9, 8}, 0), row = randomTensor(type, 1, {5}, 0);
    EXPECT(throws<std::invalid_argument>([&] { Math::ReLu(x.t, bad.t); }));
    EXPECT(throws<std::invalid_argument>([&] { Math::Add(x.t, row.t, y.t); }));  // 7 against 5 cannot broadcast
    std::vector<Shape> shapes = {x.t.shape, row.t.shape};
    Variable v1 = placeholder(type);
    std::vector<Node *> two = {&v0, &v1};
    Add add(two);
    EXPECT(throws<std::invalid_argument>([&] { add.checkShape(shapes); }));
}

TEST_GPU(eager_executor_dense_layer_with_bias_and_relu) {
    EagerExecutor executor(DeviceType::GPU);
    const size_t B = 4, K = 24, N = 16;
    Variable &x = inputParameter(&executor, {B, K});
    Variable &W = parameter(&executor, {K, N});
    Variable &b = parameter(&executor, {N});
    Variable &v = parameter(&executor, {N});
    Variable &u = inputParameter(&executor, {1, B});
    std::vector<float> hx(B * K), hW(K * N), hb(N), hv(N), hu(B, 1.f);
    u.feed(hu.data());
    for (float &f : hx) f = randInt(7) - 3.f;
    for (float &f : hW) f = randInt(7) - 3.f;
    for (float &f : hb) f = randInt(7) - 3.f;
    for (float &f : hv) f = randInt(5);
    x.feed(hx.data());
    W.feed(hW.data());
    b.feed(hb.data());
    v.feed(hv.data());

    Variable &act = relu(x * W + b);  // [B x N], the bias row shared by all rows
    Variable &out = act * v;          // [B]
    Variable &loss = u * out;         // their sum: a scalar to start the backward pass from
    EXPECT(act.shape() == Shape(1, {B, N}) && out.shape() == Shape(1, {B}) && loss.isScalar());
    std::vector<float> got(B);
    out.fetch(got.data());
    std::vector<float> pre(B * N), gb(N, 0.f), gW(K * N, 0.f);
    for (size_t i = 0; i < B; ++i) {
        float want = 0;
        for (size_t n = 0; n < N; ++n) {
            float a = hb[n];
            for (size_t k = 0; k < K; ++k) a += hx[i * K + k] * hW[k * N + n];
            pre[i * N + n] = a;
            want += (a > 0 ? a : 0.f) * hv[n];
        }
        EXPECT(got[i] == want);
    }
    backward(loss);  // d loss / d pre = v where pre > 0
    for (size_t i = 0; i < B; ++i)
        for (size_t n = 0; n < N; ++n) {
            const float g = pre[i * N + n] > 0 ? hv[n] : 0.f;
            gb[n] += g;
            for (size_t k = 0; k < K; ++k) gW[k * N + n] += hx[i * K + k] * g;
        }
    std::vector<float> rb(N), rW(K * N);
    gpu().copyFromGPUToCPU(b.gradient.raw(), rb.data(), rb.size() * 4);
    gpu().copyFromGPUToCPU(W.gradient.raw(), rW.data(), rW.size() * 4);
    EXPECT(rb == gb && rW == gW);
}

TEST_GPU(eager_executor_conv_to_scalar) {
    EagerExecutor executor(DeviceType::GPU);
    Variable &x = parameter(&executor, 1, {3, 3, 2});
    Variable &w = parameter(&executor, {1, 3, 3, 2});
    std::vector<float> hx(18), hw(18);
    for (float &f : hx) f = randInt(10);
    for (float &f : hw) f = randInt(10);
    x.feed(hx.data());
    w.feed(hw.data());
    Variable &z = x.conv2d(w, false);  // 3x3 filter over a 3x3 image, no padding: one number
    EXPECT(z.isScalar());
    float got = 0, want = 0;
    z.fetch(&got);
    for (int i = 0; i < 18; ++i) want += hx[i] * hw[i];
    EXPECT(got == want);
    backward(z);
    std::vector<float> gx(18), gw(18);
    gpu().copyFromGPUToCPU(x.gradient.raw(), gx.data(), 72);
    gpu().copyFromGPUToCPU(w.gradient.raw(), gw.data(), 72);
    EXPECT(gx == hw && gw == hx);

    EXPECT(throws<std::runtime_error>([] { EagerExecutor cpu(DeviceType::CPU); }));
}

// ---- Minus / L1Norm / L2Norm / ReduceMean nodes, AXPBY, trainers ---------------------------------------------------
TEST_GPU(loss_nodes_against_host_loops) {
    EagerExecutor executor(DeviceType::GPU);
    const size_t B = 3, R = 4, C = 5;
    Variable &x = parameter(&executor, B, {R, C});
    Variable &y = parameter(&executor, 1, {C});
    std::vector<float> hx(B * R * C), hy(C);
    for (float &f : hx) f = randInt(9) - 4.f;
    for (float &f : hy) f = randInt(9) - 4.f;
    x.feed(hx.data());
    y.feed(hy.data());

    Variable &d = x - y;  // y shared by every batch and row
    EXPECT(d.shape() == Shape(B, {R, C}));
    std::vector<float> hd(B * R * C), got(B * R * C);
    for (size_t i = 0; i < hd.size(); ++i) hd[i] = hx[i] - hy[i % C];
    d.fetch(got.data());
    EXPECT(got == hd);

    Variable &n1 = d.l1Norm();
    EXPECT(n1.shape() == Shape(B, {1}));
    std::vector<float> hn(B, 0.f), gn(B);
    for (size_t b = 0; b < B; ++b)
        for (size_t i = 0; i < R * C; ++i) hn[b] += std::fabs(hd[b * R * C + i]);
    n1.fetch(gn.data());
    EXPECT(gn == hn);

    Variable &loss = n1.reduceMean({}, false);
    EXPECT(loss.isScalar());
    float gl = 0, hl = 0;
    for (size_t b = 0; b < B; ++b) hl += hn[b];
    hl /= (float)B;
    loss.fetch(&gl);
    EXPECT(std::fabs(gl - hl) <= 1e-6f * std::fabs(hl));

    backward(loss);  // d loss / d x = sign(d) / B, d loss / d y = -sum over batch and rows of it
    std::vector<float> gx(B * R * C), gy(C), wy(C, 0.f);
    gpu().copyFromGPUToCPU(x.gradient.raw(), gx.data(), gx.size() * 4);
    gpu().copyFromGPUToCPU(y.gradient.raw(), gy.data(), gy.size() * 4);
    const float inv = 1.0f / (float)B;
    for (size_t i = 0; i < hd.size(); ++i) {
        const float g = hd[i] > 0 ? inv : (hd[i] == 0 ? 0.f : -inv);
        EXPECT(gx[i] == g);
        wy[i % C] -= g;
    }
    for (size_t c = 0; c < C; ++c) EXPECT(std::fabs(gy[c] - wy[c]) <= 1e-5f);

    // L2Norm and ReduceMean over chosen axes, explicit-tensor form
    HostTensor a = randomTensor(ElementType::from<float>(), 2, {3, 4}, 5);
    HostTensor n2 = randomTensor(ElementType::from<float>(), 2, {1}, 0);
    Math::L2Norm(a.t, n2.t);
    download(n2);
    std::vector<float> &r2 = n2.host;
    for (size_t b = 0; b < 2; ++b) {
        float sq = 0;
        for (size_t i = 0; i < 12; ++i) sq += a.host[b * 12 + i] * a.host[b * 12 + i];
        EXPECT(std::fabs(r2[b] - std::sqrt(sq)) <= 1e-6f * std::sqrt(sq) + 1e-12f);
    }
    HostTensor mean = randomTensor(ElementType::from<float>(), 1, {3, 1}, 0);
    Tensor &m = mean.t;
    Math::ReduceMean(a.t, m, {0, 2}, true);  // over the batch and the last axis
    download(mean);
    std::vector<float> &rm = mean.host;
    for (size_t r = 0; r < 3; ++r) {
        float sum = 0;
        for (size_t b = 0; b < 2; ++b)
            for (size_t c = 0; c < 4; ++c) sum += a.host[(b * 3 + r) * 4 + c];
        EXPECT(std::fabs(rm[r] - sum / 8.f) <= 1e-6f);
    }
    EXPECT(Math::ReduceMeanShape(a.t.shape, {0, 2}, false) == Shape(1, {3}));
    EXPECT(Math::ReduceMeanShape(a.t.shape, {}, false) == Shape(1, {1}));
    EXPECT(throws<std::invalid_argument>([&] { Math::ReduceMean(a.t, m, {1}, true); }));
    EXPECT(throws<std::invalid_argument>([&] { Math::L1Norm(a.t, m); }));
}

TEST_GPU(deferred_gradient_zeroing) {
    // zeroGradient() on a gradient that owns its allocation only records the fill; a reader must
    // see zeros, the first MatrixMultiply gradient overwrites, a second one adds.
    EagerExecutor executor;
    const size_t M = 6, K = 5, N = 4;
    Variable &x = parameter(&executor, {M, K});
    Variable &y = parameter(&executor, {K, N});
    std::vector<float> hx(M * K), hy(K * N), garbage(M * K, 77.f), got(M * K);
    for (float &f : hx) f = randInt(5);
    for (float &f : hy) f = randInt(5);
    x.feed(hx.data());
    y.feed(hy.data());
    gpu().copyFromCPUToGPU(garbage.data(), x.gradient.raw(), garbage.size() * 4);
    x.zeroGradient();
    gpu().copyFromGPUToCPU(x.gradient.raw(), got.data(), got.size() * 4);  // raw() performs the fill
    for (float f : got) EXPECT(f == 0.f);

    HostTensor dz = randomTensor(ElementType::from<float>(), 1, {M, N}, 5);
    Tensor z = makeTensor(gpu(), ElementType::from<float>(), 1, {M, N});
    std::vector<float> want(M * K, 0.f);
    for (size_t m = 0; m < M; ++m)
        for (size_t k = 0; k < K; ++k)
            for (size_t n = 0; n < N; ++n) want[m * K + k] += dz.host[m * N + n] * hy[k * N + n];
    gpu().copyFromCPUToGPU(garbage.data(), x.gradient.storage.ptr, garbage.size() * 4);  // behind raw()'s back
    x.zeroGradient();
    Math::MatrixMultiplyGradX(x.value, x.gradient, y.value, z, dz.t);  // overwrites the garbage
    gpu().copyFromGPUToCPU(x.gradient.raw(), got.data(), got.size() * 4);
    EXPECT(got == want);
    Math::MatrixMultiplyGradX(x.value, x.gradient, y.value, z, dz.t);  // adds
    gpu().copyFromGPUToCPU(x.gradient.raw(), got.data(), got.size() * 4);
    for (size_t i = 0; i < got.size(); ++i) EXPECT(got[i] == 2 * want[i]);
    // an element-wise gradient after a deferred zero: the fill happens first
    x.zeroGradient();
    HostTensor g = randomTensor(ElementType::from<float>(), 1, {M, K}, 9);
    Math::AddGradX(x.value, x.gradient, x.value, x.value, g.t);
    gpu().copyFromGPUToCPU(x.gradient.raw(), got.data(), got.size() * 4);
    EXPECT(got == g.host);
}

TEST_GPU(readme_regression_with_sgd_trainer) {
    // The reference README's demo: find w with [[4,-1],[2,1]] w = [10,8], i.e. w = [3,2], by
    // minimising l1NormLoss(input * w - output) with SGD.
    float hx[4] = {4, -1, 2, 1}, hy[2] = {10, 8};
    EagerExecutor executor;
    LinearDecayLearningRateIterator learningRate(2000, 0.02f, 0.f);
    SGDTrainer trainer(&learningRate);
    Variable &w = parameter(&executor, {2});
    w.gaussian();
    Variable &input = parameter(&executor, {2, 2}, false);
    Variable &output = parameter(&executor, {2}, false);
    input.feed(hx);
    output.feed(hy);
    for (int i = 0; i < 2000; ++i) {
        backward((input * w - output).l1NormLoss());
        trainer.train(&executor);
    }
    float hw[2];
    w.fetch(hw);
    printf("     w = [%f, %f]\n", hw[0], hw[1]);
    EXPECT(std::fabs(hw[0] - 3.f) < 0.05f && std::fabs(hw[1] - 2.f) < 0.05f);
    EXPECT(executor.trainableParameters().size() == 1);
}

TEST_GPU(pooling_nodes_against_host_loops) {
    EagerExecutor executor;
    const size_t B = 2, H = 6, W = 6, C = 3;
    Variable &x = parameter(&executor, B, {H, W, C});
    std::vector<float> hx(B * H * W * C);
    for (size_t i = 0; i < hx.size(); ++i) hx[i] = (float)((i * 37 + 11) % 101) - 50.f;  // distinct within any window
    x.feed(hx.data());
    Variable &mx = x.maxPooling2d(false, 2, 2, 2, 2);
    Variable &av = x.avgPooling2d(false, 2, 2, 2, 2);
    EXPECT(mx.shape() == Shape(B, {3, 3, C}) && av.shape() == Shape(B, {3, 3, C}));
    std::vector<float> gm(B * 9 * C), ga(B * 9 * C);
    mx.fetch(gm.data());
    av.fetch(ga.data());
    auto at = [&](size_t b, size_t h, size_t w, size_t c) { return hx[((b * H + h) * W + w) * C + c]; };
    for (size_t b = 0; b < B; ++b)
        for (size_t oh = 0; oh < 3; ++oh)
            for (size_t ow = 0; ow < 3; ++ow)
                for (size_t c = 0; c < C; ++c) {
                    const float v[4] = {at(b, 2 * oh, 2 * ow, c), at(b, 2 * oh, 2 * ow + 1, c), at(b, 2 * oh + 1, 2 * ow, c), at(b, 2 * oh + 1, 2 * ow + 1, c)};
                    const float m = std::max(std::max(v[0], v[1]), std::max(v[2], v[3]));
                    const size_t o = ((b * 3 + oh) * 3 + ow) * C + c;
                    EXPECT(gm[o] == m);
                    EXPECT(std::fabs(ga[o] - (v[0] + v[1] + v[2] + v[3]) * 0.25f) <= 1e-5f);
                }
    Variable &loss = (mx + av).l1NormLoss();  // both pooling gradients flow into x
    backward(loss);
    std::vector<float> gx(hx.size());
    gpu().copyFromGPUToCPU(x.gradient.raw(), gx.data(), gx.size() * 4);
    float total = 0;
    for (float g : gx) total += g;
    EXPECT(std::isfinite(total) && total != 0.f);
    std::vector<Shape> bad = {Shape(1, {3, 3})};
    std::vector<Node *> in = {&x};
    MaxPooling2d node(in, false, 2, 2, 2, 2);
    EXPECT(throws<std::invalid_argument>([&] { node.checkShape(bad); }));
    EXPECT(Math::Pooling2dShape(Shape(1, {7, 7, 4}), true, 3, 3, 2, 2) == Shape(1, {4, 4, 4}));
}

TEST_GPU(readme_cpp_demo_with_adam_trainer) {
    // The C++ demo of the reference's README, statement for statement (printing dropped).
    float x[4] = {4, -1, 2, 1};
    float y[2] = {10, 8};
    EagerExecutor executor;
    LinearDecayLearningRateIterator learningRate(1000);
    AdamTrainer trainer(&learningRate);
    auto &w = parameter(&executor, {2});
    w.gaussian();
    auto &input = parameter(&executor, {2, 2}, false);
    auto &output = parameter(&executor, {2}, false);
    input.feed(x);
    output.feed(y);
    float first = 0, last = 0;
    for (int i = 0; i < 1000; ++i) {
        auto &loss = (input * w - output).l1NormLoss();
        loss.fetch(&last);
        if (0 == i) first = last;
        backward(loss);  // the README writes loss.backward(), which is Node's no-op in the reference too (Net.h:41 is the real one)
        trainer.train(&executor, executor.trainableParameters());
    }
    float hw[2];
    w.fetch(hw);
    printf("     w = [%f, %f], loss %f -> %f\n", hw[0], hw[1], first, last);
    // lr decays from 0.01 to 0 over 1000 steps: Adam moves each weight by at most about lr per step
    // (sum = 5), enough to get from N(0, 0.01) to [3, 2]
    EXPECT(std::fabs(hw[0] - 3.f) < 0.1f && std::fabs(hw[1] - 2.f) < 0.1f && last < 0.05f * first);
}

TEST_GPU(two_layer_convnet_trains_with_sgd) {
    // conv 3x3 (4 -> 8) + bias + relu, conv 3x3 (8 -> 4), l2NormLoss against the output of a teacher
    // network of the same shape: the loss must fall steadily under plain SGD.
    EagerExecutor executor;
    ConstantLearningRateIterator learningRate(0.02f);
    SGDTrainer trainer(&learningRate);
    const size_t B = 8, H = 8, W = 8;
    std::mt19937 gen(7);
    std::normal_distribution<float> nd(0.f, 1.f);
    auto fill = [&](Variable &v, float scale) {
        std::vector<float> h(v.shape().size());
        for (float &f : h) f = nd(gen) * scale;
        v.feed(h.data());
    };
    Variable &x = parameter(&executor, B, {H, W, 4}, false);  // retained across steps, no gradient
    Variable &w1 = parameter(&executor, {8, 3, 3, 4}), &b1 = parameter(&executor, {8}), &w2 = parameter(&executor, {4, 3, 3, 8});
    Variable &t1 = parameter(&executor, {8, 3, 3, 4}, false), &tb = parameter(&executor, {8}, false), &t2 = parameter(&executor, {4, 3, 3, 8}, false);
    fill(x, 1.f);
    fill(w1, 0.2f), fill(b1, 0.1f), fill(w2, 0.2f);
    fill(t1, 0.2f), fill(tb, 0.1f), fill(t2, 0.2f);
    auto net = [&](Variable &f1, Variable &bias, Variable &f2) -> Variable & { return relu(conv2d(x, f1) + bias).conv2d(f2); };
    float first = 0, last = 0;
    for (int i = 0; i < 300; ++i) {
        Variable &loss = (net(w1, b1, w2) - net(t1, tb, t2)).l2NormLoss();
        float v = 0;
        loss.fetch(&v);
        if (0 == i) first = v;
        last = v;
        backward(loss);
        trainer.train(&executor);
    }
    printf("     loss %f -> %f\n", first, last);
    EXPECT(std::isfinite(last) && last < 0.5f * first);
    EXPECT(executor.trainableParameters().size() == 3);
}

TEST_GPU(fused_bias_relu_nodes_match_the_chain_of_nodes) {
    // relu(conv2d(x, w) + b) and relu(x2 * y + c) as chains of three nodes and as one fused node each: the same
    // values and, after backward(l2NormLoss), the same gradients of every input (Float32: bit for bit for the
    // forward values; the gradients pass through the same kernels in the same order).
    std::mt19937 gen(11);
    std::normal_distribution<float> nd(0.f, 1.f);
    auto grad = [&](Variable &v) {
        std::vector<float> h(v.shape().size());
        gpu().copyFromGPUToCPU(v.gradient.raw(), h.data(), h.size() * 4);
        return h;
    };
    auto value = [&](Variable &v) {
        std::vector<float> h(v.shape().size());
        v.fetch(h.data());
        return h;
    };
    std::vector<std::vector<float>> results[2];
    for (int fused = 0; fused < 2; ++fused) {
        EagerExecutor executor;
        gen.seed(11);
        auto fill = [&](Variable &v, float scale) {
            std::vector<float> h(v.shape().size());
            for (float &f : h) f = nd(gen) * scale;
            v.feed(h.data());
        };
        Variable &x = parameter(&executor, 4, {12, 12, 64}), &w = parameter(&executor, {64, 3, 3, 64}), &b = parameter(&executor, {64});
        Variable &x2 = parameter(&executor, 5, {40, 96}), &y = parameter(&executor, {96, 136}), &c = parameter(&executor, {136});
        // (a vector as y: z3 is [5][40] and the bias runs along x3's rows)
        Variable &x3 = parameter(&executor, 5, {40, 96}), &v = parameter(&executor, {96}), &c3 = parameter(&executor, {40});
        fill(x, 1.f), fill(w, 0.1f), fill(b, 0.5f), fill(x2, 1.f), fill(y, 0.1f), fill(c, 0.5f);
        fill(x3, 1.f), fill(v, 0.1f), fill(c3, 0.5f);
        Variable &z = fused ? conv2dBiasReLu(x, w, b) : relu(conv2d(x, w) + b);
        Variable &z2 = fused ? matrixMultiplyBiasReLu(x2, y, c) : relu(x2 * y + c);
        Variable &z3 = fused ? matrixMultiplyBiasReLu(x3, v, c3) : relu(x3 * v + c3);
        EXPECT(z.shape() == Shape(4, {12, 12, 64}) && z2.shape() == Shape(5, {40, 136}) && z3.shape() == Shape(5, {40}));
        results[fused].push_back(value(z));
        results[fused].push_back(value(z2));
        results[fused].push_back(value(z3));
        backward(z.l2NormLoss() + z2.l2NormLoss() + z3.l2NormLoss());  // (one pass: the executor drops the graph after it)
        for (Variable *p : {&x, &w, &b, &x2, &y, &c, &x3, &v, &c3}) results[fused].push_back(grad(*p));
    }
    EXPECT(results[0].size() == 12 && results[1].size() == 12);
    for (size_t k = 0; k < results[0].size(); ++k) {
        const std::vector<float> &a = results[0][k], &f = results[1][k];
        EXPECT(a.size() == f.size());
        double num = 0, den = 0;
        bool zeros = false, positives = false;
        for (size_t i = 0; i < a.size(); ++i) {
            num += (double)(a[i] - f[i]) * (a[i] - f[i]), den += (double)a[i] * a[i];
            zeros |= a[i] == 0.f, positives |= a[i] > 0.f;
        }
        if (k < 3) EXPECT(zeros && positives);  // the ReLu cut something and kept something
        EXPECT(den > 0 && std::sqrt(num / den) <= (k < 3 ? 0.0 : 1e-6));
    }
    // shape checks of the fused nodes
    EagerExecutor executor;
    Variable &x = parameter(&executor, 2, {8, 8, 4}), &w = parameter(&executor, {8, 3, 3, 4}), &bad = parameter(&executor, {7});
    EXPECT(throws<std::invalid_argument>([&] { conv2dBiasReLu(x, w, bad); }));
}

}  // namespace

// Node-level step times at the three large configurations: forward + both gradients through Function::forward /
// backward, i.e. with the scratch buffer taken from and returned to the device pool inside every call and the
// gradients zeroed before the backward pass (lazily: Tensor::zero defers the fill).  Printed, not asserted.
// The device is kept busy with the same steps for 60 ms first: the chip raises its shader clock over the first
// 35-50 ms of sustained load, and a loop timed from an idle device measures that ramp.
template <typename NodeT>
void timeNode(const char *what, NodeT &node, HostTensor &a, HostTensor &b, HostTensor &z, HostTensor &gz, HostTensor &ga,
              HostTensor &gb, double flops) {
    std::vector<const Tensor *> tin = {&a.t, &b.t};
    auto step = [&] {
        node.forward(tin, &z.t);
        ga.t.zero();
        gb.t.zero();
        node.backward(tin, &z.t, &gz.t, 0, &ga.t);
        node.backward(tin, &z.t, &gz.t, 1, &gb.t);
    };
    step();
    gpu().synchronize();
    for (const auto s0 = std::chrono::steady_clock::now(); std::chrono::steady_clock::now() - s0 < std::chrono::milliseconds(60);) {
        for (int i = 0; i < 4; ++i) step();
        gpu().synchronize();
    }
    for (int i = 0; i < 3; ++i) step();
    gpu().synchronize();
    const int reps = 20;
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < reps; ++i) step();
    gpu().synchronize();
    const double us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count() / reps;
    printf("     %-58s %8.1f us / step  %8.1f TFLOP/s\n", what, us, flops / us * 1e-6);
}

TEST_GPU(node_level_step_times) {
    {
        ElementType h16 = ElementType::from<half>();
        HostTensor x = randomTensor(h16, 1, {4096, 4096}, 2), y = randomTensor(h16, 1, {4096, 4096}, 2);
        HostTensor z = randomTensor(h16, 1, {4096, 4096}, 0), dz = randomTensor(h16, 1, {4096, 4096}, 2);
        HostTensor dx = randomTensor(h16, 1, {4096, 4096}, 0), dy = randomTensor(h16, 1, {4096, 4096}, 0);
        Variable v0 = placeholder(h16), v1 = placeholder(h16);
        std::vector<Node *> in = {&v0, &v1};
        MatrixMultiply mm(in);
        timeNode("MatrixMultiply half 4096^3 (0/1-valued operands)", mm, x, y, z, dz, dx, dy, 3 * 2.0 * 4096.0 * 4096.0 * 4096.0);
    }
    {
        ElementType f32 = ElementType::from<float>();
        HostTensor x = randomTensor(f32, 32, {56, 56, 64}, 5), w = randomTensor(f32, 1, {64, 3, 3, 64}, 5);
        HostTensor z = randomTensor(f32, 32, {56, 56, 64}, 0), gz = randomTensor(f32, 32, {56, 56, 64}, 5);
        HostTensor gx = randomTensor(f32, 32, {56, 56, 64}, 0), gw = randomTensor(f32, 1, {64, 3, 3, 64}, 0);
        Variable v0 = placeholder(f32), v1 = placeholder(f32);
        std::vector<Node *> in = {&v0, &v1};
        Conv2d conv(in, true, 1, 1, 1, 1);
        timeNode("Conv2d fp32 B32 56x56x64 3x3 -> 64", conv, x, w, z, gz, gx, gw, 3 * 2.0 * 32 * 56 * 56 * 576.0 * 64);
    }
    {
        ElementType h16 = ElementType::from<half>();
        HostTensor x = randomTensor(h16, 16, {28, 28, 128}, 2), w = randomTensor(h16, 1, {64, 4, 4, 128}, 2);
        HostTensor z = randomTensor(h16, 16, {58, 58, 64}, 0), gz = randomTensor(h16, 16, {58, 58, 64}, 2);
        HostTensor gx = randomTensor(h16, 16, {28, 28, 128}, 0), gw = randomTensor(h16, 1, {64, 4, 4, 128}, 0);
        Variable v0 = placeholder(h16), v1 = placeholder(h16);
        std::vector<Node *> in = {&v0, &v1};
        DeConv2d deconv(in, false, 2, 2);
        timeNode("DeConv2d half B16 28x28x128 4x4 s2 -> 58x58x64", deconv, x, w, z, gz, gx, gw, 3 * 2.0 * 16 * 28 * 28 * 128.0 * 64 * 16);
    }
}

int main(int argc, char **argv) {
    bool cpuOnly = false, list = false;
    std::string only;
    for (int i = 1; i < argc; ++i) {
        if (!strcmp(argv[i], "--cpu")) cpuOnly = true;
        else if (!strcmp(argv[i], "--list")) list = true;
        else only = argv[i];
    }
    int failures = 0, ran = 0;
    for (Test &t : tests()) {
        if (list) {
            printf("%s %s\n", t.needsGpu ? "gpu" : "cpu", t.name);
            continue;
        }
        if ((cpuOnly && t.needsGpu) || (!only.empty() && only != t.name)) continue;
        printf("RUN  %s\n", t.name);
        fflush(stdout);
        try {
            t.body();
            printf("PASS %s\n", t.name);
        } catch (const std::exception &e) {
            printf("FAIL %s: %s\n", t.name, e.what());
            ++failures;
        }
        fflush(stdout);
        ++ran;
    }
    if (!list) printf("%d test(s), %d failure(s)\n", ran, failures);
    return failures;
}
