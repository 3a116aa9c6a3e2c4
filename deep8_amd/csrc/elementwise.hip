// Add (numpy-style broadcasting over [batch, d0..d3]) and ReLu, forward and gradients: the steps
// that follow every MatrixMultiply / Conv2d in a Deep8 network (bias, activation).  All are
// HBM-bandwidth bound: 16-byte accesses along the contiguous axis, every output written once, and
// the broadcast-gradient reductions are two deterministic passes (no atomics).
//
// The same kernels, with a scale on the second operand or on the reduced sum and an optional
// transform of the loaded value, also serve Minus, L1Norm / L2Norm (row reductions of |x| and
// x^2), ReduceMean and its gradient; AXPBY is the trainers' update step.
//
// Replaces AddGPU / AddGradXGPU / AddGradYGPU (deep8/src/math/Add.cu:21-133 over
// deep8/include/math/GPUBinaryElementWise.h), ReLuGPU / ReLuGradGPU (deep8/src/math/ReLu.cu:20-116),
// MinusGPU / MinusGradXGPU / MinusGradYGPU (deep8/src/math/Minus.cu:21-147), L1NormGPU / L1NormGradGPU
// (deep8/src/math/L1Norm.cu:27-136), L2NormGPU / L2NormGradGPU (deep8/src/math/L2Norm.cu),
// ReduceMeanGPU / ReduceMeanGradGPU (deep8/src/math/ReduceMean.cu:30-203 over GPUReduce.h) and AXPBYGPU
// (deep8/src/math/AXPBY.cu:9-47) and AdamUpdateGPU (deep8/src/math/AdamUpdate.cu:9-47).
#include "common.h"

namespace d8 {

__device__ inline float ew_f32(float v) { return v; }
__device__ inline float ew_f32(f16 v) { return (float)v; }

static inline int ew_grid(long work, int block) {
    long blocks = (work + block - 1) / block;
    const long cap = (long)cu_count() * 32;
    if (blocks > cap) blocks = cap;
    return (int)(blocks < 1 ? 1 : blocks);
}

// Up to 5 merged axes, outermost first.  n[a] is the extent, xs / ys the element stride of the
// operand along it (0 where the operand is broadcast).
struct BroadcastGeom {
    int nd;
    int n[5];
    long xs[5], ys[5];
};

// z = x + ys * y.  A thread owns VEC consecutive elements of the innermost axis; an operand that
// is broadcast along that axis contributes one scalar to all of them.  z may be x itself when x
// is not broadcast (each thread then reads exactly the elements it writes).
template <typename T, int VEC>
__global__ __launch_bounds__(256) void add_kernel(const T *x, const T *__restrict__ y, T *z, BroadcastGeom g, long total,
                                                  float ys) {
    typedef T VT __attribute__((ext_vector_type(VEC)));
    const int last = g.nd - 1;
    const long inner = g.n[last] / VEC;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        long rem = idx / inner;
        const long i0 = (idx - rem * inner) * VEC;
        long xo = i0 * g.xs[last], yo = i0 * g.ys[last];
        for (int a = last - 1; a >= 0; --a) {
            const long q = rem / g.n[a], i = rem - q * g.n[a];
            rem = q;
            xo += i * g.xs[a];
            yo += i * g.ys[a];
        }
        float xv[VEC], yv[VEC];
        if (g.xs[last]) {
            const VT v = *(const VT *)(x + xo);
#pragma unroll
            for (int e = 0; e < VEC; ++e) xv[e] = ew_f32(v[e]);
        } else {
            const float s = ew_f32(x[xo]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) xv[e] = s;
        }
        if (g.ys[last]) {
            const VT v = *(const VT *)(y + yo);
#pragma unroll
            for (int e = 0; e < VEC; ++e) yv[e] = ew_f32(v[e]);
        } else {
            const float s = ew_f32(y[yo]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) yv[e] = s;
        }
        VT o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) o[e] = (T)(xv[e] + ys * yv[e]);
        *(VT *)(z + idx * VEC) = o;
    }
}

// What a reduction does to each value it loads.
enum { LOAD_ID = 0, LOAD_ABS = 1, LOAD_SQUARE = 2 };
template <int OP>
__device__ inline float ew_load(float v) { return OP == LOAD_ABS ? fabsf(v) : (OP == LOAD_SQUARE ? v * v : v); }

// g = keep * g + scale * op(dz), same shape.  keep is 1 (the reference's accumulate) or 0 (g's old contents are
// not read: the overwrite forms).  The same convention holds for every kernel below that takes `keep`.
template <typename T, int VEC, int OP>
__global__ __launch_bounds__(256) void accumulate_kernel(T *__restrict__ g, const T *__restrict__ dz, long total, float scale,
                                                         float keep) {
    typedef T VT __attribute__((ext_vector_type(VEC)));
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        VT a;
#pragma unroll
        for (int e = 0; e < VEC; ++e) a[e] = (T)0;
        if (keep != 0.f) a = *(const VT *)(g + idx * VEC);
        const VT b = *(const VT *)(dz + idx * VEC);
        VT o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) o[e] = (T)(ew_f32(a[e]) + scale * ew_load<OP>(ew_f32(b[e])));
        *(VT *)(g + idx * VEC) = o;
    }
}

// dz viewed [K0][R][C]; sums over R.  Block (x: column group, y: chunk of R, z: k0); TX threads
// across column vectors, 256 / TX rows in flight.  The row lanes meet in LDS in a fixed order.
// With one chunk the sums go straight into g (g += scale * sum); otherwise into
// partial[k0][chunk][C].
template <typename T, int VEC, int OP>
__global__ __launch_bounds__(256) void column_sum_kernel(const T *__restrict__ dz, T *__restrict__ g,
                                                         float *__restrict__ partial, int R, int C, int TX,
                                                         int rows_per_chunk, int chunks, float scale, float keep) {
    typedef T VT __attribute__((ext_vector_type(VEC)));
    __shared__ float part[256][VEC];
    const int tx = threadIdx.x % TX, ty = threadIdx.x / TX, lanes = 256 / TX;
    const int cv = blockIdx.x * TX + tx;
    const int k0 = blockIdx.z, chunk = blockIdx.y;
    const bool live = (long)cv * VEC < C;
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
    if (live) {
        const int r1 = min(R, (chunk + 1) * rows_per_chunk);
        const T *p = dz + ((long)k0 * R) * C + (long)cv * VEC;
        int r = chunk * rows_per_chunk + ty;
        // four rows in flight per thread; the adds keep the order of the plain loop
        for (; r + 3 * lanes < r1; r += 4 * lanes) {
            VT v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = *(const VT *)(p + (long)(r + u * lanes) * C);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[e] += ew_load<OP>(ew_f32(v[u][e]));
        }
        for (; r < r1; r += lanes) {
            const VT v = *(const VT *)(p + (long)r * C);
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] += ew_load<OP>(ew_f32(v[e]));
        }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) part[threadIdx.x][e] = acc[e];
    __syncthreads();
    if (ty == 0 && live) {
        for (int k = 1; k < lanes; ++k)
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] += part[k * TX + tx][e];
        if (chunks == 1) {
            T *o = g + (long)k0 * C + (long)cv * VEC;
#pragma unroll
            for (int e = 0; e < VEC; ++e) o[e] = (T)((keep != 0.f ? ew_f32(o[e]) : 0.f) + scale * acc[e]);
        } else {
            float *o = partial + ((long)k0 * chunks + chunk) * C + (long)cv * VEC;
#pragma unroll
            for (int e = 0; e < VEC; ++e) o[e] = acc[e];
        }
    }
}

// g[k0][c] += sum over chunks of partial[k0][chunk][c].  A block covers 16 outputs; 16 lanes per
// output each add every 16th chunk (eight loads in flight) and meet in LDS in a fixed order.
template <typename T>
__global__ __launch_bounds__(256) void column_sum_finish_kernel(const float *__restrict__ partial, T *__restrict__ g,
                                                                int C, int chunks, long total, float scale, float keep) {
    __shared__ float part[16][16];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const long idx = (long)blockIdx.x * 16 + tx;
    float v = 0.f;
    if (idx < total) {
        const long k0 = idx / C;
        const int c = (int)(idx - k0 * C);
        const float *p = partial + k0 * chunks * C + c;
        int k = ty;
        for (; k + 7 * 16 < chunks; k += 8 * 16) {
            float t[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) t[u] = p[(long)(k + u * 16) * C];
#pragma unroll
            for (int u = 0; u < 8; ++u) v += t[u];
        }
        for (; k < chunks; k += 16) v += p[(long)k * C];
    }
    part[ty][tx] = v;
    __syncthreads();
    if (ty == 0 && idx < total) {
#pragma unroll
        for (int k = 1; k < 16; ++k) v += part[k][tx];
        g[idx] = (T)((keep != 0.f ? ew_f32(g[idx]) : 0.f) + scale * v);
    }
}

// ReLuGrad and the bias gradient in one pass over a [R][C] gradient: dpre = z > 0 ? dz : 0 is written out and its
// column sums are taken on the way, with column_sum_kernel's chunks, row order and LDS meeting order, so the sums
// are bit for bit those of d8_add_grad run on dpre afterwards.  z is the layer's output relu(pre): z > 0 exactly
// where pre > 0 (deep8/src/math/ReLu.cu:61-116 gates on pre; Add.cu:64-133 sums).  dpre may be dz (in place).
template <typename T, int VEC>
__global__ __launch_bounds__(256) void relu_gate_column_sum_kernel(const T *__restrict__ z, const T *dz, T *dpre,
                                                                   T *__restrict__ g, float *__restrict__ partial, int R, int C,
                                                                   int TX, int rows_per_chunk, int chunks, float keep) {
    typedef T VT __attribute__((ext_vector_type(VEC)));
    __shared__ float part[256][VEC];
    const int tx = threadIdx.x % TX, ty = threadIdx.x / TX, lanes = 256 / TX;
    const int cv = blockIdx.x * TX + tx;
    const int chunk = blockIdx.y;
    const bool live = (long)cv * VEC < C;
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
    if (live) {
        const int r1 = min(R, (chunk + 1) * rows_per_chunk);
        const long col = (long)cv * VEC;
        int r = chunk * rows_per_chunk + ty;
        for (; r + 3 * lanes < r1; r += 4 * lanes) {
            VT a[4], b[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                a[u] = *(const VT *)(z + (long)(r + u * lanes) * C + col);
                b[u] = *(const VT *)(dz + (long)(r + u * lanes) * C + col);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    if (!(ew_f32(a[u][e]) > 0.f)) b[u][e] = (T)0.f;
                    acc[e] += ew_f32(b[u][e]);
                }
                *(VT *)(dpre + (long)(r + u * lanes) * C + col) = b[u];
            }
        }
        for (; r < r1; r += lanes) {
            const VT a = *(const VT *)(z + (long)r * C + col);
            VT b = *(const VT *)(dz + (long)r * C + col);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                if (!(ew_f32(a[e]) > 0.f)) b[e] = (T)0.f;
                acc[e] += ew_f32(b[e]);
            }
            *(VT *)(dpre + (long)r * C + col) = b;
        }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) part[threadIdx.x][e] = acc[e];
    __syncthreads();
    if (ty == 0 && live) {
        for (int k = 1; k < lanes; ++k)
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] += part[k * TX + tx][e];
        if (chunks == 1) {
            T *o = g + (long)cv * VEC;
#pragma unroll
            for (int e = 0; e < VEC; ++e) o[e] = (T)((keep != 0.f ? ew_f32(o[e]) : 0.f) + acc[e]);
        } else {
            float *o = partial + (long)chunk * C + (long)cv * VEC;
#pragma unroll
            for (int e = 0; e < VEC; ++e) o[e] = acc[e];
        }
    }
}

// z[r][c] = relu?(z[r][c] + bias[c]) in place: the one-pass fallback of the fused GEMM store.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void bias_relu_kernel(T *z, const T *__restrict__ bias, long nvec, int CV, int relu) {
    typedef T VT __attribute__((ext_vector_type(VEC)));
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < nvec; idx += (long)gridDim.x * blockDim.x) {
        VT v = *(const VT *)(z + idx * VEC);
        const int c = (int)(idx % CV) * VEC;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float f = ew_f32(v[e]);
            if (bias) f = ew_f32((T)(f + ew_f32(bias[c + e])));  // rounded as the separate Add pass rounds it
            v[e] = (T)(relu && !(f > 0.f) ? 0.f : f);
        }
        *(VT *)(z + idx * VEC) = v;
    }
}

// Any other pattern of kept and summed axes: a thread per element of g walks the summed index
// space in memory order (the order of the reference kernel, GPUBinaryElementWise.h:42-95).
struct ReduceGeom {
    int n[5];      // extents of dz
    int kept[5];   // 1 where g has the same extent, 0 where it is summed (or the extent is 1)
};

template <typename T, int OP>
__global__ __launch_bounds__(256) void broadcast_sum_kernel(const T *__restrict__ dz, T *__restrict__ g, ReduceGeom q,
                                                            long total, float scale, float keep) {
    long zs[5];
    zs[4] = 1;
    for (int a = 3; a >= 0; --a) zs[a] = zs[a + 1] * q.n[a + 1];
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        long rem = idx, base = 0;
        for (int a = 4; a >= 0; --a)
            if (q.kept[a]) {
                const long t = rem / q.n[a];
                base += (rem - t * q.n[a]) * zs[a];
                rem = t;
            }
        float acc = 0.f;
        int i[5] = {0, 0, 0, 0, 0};
        while (true) {
            long off = base;
            for (int a = 0; a < 5; ++a) off += (long)i[a] * zs[a];
            acc += ew_load<OP>(ew_f32(dz[off]));
            int a = 4;
            for (; a >= 0; --a) {
                if (q.kept[a]) continue;
                if (++i[a] < q.n[a]) break;
                i[a] = 0;
            }
            if (a < 0) break;
        }
        g[idx] = (T)((keep != 0.f ? ew_f32(g[idx]) : 0.f) + scale * acc);
    }
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void relu_kernel(const T *__restrict__ x, T *__restrict__ y, long total) {
    typedef T VT __attribute__((ext_vector_type(VEC)));
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const VT v = *(const VT *)(x + idx * VEC);
        VT o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) o[e] = v[e] > (T)0 ? v[e] : (T)0;
        *(VT *)(y + idx * VEC) = o;
    }
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void relu_grad_kernel(const T *__restrict__ x, T *__restrict__ dx,
                                                        const T *__restrict__ dy, long total, float keep) {
    typedef T VT __attribute__((ext_vector_type(VEC)));
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const VT v = *(const VT *)(x + idx * VEC), d = *(const VT *)(dy + idx * VEC);
        VT old;
#pragma unroll
        for (int e = 0; e < VEC; ++e) old[e] = (T)0;
        if (keep != 0.f) old = *(const VT *)(dx + idx * VEC);
        VT o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) o[e] = (T)(ew_f32(old[e]) + (v[e] > (T)0 ? ew_f32(d[e]) : 0.f));
        *(VT *)(dx + idx * VEC) = o;
    }
}

// dx[b][i] += dy[b] * sign(x[b][i])        (L1, deep8/src/math/L1Norm.cu:77-95)
// dx[b][i] += dy[b] / y[b] * x[b][i]       (L2)
template <typename T, int VEC, bool L2>
__global__ __launch_bounds__(256) void norm_grad_kernel(const T *__restrict__ x, T *__restrict__ dx, const T *__restrict__ y,
                                                        const T *__restrict__ dy, long row_vecs, long total) {
    typedef T VT __attribute__((ext_vector_type(VEC)));
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const long b = idx / row_vecs;
        const float s = L2 ? ew_f32(dy[b]) / ew_f32(y[b]) : ew_f32(dy[b]);
        const VT v = *(const VT *)(x + idx * VEC), old = *(const VT *)(dx + idx * VEC);
        VT o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float xv = ew_f32(v[e]);
            const float gx = L2 ? s * xv : (xv > 0.f ? s : (xv == 0.f ? 0.f : -s));
            o[e] = (T)(ew_f32(old[e]) + gx);
        }
        *(VT *)(dx + idx * VEC) = o;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void sqrt_kernel(T *p, long n) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) p[i] = (T)sqrtf(ew_f32(p[i]));
}

template <typename T>
__global__ __launch_bounds__(256) void ew_zero_kernel(T *p, long n) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) p[i] = (T)0;
}

// z = alpha * x + beta * y (z may be x or y)
template <typename T, int VEC>
__global__ __launch_bounds__(256) void axpby_kernel(const T *x, float alpha, const T *y, float beta, T *z, long total) {
    typedef T VT __attribute__((ext_vector_type(VEC)));
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const VT a = *(const VT *)(x + idx * VEC), b = *(const VT *)(y + idx * VEC);
        VT o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) o[e] = (T)(alpha * ew_f32(a[e]) + beta * ew_f32(b[e]));
        *(VT *)(z + idx * VEC) = o;
    }
}

// One Adam step (deep8/src/math/AdamUpdate.cu:9-20): g += wd * value; m = b1 m + (1 - b1) g;
// v = b2 v + (1 - b2) g^2; value -= ratio * m / (sqrt(v) + eps).  All four tensors are read and
// written once.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void adam_kernel(T *__restrict__ value, T *__restrict__ grad, T *__restrict__ m,
                                                   T *__restrict__ v, float b1, float b2, float eps, float wd, float ratio,
                                                   long total) {
    typedef T VT __attribute__((ext_vector_type(VEC)));
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        VT x = *(const VT *)(value + idx * VEC), g = *(const VT *)(grad + idx * VEC);
        VT mt = *(const VT *)(m + idx * VEC), vt = *(const VT *)(v + idx * VEC);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float xe = ew_f32(x[e]);
            const float ge = ew_f32(g[e]) + xe * wd;
            const float me = ew_f32(mt[e]) * b1 + (1.f - b1) * ge;
            const float ve = ew_f32(vt[e]) * b2 + ge * ge * (1.f - b2);
            g[e] = (T)ge, mt[e] = (T)me, vt[e] = (T)ve;
            x[e] = (T)(xe - me / (sqrtf(ve) + eps) * ratio);
        }
        *(VT *)(value + idx * VEC) = x;
        *(VT *)(grad + idx * VEC) = g;
        *(VT *)(m + idx * VEC) = mt;
        *(VT *)(v + idx * VEC) = vt;
    }
}

static inline bool al16(const void *p) { return ((size_t)p & 15) == 0; }

static int check_dims(const char *who, const int *d, const int *zd) {
    for (int a = 0; a < 5; ++a) {
        D8_REQUIRE(d[a] >= 1 && zd[a] >= 1, "%s: extents must be positive", who);
        D8_REQUIRE(d[a] == 1 || d[a] == zd[a], "%s: the shape is error (axis %d: %d against %d)", who, a, d[a], zd[a]);
    }
    return 0;
}

static long prod5(const int *d) {
    long n = 1;
    for (int a = 0; a < 5; ++a) n *= d[a];
    return n;
}

// The gradient's reduction, with consecutive axes of the same kind merged:
// kind 0: g += dz; kind 1: dz is [K0][R][C], summed over R; kind 2: anything else.
struct ReducePlan {
    int kind;
    long K0, R, C;
    int chunks, rows_per_chunk;
};

static ReducePlan plan_reduce(const int *d, const int *zd) {
    int kinds[5], ext[5], n = 0;  // 1 kept, 0 summed; extent-1 axes dropped
    for (int a = 0; a < 5; ++a) {
        if (zd[a] == 1) continue;
        const int k = d[a] == zd[a];
        if (n && kinds[n - 1] == k) ext[n - 1] *= zd[a];
        else kinds[n] = k, ext[n] = zd[a], ++n;
    }
    ReducePlan p = {2, 1, 1, 1, 1, 1};
    if (n == 0 || (n == 1 && kinds[0] == 1)) {
        p.kind = 0;
        return p;
    }
    if (n == 1) p.kind = 1, p.R = ext[0];                                              // [R]
    else if (n == 2 && kinds[0] == 0) p.kind = 1, p.R = ext[0], p.C = ext[1];          // [R][C]
    else if (n == 2) p.kind = 1, p.K0 = ext[0], p.R = ext[1];                          // [K0][R]
    else if (n == 3 && kinds[0] == 1) p.kind = 1, p.K0 = ext[0], p.R = ext[1], p.C = ext[2];  // [K0][R][C]
    if (p.kind == 1) {
        if (p.K0 > 65535 || p.R >= (1L << 31) || p.C >= (1L << 31)) {
            p.kind = 2;
            return p;
        }
        const long colblocks = (p.C + 255) / 256;  // upper bound on column groups
        long chunks = (4L * cu_count()) / (colblocks * p.K0);
        const long max_chunks = (p.R + 63) / 64;
        if (chunks > max_chunks) chunks = max_chunks;
        if (chunks > 512) chunks = 512;
        if (chunks < 1) chunks = 1;
        p.rows_per_chunk = (int)((p.R + chunks - 1) / chunks);
        p.chunks = (int)((p.R + p.rows_per_chunk - 1) / p.rows_per_chunk);
    }
    return p;
}

// g = keep * g + scale * (op(dz) summed over the axes where g has extent 1 and dz does not)
template <typename T, int WIDE, int OP = LOAD_ID>
static int reduce_t(T *g, const int *d, const T *dz, const int *zd, void *scratch, size_t scratch_bytes, hipStream_t s,
                    float scale = 1.f, float keep = 1.f) {
    const ReducePlan p = plan_reduce(d, zd);
    const long ng = prod5(d);
    if (p.kind == 0) {
        if (ng % WIDE == 0 && al16(g) && al16(dz))
            hipLaunchKernelGGL((accumulate_kernel<T, WIDE, OP>), dim3(ew_grid(ng / WIDE, 256)), dim3(256), 0, s, g, dz, ng / WIDE, scale, keep);
        else
            hipLaunchKernelGGL((accumulate_kernel<T, 1, OP>), dim3(ew_grid(ng, 256)), dim3(256), 0, s, g, dz, ng, scale, keep);
    } else if (p.kind == 1) {
        int chunks = p.chunks, rpc = p.rows_per_chunk;
        const size_t need = (size_t)p.K0 * chunks * p.C * sizeof(float);
        if (chunks > 1 && (!scratch || scratch_bytes < need || !al16(scratch))) chunks = 1, rpc = (int)p.R;  // one pass, still exact
        const bool wide = p.C % WIDE == 0 && al16(g) && al16(dz);
        const int vec = wide ? WIDE : 1;
        const long cvs = p.C / vec;
        int TX = 1;
        while (TX < 32 && TX < cvs) TX *= 2;
        dim3 grid((unsigned)((cvs + TX - 1) / TX), (unsigned)chunks, (unsigned)p.K0);
        if (wide)
            hipLaunchKernelGGL((column_sum_kernel<T, WIDE, OP>), grid, dim3(256), 0, s, dz, g, (float *)scratch, (int)p.R, (int)p.C,
                               TX, rpc, chunks, scale, keep);
        else
            hipLaunchKernelGGL((column_sum_kernel<T, 1, OP>), grid, dim3(256), 0, s, dz, g, (float *)scratch, (int)p.R, (int)p.C,
                               TX, rpc, chunks, scale, keep);
        if (chunks > 1) {
            D8_LAUNCH_CHECK();
            hipLaunchKernelGGL((column_sum_finish_kernel<T>), dim3((unsigned)((ng + 15) / 16)), dim3(256), 0, s,
                               (const float *)scratch, g, (int)p.C, chunks, ng, scale, keep);
        }
    } else {
        ReduceGeom q;
        for (int a = 0; a < 5; ++a) q.n[a] = zd[a], q.kept[a] = (d[a] == zd[a] && zd[a] > 1) ? 1 : 0;
        hipLaunchKernelGGL((broadcast_sum_kernel<T, OP>), dim3(ew_grid(ng, 256)), dim3(256), 0, s, dz, g, q, ng, scale, keep);
    }
    D8_LAUNCH_CHECK();
    return 0;
}

template <typename T, int WIDE>
static int add_t(const T *x, const int *xd, const T *y, const int *yd, T *z, const int *zd, hipStream_t s, float ys = 1.f) {
    // merge consecutive axes on which both operands behave the same way
    BroadcastGeom g;
    int kx[5], ky[5];
    g.nd = 0;
    for (int a = 0; a < 5; ++a) {
        if (zd[a] == 1) continue;
        const int fx = xd[a] != 1, fy = yd[a] != 1;
        if (g.nd && kx[g.nd - 1] == fx && ky[g.nd - 1] == fy) g.n[g.nd - 1] *= zd[a];
        else kx[g.nd] = fx, ky[g.nd] = fy, g.n[g.nd] = zd[a], ++g.nd;
    }
    if (g.nd == 0) g.nd = 1, g.n[0] = 1, kx[0] = ky[0] = 1;
    long sx = 1, sy = 1;
    for (int a = g.nd - 1; a >= 0; --a) {
        g.xs[a] = kx[a] ? sx : 0;
        g.ys[a] = ky[a] ? sy : 0;
        if (kx[a]) sx *= g.n[a];
        if (ky[a]) sy *= g.n[a];
    }
    const long n = prod5(zd);
    if (g.n[g.nd - 1] % WIDE == 0 && al16(x) && al16(y) && al16(z))
        hipLaunchKernelGGL((add_kernel<T, WIDE>), dim3(ew_grid(n / WIDE, 256)), dim3(256), 0, s, x, y, z, g, n / WIDE, ys);
    else
        hipLaunchKernelGGL((add_kernel<T, 1>), dim3(ew_grid(n, 256)), dim3(256), 0, s, x, y, z, g, n, ys);
    D8_LAUNCH_CHECK();
    return 0;
}

// y[b] = sum over i of op(x[b][i]) (then the square root for L2): zero, reduce, finish.
template <typename T, int WIDE, int OP>
static int norm_t(const T *x, T *y, int batch, long size, void *scratch, size_t scratch_bytes, hipStream_t s) {
    const int yd[5] = {batch, 1, 1, 1, 1}, xd[5] = {batch, 1, 1, 1, (int)size};
    hipLaunchKernelGGL((ew_zero_kernel<T>), dim3(ew_grid(batch, 256)), dim3(256), 0, s, y, (long)batch);
    D8_LAUNCH_CHECK();
    if (int rc = reduce_t<T, WIDE, OP>(y, yd, x, xd, scratch, scratch_bytes, s)) return rc;
    if (OP == LOAD_SQUARE) {
        hipLaunchKernelGGL((sqrt_kernel<T>), dim3(ew_grid(batch, 256)), dim3(256), 0, s, y, (long)batch);
        D8_LAUNCH_CHECK();
    }
    return 0;
}

template <typename T, int WIDE, bool L2>
static int norm_grad_t(const T *x, T *dx, const T *y, const T *dy, int batch, long size, hipStream_t s) {
    const long n = (long)batch * size;
    if (size % WIDE == 0 && al16(x) && al16(dx))
        hipLaunchKernelGGL((norm_grad_kernel<T, WIDE, L2>), dim3(ew_grid(n / WIDE, 256)), dim3(256), 0, s, x, dx, y, dy, size / WIDE, n / WIDE);
    else
        hipLaunchKernelGGL((norm_grad_kernel<T, 1, L2>), dim3(ew_grid(n, 256)), dim3(256), 0, s, x, dx, y, dy, size, n);
    D8_LAUNCH_CHECK();
    return 0;
}

static int check_norm(const char *who, int dtype, const void *x, const void *y, int batch, long size) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32) return fail(D8_ERR_DTYPE, "%s: element type %d is not supported", who, dtype);
    D8_REQUIRE(x && y, "%s: null tensor", who);
    D8_REQUIRE(batch >= 1 && size >= 1 && size < (1L << 31), "%s: the shape is error", who);
    return 0;
}

template <typename T, int WIDE>
static int bias_relu_t(T *z, const T *bias, long rows, int cols, int relu, hipStream_t s) {
    const long n = rows * cols;
    if (cols % WIDE == 0 && al16(z) && al16(bias))
        hipLaunchKernelGGL((bias_relu_kernel<T, WIDE>), dim3(ew_grid(n / WIDE, 256)), dim3(256), 0, s, z, bias, n / WIDE, cols / WIDE, relu);
    else
        hipLaunchKernelGGL((bias_relu_kernel<T, 1>), dim3(ew_grid(n, 256)), dim3(256), 0, s, z, bias, n, cols, relu);
    D8_LAUNCH_CHECK();
    return 0;
}

int launch_bias_relu(int dtype, void *z, const void *bias, long rows, int cols, int relu, hipStream_t stream) {
    if (rows <= 0 || cols <= 0 || (!bias && !relu)) return 0;
    if (dtype == D8_FLOAT32) return bias_relu_t<float, 4>((float *)z, (const float *)bias, rows, cols, relu, stream);
    if (dtype == D8_FLOAT16) return bias_relu_t<f16, 8>((f16 *)z, (const f16 *)bias, rows, cols, relu, stream);
    return fail(D8_ERR_DTYPE, "bias / ReLu store: element type %d is not supported", dtype);
}

// dpre = z > 0 ? dz : 0;  g = keep * g + column sums of dpre.  Same plan as reduce_t on a [R][C] tensor.
template <typename T, int WIDE>
static int relu_gate_sum_t(const T *z, const T *dz, T *dpre, T *g, long rows, int cols, void *scratch, size_t scratch_bytes,
                           float keep, hipStream_t s) {
    const int gd[5] = {1, 1, 1, 1, cols}, zd[5] = {1, 1, 1, (int)rows, cols};
    const ReducePlan p = plan_reduce(gd, zd);
    // (a single row has nothing to sum: one chunk, the sums are the row itself)
    int chunks = p.kind == 1 ? p.chunks : 1, rpc = p.kind == 1 ? p.rows_per_chunk : (int)rows;
    const size_t need = (size_t)chunks * cols * sizeof(float);
    if (chunks > 1 && (!scratch || scratch_bytes < need || !al16(scratch))) chunks = 1, rpc = (int)rows;
    const bool wide = cols % WIDE == 0 && al16(g) && al16(dz) && al16(z) && al16(dpre);
    const long cvs = cols / (wide ? WIDE : 1);
    int TX = 1;
    while (TX < 32 && TX < cvs) TX *= 2;
    dim3 grid((unsigned)((cvs + TX - 1) / TX), (unsigned)chunks, 1);
    if (wide)
        hipLaunchKernelGGL((relu_gate_column_sum_kernel<T, WIDE>), grid, dim3(256), 0, s, z, dz, dpre, g, (float *)scratch, (int)rows, cols, TX, rpc, chunks, keep);
    else
        hipLaunchKernelGGL((relu_gate_column_sum_kernel<T, 1>), grid, dim3(256), 0, s, z, dz, dpre, g, (float *)scratch, (int)rows, cols, TX, rpc, chunks, keep);
    D8_LAUNCH_CHECK();
    if (chunks > 1) {
        hipLaunchKernelGGL((column_sum_finish_kernel<T>), dim3((unsigned)((cols + 15) / 16)), dim3(256), 0, s,
                           (const float *)scratch, g, cols, chunks, (long)cols, 1.f, keep);
        D8_LAUNCH_CHECK();
    }
    return 0;
}

}  // namespace d8

using namespace d8;

extern "C" {

size_t d8_bias_relu_grad_scratch_bytes(int dtype, long rows, int cols) {
    if (rows < 1 || cols < 1 || rows >= (1L << 31)) return 0;
    const int gd[5] = {1, 1, 1, 1, cols}, zd[5] = {1, 1, 1, (int)rows, cols};
    return d8_add_grad_scratch_bytes(dtype, gd, zd);
}

int d8_bias_relu_grad(int dtype, const void *z, const void *dz, void *dpre, void *dbias, long rows, int cols,
                      int accumulate_bias, void *scratch, size_t scratch_bytes, void *stream) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32)
        return fail(D8_ERR_DTYPE, "d8_bias_relu_grad: element type %d is not supported", dtype);
    D8_REQUIRE(z && dz && dpre && dbias, "d8_bias_relu_grad: null tensor");
    D8_REQUIRE(rows > 0 && cols > 0 && rows < (1L << 31), "d8_bias_relu_grad: %ld rows x %d columns", rows, cols);
    const float keep = accumulate_bias ? 1.f : 0.f;
    return dtype == D8_FLOAT32
               ? relu_gate_sum_t<float, 4>((const float *)z, (const float *)dz, (float *)dpre, (float *)dbias, rows, cols, scratch, scratch_bytes, keep, as_stream(stream))
               : relu_gate_sum_t<f16, 8>((const f16 *)z, (const f16 *)dz, (f16 *)dpre, (f16 *)dbias, rows, cols, scratch, scratch_bytes, keep, as_stream(stream));
}

int d8_add(int dtype, const void *x, const int *xdims, const void *y, const int *ydims, void *z, const int *zdims,
           void *stream) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32) return fail(D8_ERR_DTYPE, "d8_add: element type %d is not supported", dtype);
    D8_REQUIRE(x && y && z && xdims && ydims && zdims, "d8_add: null argument");
    if (int rc = check_dims("d8_add", xdims, zdims)) return rc;
    if (int rc = check_dims("d8_add", ydims, zdims)) return rc;
    for (int a = 0; a < 5; ++a)
        D8_REQUIRE(zdims[a] == (xdims[a] > ydims[a] ? xdims[a] : ydims[a]), "d8_add: the shape is error (axis %d)", a);
    return dtype == D8_FLOAT32 ? add_t<float, 4>((const float *)x, xdims, (const float *)y, ydims, (float *)z, zdims, as_stream(stream))
                               : add_t<f16, 8>((const f16 *)x, xdims, (const f16 *)y, ydims, (f16 *)z, zdims, as_stream(stream));
}

size_t d8_add_grad_scratch_bytes(int dtype, const int *gdims, const int *zdims) {
    (void)dtype;
    if (!gdims || !zdims) return 0;
    for (int a = 0; a < 5; ++a)
        if (gdims[a] < 1 || zdims[a] < 1 || (gdims[a] != 1 && gdims[a] != zdims[a])) return 0;
    const ReducePlan p = plan_reduce(gdims, zdims);
    return p.kind == 1 && p.chunks > 1 ? (size_t)p.K0 * p.chunks * p.C * sizeof(float) : 0;
}

static int add_grad_impl(int dtype, void *g, const int *gdims, const void *dz, const int *zdims,
                         void *scratch, size_t scratch_bytes, void *stream, float keep) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32)
        return fail(D8_ERR_DTYPE, "d8_add_grad: element type %d is not supported", dtype);
    D8_REQUIRE(g && dz && gdims && zdims, "d8_add_grad: null argument");
    if (int rc = check_dims("d8_add_grad", gdims, zdims)) return rc;
    return dtype == D8_FLOAT32
               ? reduce_t<float, 4>((float *)g, gdims, (const float *)dz, zdims, scratch, scratch_bytes, as_stream(stream), 1.f, keep)
               : reduce_t<f16, 8>((f16 *)g, gdims, (const f16 *)dz, zdims, scratch, scratch_bytes, as_stream(stream), 1.f, keep);
}

int d8_add_grad(int dtype, void *g, const int *gdims, const void *dz, const int *zdims,
                void *scratch, size_t scratch_bytes, void *stream) {
    return add_grad_impl(dtype, g, gdims, dz, zdims, scratch, scratch_bytes, stream, 1.f);
}

int d8_add_grad_overwrite(int dtype, void *g, const int *gdims, const void *dz, const int *zdims,
                          void *scratch, size_t scratch_bytes, void *stream) {
    return add_grad_impl(dtype, g, gdims, dz, zdims, scratch, scratch_bytes, stream, 0.f);
}

int d8_relu(int dtype, const void *x, void *y, long n, void *stream) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32) return fail(D8_ERR_DTYPE, "d8_relu: element type %d is not supported", dtype);
    D8_REQUIRE(n >= 0, "d8_relu: negative size");
    if (n == 0) return 0;
    D8_REQUIRE(x && y, "d8_relu: null tensor");
    hipStream_t s = as_stream(stream);
    const bool al = al16(x) && al16(y);
    if (dtype == D8_FLOAT32) {
        if (al && n % 4 == 0) hipLaunchKernelGGL((relu_kernel<float, 4>), dim3(ew_grid(n / 4, 256)), dim3(256), 0, s, (const float *)x, (float *)y, n / 4);
        else hipLaunchKernelGGL((relu_kernel<float, 1>), dim3(ew_grid(n, 256)), dim3(256), 0, s, (const float *)x, (float *)y, n);
    } else {
        if (al && n % 8 == 0) hipLaunchKernelGGL((relu_kernel<f16, 8>), dim3(ew_grid(n / 8, 256)), dim3(256), 0, s, (const f16 *)x, (f16 *)y, n / 8);
        else hipLaunchKernelGGL((relu_kernel<f16, 1>), dim3(ew_grid(n, 256)), dim3(256), 0, s, (const f16 *)x, (f16 *)y, n);
    }
    D8_LAUNCH_CHECK();
    return 0;
}

static int relu_grad_impl(int dtype, const void *x, void *dx, const void *dy, long n, void *stream, float keep) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32)
        return fail(D8_ERR_DTYPE, "d8_relu_grad: element type %d is not supported", dtype);
    D8_REQUIRE(n >= 0, "d8_relu_grad: negative size");
    if (n == 0) return 0;
    D8_REQUIRE(x && dx && dy, "d8_relu_grad: null tensor");
    hipStream_t s = as_stream(stream);
    const bool al = al16(x) && al16(dx) && al16(dy);
    if (dtype == D8_FLOAT32) {
        if (al && n % 4 == 0) hipLaunchKernelGGL((relu_grad_kernel<float, 4>), dim3(ew_grid(n / 4, 256)), dim3(256), 0, s, (const float *)x, (float *)dx, (const float *)dy, n / 4, keep);
        else hipLaunchKernelGGL((relu_grad_kernel<float, 1>), dim3(ew_grid(n, 256)), dim3(256), 0, s, (const float *)x, (float *)dx, (const float *)dy, n, keep);
    } else {
        if (al && n % 8 == 0) hipLaunchKernelGGL((relu_grad_kernel<f16, 8>), dim3(ew_grid(n / 8, 256)), dim3(256), 0, s, (const f16 *)x, (f16 *)dx, (const f16 *)dy, n / 8, keep);
        else hipLaunchKernelGGL((relu_grad_kernel<f16, 1>), dim3(ew_grid(n, 256)), dim3(256), 0, s, (const f16 *)x, (f16 *)dx, (const f16 *)dy, n, keep);
    }
    D8_LAUNCH_CHECK();
    return 0;
}

int d8_relu_grad(int dtype, const void *x, void *dx, const void *dy, long n, void *stream) {
    return relu_grad_impl(dtype, x, dx, dy, n, stream, 1.f);
}

int d8_relu_grad_overwrite(int dtype, const void *x, void *dx, const void *dy, long n, void *stream) {
    return relu_grad_impl(dtype, x, dx, dy, n, stream, 0.f);
}

int d8_minus(int dtype, const void *x, const int *xdims, const void *y, const int *ydims, void *z, const int *zdims,
             void *stream) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32) return fail(D8_ERR_DTYPE, "d8_minus: element type %d is not supported", dtype);
    D8_REQUIRE(x && y && z && xdims && ydims && zdims, "d8_minus: null argument");
    if (int rc = check_dims("d8_minus", xdims, zdims)) return rc;
    if (int rc = check_dims("d8_minus", ydims, zdims)) return rc;
    for (int a = 0; a < 5; ++a)
        D8_REQUIRE(zdims[a] == (xdims[a] > ydims[a] ? xdims[a] : ydims[a]), "d8_minus: the shape is error (axis %d)", a);
    return dtype == D8_FLOAT32
               ? add_t<float, 4>((const float *)x, xdims, (const float *)y, ydims, (float *)z, zdims, as_stream(stream), -1.f)
               : add_t<f16, 8>((const f16 *)x, xdims, (const f16 *)y, ydims, (f16 *)z, zdims, as_stream(stream), -1.f);
}

int d8_minus_grad_y(int dtype, void *g, const int *gdims, const void *dz, const int *zdims,
                    void *scratch, size_t scratch_bytes, void *stream) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32)
        return fail(D8_ERR_DTYPE, "d8_minus_grad_y: element type %d is not supported", dtype);
    D8_REQUIRE(g && dz && gdims && zdims, "d8_minus_grad_y: null argument");
    if (int rc = check_dims("d8_minus_grad_y", gdims, zdims)) return rc;
    return dtype == D8_FLOAT32
               ? reduce_t<float, 4>((float *)g, gdims, (const float *)dz, zdims, scratch, scratch_bytes, as_stream(stream), -1.f)
               : reduce_t<f16, 8>((f16 *)g, gdims, (const f16 *)dz, zdims, scratch, scratch_bytes, as_stream(stream), -1.f);
}

int d8_l1norm(int dtype, const void *x, void *y, int batch, long size, void *scratch, size_t scratch_bytes, void *stream) {
    if (int rc = check_norm("d8_l1norm", dtype, x, y, batch, size)) return rc;
    return dtype == D8_FLOAT32
               ? norm_t<float, 4, LOAD_ABS>((const float *)x, (float *)y, batch, size, scratch, scratch_bytes, as_stream(stream))
               : norm_t<f16, 8, LOAD_ABS>((const f16 *)x, (f16 *)y, batch, size, scratch, scratch_bytes, as_stream(stream));
}

int d8_l1norm_grad(int dtype, const void *x, void *dx, const void *dy, int batch, long size, void *stream) {
    if (int rc = check_norm("d8_l1norm_grad", dtype, x, dx, batch, size)) return rc;
    D8_REQUIRE(dy, "d8_l1norm_grad: null tensor");
    return dtype == D8_FLOAT32
               ? norm_grad_t<float, 4, false>((const float *)x, (float *)dx, (const float *)dy, (const float *)dy, batch, size, as_stream(stream))
               : norm_grad_t<f16, 8, false>((const f16 *)x, (f16 *)dx, (const f16 *)dy, (const f16 *)dy, batch, size, as_stream(stream));
}

int d8_l2norm(int dtype, const void *x, void *y, int batch, long size, void *scratch, size_t scratch_bytes, void *stream) {
    if (int rc = check_norm("d8_l2norm", dtype, x, y, batch, size)) return rc;
    return dtype == D8_FLOAT32
               ? norm_t<float, 4, LOAD_SQUARE>((const float *)x, (float *)y, batch, size, scratch, scratch_bytes, as_stream(stream))
               : norm_t<f16, 8, LOAD_SQUARE>((const f16 *)x, (f16 *)y, batch, size, scratch, scratch_bytes, as_stream(stream));
}

int d8_l2norm_grad(int dtype, const void *x, void *dx, const void *y, const void *dy, int batch, long size, void *stream) {
    if (int rc = check_norm("d8_l2norm_grad", dtype, x, dx, batch, size)) return rc;
    D8_REQUIRE(y && dy, "d8_l2norm_grad: null tensor");
    return dtype == D8_FLOAT32
               ? norm_grad_t<float, 4, true>((const float *)x, (float *)dx, (const float *)y, (const float *)dy, batch, size, as_stream(stream))
               : norm_grad_t<f16, 8, true>((const f16 *)x, (f16 *)dx, (const f16 *)y, (const f16 *)dy, batch, size, as_stream(stream));
}

static int mean_count(const char *who, const int *xdims, const int *ydims, double *count) {
    if (int rc = check_dims(who, ydims, xdims)) return rc;
    *count = (double)prod5(xdims) / (double)prod5(ydims);
    return 0;
}

int d8_reduce_mean(int dtype, const void *x, const int *xdims, void *y, const int *ydims,
                   void *scratch, size_t scratch_bytes, void *stream) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32)
        return fail(D8_ERR_DTYPE, "d8_reduce_mean: element type %d is not supported", dtype);
    D8_REQUIRE(x && y && xdims && ydims, "d8_reduce_mean: null argument");
    double count = 1;
    if (int rc = mean_count("d8_reduce_mean", xdims, ydims, &count)) return rc;
    hipStream_t s = as_stream(stream);
    const long ny = prod5(ydims);
    const float scale = (float)(1.0 / count);
    if (dtype == D8_FLOAT32) {
        hipLaunchKernelGGL((ew_zero_kernel<float>), dim3(ew_grid(ny, 256)), dim3(256), 0, s, (float *)y, ny);
        D8_LAUNCH_CHECK();
        return reduce_t<float, 4>((float *)y, ydims, (const float *)x, xdims, scratch, scratch_bytes, s, scale);
    }
    hipLaunchKernelGGL((ew_zero_kernel<f16>), dim3(ew_grid(ny, 256)), dim3(256), 0, s, (f16 *)y, ny);
    D8_LAUNCH_CHECK();
    return reduce_t<f16, 8>((f16 *)y, ydims, (const f16 *)x, xdims, scratch, scratch_bytes, s, scale);
}

int d8_reduce_mean_grad(int dtype, void *dx, const int *xdims, const void *dy, const int *ydims, void *stream) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32)
        return fail(D8_ERR_DTYPE, "d8_reduce_mean_grad: element type %d is not supported", dtype);
    D8_REQUIRE(dx && dy && xdims && ydims, "d8_reduce_mean_grad: null argument");
    double count = 1;
    if (int rc = mean_count("d8_reduce_mean_grad", xdims, ydims, &count)) return rc;
    const float ys = (float)(1.0 / count);
    return dtype == D8_FLOAT32
               ? add_t<float, 4>((const float *)dx, xdims, (const float *)dy, ydims, (float *)dx, xdims, as_stream(stream), ys)
               : add_t<f16, 8>((const f16 *)dx, xdims, (const f16 *)dy, ydims, (f16 *)dx, xdims, as_stream(stream), ys);
}

int d8_axpby(int dtype, const void *x, float alpha, const void *y, float beta, void *z, long n, void *stream) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32) return fail(D8_ERR_DTYPE, "d8_axpby: element type %d is not supported", dtype);
    D8_REQUIRE(n >= 0, "d8_axpby: negative size");
    if (n == 0) return 0;
    D8_REQUIRE(x && y && z, "d8_axpby: null tensor");
    hipStream_t s = as_stream(stream);
    const bool al = al16(x) && al16(y) && al16(z);
    if (dtype == D8_FLOAT32) {
        if (al && n % 4 == 0) hipLaunchKernelGGL((axpby_kernel<float, 4>), dim3(ew_grid(n / 4, 256)), dim3(256), 0, s, (const float *)x, alpha, (const float *)y, beta, (float *)z, n / 4);
        else hipLaunchKernelGGL((axpby_kernel<float, 1>), dim3(ew_grid(n, 256)), dim3(256), 0, s, (const float *)x, alpha, (const float *)y, beta, (float *)z, n);
    } else {
        if (al && n % 8 == 0) hipLaunchKernelGGL((axpby_kernel<f16, 8>), dim3(ew_grid(n / 8, 256)), dim3(256), 0, s, (const f16 *)x, alpha, (const f16 *)y, beta, (f16 *)z, n / 8);
        else hipLaunchKernelGGL((axpby_kernel<f16, 1>), dim3(ew_grid(n, 256)), dim3(256), 0, s, (const f16 *)x, alpha, (const f16 *)y, beta, (f16 *)z, n);
    }
    D8_LAUNCH_CHECK();
    return 0;
}

int d8_adam_update(int dtype, void *value, void *gradient, void *m, void *v, float beta1, float beta2, float epsilon,
                   float learning_rate, float weight_decay, long steps, long n, void *stream) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32)
        return fail(D8_ERR_DTYPE, "d8_adam_update: element type %d is not supported", dtype);
    D8_REQUIRE(n >= 0, "d8_adam_update: negative size");
    if (n == 0) return 0;
    D8_REQUIRE(value && gradient && m && v, "d8_adam_update: null tensor");
    if (steps <= 0) steps = 1;  // avoid a division by zero (deep8/src/math/AdamUpdate.cpp:11-14)
    const float ratio = learning_rate * sqrtf(1.0f - powf(beta2, (float)steps)) / (1.0f - powf(beta1, (float)steps));
    hipStream_t s = as_stream(stream);
    const bool al = al16(value) && al16(gradient) && al16(m) && al16(v);
    if (dtype == D8_FLOAT32) {
        if (al && n % 4 == 0) hipLaunchKernelGGL((adam_kernel<float, 4>), dim3(ew_grid(n / 4, 256)), dim3(256), 0, s, (float *)value, (float *)gradient, (float *)m, (float *)v, beta1, beta2, epsilon, weight_decay, ratio, n / 4);
        else hipLaunchKernelGGL((adam_kernel<float, 1>), dim3(ew_grid(n, 256)), dim3(256), 0, s, (float *)value, (float *)gradient, (float *)m, (float *)v, beta1, beta2, epsilon, weight_decay, ratio, n);
    } else {
        if (al && n % 8 == 0) hipLaunchKernelGGL((adam_kernel<f16, 8>), dim3(ew_grid(n / 8, 256)), dim3(256), 0, s, (f16 *)value, (f16 *)gradient, (f16 *)m, (f16 *)v, beta1, beta2, epsilon, weight_decay, ratio, n / 8);
        else hipLaunchKernelGGL((adam_kernel<f16, 1>), dim3(ew_grid(n, 256)), dim3(256), 0, s, (f16 *)value, (f16 *)gradient, (f16 *)m, (f16 *)v, beta1, beta2, epsilon, weight_decay, ratio, n);
    }
    D8_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
