// MaxPooling2d and AvgPooling2d, forward and gradients, NHWC.  All four are gathers with one write
// per destination element (no atomics): HBM-bandwidth bound, 16-byte accesses along the channels.
//
// Semantics are those of Deep8's CPU path:
//   * forward (deep8/src/math/MaxPooling2d.cpp:99-142, AvgPooling2d.cpp:99-142): the window is cut
//     from the image padded with ZEROS (extract_image_patches(..., padding value 0)), so a window that
//     sticks out of the image takes part of its maximum / mean from zeros; the mean divides by the
//     full window size;
//   * MaxPooling2dGrad (MaxPooling2d.cpp:199-251): dy goes to the first maximum (row-major scan,
//     strict >) of the window CLIPPED to the image -- padding plays no part here;
//   * AvgPooling2dGrad (AvgPooling2d.cpp:199-245): every in-image element of the window receives
//     dy / (FH * FW).
// The reference's GPU path calls cuDNN for max pooling (deep8/src/math/MaxPooling2d.cu:41-147),
// whose padding behaves differently; the CPU path is the one the checker restates.
#include "common.h"

namespace d8 {

__device__ inline float pool_f32(float v) { return v; }
__device__ inline float pool_f32(f16 v) { return (float)v; }

struct PoolGeom {
    int B, IH, IW, C, OH, OW, FH, FW, sy, sx, pt, pl;
};

static inline int pool_grid(long work) {
    long blocks = (work + 255) / 256;
    const long cap = (long)cu_count() * 32;
    if (blocks > cap) blocks = cap;
    return (int)(blocks < 1 ? 1 : blocks);
}

template <typename T, int VEC, bool MAX>
__global__ __launch_bounds__(256) void pool_forward_kernel(const T *__restrict__ x, T *__restrict__ y, PoolGeom g, long total) {
    typedef T VT __attribute__((ext_vector_type(VEC)));
    const int cv = g.C / VEC;
    const float inv = 1.0f / ((float)g.FH * (float)g.FW);
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const int c = (int)(idx % cv) * VEC;
        long p = idx / cv;
        const int ow = (int)(p % g.OW);
        p /= g.OW;
        const int oh = (int)(p % g.OH), b = (int)(p / g.OH);
        float acc[VEC];
        bool first = true;
        for (int fh = 0; fh < g.FH; ++fh) {
            const int ih = oh * g.sy + fh - g.pt;
            for (int fw = 0; fw < g.FW; ++fw) {
                const int iw = ow * g.sx + fw - g.pl;
                float v[VEC];
                if (ih >= 0 && ih < g.IH && iw >= 0 && iw < g.IW) {
                    const VT t = *(const VT *)(x + (((long)b * g.IH + ih) * g.IW + iw) * g.C + c);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) v[e] = pool_f32(t[e]);
                } else {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) v[e] = 0.f;
                }
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[e] = first ? v[e] : (MAX ? fmaxf(acc[e], v[e]) : acc[e] + v[e]);
                first = false;
            }
        }
        VT o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) o[e] = (T)(MAX ? acc[e] : acc[e] * inv);
        *(VT *)(y + idx * VEC) = o;
    }
}

// dx[b][ih][iw][c] += sum over the windows (oh, ow) that contain (ih, iw) of
//   MAX: dy[oh][ow][c] if (ih, iw) is the first maximum of the clipped window, else 0
//   AVG: dy[oh][ow][c] / (FH * FW)
template <typename T, int VEC, bool MAX>
__global__ __launch_bounds__(256) void pool_backward_kernel(const T *__restrict__ x, T *__restrict__ dx, const T *__restrict__ dy,
                                                            PoolGeom g, long total, float keep) {
    typedef T VT __attribute__((ext_vector_type(VEC)));
    const int cv = g.C / VEC;
    const float inv = 1.0f / ((float)g.FH * (float)g.FW);
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const int c = (int)(idx % cv) * VEC;
        long p = idx / cv;
        const int iw = (int)(p % g.IW);
        p /= g.IW;
        const int ih = (int)(p % g.IH), b = (int)(p / g.IH);
        // windows containing the element: oh * sy - pt <= ih < oh * sy - pt + FH
        int oh0 = ih + g.pt - g.FH + 1;
        oh0 = oh0 <= 0 ? 0 : (oh0 + g.sy - 1) / g.sy;
        int ow0 = iw + g.pl - g.FW + 1;
        ow0 = ow0 <= 0 ? 0 : (ow0 + g.sx - 1) / g.sx;
        const int oh1 = min(g.OH - 1, (ih + g.pt) / g.sy), ow1 = min(g.OW - 1, (iw + g.pl) / g.sx);
        const T *xb = x + (long)b * g.IH * g.IW * g.C + c;
        float acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
        float mine[VEC];
        if (MAX) {
            const VT t = *(const VT *)(xb + ((long)ih * g.IW + iw) * g.C);
#pragma unroll
            for (int e = 0; e < VEC; ++e) mine[e] = pool_f32(t[e]);
        }
        for (int oh = oh0; oh <= oh1; ++oh)
            for (int ow = ow0; ow <= ow1; ++ow) {
                const VT d = *(const VT *)(dy + (((long)b * g.OH + oh) * g.OW + ow) * g.C + c);
                if (!MAX) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc[e] += pool_f32(d[e]) * inv;
                    continue;
                }
                // this element wins the window iff nothing before it (scan order) is >= it and
                // nothing after it is > it
                const int h0 = max(0, oh * g.sy - g.pt), h1 = min(g.IH, oh * g.sy - g.pt + g.FH);
                const int w0 = max(0, ow * g.sx - g.pl), w1 = min(g.IW, ow * g.sx - g.pl + g.FW);
                bool win[VEC];
#pragma unroll
                for (int e = 0; e < VEC; ++e) win[e] = true;
                for (int h = h0; h < h1; ++h)
                    for (int w = w0; w < w1; ++w) {
                        if (h == ih && w == iw) continue;
                        const bool before = h < ih || (h == ih && w < iw);
                        const VT t = *(const VT *)(xb + ((long)h * g.IW + w) * g.C);
#pragma unroll
                        for (int e = 0; e < VEC; ++e) {
                            const float o = pool_f32(t[e]);
                            if (before ? !(mine[e] > o) : (o > mine[e])) win[e] = false;
                        }
                    }
#pragma unroll
                for (int e = 0; e < VEC; ++e)
                    if (win[e]) acc[e] += pool_f32(d[e]);
            }
        VT o;  // keep = 1: added to what dx holds (the reference's accumulate); 0: dx's old contents are not read
#pragma unroll
        for (int e = 0; e < VEC; ++e) o[e] = (T)0;
        if (keep != 0.f) o = *(const VT *)(dx + idx * VEC);
#pragma unroll
        for (int e = 0; e < VEC; ++e) o[e] = (T)(pool_f32(o[e]) + acc[e]);
        *(VT *)(dx + idx * VEC) = o;
    }
}

// The same gradients when the windows do not overlap (stride >= filter in both directions, the usual
// 2x2 / 2 pooling): a thread per window and channel vector reads the window once, finds the first
// maximum exactly as the reference scans for it (start from the first element of the clipped window,
// replace on strict >, deep8/src/math/MaxPooling2d.cpp:228-243), reads dy once and writes the stride
// cell the window sits in -- the image is cut into OH x OW cells, cell (oh, ow) starting where window
// (oh, ow) starts and the border cells reaching the image's edges, so that every element of dx is
// written by exactly one thread.  Elements of a cell outside its window receive nothing: untouched
// with keep = 1, zero with keep = 0.  Every tensor is read or written once.
template <typename T, int VEC, bool MAX>
__global__ __launch_bounds__(256) void pool_backward_cells_kernel(const T *__restrict__ x, T *__restrict__ dx,
                                                                  const T *__restrict__ dy, PoolGeom g, long total, float keep) {
    typedef T VT __attribute__((ext_vector_type(VEC)));
    const int cv = g.C / VEC;
    const float inv = 1.0f / ((float)g.FH * (float)g.FW);
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const int c = (int)(idx % cv) * VEC;
        long p = idx / cv;
        const int ow = (int)(p % g.OW);
        p /= g.OW;
        const int oh = (int)(p % g.OH), b = (int)(p / g.OH);
        const int wh0 = max(0, oh * g.sy - g.pt), wh1 = min(g.IH, oh * g.sy - g.pt + g.FH);
        const int ww0 = max(0, ow * g.sx - g.pl), ww1 = min(g.IW, ow * g.sx - g.pl + g.FW);
        const int ch0 = oh == 0 ? 0 : oh * g.sy - g.pt, ch1 = oh == g.OH - 1 ? g.IH : (oh + 1) * g.sy - g.pt;
        const int cw0 = ow == 0 ? 0 : ow * g.sx - g.pl, cw1 = ow == g.OW - 1 ? g.IW : (ow + 1) * g.sx - g.pl;
        const long img = (long)b * g.IH * g.IW * g.C + c;
        const VT d = *(const VT *)(dy + idx * VEC);
        int pos[VEC];  // h * IW + w of the winner, per channel
        if (MAX) {
            float best[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) best[e] = 0.f, pos[e] = -1;
            bool first = true;
            for (int h = wh0; h < wh1; ++h)
                for (int w = ww0; w < ww1; ++w) {
                    const VT t = *(const VT *)(x + img + ((long)h * g.IW + w) * g.C);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const float v = pool_f32(t[e]);
                        if (first || v > best[e]) best[e] = v, pos[e] = h * g.IW + w;
                    }
                    first = false;
                }
        }
        for (int h = ch0; h < ch1; ++h)
            for (int w = cw0; w < cw1; ++w) {
                const bool inwin = h >= wh0 && h < wh1 && w >= ww0 && w < ww1;
                if (!inwin && keep != 0.f) continue;
                T *q = dx + img + ((long)h * g.IW + w) * g.C;
                VT o;
#pragma unroll
                for (int e = 0; e < VEC; ++e) o[e] = (T)0;
                if (keep != 0.f) o = *(const VT *)q;
                if (inwin) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const float add = MAX ? (pos[e] == h * g.IW + w ? pool_f32(d[e]) : 0.f) : pool_f32(d[e]) * inv;
                        o[e] = (T)(pool_f32(o[e]) + add);
                    }
                }
                *(VT *)q = o;
            }
    }
}

static int pool_geometry(const char *who, int dtype, int B, int IH, int IW, int C, int FH, int FW, int covered, int sy, int sx,
                         PoolGeom &g) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32) return fail(D8_ERR_DTYPE, "%s: element type %d is not supported", who, dtype);
    D8_REQUIRE(B > 0 && IH > 0 && IW > 0 && C > 0, "%s: sizes must be positive", who);
    D8_REQUIRE(FH >= 1 && FW >= 1 && sy >= 1 && sx >= 1, "%s: the params is error", who);
    int geo[4];
    if (int rc = d8_conv2d_geometry(IH, IW, FH, FW, covered, sy, sx, 1, 1, geo)) return rc;
    D8_REQUIRE(geo[0] >= 1 && geo[1] >= 1, "%s: the shape is error", who);
    g = {B, IH, IW, C, geo[0], geo[1], FH, FW, sy, sx, geo[2], geo[3]};
    return 0;
}

template <bool MAX>
static int pool_forward(int dtype, const void *x, void *y, const PoolGeom &g, hipStream_t s) {
    const long pixels = (long)g.B * g.OH * g.OW;
    const bool al = (((size_t)x | (size_t)y) & 15) == 0;
    if (dtype == D8_FLOAT32) {
        if (al && g.C % 4 == 0) hipLaunchKernelGGL((pool_forward_kernel<float, 4, MAX>), dim3(pool_grid(pixels * g.C / 4)), dim3(256), 0, s, (const float *)x, (float *)y, g, pixels * g.C / 4);
        else hipLaunchKernelGGL((pool_forward_kernel<float, 1, MAX>), dim3(pool_grid(pixels * g.C)), dim3(256), 0, s, (const float *)x, (float *)y, g, pixels * g.C);
    } else {
        if (al && g.C % 8 == 0) hipLaunchKernelGGL((pool_forward_kernel<f16, 8, MAX>), dim3(pool_grid(pixels * g.C / 8)), dim3(256), 0, s, (const f16 *)x, (f16 *)y, g, pixels * g.C / 8);
        else hipLaunchKernelGGL((pool_forward_kernel<f16, 1, MAX>), dim3(pool_grid(pixels * g.C)), dim3(256), 0, s, (const f16 *)x, (f16 *)y, g, pixels * g.C);
    }
    D8_LAUNCH_CHECK();
    return 0;
}

template <bool MAX>
static int pool_backward(int dtype, const void *x, void *dx, const void *dy, const PoolGeom &g, hipStream_t s, float keep) {
    const long pixels = (long)g.B * g.IH * g.IW;
    const bool al = (((size_t)x | (size_t)dx | (size_t)dy) & 15) == 0;
    // windows that do not overlap, and an image that fits the cell kernel's 32-bit pixel index
    if (g.sy >= g.FH && g.sx >= g.FW && g.pt < g.sy && g.pl < g.sx && (long)g.IH * g.IW < (1L << 31)) {
        const long wins = (long)g.B * g.OH * g.OW;
        if (dtype == D8_FLOAT32) {
            if (al && g.C % 4 == 0) hipLaunchKernelGGL((pool_backward_cells_kernel<float, 4, MAX>), dim3(pool_grid(wins * g.C / 4)), dim3(256), 0, s, (const float *)x, (float *)dx, (const float *)dy, g, wins * g.C / 4, keep);
            else hipLaunchKernelGGL((pool_backward_cells_kernel<float, 1, MAX>), dim3(pool_grid(wins * g.C)), dim3(256), 0, s, (const float *)x, (float *)dx, (const float *)dy, g, wins * g.C, keep);
        } else {
            if (al && g.C % 8 == 0) hipLaunchKernelGGL((pool_backward_cells_kernel<f16, 8, MAX>), dim3(pool_grid(wins * g.C / 8)), dim3(256), 0, s, (const f16 *)x, (f16 *)dx, (const f16 *)dy, g, wins * g.C / 8, keep);
            else hipLaunchKernelGGL((pool_backward_cells_kernel<f16, 1, MAX>), dim3(pool_grid(wins * g.C)), dim3(256), 0, s, (const f16 *)x, (f16 *)dx, (const f16 *)dy, g, wins * g.C, keep);
        }
        D8_LAUNCH_CHECK();
        return 0;
    }
    if (dtype == D8_FLOAT32) {
        if (al && g.C % 4 == 0) hipLaunchKernelGGL((pool_backward_kernel<float, 4, MAX>), dim3(pool_grid(pixels * g.C / 4)), dim3(256), 0, s, (const float *)x, (float *)dx, (const float *)dy, g, pixels * g.C / 4, keep);
        else hipLaunchKernelGGL((pool_backward_kernel<float, 1, MAX>), dim3(pool_grid(pixels * g.C)), dim3(256), 0, s, (const float *)x, (float *)dx, (const float *)dy, g, pixels * g.C, keep);
    } else {
        if (al && g.C % 8 == 0) hipLaunchKernelGGL((pool_backward_kernel<f16, 8, MAX>), dim3(pool_grid(pixels * g.C / 8)), dim3(256), 0, s, (const f16 *)x, (f16 *)dx, (const f16 *)dy, g, pixels * g.C / 8, keep);
        else hipLaunchKernelGGL((pool_backward_kernel<f16, 1, MAX>), dim3(pool_grid(pixels * g.C)), dim3(256), 0, s, (const f16 *)x, (f16 *)dx, (const f16 *)dy, g, pixels * g.C, keep);
    }
    D8_LAUNCH_CHECK();
    return 0;
}

}  // namespace d8

using namespace d8;

extern "C" {

int d8_maxpool2d(int dtype, const void *x, void *y, int B, int IH, int IW, int C, int FH, int FW, int covered, int sy, int sx,
                 void *stream) {
    PoolGeom g;
    if (int rc = pool_geometry("d8_maxpool2d", dtype, B, IH, IW, C, FH, FW, covered, sy, sx, g)) return rc;
    D8_REQUIRE(x && y, "d8_maxpool2d: null tensor");
    return pool_forward<true>(dtype, x, y, g, as_stream(stream));
}

int d8_maxpool2d_grad(int dtype, const void *x, void *dx, const void *dy, int B, int IH, int IW, int C, int FH, int FW,
                      int covered, int sy, int sx, void *stream) {
    PoolGeom g;
    if (int rc = pool_geometry("d8_maxpool2d_grad", dtype, B, IH, IW, C, FH, FW, covered, sy, sx, g)) return rc;
    D8_REQUIRE(x && dx && dy, "d8_maxpool2d_grad: null tensor");
    return pool_backward<true>(dtype, x, dx, dy, g, as_stream(stream), 1.f);
}

int d8_maxpool2d_grad_overwrite(int dtype, const void *x, void *dx, const void *dy, int B, int IH, int IW, int C, int FH, int FW,
                                int covered, int sy, int sx, void *stream) {
    PoolGeom g;
    if (int rc = pool_geometry("d8_maxpool2d_grad_overwrite", dtype, B, IH, IW, C, FH, FW, covered, sy, sx, g)) return rc;
    D8_REQUIRE(x && dx && dy, "d8_maxpool2d_grad_overwrite: null tensor");
    return pool_backward<true>(dtype, x, dx, dy, g, as_stream(stream), 0.f);
}

int d8_avgpool2d(int dtype, const void *x, void *y, int B, int IH, int IW, int C, int FH, int FW, int covered, int sy, int sx,
                 void *stream) {
    PoolGeom g;
    if (int rc = pool_geometry("d8_avgpool2d", dtype, B, IH, IW, C, FH, FW, covered, sy, sx, g)) return rc;
    D8_REQUIRE(x && y, "d8_avgpool2d: null tensor");
    return pool_forward<false>(dtype, x, y, g, as_stream(stream));
}

int d8_avgpool2d_grad(int dtype, void *dx, const void *dy, int B, int IH, int IW, int C, int FH, int FW, int covered, int sy,
                      int sx, void *stream) {
    PoolGeom g;
    if (int rc = pool_geometry("d8_avgpool2d_grad", dtype, B, IH, IW, C, FH, FW, covered, sy, sx, g)) return rc;
    D8_REQUIRE(dx && dy, "d8_avgpool2d_grad: null tensor");
    return pool_backward<false>(dtype, dx, dx, dy, g, as_stream(stream), 1.f);
}

int d8_avgpool2d_grad_overwrite(int dtype, void *dx, const void *dy, int B, int IH, int IW, int C, int FH, int FW, int covered,
                                int sy, int sx, void *stream) {
    PoolGeom g;
    if (int rc = pool_geometry("d8_avgpool2d_grad_overwrite", dtype, B, IH, IW, C, FH, FW, covered, sy, sx, g)) return rc;
    D8_REQUIRE(dx && dy, "d8_avgpool2d_grad_overwrite: null tensor");
    return pool_backward<false>(dtype, dx, dx, dy, g, as_stream(stream), 0.f);
}

}  // extern "C"
