// The four gather maps behind Conv2d / DeConv2d: im2col, col2im, and DeConv2d's col2im / im2col.
// All are HBM-bandwidth bound; every output element is written exactly once, every launch is a
// grid-stride loop over 16-byte vectors along the contiguous axis wherever the geometry allows.
//
// Replaces Conv2dIm2ColKernel / Conv2dCol2ImKernel (deep8/src/math/Conv2d.cu:10-118) and
// DeConv2dCol2ImKernel / DeConv2dIm2ColKernel (deep8/src/math/DeConv2d.cu:11-58,310-351).
#include "conv_maps.h"

namespace d8 {

static inline int grid_for(long work, int block) {
    long blocks = (work + block - 1) / block;
    const long cap = (long)cu_count() * 32;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return (int)blocks;
}

// ---- im2col: pure copy, V is the raw vector moved per thread (bit-exact) -------------------
// Sums are carried in fp32 for half and float images, in fp64 for double ones.
template <typename T>
struct Wide {
    typedef float type;
};
template <>
struct Wide<double> {
    typedef double type;
};

template <typename V>
__global__ __launch_bounds__(256) void im2col_kernel(const V *__restrict__ im, V *__restrict__ col,
                                                     MapGeom g, int CV, long total) {
    const int taps = g.FH * g.FW;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int cv = (int)(idx % CV);
        const long t = idx / CV;
        const int tap = (int)(t % taps);
        const long r = t / taps;
        const int fx = tap % g.FW, fy = tap / g.FW;
        const int ox = (int)(r % g.OW);
        const long q = r / g.OW;
        const int oy = (int)(q % g.OH), b = (int)(q / g.OH);
        const int iy = oy * g.sy + fy * g.dy - g.pt;
        const int ix = ox * g.sx + fx * g.dx - g.pl;
        V v;
        memset(&v, 0, sizeof(V));
        if (iy >= 0 && iy < g.IH && ix >= 0 && ix < g.IW)
            v = im[(((long)b * g.IH + iy) * g.IW + ix) * CV + cv];
        col[idx] = v;
    }
}

// Division of a number below 2^31 by a runtime constant as a multiply-high, an add and a shift (the round-up
// method: with s = ceil(log2 d) and m = floor(2^32 (2^s - d) / d) + 1, n / d = (mulhi(n, m) + n) >> s).
struct FastDiv {
    unsigned m;
    int s;
};
static FastDiv fast_div(unsigned d) {
    int s = 0;
    while ((1ull << s) < d) ++s;
    return FastDiv{(unsigned)((((1ull << s) - d) << 32) / d + 1), s};
}
__device__ __forceinline__ unsigned div_by(unsigned n, FastDiv d) { return (__umulhi(n, d.m) + n) >> d.s; }

typedef unsigned u32x4v __attribute__((ext_vector_type(4)));

// im2col in 16-byte pieces for the common case (channel rows that are multiples of 16 bytes, fewer than 2^31
// patch rows).  A workgroup owns `rows_per_block` consecutive patch rows, i.e. one contiguous stretch of col,
// and walks it 256 pieces at a time, four stretches per round: four image reads in flight per thread, then
// four stores.  All index arithmetic is 32-bit, with the divisions by runtime constants done by multiplication
// (the 64-bit divisions of the generic kernel above cost more than the copy).  The patch matrix is written once
// and not read again by this kernel, so its stores are streamed past the cache, which stays with the image
// (every pixel is read FH * FW times).
struct Im2colVec {
    int CV, K16;  // 16-byte pieces per tap and per patch row
    FastDiv by_K16, by_CV, by_FW, by_OW, by_OH;
    long rows;
    int rows_per_block;
};

__global__ __launch_bounds__(256) void im2col_vec_kernel(const u32x4v *__restrict__ im, u32x4v *__restrict__ col,
                                                         MapGeom g, Im2colVec q) {
    // workgroup ids congruent modulo 8 run on the same XCD: each XCD takes one contiguous eighth of the patch
    // rows, so its L2 fetches one eighth of the image (plus a halo) instead of most of it
    const unsigned chunk = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const long row0 = (long)chunk * q.rows_per_block;
    const long left = q.rows - row0;
    if (left <= 0) return;
    const unsigned nrows = (unsigned)(left < q.rows_per_block ? left : q.rows_per_block);
    const unsigned span = nrows * (unsigned)q.K16;
    u32x4v *out = col + row0 * q.K16;
    constexpr int U = 4;
    for (unsigned base = threadIdx.x; base < span; base += 256 * U) {
        u32x4v v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const unsigned l = base + 256 * u;
            v[u] = u32x4v{0u, 0u, 0u, 0u};
            if (l < span) {
                const unsigned rl = div_by(l, q.by_K16), piece = l - rl * q.K16;
                const unsigned tap = div_by(piece, q.by_CV), cv = piece - tap * q.CV;
                const unsigned fy = div_by(tap, q.by_FW), fx = tap - fy * g.FW;
                const unsigned r = (unsigned)row0 + rl;
                const unsigned t = div_by(r, q.by_OW), ox = r - t * g.OW;
                const unsigned b = div_by(t, q.by_OH), oy = t - b * g.OH;
                const int iy = (int)oy * g.sy + (int)fy * g.dy - g.pt;
                const int ix = (int)ox * g.sx + (int)fx * g.dx - g.pl;
                if (iy >= 0 && iy < g.IH && ix >= 0 && ix < g.IW)
                    v[u] = im[(((long)b * g.IH + iy) * g.IW + ix) * q.CV + cv];
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const unsigned l = base + 256 * u;
            if (l < span) __builtin_nontemporal_store(v[u], out + l);
        }
    }
}

// The same with rows padded to `pitch` elements (a patch row whose own length cannot be moved in 16-byte
// pieces: 1- and 3-channel images); the padding is written as zeros.  A thread gathers the NV elements of one
// 16-byte piece of a row (the pitch is a multiple of that) and stores them at once.
template <typename V, int NV>
__global__ __launch_bounds__(256) void im2col_padded_kernel(const V *__restrict__ im, V *__restrict__ col, MapGeom g, long total) {
    typedef V VV __attribute__((ext_vector_type(NV)));
    const int K = g.FH * g.FW * g.C, pieces = g.pitch / NV;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const int j0 = (int)(idx % pieces) * NV;
        const long r = idx / pieces;
        const int ox = (int)(r % g.OW);
        const long q = r / g.OW;
        const int oy = (int)(q % g.OH), b = (int)(q / g.OH);
        const V *img = im + (long)b * g.IH * g.IW * g.C;
        VV v;
#pragma unroll
        for (int e = 0; e < NV; ++e) {
            const int j = j0 + e;
            V s = 0;
            if (j < K) {
                const int tap = j / g.C, c = j - tap * g.C, fx = tap % g.FW, fy = tap / g.FW;
                const int iy = oy * g.sy + fy * g.dy - g.pt, ix = ox * g.sx + fx * g.dx - g.pl;
                if (iy >= 0 && iy < g.IH && ix >= 0 && ix < g.IW) s = img[((long)iy * g.IW + ix) * g.C + c];
            }
            v[e] = s;
        }
        *(VV *)(col + r * g.pitch + j0) = v;
    }
}

template <typename V>
__global__ __launch_bounds__(256) void pad_rows_kernel(const V *__restrict__ src, V *__restrict__ dst, int K, int pitch, long total) {
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const int j = (int)(idx % pitch);
        const long r = idx / pitch;
        dst[idx] = j < K ? src[r * K + j] : (V)0;
    }
}

// ---- col2im: one thread owns VEC channels of one image pixel; taps are added in (fy, fx)
// ascending order into registers, then the pixel is written once. -----------------------------
template <typename T, int VEC, bool ACC>
__global__ __launch_bounds__(256) void col2im_kernel(const T *__restrict__ col, T *__restrict__ im,
                                                     MapGeom g, long total) {
    typedef T VT __attribute__((ext_vector_type(VEC)));
    const int CV = g.C / VEC;
    const long K = (long)g.FH * g.FW * g.C;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int cv = (int)(idx % CV);
        const long p = idx / CV;
        const int ix = (int)(p % g.IW);
        const long q = p / g.IW;
        const int iy = (int)(q % g.IH), b = (int)(q / g.IH);
        T *dst = im + p * g.C + (long)cv * VEC;
        typedef typename Wide<T>::type W;
        W acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = 0;
        if (ACC) {
            VT v = *(const VT *)dst;
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] = (W)v[e];
        }
        for (int fy = 0; fy < g.FH; ++fy) {
            const int ty = iy + g.pt - fy * g.dy;
            if (ty < 0 || ty % g.sy) continue;
            const int oy = ty / g.sy;
            if (oy >= g.OH) continue;
            for (int fx = 0; fx < g.FW; ++fx) {
                const int tx = ix + g.pl - fx * g.dx;
                if (tx < 0 || tx % g.sx) continue;
                const int ox = tx / g.sx;
                if (ox >= g.OW) continue;
                const VT v = *(const VT *)(col + (((long)b * g.OH + oy) * g.OW + ox) * K +
                                           (long)(fy * g.FW + fx) * g.C + (long)cv * VEC);
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[e] += (W)v[e];
            }
        }
        VT o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) o[e] = (T)acc[e];
        *(VT *)dst = o;
    }
}

template <typename T, bool ACC>
__global__ __launch_bounds__(256) void col2im_scalar_kernel(const T *__restrict__ col, T *__restrict__ im,
                                                            MapGeom g, long total) {
    const long K = g.pitch ? (long)g.pitch : (long)g.FH * g.FW * g.C;  // row pitch of col
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int c = (int)(idx % g.C);
        const long p = idx / g.C;
        const int ix = (int)(p % g.IW);
        const long q = p / g.IW;
        const int iy = (int)(q % g.IH), b = (int)(q / g.IH);
        typedef typename Wide<T>::type W;
        W acc = ACC ? (W)im[idx] : (W)0;
        for (int fy = 0; fy < g.FH; ++fy) {
            const int ty = iy + g.pt - fy * g.dy;
            if (ty < 0 || ty % g.sy) continue;
            const int oy = ty / g.sy;
            if (oy >= g.OH) continue;
            for (int fx = 0; fx < g.FW; ++fx) {
                const int tx = ix + g.pl - fx * g.dx;
                if (tx < 0 || tx % g.sx) continue;
                const int ox = tx / g.sx;
                if (ox >= g.OW) continue;
                acc += (W)col[(((long)b * g.OH + oy) * g.OW + ox) * K + (long)(fy * g.FW + fx) * g.C + c];
            }
        }
        im[idx] = (T)acc;
    }
}

// ---- DeConv2d col2im (gather, overwrite) -------------------------------------------------------
// In MapGeom for the two DeConv2d maps: C = OC, (IH,IW) = deconv input, (OH,OW) = deconv output.
template <typename T>
__global__ __launch_bounds__(256) void deconv_col2im_kernel(const T *__restrict__ zmat, T *__restrict__ z,
                                                            MapGeom g, long total) {
    const int taps = g.FH * g.FW;
    const long N = (long)g.C * taps;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int oc = (int)(idx % g.C);
        const long p = idx / g.C;
        const int ox = (int)(p % g.OW);
        const long q = p / g.OW;
        const int oy = (int)(q % g.OH), b = (int)(q / g.OH);
        typedef typename Wide<T>::type W;
        W acc = 0;
        for (int fy = 0; fy < g.FH; ++fy) {
            const int ty = oy - g.pt + fy;
            if (ty < 0 || ty % g.sy) continue;
            const int iy = ty / g.sy;
            if (iy >= g.IH) continue;
            for (int fx = 0; fx < g.FW; ++fx) {
                const int tx = ox - g.pl + fx;
                if (tx < 0 || tx % g.sx) continue;
                const int ix = tx / g.sx;
                if (ix >= g.IW) continue;
                acc += (W)zmat[(((long)b * g.IH + iy) * g.IW + ix) * N + (long)oc * taps + fy * g.FW + fx];
            }
        }
        z[idx] = (T)acc;
    }
}

// ---- DeConv2d im2col (pure copy) ------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void deconv_im2col_kernel(const T *__restrict__ dz, T *__restrict__ dzmat,
                                                            MapGeom g, long total) {
    const int taps = g.FH * g.FW;
    const int N = g.C * taps;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int col = (int)(idx % N);
        const long r = idx / N;
        const int ix = (int)(r % g.IW);
        const long q = r / g.IW;
        const int iy = (int)(q % g.IH), b = (int)(q / g.IH);
        const int oc = col / taps, tap = col % taps;
        const int fy = tap / g.FW, fx = tap % g.FW;
        const int oy = iy * g.sy + g.pt - fy;
        const int ox = ix * g.sx + g.pl - fx;
        T v = (T)0;
        if (oy >= 0 && oy < g.OH && ox >= 0 && ox < g.OW)
            v = dz[(((long)b * g.OH + oy) * g.OW + ox) * g.C + oc];
        dzmat[idx] = v;
    }
}

// ---- the two DeConv2d maps staged through LDS ------------------------------------------------------------------
// The reference's matrix layout [B*IH*IW][OC][FH*FW] puts the channels of one tap FH*FW elements apart, so a thread
// per element (the kernels above) moves 2 or 4 bytes at a time.  These forms move 16 bytes per lane on the matrix
// side and on the image side and turn the layout around in LDS.
//
// col2im: a workgroup owns one output row (b, oy).  For each filter row fy that reaches it (ascending, then fx
// ascending inside: the reference's addition order, so sums round identically) the slab
// zmat[(b, iy, ix)][oc][fy][0 .. FW) of all ix, oc is copied into LDS as [ix][fx][oc]; a thread then owns VEC
// channels of one output pixel, adds its taps from LDS into fp32 registers and, after the last fy, writes once.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void deconv_col2im_lds_kernel(const T *__restrict__ zmat, T *__restrict__ z, MapGeom g, FastDiv by_C,
                                                                FastDiv by_CV, FastDiv by_sx) {
    extern __shared__ __attribute__((aligned(16))) unsigned char deconv_lds[];
    T *slab = (T *)deconv_lds;  // [IW][FW][C]
    typedef T VT __attribute__((ext_vector_type(VEC)));
    // (workgroup ids congruent mod 8 share an XCD: each XCD takes a contiguous eighth of the rows, so neighbouring
    // output rows, which read the same matrix rows, meet in one L2)
    const unsigned line = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    if (line >= (unsigned)(g.B * g.OH)) return;
    const int oy = line % g.OH, b = line / g.OH;
    const int taps = g.FH * g.FW, C = g.C, CV = C / VEC;
    const long N = (long)C * taps;
    const int pairs = g.IW * C;      // (ix, oc) pairs staged per filter row
    const int outs = g.OW * CV;      // (ox, channel vector) outputs of this row
    // each thread keeps the sums of up to MAXO of the row's outputs (outs <= 256 * MAXO is checked by the launcher)
    constexpr int MAXO = 4;
    float acc[MAXO][VEC];
#pragma unroll
    for (int o = 0; o < MAXO; ++o)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[o][e] = 0.f;
    // the taps of the slab now in LDS into this thread's sums
    auto accumulate = [&]() {
#pragma unroll
        for (int o = 0; o < MAXO; ++o) {
            const int q = threadIdx.x + 256 * o;
            if (q < outs) {
                const int ox = (int)div_by((unsigned)q, by_CV), cv = q - ox * CV;
                for (int fx = 0; fx < g.FW; ++fx) {
                    const int tx = ox - g.pl + fx;
                    if (tx < 0) continue;
                    const int ix = (int)div_by((unsigned)tx, by_sx);  // (a division by a multiplication: the stride is a run-time value)
                    if (ix * g.sx != tx || ix >= g.IW) continue;
                    const VT v = *(const VT *)(slab + (ix * g.FW + fx) * C + cv * VEC);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc[o][e] += (float)v[e];
                }
            }
        }
    };
    // which input row filter row fy reads for this output row, if any (uniform over the workgroup)
    auto reaches = [&](int fy, int &iy) -> bool {
        const int ty = oy - g.pt + fy;
        if (ty < 0 || ty % g.sy) return false;
        iy = ty / g.sy;
        return iy < g.IH;
    };
    // a filter row of a channel is FW contiguous elements: fetched as one 8- or 16-byte piece where it is one
    const bool row8 = g.FW * sizeof(T) == 8 && (taps * sizeof(T)) % 8 == 0 && ((size_t)zmat & 7) == 0;
    const bool row16 = g.FW * sizeof(T) == 16 && (taps * sizeof(T)) % 16 == 0 && ((size_t)zmat & 15) == 0;
    constexpr int U = 8;
    if ((row8 || row16) && pairs <= 256 * U) {
        // Every thread's pieces of a slab fit its registers: the next filter row's pieces are requested before the
        // present slab is added up, so their way from memory runs under that work instead of after it.
        u32x4v v[U];
        auto fetch = [&](int fy, int iy) {
            const unsigned char *base = (const unsigned char *)(zmat + ((long)b * g.IH + iy) * g.IW * N + (long)fy * g.FW);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int q = threadIdx.x + 256 * u;  // (ix * C + oc): its filter rows start q * taps elements in
                if (q < pairs) {
                    const unsigned char *p = base + (long)q * taps * sizeof(T);
                    if (row16) {
                        v[u] = *(const u32x4v *)p;
                    } else {
                        const uint2 w = *(const uint2 *)p;
                        v[u] = u32x4v{w.x, w.y, 0u, 0u};
                    }
                }
            }
        };
        int fy = 0, iy = 0;
        while (fy < g.FH && !reaches(fy, iy)) ++fy;
        if (fy < g.FH) fetch(fy, iy);
        while (fy < g.FH) {
            __syncthreads();  // the previous slab has been consumed
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int q = threadIdx.x + 256 * u;
                if (q < pairs) {
                    const int ix = (int)div_by((unsigned)q, by_C), oc = q - ix * C;
                    T *d = slab + ix * g.FW * C + oc;
#pragma unroll
                    for (int fx = 0; fx < (int)(16 / sizeof(T)); ++fx) {
                        if (fx < g.FW) {
                            if constexpr (sizeof(T) == 4) ((unsigned *)d)[fx * C] = v[u][fx & 3];
                            else ((unsigned short *)d)[fx * C] = (unsigned short)(v[u][(fx >> 1) & 3] >> (16 * (fx & 1)));
                        }
                    }
                }
            }
            int nfy = fy + 1, niy = 0;
            while (nfy < g.FH && !reaches(nfy, niy)) ++nfy;
            if (nfy < g.FH) fetch(nfy, niy);
            __syncthreads();
            accumulate();
            fy = nfy;
        }
    } else
    for (int fy = 0; fy < g.FH; ++fy) {
        const int ty = oy - g.pt + fy;
        if (ty < 0 || ty % g.sy) continue;  // (uniform over the workgroup)
        const int iy = ty / g.sy;
        if (iy >= g.IH) continue;
        __syncthreads();  // the previous slab has been consumed
        const T *src = zmat + ((long)b * g.IH + iy) * g.IW * N + (long)fy * g.FW;
        for (int q = threadIdx.x; q < pairs; q += 256) {
            const int ix = (int)div_by((unsigned)q, by_C), oc = q - ix * C;
            const T *p = src + (long)ix * N + (long)oc * taps;
            T *d = slab + ix * g.FW * C + oc;
            if (row8) {
                typedef T V8 __attribute__((ext_vector_type(8 / sizeof(T))));
                const V8 v = *(const V8 *)p;
#pragma unroll
                for (int fx = 0; fx < (int)(8 / sizeof(T)); ++fx) d[fx * C] = v[fx];
            } else if (row16) {
                typedef T V16 __attribute__((ext_vector_type(16 / sizeof(T))));
                const V16 v = *(const V16 *)p;
#pragma unroll
                for (int fx = 0; fx < (int)(16 / sizeof(T)); ++fx) d[fx * C] = v[fx];
            } else {
                for (int fx = 0; fx < g.FW; ++fx) d[fx * C] = p[fx];
            }
        }
        __syncthreads();
        accumulate();
    }
    T *row = z + ((long)b * g.OH + oy) * g.OW * C;
#pragma unroll
    for (int o = 0; o < MAXO; ++o) {
        const int q = threadIdx.x + 256 * o;
        if (q < outs) {
            VT out;
#pragma unroll
            for (int e = 0; e < VEC; ++e) out[e] = (T)acc[o][e];
            *(VT *)(row + (long)q * VEC) = out;
        }
    }
}

// im2col where a thread writes whole filter windows: a workgroup owns one input row (b, iy).  The FH rows of dz its taps
// read are copied into LDS as [fy][ox][oc] (zeros where the row lies outside the image; eight 16-byte pieces fetched per
// thread before the first is written).  A thread then owns the FH * FW consecutive matrix columns of one (ix, oc): it
// walks (fy, fx) with two counters, gathers VEC values at a time from LDS and stores them as one 16-byte piece (FH * FW
// a multiple of VEC).  A pure copy: bit-exact.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void deconv_im2col_windows_kernel(const T *__restrict__ dz, T *__restrict__ dzmat, MapGeom g, FastDiv by_C,
                                                                    FastDiv by_row) {
    extern __shared__ __attribute__((aligned(16))) unsigned char deconv_lds[];
    T *rows = (T *)deconv_lds;  // [FH][OW][C]
    typedef T VT __attribute__((ext_vector_type(VEC)));
    const unsigned line = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);  // contiguous rows per XCD, as above
    if (line >= (unsigned)(g.B * g.IH)) return;
    const int iy = line % g.IH, b = line / g.IH;
    const int taps = g.FH * g.FW, C = g.C;
    const int N = C * taps, rowlen = g.OW * C, rowv = rowlen / VEC;  // rowlen is a multiple of VEC (C is)
    constexpr int U = 8;
    const int pieces = g.FH * rowv;
    for (int p0 = threadIdx.x; p0 < pieces; p0 += 256 * U) {
        VT v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const unsigned p = p0 + 256 * u;
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[u][e] = (T)0;
            if (p < (unsigned)pieces) {
                const unsigned fy = div_by(p, by_row), q = p - fy * rowv;
                const int oy = iy * g.sy + g.pt - (int)fy;
                if (oy >= 0 && oy < g.OH) v[u] = *(const VT *)(dz + ((long)b * g.OH + oy) * rowlen + (long)q * VEC);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const unsigned p = p0 + 256 * u;
            if (p < (unsigned)pieces) *(VT *)(rows + (long)p * VEC) = v[u];
        }
    }
    __syncthreads();
    T *out = dzmat + ((long)b * g.IH + iy) * g.IW * N;
    const int cells = g.IW * C;
    for (int p = threadIdx.x; p < cells; p += 256) {
        const unsigned ix = div_by((unsigned)p, by_C), oc = (unsigned)p - ix * C;
        T *dst = out + (long)ix * N + (long)oc * taps;
        int fy = 0, fx = 0;
        for (int t0 = 0; t0 < taps; t0 += VEC) {
            VT v;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const int ox = (int)ix * g.sx + g.pl - fx;
                v[e] = (ox >= 0 && ox < g.OW) ? rows[((long)fy * g.OW + ox) * C + oc] : (T)0;
                if (++fx == g.FW) fx = 0, ++fy;
            }
            *(VT *)(dst + t0) = v;
        }
    }
}

// im2col for the usual filters (FH x FW known at compile time: 4 x 4, 3 x 3, 2 x 2), 16 bytes of channels per thread:
// the same staging, with each pixel's channels at a pitch that keeps the 16-byte LDS reads of lanes on neighbouring
// input pixels in different banks.  A thread owns one input pixel and OCV = 16 / ES consecutive channels: it reads
// the OCV channels of every tap with one 16-byte LDS read (zeros outside the image), which gives it the
// [OCV][FH * FW] block of the matrix row -- 16 * FH * FW contiguous bytes -- transposed; it turns the block around in
// registers (a byte permute per two halves, a move per float) and writes it in 16-byte pieces.  Some 0.6
// instructions per byte stored, against 3 when every element is read from LDS on its own.  A pure copy: bit-exact.
template <int ES, int FH_, int FW_>
__global__ __launch_bounds__(256) void deconv_im2col_blocks_kernel(const unsigned char *__restrict__ dz, unsigned char *__restrict__ dzmat,
                                                                   MapGeom g, int pitch, FastDiv by_groups, FastDiv by_row) {
    extern __shared__ __attribute__((aligned(16))) unsigned char deconv_lds[];  // [FH][OW] pixels of `pitch` bytes
    constexpr int TAPS = FH_ * FW_, OCV = 16 / ES;
    const unsigned slot = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);  // contiguous rows per XCD, as above
    const unsigned line = slot;
    if (line >= (unsigned)(g.B * g.IH)) return;
    const int iy = line % g.IH, b = line / g.IH;
    const int groups = g.C / OCV;                    // 16-byte pieces per pixel
    const int rowv = g.OW * groups, pieces = FH_ * rowv;
    const long rowbytes = (long)g.OW * g.C * ES;
    constexpr int U = 8;
    for (int p0 = threadIdx.x; p0 < pieces; p0 += 256 * U) {
        u32x4v v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const unsigned p = p0 + 256 * u;
            v[u] = u32x4v{0u, 0u, 0u, 0u};
            if (p < (unsigned)pieces) {
                const unsigned fy = div_by(p, by_row), q = p - fy * rowv;
                const int oy = iy * g.sy + g.pt - (int)fy;
                if (oy >= 0 && oy < g.OH) v[u] = *(const u32x4v *)(dz + ((long)b * g.OH + oy) * rowbytes + (long)q * 16);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const unsigned p = p0 + 256 * u;
            if (p < (unsigned)pieces) {
                const unsigned fy = div_by(p, by_row), q = p - fy * rowv, px = div_by(q, by_groups), part = q - px * groups;
                *(u32x4v *)(deconv_lds + (fy * g.OW + px) * pitch + part * 16) = v[u];
            }
        }
    }
    __syncthreads();

    const long N = (long)g.C * TAPS;  // elements per matrix row
    unsigned char *out = dzmat + ((long)b * g.IH + iy) * g.IW * N * ES;
    const int cells = g.IW * groups;
    // A row of at most 256 cells (one per thread): the turned blocks go back through LDS -- over the staged rows, which
    // every thread has read by then -- so that the lanes of a wave store consecutive 16-byte pieces of the matrix
    // (the workgroup's output is one contiguous run of bytes).  A thread storing its own block piece by piece writes
    // a sixteenth of 64 different lines per instruction: 11.6 us for C5's matrix where a plain fill takes 5.4.
    if (cells <= 256) {
        constexpr int CELL = 16 * TAPS + 16;  // bytes between two cells' blocks in LDS (the pad spreads them over the banks)
        const int p = threadIdx.x;
        u32x4v r[TAPS];
        if (p < cells) {
            const unsigned ix = div_by((unsigned)p, by_groups), og = (unsigned)p - ix * groups;
#pragma unroll
            for (int t = 0; t < TAPS; ++t) {
                const int fy = t / FW_, fx = t % FW_;
                const int ox = (int)ix * g.sx + g.pl - fx;
                r[t] = u32x4v{0u, 0u, 0u, 0u};
                if (ox >= 0 && ox < g.OW) r[t] = *(const u32x4v *)(deconv_lds + (fy * g.OW + ox) * pitch + og * 16);
            }
        }
        __syncthreads();
        if (p < cells) {
#pragma unroll
            for (int j = 0; j < TAPS; ++j) {
                u32x4v o;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    if constexpr (ES == 4) {
                        const int e = 4 * j + w;
                        o[w] = r[e % TAPS][e / TAPS];
                    } else {
                        const int e0 = 8 * j + 2 * w, e1 = e0 + 1;
                        const int c0 = e0 / TAPS, c1 = e1 / TAPS;
                        const unsigned lo = r[e0 % TAPS][c0 / 2], hi = r[e1 % TAPS][c1 / 2];
                        const unsigned b0 = 2 * (c0 & 1), b1 = 4 + 2 * (c1 & 1);
                        o[w] = __builtin_amdgcn_perm(hi, lo, b0 | (b0 + 1) << 8 | b1 << 16 | (b1 + 1) << 24);
                    }
                }
                *(u32x4v *)(deconv_lds + p * CELL + 16 * j) = o;
            }
        }
        __syncthreads();
        for (int q = threadIdx.x; q < cells * TAPS; q += 256) {
            const int cell = q / TAPS, j = q - cell * TAPS;
            *(u32x4v *)(out + (long)q * 16) = *(const u32x4v *)(deconv_lds + cell * CELL + 16 * j);
        }
        return;
    }
    for (int p = threadIdx.x; p < cells; p += 256) {
        const unsigned ix = div_by((unsigned)p, by_groups), og = (unsigned)p - ix * groups;
        u32x4v r[TAPS];
#pragma unroll
        for (int t = 0; t < TAPS; ++t) {
            const int fy = t / FW_, fx = t % FW_;
            const int ox = (int)ix * g.sx + g.pl - fx;
            r[t] = u32x4v{0u, 0u, 0u, 0u};
            if (ox >= 0 && ox < g.OW) r[t] = *(const u32x4v *)(deconv_lds + (fy * g.OW + ox) * pitch + og * 16);
        }
        unsigned char *dst = out + ((long)ix * N + (long)og * OCV * TAPS) * ES;
#pragma unroll
        for (int j = 0; j < TAPS; ++j) {  // piece j of the [OCV][TAPS] block: elements 16 / ES * j ...
            u32x4v o;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                if constexpr (ES == 4) {
                    const int e = 4 * j + w;
                    o[w] = r[e % TAPS][e / TAPS];
                } else {
                    const int e0 = 8 * j + 2 * w, e1 = e0 + 1;
                    const int c0 = e0 / TAPS, c1 = e1 / TAPS;  // channels of the two halves
                    const unsigned lo = r[e0 % TAPS][c0 / 2], hi = r[e1 % TAPS][c1 / 2];
                    const unsigned b0 = 2 * (c0 & 1), b1 = 4 + 2 * (c1 & 1);  // byte positions in {hi : lo}
                    o[w] = __builtin_amdgcn_perm(hi, lo, b0 | (b0 + 1) << 8 | b1 << 16 | (b1 + 1) << 24);
                }
            }
            *(u32x4v *)(dst + 16 * j) = o;
        }
    }
}

template <int ES>
static bool launch_im2col_blocks(const void *dz, void *dzmat, const MapGeom &g, hipStream_t s) {
    const int row = g.C * ES;
    // a pitch that puts lanes on neighbouring input pixels (sx output pixels apart) 128 bytes apart modulo 256
    int pitch = row;
    for (int pad = 0; pad <= 256; pad += 16)
        if (((long)g.sx * (row + pad)) % 256 == 128) {
            pitch = row + pad;
            break;
        }
    size_t lds = (size_t)g.FH * g.OW * pitch;
    const size_t cells = (size_t)g.IW * (row / 16), turned = cells * (16 * g.FH * g.FW + 16);  // the blocks on their way out
    if (cells <= 256 && turned > lds) lds = turned;
    if (lds > 64 * 1024) return false;
    const FastDiv by_groups = fast_div((unsigned)(row / 16)), by_row = fast_div((unsigned)(g.OW * (row / 16)));
    const dim3 grid((g.B * g.IH + 7) & ~7), block(256);
    const unsigned char *src = (const unsigned char *)dz;
    unsigned char *dst = (unsigned char *)dzmat;
    if (g.FH == 4 && g.FW == 4)
        hipLaunchKernelGGL((deconv_im2col_blocks_kernel<ES, 4, 4>), grid, block, lds, s, src, dst, g, pitch, by_groups, by_row);
    else if (g.FH == 3 && g.FW == 3)
        hipLaunchKernelGGL((deconv_im2col_blocks_kernel<ES, 3, 3>), grid, block, lds, s, src, dst, g, pitch, by_groups, by_row);
    else if (g.FH == 2 && g.FW == 2)
        hipLaunchKernelGGL((deconv_im2col_blocks_kernel<ES, 2, 2>), grid, block, lds, s, src, dst, g, pitch, by_groups, by_row);
    else
        return false;
    return true;
}

// im2col: a workgroup owns one input row (b, iy).  The FH rows of dz its taps read are copied into LDS as
// [fy][ox][oc] (zeros where the row lies outside the image); a thread then assembles VEC consecutive columns
// (oc, fy, fx) of a matrix row from LDS and stores them at once.  A pure copy: bit-exact.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void deconv_im2col_lds_kernel(const T *__restrict__ dz, T *__restrict__ dzmat, MapGeom g,
                                                                FastDiv by_T, FastDiv by_FW, FastDiv by_NV) {
    extern __shared__ __attribute__((aligned(16))) unsigned char deconv_lds[];
    T *rows = (T *)deconv_lds;  // [FH][OW][C]
    typedef T VT __attribute__((ext_vector_type(VEC)));
    const unsigned line = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);  // contiguous rows per XCD, as above
    if (line >= (unsigned)(g.B * g.IH)) return;
    const int iy = line % g.IH, b = line / g.IH;
    const int taps = g.FH * g.FW, C = g.C;
    const int N = C * taps, NV = N / VEC, rowlen = g.OW * C;
    for (int fy = 0; fy < g.FH; ++fy) {
        const int oy = iy * g.sy + g.pt - fy;
        const bool inside = oy >= 0 && oy < g.OH;
        const T *src = dz + ((long)b * g.OH + (inside ? oy : 0)) * rowlen;
        for (int q = threadIdx.x * VEC; q < rowlen; q += 256 * VEC) {  // rowlen is a multiple of VEC (C is)
            VT v;
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[e] = (T)0;
            if (inside) v = *(const VT *)(src + q);
            *(VT *)(rows + (long)fy * rowlen + q) = v;
        }
    }
    __syncthreads();
    T *out = dzmat + ((long)b * g.IH + iy) * g.IW * N;
    const int chunks = g.IW * NV;
    for (int q = threadIdx.x; q < chunks; q += 256) {
        const unsigned ix = div_by((unsigned)q, by_NV), c0 = ((unsigned)q - ix * NV) * VEC;
        VT v;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const unsigned col = c0 + e, oc = div_by(col, by_T), tap = col - oc * taps;
            const unsigned fy = div_by(tap, by_FW), fx = tap - fy * g.FW;
            const int ox = (int)ix * g.sx + g.pl - (int)fx;
            v[e] = (ox >= 0 && ox < g.OW) ? rows[((long)fy * g.OW + ox) * C + oc] : (T)0;
        }
        *(VT *)(out + (long)q * VEC) = v;
    }
}

static int check_geom(const char *who, int dtype, const void *a, const void *b, const MapGeom &g) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32 && dtype != D8_FLOAT64)
        return fail(D8_ERR_DTYPE, "%s: element type %d is not supported", who, dtype);
    D8_REQUIRE(g.B >= 0 && g.IH > 0 && g.IW > 0 && g.C > 0 && g.OH > 0 && g.OW > 0 && g.FH > 0 && g.FW > 0,
               "%s: sizes must be positive", who);
    D8_REQUIRE(g.sy >= 1 && g.sx >= 1 && g.dy >= 1 && g.dx >= 1, "%s: stride and dilation must be >= 1", who);
    D8_REQUIRE(g.pt >= 0 && g.pl >= 0, "%s: padding must be >= 0", who);
    D8_REQUIRE(g.B == 0 || (a && b), "%s: null pointer", who);
    return 0;
}

static inline bool aligned16(const void *p) { return ((size_t)p & 15) == 0; }

template <typename T>
__global__ __launch_bounds__(256) void unpad_add_kernel(const T *__restrict__ src, T *__restrict__ dst, int K, int pitch, long total, float beta) {
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const long r = idx / K;
        const int j = (int)(idx - r * K);
        float v = (float)src[r * pitch + j];
        if (beta != 0.f) v += (float)dst[idx];
        dst[idx] = (T)v;
    }
}

int launch_unpad_add(int dtype, const void *src, void *dst, long rows, int K, int pitch, float beta, hipStream_t s) {
    const long total = rows * K;
    if (total == 0) return 0;
    if (dtype == D8_FLOAT32)
        hipLaunchKernelGGL((unpad_add_kernel<float>), dim3(grid_for(total, 256)), dim3(256), 0, s, (const float *)src, (float *)dst, K, pitch, total, beta);
    else
        hipLaunchKernelGGL((unpad_add_kernel<f16>), dim3(grid_for(total, 256)), dim3(256), 0, s, (const f16 *)src, (f16 *)dst, K, pitch, total, beta);
    D8_LAUNCH_CHECK();
    return 0;
}

int launch_pad_rows(int dtype, const void *src, void *dst, long rows, int K, int pitch, hipStream_t s) {
    const long total = rows * pitch;
    if (total == 0) return 0;
    if (dtype_bytes(dtype) == 4)
        hipLaunchKernelGGL((pad_rows_kernel<unsigned>), dim3(grid_for(total, 256)), dim3(256), 0, s, (const unsigned *)src, (unsigned *)dst, K, pitch, total);
    else
        hipLaunchKernelGGL((pad_rows_kernel<unsigned short>), dim3(grid_for(total, 256)), dim3(256), 0, s, (const unsigned short *)src, (unsigned short *)dst, K, pitch, total);
    D8_LAUNCH_CHECK();
    return 0;
}

int launch_im2col(int dtype, const void *im, void *col, const MapGeom &g, hipStream_t s) {
    if (g.B == 0) return 0;
    const size_t es = dtype_bytes(dtype);
    if (g.pitch) {  // padded rows: fp32 and half only (the callers' choice)
        // the pitch is a multiple of 16 bytes and col is 16-byte aligned (the operator's own scratch)
        const long total = (long)g.B * g.OH * g.OW * (g.pitch / (int)(16 / es));
        if (es == 4)
            hipLaunchKernelGGL((im2col_padded_kernel<unsigned, 4>), dim3(grid_for(total, 256)), dim3(256), 0, s, (const unsigned *)im, (unsigned *)col, g, total);
        else
            hipLaunchKernelGGL((im2col_padded_kernel<unsigned short, 8>), dim3(grid_for(total, 256)), dim3(256), 0, s, (const unsigned short *)im, (unsigned short *)col, g, total);
        D8_LAUNCH_CHECK();
        return 0;
    }
    const long elems = (long)g.B * g.OH * g.OW * g.FH * g.FW * g.C;
    const size_t row_bytes = (size_t)g.C * es;
    const long rows = (long)g.B * g.OH * g.OW;
    if (row_bytes % 16 == 0 && aligned16(im) && aligned16(col) && rows < (1L << 31) && (long)g.FH * g.FW * row_bytes / 16 < (1L << 20)) {
        Im2colVec q;
        q.CV = (int)(row_bytes / 16);
        q.K16 = g.FH * g.FW * q.CV;
        q.rows = rows;
        // about 32 workgroups per CU, whole patch rows each, a stretch of fewer than 2^31 pieces
        long per = (rows + (long)cu_count() * 32 - 1) / ((long)cu_count() * 32);
        per = (per + 3) & ~3L;
        while (per > 4 && per * q.K16 >= (1L << 31)) per /= 2;
        q.rows_per_block = (int)per;
        q.by_K16 = fast_div(q.K16), q.by_CV = fast_div(q.CV), q.by_FW = fast_div(g.FW), q.by_OW = fast_div(g.OW), q.by_OH = fast_div(g.OH);
        const unsigned blocks = ((unsigned)((rows + per - 1) / per) + 7u) & ~7u;  // a multiple of 8 (see the kernel)
        hipLaunchKernelGGL(im2col_vec_kernel, dim3(blocks), dim3(256), 0, s,
                           (const u32x4v *)im, (u32x4v *)col, g, q);
    } else if (row_bytes % 16 == 0 && aligned16(im) && aligned16(col)) {
        const int CV = (int)(row_bytes / 16);
        const long total = elems / (16 / es);
        hipLaunchKernelGGL((im2col_kernel<uint4>), dim3(grid_for(total, 256)), dim3(256), 0, s,
                           (const uint4 *)im, (uint4 *)col, g, CV, total);
    } else if (es == 8) {
        hipLaunchKernelGGL((im2col_kernel<unsigned long long>), dim3(grid_for(elems, 256)), dim3(256), 0, s,
                           (const unsigned long long *)im, (unsigned long long *)col, g, g.C, elems);
    } else if (es == 4) {
        hipLaunchKernelGGL((im2col_kernel<unsigned>), dim3(grid_for(elems, 256)), dim3(256), 0, s,
                           (const unsigned *)im, (unsigned *)col, g, g.C, elems);
    } else {
        hipLaunchKernelGGL((im2col_kernel<unsigned short>), dim3(grid_for(elems, 256)), dim3(256), 0, s,
                           (const unsigned short *)im, (unsigned short *)col, g, g.C, elems);
    }
    D8_LAUNCH_CHECK();
    return 0;
}

template <typename T, int VEC, bool ACC>
static void launch_col2im_t(const void *col, void *im, const MapGeom &g, bool vec, long elems, hipStream_t s) {
    if (vec)
        hipLaunchKernelGGL((col2im_kernel<T, VEC, ACC>), dim3(grid_for(elems / VEC, 256)), dim3(256), 0, s,
                           (const T *)col, (T *)im, g, elems / VEC);
    else
        hipLaunchKernelGGL((col2im_scalar_kernel<T, ACC>), dim3(grid_for(elems, 256)), dim3(256), 0, s,
                           (const T *)col, (T *)im, g, elems);
}

int launch_col2im(int dtype, const void *col, void *im, const MapGeom &g, bool accumulate, hipStream_t s) {
    if (g.B == 0) return 0;
    const long elems = (long)g.B * g.IH * g.IW * g.C;
    const bool al = aligned16(im) && aligned16(col);
    if (dtype == D8_FLOAT64) {
        if (accumulate) launch_col2im_t<double, 2, true>(col, im, g, g.C % 2 == 0 && al && !g.pitch, elems, s);
        else launch_col2im_t<double, 2, false>(col, im, g, g.C % 2 == 0 && al && !g.pitch, elems, s);
    } else if (dtype == D8_FLOAT32) {
        if (accumulate) launch_col2im_t<float, 4, true>(col, im, g, g.C % 4 == 0 && al && !g.pitch, elems, s);
        else launch_col2im_t<float, 4, false>(col, im, g, g.C % 4 == 0 && al && !g.pitch, elems, s);
    } else {
        if (accumulate) launch_col2im_t<f16, 8, true>(col, im, g, g.C % 8 == 0 && al && !g.pitch, elems, s);
        else launch_col2im_t<f16, 8, false>(col, im, g, g.C % 8 == 0 && al && !g.pitch, elems, s);
    }
    D8_LAUNCH_CHECK();
    return 0;
}

}  // namespace d8

using namespace d8;

extern "C" {

int d8_im2col(int dtype, const void *im, void *col,
              int B, int IH, int IW, int C, int OH, int OW, int FH, int FW,
              int sy, int sx, int dy, int dx, int padTop, int padLeft, void *stream) {
    MapGeom g = {B, IH, IW, C, OH, OW, FH, FW, sy, sx, dy, dx, padTop, padLeft};
    if (int rc = check_geom("d8_im2col", dtype, im, col, g)) return rc;
    return launch_im2col(dtype, im, col, g, as_stream(stream));
}

int d8_col2im(int dtype, const void *col, void *im,
              int B, int IH, int IW, int C, int OH, int OW, int FH, int FW,
              int sy, int sx, int dy, int dx, int padTop, int padLeft, void *stream) {
    MapGeom g = {B, IH, IW, C, OH, OW, FH, FW, sy, sx, dy, dx, padTop, padLeft};
    if (int rc = check_geom("d8_col2im", dtype, col, im, g)) return rc;
    return launch_col2im(dtype, col, im, g, true, as_stream(stream));
}

int d8_deconv_col2im(int dtype, const void *zmat, void *z,
                     int B, int IH, int IW, int OH, int OW, int OC, int FH, int FW,
                     int sy, int sx, int padTop, int padLeft, void *stream) {
    MapGeom g = {B, IH, IW, OC, OH, OW, FH, FW, sy, sx, 1, 1, padTop, padLeft};
    if (int rc = check_geom("d8_deconv_col2im", dtype, zmat, z, g)) return rc;
    if (B == 0) return 0;
    const long elems = (long)B * OH * OW * OC;
    hipStream_t s = as_stream(stream);
    {   // the LDS-staged form: 16-byte channel vectors, a slab of one filter row in LDS, at most 1024 outputs per row
        const size_t es = dtype_bytes(dtype), vec = 16 / es, lds = (size_t)IW * FW * OC * es;
        if (es <= 4 && OC % vec == 0 && aligned16(z) && lds <= 60 * 1024 && (long)OW * (OC / vec) <= 1024 && (long)B * OH < (1L << 31)) {
            if (es == 4)
                hipLaunchKernelGGL((deconv_col2im_lds_kernel<float, 4>), dim3((B * OH + 7) & ~7), dim3(256), lds, s, (const float *)zmat, (float *)z, g,
                                   fast_div((unsigned)OC), fast_div((unsigned)(OC / vec)), fast_div((unsigned)sx));
            else
                hipLaunchKernelGGL((deconv_col2im_lds_kernel<f16, 8>), dim3((B * OH + 7) & ~7), dim3(256), lds, s, (const f16 *)zmat, (f16 *)z, g,
                                   fast_div((unsigned)OC), fast_div((unsigned)(OC / vec)), fast_div((unsigned)sx));
            D8_LAUNCH_CHECK();
            return 0;
        }
    }
    if (dtype == D8_FLOAT64)
        hipLaunchKernelGGL((deconv_col2im_kernel<double>), dim3(grid_for(elems, 256)), dim3(256), 0, s,
                           (const double *)zmat, (double *)z, g, elems);
    else if (dtype == D8_FLOAT32)
        hipLaunchKernelGGL((deconv_col2im_kernel<float>), dim3(grid_for(elems, 256)), dim3(256), 0, s,
                           (const float *)zmat, (float *)z, g, elems);
    else
        hipLaunchKernelGGL((deconv_col2im_kernel<f16>), dim3(grid_for(elems, 256)), dim3(256), 0, s,
                           (const f16 *)zmat, (f16 *)z, g, elems);
    D8_LAUNCH_CHECK();
    return 0;
}

int d8_deconv_im2col(int dtype, const void *dz, void *dzmat,
                     int B, int IH, int IW, int OH, int OW, int OC, int FH, int FW,
                     int sy, int sx, int padTop, int padLeft, void *stream) {
    MapGeom g = {B, IH, IW, OC, OH, OW, FH, FW, sy, sx, 1, 1, padTop, padLeft};
    if (int rc = check_geom("d8_deconv_im2col", dtype, dz, dzmat, g)) return rc;
    if (B == 0) return 0;
    const long elems = (long)B * IH * IW * OC * FH * FW;
    hipStream_t s = as_stream(stream);
    {   // the LDS-staged form: the FH rows of dz an input row reads in LDS, 16-byte pieces of the matrix rows written
        const size_t es = dtype_bytes(dtype), vec = 16 / es, lds = (size_t)FH * OW * OC * es;
        const long N = (long)OC * FH * FW;
        if (es <= 4 && OC % vec == 0 && N % vec == 0 && aligned16(dz) && aligned16(dzmat) && lds <= 60 * 1024 && N < (1L << 24) &&
            (long)IW * N < (1L << 31) && (long)B * IH < (1L << 31)) {
            if ((long)FH * OW * OC * es < (1L << 24) && (long)IW * N * es < (1L << 31)) {  // 16 bytes of channels per thread, the block turned in registers
                if (es == 4 ? launch_im2col_blocks<4>(dz, dzmat, g, s) : launch_im2col_blocks<2>(dz, dzmat, g, s)) {
                    D8_LAUNCH_CHECK();
                    return 0;
                }
            }
            if ((FH * FW) % vec == 0 && (long)FH * OW * OC < (1L << 31)) {  // whole filter windows per thread
                const FastDiv by_C = fast_div((unsigned)OC), by_row = fast_div((unsigned)(OW * OC / vec));
                if (es == 4)
                    hipLaunchKernelGGL((deconv_im2col_windows_kernel<unsigned, 4>), dim3((B * IH + 7) & ~7), dim3(256), lds, s, (const unsigned *)dz, (unsigned *)dzmat, g, by_C, by_row);
                else
                    hipLaunchKernelGGL((deconv_im2col_windows_kernel<unsigned short, 8>), dim3((B * IH + 7) & ~7), dim3(256), lds, s, (const unsigned short *)dz, (unsigned short *)dzmat, g, by_C, by_row);
                D8_LAUNCH_CHECK();
                return 0;
            }
            const FastDiv by_T = fast_div((unsigned)(FH * FW)), by_FW = fast_div((unsigned)FW), by_NV = fast_div((unsigned)(N / vec));
            if (es == 4)
                hipLaunchKernelGGL((deconv_im2col_lds_kernel<unsigned, 4>), dim3((B * IH + 7) & ~7), dim3(256), lds, s, (const unsigned *)dz, (unsigned *)dzmat, g, by_T, by_FW, by_NV);
            else
                hipLaunchKernelGGL((deconv_im2col_lds_kernel<unsigned short, 8>), dim3((B * IH + 7) & ~7), dim3(256), lds, s, (const unsigned short *)dz, (unsigned short *)dzmat, g, by_T, by_FW, by_NV);
            D8_LAUNCH_CHECK();
            return 0;
        }
    }
    if (dtype == D8_FLOAT64)
        hipLaunchKernelGGL((deconv_im2col_kernel<unsigned long long>), dim3(grid_for(elems, 256)), dim3(256), 0, s,
                           (const unsigned long long *)dz, (unsigned long long *)dzmat, g, elems);
    else if (dtype == D8_FLOAT32)
        hipLaunchKernelGGL((deconv_im2col_kernel<unsigned>), dim3(grid_for(elems, 256)), dim3(256), 0, s,
                           (const unsigned *)dz, (unsigned *)dzmat, g, elems);
    else
        hipLaunchKernelGGL((deconv_im2col_kernel<unsigned short>), dim3(grid_for(elems, 256)), dim3(256), 0, s,
                           (const unsigned short *)dz, (unsigned short *)dzmat, g, elems);
    D8_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
