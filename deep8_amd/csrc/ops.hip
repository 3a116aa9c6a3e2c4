// Whole-operator entry points: the shape cases, pad formulas, scratch layout and
// overwrite / accumulate semantics of Deep8's MatrixMultiply, Conv2d and DeConv2d GPU paths,
// expressed as d8_gemm plus the four gather maps.
//
//   MatrixMultiply   deep8/src/math/MatrixMultiply.cu:21-57 (fwd), :193-232 (GradX), :381-420 (GradY)
//   Conv2d           deep8/src/math/Conv2d.cu:145-196, :440-492, :750-802, pads :332-336
//   DeConv2d         deep8/src/math/DeConv2d.cu:76-131, :371-429, :642-700, pads :99-100
#include <atomic>

#include "conv_maps.h"
#include "gemm_args.h"

namespace d8 {

static inline size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

struct Gemm {
    int ta, tb, M, N, K;
    const void *A;
    int lda;
    long sA;
    const void *B;
    int ldb;
    long sB;
    float beta;
    void *C;
    int ldc;
    long sC;
    int batch;
};

static size_t gemm_ws(int dtype, const Gemm &g) {
    return d8_gemm_workspace_bytes(dtype, g.ta, g.tb, g.M, g.N, g.K, g.batch, g.sC);
}

static int run(int dtype, const Gemm &g, void *ws, size_t ws_bytes, void *stream) {
    return d8_gemm(dtype, g.ta, g.tb, g.M, g.N, g.K, g.A, g.lda, g.sA, g.B, g.ldb, g.sB, g.beta,
                   g.C, g.ldc, g.sC, g.batch, ws, ws_bytes, stream);
}

// The same product as a GemmArgs block (what d8_gemm builds from its arguments), for the planners that take one.
static GemmArgs to_args(const Gemm &p) {
    GemmArgs g;
    memset(&g, 0, sizeof(g));
    g.A = p.A, g.B = p.B, g.C = p.C;
    g.M = p.M, g.N = p.N, g.K = p.K;
    g.lda = p.lda, g.ldb = p.ldb, g.ldc = p.ldc;
    g.sA = p.sA, g.sB = p.sB, g.sC = p.sC;
    g.beta = p.beta;
    g.red = (p.sC == 0 && p.batch > 1) ? p.batch : 1;
    g.batch = g.red > 1 ? 1 : p.batch;
    g.splits = 1;
    g.virt = VIRT_NONE;
    return g;
}

// A forward product followed by Add (bias[n] onto column n) and ReLu: in the product's own store where the kernel
// that runs it has one, else the product and one in-place pass over its result.
static int run_bias_relu(int dtype, const Gemm &p, const void *bias, int relu, void *ws, size_t ws_bytes, void *stream) {
    if (bias || relu) {
        GemmArgs g = to_args(p);
        g.bias = bias, g.relu = relu;
        if (gemm_fuses_store(dtype, g, p.ta, p.tb)) return gemm_run_fused(dtype, g, p.ta, p.tb, ws, ws_bytes, as_stream(stream));
    }
    if (int rc = run(dtype, p, ws, ws_bytes, stream)) return rc;
    return launch_bias_relu(dtype, p.C, bias, (long)p.M * p.batch, p.N, relu, as_stream(stream));
}

// The staged (im2col / col2im) route needs its interim matrix.  The size query plans with aligned tensors, so a
// tensor that is not 16-byte aligned (a view at an odd offset) can land here with a scratch sized for the route
// that stages nothing: the message says so.
static int need_scratch(const char *who, const void *scratch, size_t have, size_t need, const void *a, const void *b, const void *c) {
    if (scratch && have >= need) return 0;
    const bool odd = (((size_t)a | (size_t)b | (size_t)c) & 15) != 0;
    return fail(D8_ERR_ARGUMENT, "%s: the interim matrix needs %zu bytes of scratch, %zu given%s", who, need, scratch ? have : (size_t)0,
                odd ? " (a tensor is not 16-byte aligned: it cannot be read by the tile loader, which the size query assumed)" : "");
}

static int check_mm(const char *who, int dtype, int xb, int xr, int xc, int yb, int yr, int yc) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32 && dtype != D8_FLOAT64)
        return fail(D8_ERR_DTYPE, "%s: element type %d is not supported", who, dtype);
    D8_REQUIRE(xb > 0 && xr > 0 && xc > 0 && yb > 0 && yr > 0 && yc > 0, "%s: sizes must be positive", who);
    D8_REQUIRE(xb == yb || xb == 1 || yb == 1, "%s: batch %d vs %d", who, xb, yb);
    D8_REQUIRE(xc == yr, "%s: inner dimensions %d vs %d", who, xc, yr);
    // (a shared y collapses x's batch into the rows of one product, whose row count is an int)
    D8_REQUIRE((long)xb * xr < (1L << 31), "%s: %d x %d rows of x exceed 2^31 - 1", who, xb, xr);
    return 0;
}

// which: 0 forward, 1 gradient of x, 2 gradient of y.  Pointers may be null when only the
// shape is wanted (workspace query).
static Gemm mm_plan(int which, const void *x, int xb, int xr, int xc, const void *y, int yb, int yr, int yc,
                    const void *z, float grad_beta = 1.f) {
    const int zb = xb > yb ? xb : yb;
    const long xs = (long)xr * xc, ys = (long)yr * yc, zs = (long)xr * yc;
    Gemm g;
    if (which == 0) {
        if (yb == 1) g = {0, 0, xb * xr, yc, xc, x, xc, 0, y, yc, 0, 0.f, (void *)z, yc, 0, 1};
        else if (xb == 1 && yc == 1) g = {0, 1, yb, xr, xc, y, xc, 0, x, xc, 0, 0.f, (void *)z, xr, 0, 1};
        else g = {0, 0, xr, yc, xc, x, xc, xb == 1 ? 0 : xs, y, yc, ys, 0.f, (void *)z, yc, zs, zb};
    } else if (which == 1) {  // x plays dx (output), z plays dz
        if (yb == 1) g = {0, 1, xb * xr, xc, yc, z, yc, 0, y, yc, 0, grad_beta, (void *)x, xc, 0, 1};
        else if (xb == 1 && yc == 1) g = {1, 0, xr, xc, yb, z, xr, 0, y, xc, 0, grad_beta, (void *)x, xc, 0, 1};
        else g = {0, 1, xr, xc, yc, z, yc, zs, y, yc, ys, grad_beta, (void *)x, xc, xb == 1 ? 0 : xs, zb};
    } else {  // y plays dy (output), z plays dz
        if (yb == 1) g = {1, 0, yr, yc, xb * xr, x, xc, 0, z, yc, 0, grad_beta, (void *)y, yc, 0, 1};
        else if (xb == 1 && yc == 1) g = {0, 0, yb, xc, xr, z, xr, 0, x, xc, 0, grad_beta, (void *)y, xc, 0, 1};
        else g = {1, 0, yr, yc, xr, x, xc, xb == 1 ? 0 : xs, z, yc, zs, grad_beta, (void *)y, yc, ys, zb};
    }
    return g;
}

static int check_conv(const char *who, int dtype, int B, int IH, int IW, int IC, int OC, int FH, int FW,
                      int sy, int sx, int dy, int dx) {
    if (dtype != D8_FLOAT16 && dtype != D8_FLOAT32 && dtype != D8_FLOAT64)
        return fail(D8_ERR_DTYPE, "%s: element type %d is not supported", who, dtype);
    D8_REQUIRE(B > 0 && IH > 0 && IW > 0 && IC > 0 && OC > 0 && FH > 0 && FW > 0, "%s: sizes must be positive", who);
    D8_REQUIRE(sy >= 1 && sx >= 1 && dy >= 1 && dx >= 1, "%s: the stride and dilation must >= 1", who);
    // row and column counts of the products are ints: pixels of the batch, elements of a patch row / of a filter's taps
    D8_REQUIRE((long)B * IH * IW < (1L << 31) && (long)FH * FW * IC < (1L << 31) && (long)FH * FW * OC < (1L << 31),
               "%s: %d x %d x %d pixels or a %d x %d filter over %d -> %d channels exceed 2^31 - 1 rows or columns", who, B, IH, IW, FH,
               FW, IC, OC);
    return 0;
}

// ---- implicit convolution: the patch matrix is read straight from the image by the GEMM's tile
// loader instead of being written out and read back.  which: 0 forward, 1 gradient of x (stride 1
// only), 2 gradient of the filter.  Returns false when the shape does not qualify; the caller then
// takes the im2col / col2im route.
struct ConvShape {
    int B, IH, IW, IC, OC, FH, FW, OH, OW, sy, sx, dy, dx, pt, pl;
};

static unsigned magic_of(unsigned d) { return d <= 1 ? 0xFFFFFFFFu : (unsigned)((1ull << 32) / d); }

// Whether a product with a patch-matrix operand can run: the tiled kernels have their alignment and size rules,
// the fp64 kernel moves single elements and takes any shape.
static bool implicit_eligible(int dtype, const GemmArgs &g, int ta, int tb) {
    return dtype == D8_FLOAT64 ? true : gemm_tiled_eligible(dtype, g, ta, tb);
}
// Workspace such a product may use (the split of its reduction).
static size_t implicit_workspace(int dtype, const GemmArgs &g) {
    if (dtype == D8_FLOAT64) {
        if (g.virt == VIRT_A_CLASSES) return 0;
        int tps = 0;
        const int pieces = gemm_f64_splits(g.M, g.N, g.K, g.batch, g.red, (size_t)-1, &tps);
        return pieces > 1 ? (size_t)pieces * g.batch * g.M * g.N * sizeof(double) : 0;
    }
    return gemm_tiled_workspace(dtype, g.M, g.N, g.K, g.red, g.virt);
}
static int implicit_run(int dtype, GemmArgs &g, int ta, int tb, void *scratch, size_t scratch_bytes, hipStream_t stream) {
    if (dtype == D8_FLOAT64) {
        g.ws = (float *)scratch, g.ws_bytes = scratch ? scratch_bytes : 0;
        return gemm_f64_launch(g, ta, tb, stream);
    }
    if (g.virt == VIRT_A_CLASSES) return gemm_tiled_launch(dtype, g, ta, tb, stream);
    return gemm_tiled_run(dtype, g, ta, tb, scratch, scratch_bytes, stream);
}

// Float64 gradient of x: the product's N is the input channel count, and under 128 channels the fp64 kernel is
// left with its 64 x 64 tiles, half the flops per operand byte of the 128 x 128 tiles that the staged product
// ([patch rows] x [taps x channels]) runs on -- measured at B32 56x56x64 3x3: 0.53 ms against 0.42 ms staged,
// col2im included.  From 128 channels on the patch product fills the large tiles too.
static bool f64_grad_x_fills_tiles(int dtype, int IC) { return dtype != D8_FLOAT64 || IC >= 128; }

static bool conv_implicit_plan(int dtype, int which, const ConvShape &c, const void *x, const void *w, const void *z,
                               GemmArgs &g, int &ta, int &tb) {
    const bool off = getenv("D8_CONV_EXPLICIT") != nullptr;  // tuning and test aid: force the im2col route
    if (off) return false;
    const long es = (long)dtype_bytes(dtype);
    const long taps = (long)c.FH * c.FW, M = (long)c.B * c.OH * c.OW, K = taps * c.IC;
    if (M >= (1L << 31) || K >= (1L << 31) || (long)c.B * c.IH * c.IW * c.IC * es >= (1L << 31) || M * c.OC * es >= (1L << 31))
        return false;
    memset(&g, 0, sizeof(g));
    g.batch = 1;
    g.red = 1;
    g.splits = 1;
    PatchGeom &pg = g.pg;
    if (which == 1) {  // dx[(b,iy,ix)][ic] += sum over taps of dz[b][iy + pt - fy*dy][ix + pl - fx*dx][:] . w[:][tap][ic]
        if (c.sy != 1 || c.sx != 1) return false;
        if (!f64_grad_x_fills_tiles(dtype, c.IC)) return false;
        pg = {c.OH, c.OW, c.OC, c.IH, c.IW, c.FW, 1, 1, -c.dy, -c.dx, -c.pt, -c.pl, 0, 0, (unsigned)(M * c.OC * es)};
        g.virt = VIRT_A_ROWS;
        g.A = z, g.B = w, g.C = (void *)x;
        g.M = c.B * c.IH * c.IW, g.N = c.IC, g.K = c.OC;
        g.ldb = (int)K, g.sB = c.IC, g.ldc = c.IC, g.red = (int)taps, g.beta = 1.f;
        ta = 0, tb = 0;
    } else {
        pg = {c.IH, c.IW, c.IC, c.OH, c.OW, c.FW, c.sy, c.sx, c.dy, c.dx, c.pt, c.pl, 0, 0,
              (unsigned)((long)c.B * c.IH * c.IW * c.IC * es)};
        if (which == 0) {  // z[(b,oy,ox)][oc] = sum over taps of patch_tap(x) . w[oc][tap][:]
            g.virt = VIRT_A_ROWS;
            g.A = x, g.B = w, g.C = (void *)z;
            g.M = (int)M, g.N = c.OC, g.K = c.IC;
            g.ldb = (int)K, g.sB = c.IC, g.ldc = c.OC, g.red = (int)taps, g.beta = 0.f;
            ta = 0, tb = 1;
        } else {  // dw[oc][(tap,ic)] += sum over patch rows of dz[row][oc] . patch(x)[row][(tap,ic)]
            g.virt = VIRT_B_KROWS;
            g.A = z, g.B = x, g.C = (void *)w;
            g.M = c.OC, g.N = (int)K, g.K = (int)M;
            g.lda = c.OC, g.ldc = (int)K, g.beta = 1.f;
            ta = 1, tb = 0;
        }
    }
    pg.mg_plane = magic_of((unsigned)pg.OH * pg.OW);
    pg.mg_ow = magic_of((unsigned)pg.OW);
    return implicit_eligible(dtype, g, ta, tb);
}

// Conv2d's gradient of x for a stride above 1, input pixel by input pixel: the pixels of dx with one residue (py, px)
// modulo the stride receive the taps fy with fy * dy = py + pt (mod sy) -- fy = f0y + (sy / gcd(sy, dy)) * j -- from
// dz[b][y' + (py + pt - f0y * dy) / sy - j * dy / gcd(sy, dy)][..]: a stride-1 patch product with a negative dilation
// per class (OutClass), all classes in one launch, nothing staged.  A class that no tap reaches (a filter smaller
// than the stride; a dilation that shares a factor with the stride, which leaves whole rows of x unread) gets no
// product: *untouched tells the caller, who zero-fills dx before an overwriting call.
static int gcd_of(int a, int b) { return b ? gcd_of(b, a % b) : a; }

static bool conv_classes_grad_x(int dtype, const ConvShape &c, const void *gx, const void *w, const void *gz, GemmArgs &g, bool *untouched) {
    *untouched = false;
    if (getenv("D8_CONV_EXPLICIT") != nullptr) return false;
    if ((c.sy == 1 && c.sx == 1) || c.sy * c.sx > MAX_CLASSES) return false;
    if (c.IH < c.sy || c.IW < c.sx) return false;
    if (!f64_grad_x_fills_tiles(dtype, c.IC)) return false;
    const long es = (long)dtype_bytes(dtype), T = (long)c.FH * c.FW;
    const long zbytes = (long)c.B * c.OH * c.OW * c.OC * es;
    if (zbytes >= (1L << 31) || (long)c.B * c.IH * c.IW * c.IC * es >= (1L << 31) || T * c.IC * c.OC * es >= (1L << 31))
        return false;
    const int gy = gcd_of(c.sy, c.dy), gw = gcd_of(c.sx, c.dx), stepy = c.sy / gy, stepx = c.sx / gw;
    memset(&g, 0, sizeof(g));
    g.pg = {c.OH, c.OW, c.OC, 0, 0, 0, 1, 1, -(c.dy / gy), -(c.dx / gw), 0, 0, 0, 0, (unsigned)zbytes};
    g.virt = VIRT_A_CLASSES;
    g.A = gz, g.B = w, g.C = (void *)gx;
    g.N = c.IC, g.K = c.OC;
    g.ldb = (int)(T * c.IC), g.sB = (long)stepx * c.IC, g.sB_row = (long)stepy * c.FW * c.IC, g.ldc = c.IC;
    g.batch = 1, g.red = 1, g.splits = 1, g.beta = 1.f;
    g.out_H = c.IH, g.out_W = c.IW, g.out_sy = c.sy, g.out_sx = c.sx;
    // the first tap f < n with f * d = v (mod s), or -1
    auto first_tap = [](int v, int d, int s, int step, int n) {
        for (int f = 0; f < step && f < n; ++f)
            if ((((v - f * d) % s) + s) % s == 0) return f;
        return -1;
    };
    int largest = 0, smallest = 0x7fffffff, most_taps = 0;
    for (int py = 0; py < c.sy; ++py)
        for (int px = 0; px < c.sx; ++px) {
            const int f0y = first_tap(py + c.pt, c.dy, c.sy, stepy, c.FH), f0x = first_tap(px + c.pl, c.dx, c.sx, stepx, c.FW);
            if (f0y < 0 || f0x < 0) {
                *untouched = true;
                continue;
            }
            OutClass &k = g.cls[g.ncls++];
            k.OH = (c.IH - py + c.sy - 1) / c.sy, k.OW = (c.IW - px + c.sx - 1) / c.sx;
            k.M = c.B * k.OH * k.OW;
            k.taps_w = (c.FW - f0x + stepx - 1) / stepx;
            k.red = ((c.FH - f0y + stepy - 1) / stepy) * k.taps_w;
            k.pt = -((py + c.pt - f0y * c.dy) / c.sy), k.pl = -((px + c.pl - f0x * c.dx) / c.sx);  // (exact divisions)
            k.py = py, k.px = px;
            k.b_off = (unsigned)((f0y * c.FW + f0x) * c.IC);
            largest = k.M > largest ? k.M : largest;
            smallest = k.M < smallest ? k.M : smallest;
            most_taps = k.red > most_taps ? k.red : most_taps;
        }
    if (g.ncls == 0) return false;
    g.tiles_per_split = most_taps * (c.OC / (dtype == D8_FLOAT64 ? 16 : gemm_tiled_k_step(dtype)) + 1);
    g.M = smallest;
    const bool ok = implicit_eligible(dtype, g, 0, 0);
    g.M = largest;
    return ok;
}

}  // namespace d8

using namespace d8;

extern "C" {

// ---------------------------------------------------------------------------------------------
size_t d8_matmul_scratch_bytes(int dtype, int which, int xb, int xr, int xc, int yb, int yr, int yc) {
    if (check_mm("d8_matmul_scratch_bytes", dtype, xb, xr, xc, yb, yr, yc)) return 0;
    if (which == 3)  // for d8_matmul_grad_xy: both gradients' scratch side by side (they may share a launch)
        return align256(d8_matmul_scratch_bytes(dtype, 1, xb, xr, xc, yb, yr, yc)) + d8_matmul_scratch_bytes(dtype, 2, xb, xr, xc, yb, yr, yc);
    return gemm_ws(dtype, mm_plan(which, nullptr, xb, xr, xc, nullptr, yb, yr, yc, nullptr));
}

int d8_matmul(int dtype, const void *x, int xb, int xr, int xc, const void *y, int yb, int yr, int yc,
              void *z, void *scratch, size_t scratch_bytes, void *stream) {
    if (int rc = check_mm("d8_matmul", dtype, xb, xr, xc, yb, yr, yc)) return rc;
    D8_REQUIRE(x && y && z, "d8_matmul: null tensor");
    return run(dtype, mm_plan(0, x, xb, xr, xc, y, yb, yr, yc, z), scratch, scratch_bytes, stream);
}

int d8_matmul_bias_relu(int dtype, const void *x, int xb, int xr, int xc, const void *y, int yb, int yr, int yc,
                        const void *bias, int relu, void *z, void *scratch, size_t scratch_bytes, void *stream) {
    if (int rc = check_mm("d8_matmul_bias_relu", dtype, xb, xr, xc, yb, yr, yc)) return rc;
    if (dtype == D8_FLOAT64) return fail(D8_ERR_DTYPE, "d8_matmul_bias_relu: element type %d is not supported", dtype);
    D8_REQUIRE(x && y && z, "d8_matmul_bias_relu: null tensor");
    const Gemm p = mm_plan(0, x, xb, xr, xc, y, yb, yr, yc, z);
    if (yc == 1 && !(xb == 1 && yb > 1) && (bias || relu)) {
        // y is a vector (or a batch of vectors): z is [batch][xr] and its last axis -- the one the bias runs along -- is
        // x's rows, which this plan puts on the product's M side.  The product, then one pass over z as [batch][xr].
        if (int rc = run(dtype, p, scratch, scratch_bytes, stream)) return rc;
        return launch_bias_relu(dtype, z, bias, (long)(xb > yb ? xb : yb), xr, relu, as_stream(stream));
    }
    return run_bias_relu(dtype, p, bias, relu, scratch, scratch_bytes, stream);
}

int d8_matmul_grad_x(int dtype, void *dx, int xb, int xr, int xc, const void *y, int yb, int yr, int yc,
                     const void *dz, void *scratch, size_t scratch_bytes, void *stream) {
    if (int rc = check_mm("d8_matmul_grad_x", dtype, xb, xr, xc, yb, yr, yc)) return rc;
    D8_REQUIRE(dx && y && dz, "d8_matmul_grad_x: null tensor");
    return run(dtype, mm_plan(1, dx, xb, xr, xc, y, yb, yr, yc, dz), scratch, scratch_bytes, stream);
}

int d8_matmul_grad_y(int dtype, const void *x, int xb, int xr, int xc, void *dy, int yb, int yr, int yc,
                     const void *dz, void *scratch, size_t scratch_bytes, void *stream) {
    if (int rc = check_mm("d8_matmul_grad_y", dtype, xb, xr, xc, yb, yr, yc)) return rc;
    D8_REQUIRE(x && dy && dz, "d8_matmul_grad_y: null tensor");
    return run(dtype, mm_plan(2, x, xb, xr, xc, dy, yb, yr, yc, dz), scratch, scratch_bytes, stream);
}

int d8_matmul_grad_x_overwrite(int dtype, void *dx, int xb, int xr, int xc, const void *y, int yb, int yr, int yc,
                               const void *dz, void *scratch, size_t scratch_bytes, void *stream) {
    if (int rc = check_mm("d8_matmul_grad_x_overwrite", dtype, xb, xr, xc, yb, yr, yc)) return rc;
    D8_REQUIRE(dx && y && dz, "d8_matmul_grad_x_overwrite: null tensor");
    return run(dtype, mm_plan(1, dx, xb, xr, xc, y, yb, yr, yc, dz, 0.f), scratch, scratch_bytes, stream);
}

int d8_matmul_grad_y_overwrite(int dtype, const void *x, int xb, int xr, int xc, void *dy, int yb, int yr, int yc,
                               const void *dz, void *scratch, size_t scratch_bytes, void *stream) {
    if (int rc = check_mm("d8_matmul_grad_y_overwrite", dtype, xb, xr, xc, yb, yr, yc)) return rc;
    D8_REQUIRE(x && dy && dz, "d8_matmul_grad_y_overwrite: null tensor");
    return run(dtype, mm_plan(2, x, xb, xr, xc, dy, yb, yr, yc, dz, 0.f), scratch, scratch_bytes, stream);
}

static std::atomic<unsigned long> matmul_pair_launches{0};
unsigned long d8_matmul_grad_pair_launches(void) { return matmul_pair_launches.load(); }

int d8_matmul_grad_xy(int dtype, const void *x, void *dx, int xb, int xr, int xc, const void *y, void *dy, int yb, int yr,
                      int yc, const void *dz, int overwrite, void *scratch, size_t scratch_bytes, void *stream) {
    if (int rc = check_mm("d8_matmul_grad_xy", dtype, xb, xr, xc, yb, yr, yc)) return rc;
    D8_REQUIRE(x && dx && y && dy && dz, "d8_matmul_grad_xy: null tensor");
    D8_REQUIRE(dx != dy, "d8_matmul_grad_xy: dx and dy are the same tensor");
    const Gemm px = mm_plan(1, dx, xb, xr, xc, y, yb, yr, yc, dz, (overwrite & 1) ? 0.f : 1.f);
    const Gemm py = mm_plan(2, x, xb, xr, xc, dy, yb, yr, yc, dz, (overwrite & 2) ? 0.f : 1.f);
    if (dtype == D8_FLOAT16) {
        // both products large enough for the 256 x 256-tile kernel: one launch whose workgroups go from a tile of
        // dX straight on to a tile of dY
        static const char *wide = getenv("D8_GEMM_WIDE");  // tuning aid: 0 keeps the products apart
        GemmArgs gx = to_args(px);
        const GemmArgs gy = to_args(py);
        gx.ws = (float *)scratch, gx.ws_bytes = scratch_bytes;  // (only ever used for the kernel's phase record, a measurement aid)
        const long tx = (long)ceil_div(gx.M, 256) * ceil_div(gx.N, 256) * gx.batch;
        const long ty = (long)ceil_div(gy.M, 256) * ceil_div(gy.N, 256) * gy.batch;
        const long most = (long)cu_count() * 3 / 4;
        if (!(wide && atoi(wide) == 0) && gx.red == 1 && gy.red == 1 && tx >= most && ty >= most && tx + ty < 0x3fffffffL &&
            gemm_wide_eligible(gx, px.ta, px.tb) && gemm_wide_eligible(gy, py.ta, py.tb)) {
            ++matmul_pair_launches;
            return gemm_wide_pair_launch(gx, px.ta, px.tb, gy, py.ta, py.tb, as_stream(stream));
        }
    }
    {  // both products small: one launch of the small-product kernel's workgroups for both
        int rc = 0;
        if (gemm_small_pair_run(dtype, to_args(px), px.ta, px.tb, to_args(py), py.ta, py.tb, as_stream(stream), &rc)) {
            ++matmul_pair_launches;
            return rc;
        }
    }
    {  // both on the tiled kernels with all their workgroups resident at once: one launch, then their split reductions
        int rc = 0;
        GemmArgs gx = to_args(px), gy = to_args(py);
        if (gemm_tiled_run_plain_pair(dtype, gx, px.ta, px.tb, gy, py.ta, py.tb, scratch, scratch_bytes, as_stream(stream), &rc)) {
            ++matmul_pair_launches;
            return rc;
        }
    }
    if (int rc = run(dtype, px, scratch, scratch_bytes, stream)) return rc;
    return run(dtype, py, scratch, scratch_bytes, stream);
}

// ---------------------------------------------------------------------------------------------
int d8_conv2d_geometry(int IH, int IW, int FH, int FW, int covered, int sy, int sx, int dy, int dx, int *out) {
    D8_REQUIRE(out, "d8_conv2d_geometry: out is null");
    D8_REQUIRE(IH > 0 && IW > 0 && FH > 0 && FW > 0 && sy >= 1 && sx >= 1 && dy >= 1 && dx >= 1,
               "d8_conv2d_geometry: bad geometry");
    const int rfh = FH + (FH - 1) * (dy - 1), rfw = FW + (FW - 1) * (dx - 1);
    int OH, OW;
    if (!covered) {
        OH = (IH - rfh) / sy + 1;
        OW = (IW - rfw) / sx + 1;
        D8_REQUIRE(rfh <= IH && rfw <= IW, "d8_conv2d_geometry: the filter is larger than the input");
    } else {
        OH = (IH - 1) / sy + 1;
        OW = (IW - 1) / sx + 1;
    }
    out[0] = OH;
    out[1] = OW;
    const int py = (OH - 1) * sy + rfh - IH, px = (OW - 1) * sx + rfw - IW;
    out[2] = (py > 0 ? py : 0) / 2;
    out[3] = (px > 0 ? px : 0) / 2;
    return 0;
}

int d8_deconv2d_geometry(int IH, int IW, int FH, int FW, int covered, int sy, int sx, int *out) {
    D8_REQUIRE(out, "d8_deconv2d_geometry: out is null");
    D8_REQUIRE(IH > 0 && IW > 0 && FH > 0 && FW > 0 && sy >= 1 && sx >= 1, "d8_deconv2d_geometry: bad geometry");
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
    const int py = OH + FH - (IH - 1) * sy - 2, px = OW + FW - (IW - 1) * sx - 2;
    out[2] = (py > 0 ? py : 0) / 2;
    out[3] = (px > 0 ? px : 0) / 2;
    return 0;
}

// Conv2d GEMMs on the patch matrix [M x K], M = B*OH*OW, K = FH*FW*IC.
static Gemm conv_plan(int which, int M, int K, int OC, const void *col, const void *w, const void *zz) {
    if (which == 0) return {0, 1, M, OC, K, col, K, 0, w, K, 0, 0.f, (void *)zz, OC, 0, 1};   // z = xcol W^T
    if (which == 1) return {0, 0, M, K, OC, zz, OC, 0, w, K, 0, 0.f, (void *)col, K, 0, 1};   // dxcol = dz W
    return {1, 0, OC, K, M, zz, OC, 0, col, K, 0, 1.f, (void *)w, K, 0, 1};                   // dW += dz^T xcol
}

// A patch row of K = FH * FW * IC elements that cannot be moved in 16-byte pieces (1- and 3-channel images) keeps
// all three products off the tiled kernels.  Such a layer runs on a patch matrix whose rows are padded with zeros
// to the next multiple of 16 bytes, against a copy of the filter in the same pitch: the products then have
// K (forward) or N (gradients) = the pitch, and the padding contributes exact zeros.  Returns that pitch, or 0
// where the plain route applies (K already fits, OC would not, Float64, or a patch row so short -- below 64
// elements -- that the products stay small either way and the extra copies cost more than they save).
static int conv_padded_pitch(int dtype, int K, int OC) {
    if (dtype == D8_FLOAT64) return 0;
    const int epv = 16 / (int)dtype_bytes(dtype);
    if (K % epv == 0 || OC % epv != 0 || K < 64) return 0;
    return (K + epv - 1) / epv * epv;
}

// scratch of the padded route: patch matrix [M][pitch] | filter or filter gradient [OC][pitch] | GEMM workspace
struct PaddedScratch {
    size_t col, filt, total;
};
static PaddedScratch conv_padded_scratch(int dtype, int which, int M, int OC, int pitch) {
    PaddedScratch s;
    s.col = align256((size_t)M * pitch * dtype_bytes(dtype));
    s.filt = align256((size_t)OC * pitch * dtype_bytes(dtype));
    s.total = s.col + s.filt + gemm_ws(dtype, conv_plan(which, M, pitch, OC, nullptr, nullptr, nullptr));
    return s;
}

size_t d8_conv2d_scratch_bytes(int dtype, int which, int B, int IH, int IW, int IC,
                               int OC, int FH, int FW, int covered, int sy, int sx, int dy, int dx) {
    if (which == 3)  // for d8_conv2d_grad_xy: both gradients' scratch side by side (they may share a launch)
        return align256(d8_conv2d_scratch_bytes(dtype, 2, B, IH, IW, IC, OC, FH, FW, covered, sy, sx, dy, dx)) +
               d8_conv2d_scratch_bytes(dtype, 1, B, IH, IW, IC, OC, FH, FW, covered, sy, sx, dy, dx);
    int g[4];
    if (check_conv("d8_conv2d_scratch_bytes", dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, dy, dx)) return 0;
    if (d8_conv2d_geometry(IH, IW, FH, FW, covered, sy, sx, dy, dx, g)) return 0;
    const int M = B * g[0] * g[1], K = FH * FW * IC;
    const ConvShape cs = {B, IH, IW, IC, OC, FH, FW, g[0], g[1], sy, sx, dy, dx, g[2], g[3]};
    GemmArgs ga;
    int ta, tb;
    if (conv_implicit_plan(dtype, which, cs, nullptr, nullptr, nullptr, ga, ta, tb))
        return implicit_workspace(dtype, ga);
    bool untouched = false;
    if (which == 1 && conv_classes_grad_x(dtype, cs, nullptr, nullptr, nullptr, ga, &untouched)) return 0;
    const size_t col = align256((size_t)M * K * dtype_bytes(dtype));
    const size_t plain = col + gemm_ws(dtype, conv_plan(which, M, K, OC, nullptr, nullptr, nullptr));
    if (const int pitch = conv_padded_pitch(dtype, K, OC)) {
        const size_t padded = conv_padded_scratch(dtype, which, M, OC, pitch).total;
        return padded > plain ? padded : plain;
    }
    return plain;
}

static int conv2d_impl(int dtype, const void *x, int B, int IH, int IW, int IC,
                       const void *w, int OC, int FH, int FW, void *z,
                       int covered, int sy, int sx, int dy, int dx,
                       void *scratch, size_t scratch_bytes, void *stream, const void *bias, int relu) {
    int g[4];
    if (int rc = check_conv("d8_conv2d", dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, dy, dx)) return rc;
    if (int rc = d8_conv2d_geometry(IH, IW, FH, FW, covered, sy, sx, dy, dx, g)) return rc;
    const int M = B * g[0] * g[1], K = FH * FW * IC;
    const size_t col = align256((size_t)M * K * dtype_bytes(dtype));
    D8_REQUIRE(x && w && z, "d8_conv2d: null tensor");
    {
        const ConvShape cs = {B, IH, IW, IC, OC, FH, FW, g[0], g[1], sy, sx, dy, dx, g[2], g[3]};
        GemmArgs ga;
        int ta, tb;
        if (conv_implicit_plan(dtype, 0, cs, x, w, z, ga, ta, tb)) {
            ga.bias = bias, ga.relu = relu;  // applied in the tile store (and in the remainder band's reduction)
            return implicit_run(dtype, ga, ta, tb, scratch, scratch_bytes, as_stream(stream));
        }
    }
    if (int rc = need_scratch("d8_conv2d", scratch, scratch_bytes, (size_t)M * K * dtype_bytes(dtype), x, w, z)) return rc;
    if (const int pitch = conv_padded_pitch(dtype, K, OC)) {
        const PaddedScratch ps = conv_padded_scratch(dtype, 0, M, OC, pitch);
        if (scratch_bytes >= ps.total && ((size_t)scratch & 15) == 0) {  // a smaller scratch still serves the plain route
            char *colp = (char *)scratch, *wp = colp + ps.col, *ws = wp + ps.filt;
            const MapGeom mg = {B, IH, IW, IC, g[0], g[1], FH, FW, sy, sx, dy, dx, g[2], g[3], pitch};
            if (int rc = launch_im2col(dtype, x, colp, mg, as_stream(stream))) return rc;
            if (int rc = launch_pad_rows(dtype, w, wp, OC, K, pitch, as_stream(stream))) return rc;
            Gemm plan = conv_plan(0, M, pitch, OC, colp, wp, z);  // z = xcol W^T over K = pitch
            return run_bias_relu(dtype, plan, bias, relu, ws, scratch_bytes - ps.col - ps.filt, stream);
        }
    }
    if (int rc = d8_im2col(dtype, x, scratch, B, IH, IW, IC, g[0], g[1], FH, FW, sy, sx, dy, dx, g[2], g[3], stream))
        return rc;
    const size_t ws = scratch_bytes > col ? scratch_bytes - col : 0;
    return run_bias_relu(dtype, conv_plan(0, M, K, OC, scratch, w, z), bias, relu, ws ? (char *)scratch + col : nullptr, ws, stream);
}

int d8_conv2d(int dtype, const void *x, int B, int IH, int IW, int IC,
              const void *w, int OC, int FH, int FW, void *z,
              int covered, int sy, int sx, int dy, int dx,
              void *scratch, size_t scratch_bytes, void *stream) {
    return conv2d_impl(dtype, x, B, IH, IW, IC, w, OC, FH, FW, z, covered, sy, sx, dy, dx, scratch, scratch_bytes, stream, nullptr, 0);
}

int d8_conv2d_bias_relu(int dtype, const void *x, int B, int IH, int IW, int IC,
                        const void *w, int OC, int FH, int FW, const void *bias, int relu, void *z,
                        int covered, int sy, int sx, int dy, int dx,
                        void *scratch, size_t scratch_bytes, void *stream) {
    if (dtype == D8_FLOAT64) return fail(D8_ERR_DTYPE, "d8_conv2d_bias_relu: element type %d is not supported", dtype);
    return conv2d_impl(dtype, x, B, IH, IW, IC, w, OC, FH, FW, z, covered, sy, sx, dy, dx, scratch, scratch_bytes, stream, bias, relu);
}

static int d8_conv2d_grad_x_impl(int dtype, void *gx, int B, int IH, int IW, int IC,
                     const void *w, int OC, int FH, int FW, const void *gz,
                     int covered, int sy, int sx, int dy, int dx,
                     void *scratch, size_t scratch_bytes, void *stream, float beta) {
    int g[4];
    if (int rc = check_conv("d8_conv2d_grad_x", dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, dy, dx)) return rc;
    if (int rc = d8_conv2d_geometry(IH, IW, FH, FW, covered, sy, sx, dy, dx, g)) return rc;
    const int M = B * g[0] * g[1], K = FH * FW * IC;
    const size_t col = align256((size_t)M * K * dtype_bytes(dtype));
    D8_REQUIRE(gx && w && gz, "d8_conv2d_grad_x: null tensor");
    {
        const ConvShape cs = {B, IH, IW, IC, OC, FH, FW, g[0], g[1], sy, sx, dy, dx, g[2], g[3]};
        GemmArgs ga;
        int ta, tb;
        if (conv_implicit_plan(dtype, 1, cs, gx, w, gz, ga, ta, tb)) {
            ga.beta = beta;
            return implicit_run(dtype, ga, ta, tb, scratch, scratch_bytes, as_stream(stream));
        }
        bool untouched = false;
        if (conv_classes_grad_x(dtype, cs, gx, w, gz, ga, &untouched)) {
            if (untouched && beta == 0.f) {  // pixels of dx that no tap reaches: zero, and the classes add to that
                if (int rc = d8_fill(dtype, gx, (size_t)B * IH * IW * IC, 0.f, stream)) return rc;
                beta = 1.f;
            }
            ga.beta = beta;
            return implicit_run(dtype, ga, 0, 0, nullptr, 0, as_stream(stream));
        }
    }
    if (int rc = need_scratch("d8_conv2d_grad_x", scratch, scratch_bytes, (size_t)M * K * dtype_bytes(dtype), gx, w, gz)) return rc;
    if (const int pitch = conv_padded_pitch(dtype, K, OC)) {
        const PaddedScratch ps = conv_padded_scratch(dtype, 1, M, OC, pitch);
        if (scratch_bytes >= ps.total && ((size_t)scratch & 15) == 0) {
            char *colp = (char *)scratch, *wp = colp + ps.col, *ws = wp + ps.filt;
            if (int rc = launch_pad_rows(dtype, w, wp, OC, K, pitch, as_stream(stream))) return rc;
            Gemm plan = conv_plan(1, M, pitch, OC, colp, wp, gz);  // dxcol [M][pitch] = dz W, the padding columns come out 0
            if (int rc = run(dtype, plan, ws, scratch_bytes - ps.col - ps.filt, stream)) return rc;
            if (beta == 0.f)  // col2im adds into its destination
                if (int rc = d8_fill(dtype, gx, (size_t)B * IH * IW * IC, 0.f, stream)) return rc;
            const MapGeom mg = {B, IH, IW, IC, g[0], g[1], FH, FW, sy, sx, dy, dx, g[2], g[3], pitch};
            return launch_col2im(dtype, colp, gx, mg, true, as_stream(stream));
        }
    }
    const size_t ws = scratch_bytes > col ? scratch_bytes - col : 0;
    if (int rc = run(dtype, conv_plan(1, M, K, OC, scratch, w, gz), ws ? (char *)scratch + col : nullptr, ws, stream))
        return rc;
    if (beta == 0.f)  // col2im adds into its destination
        if (int rc = d8_fill(dtype, gx, (size_t)B * IH * IW * IC, 0.f, stream)) return rc;
    return d8_col2im(dtype, scratch, gx, B, IH, IW, IC, g[0], g[1], FH, FW, sy, sx, dy, dx, g[2], g[3], stream);
}

static int d8_conv2d_grad_y_impl(int dtype, const void *x, int B, int IH, int IW, int IC,
                     void *gw, int OC, int FH, int FW, const void *gz,
                     int covered, int sy, int sx, int dy, int dx,
                     void *scratch, size_t scratch_bytes, void *stream, float beta) {
    int g[4];
    if (int rc = check_conv("d8_conv2d_grad_y", dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, dy, dx)) return rc;
    if (int rc = d8_conv2d_geometry(IH, IW, FH, FW, covered, sy, sx, dy, dx, g)) return rc;
    const int M = B * g[0] * g[1], K = FH * FW * IC;
    const size_t col = align256((size_t)M * K * dtype_bytes(dtype));
    D8_REQUIRE(x && gw && gz, "d8_conv2d_grad_y: null tensor");
    {
        const ConvShape cs = {B, IH, IW, IC, OC, FH, FW, g[0], g[1], sy, sx, dy, dx, g[2], g[3]};
        GemmArgs ga;
        int ta, tb;
        if (conv_implicit_plan(dtype, 2, cs, x, gw, gz, ga, ta, tb)) {
            ga.beta = beta;
            return implicit_run(dtype, ga, ta, tb, scratch, scratch_bytes, as_stream(stream));
        }
    }
    if (int rc = need_scratch("d8_conv2d_grad_y", scratch, scratch_bytes, (size_t)M * K * dtype_bytes(dtype), x, gw, gz)) return rc;
    if (const int pitch = conv_padded_pitch(dtype, K, OC)) {
        const PaddedScratch ps = conv_padded_scratch(dtype, 2, M, OC, pitch);
        if (scratch_bytes >= ps.total && ((size_t)scratch & 15) == 0) {
            char *colp = (char *)scratch, *gwp = colp + ps.col, *ws = gwp + ps.filt;
            const MapGeom mg = {B, IH, IW, IC, g[0], g[1], FH, FW, sy, sx, dy, dx, g[2], g[3], pitch};
            if (int rc = launch_im2col(dtype, x, colp, mg, as_stream(stream))) return rc;
            Gemm plan = conv_plan(2, M, pitch, OC, colp, gwp, gz);  // [OC][pitch] = dz^T xcol
            plan.beta = 0.f;
            if (int rc = run(dtype, plan, ws, scratch_bytes - ps.col - ps.filt, stream)) return rc;
            return launch_unpad_add(dtype, gwp, gw, OC, K, pitch, beta, as_stream(stream));  // gw (+)= its first K columns
        }
    }
    if (int rc = d8_im2col(dtype, x, scratch, B, IH, IW, IC, g[0], g[1], FH, FW, sy, sx, dy, dx, g[2], g[3], stream))
        return rc;
    const size_t ws = scratch_bytes > col ? scratch_bytes - col : 0;
    Gemm plan = conv_plan(2, M, K, OC, scratch, gw, gz);
    plan.beta = beta;
    return run(dtype, plan, ws ? (char *)scratch + col : nullptr, ws, stream);
}

// ---------------------------------------------------------------------------------------------
// DeConv2d.  The interim matrix is kept tap-major, [B*IH*IW][FH*FW][OC] (the reference's kernels use
// [.][OC][FH*FW]; the layout is private to the operator), so that both gather maps move whole
// channel vectors: they are then exactly the Conv2d maps of a mirrored geometry -- image = the
// DeConv2d output, patch grid = the DeConv2d input, dilation -1, negated pads -- and the GEMMs
// become one product per tap against the filter slice w[:, tap, :] (row stride FH*FW*IC).
static MapGeom deconv_mirror(int B, int IH, int IW, int OC, int FH, int FW, int sy, int sx, const int *g) {
    return {B, g[0], g[1], OC, IH, IW, FH, FW, sy, sx, -1, -1, -g[2], -g[3]};
}

static Gemm deconv_plan(int which, int M, int T, int OC, int IC, const void *mat, const void *w, const void *xx) {
    const int NP = T * OC, KW = T * IC;
    if (which == 0) return {0, 1, M, OC, IC, xx, IC, 0, w, KW, IC, 0.f, (void *)mat, NP, OC, T};  // zmat[:, t, :] = x w_t^T
    if (which == 1) return {0, 0, M, IC, OC, mat, NP, OC, w, KW, IC, 1.f, (void *)xx, IC, 0, T};  // dx += sum_t dzmat[:, t, :] w_t
    return {1, 0, OC, IC, M, mat, NP, OC, xx, IC, 0, 1.f, (void *)w, KW, IC, T};                  // dw_t += dzmat[:, t, :]^T x
}

// dx += sum over taps of (rows of dz gathered for that tap) . w_t, the gather done by the GEMM's loader
static bool deconv_implicit_grad_x(int dtype, int B, int IH, int IW, int IC, int OC, int FH, int FW, int sy, int sx,
                                   const int *geo, const void *gx, const void *w, const void *gz, GemmArgs &g) {
    if (getenv("D8_CONV_EXPLICIT") != nullptr) return false;
    const long es = (long)dtype_bytes(dtype), T = (long)FH * FW;
    const long zbytes = (long)B * geo[0] * geo[1] * OC * es;
    if (zbytes >= (1L << 31) || (long)B * IH * IW >= (1L << 31) || T * IC >= (1L << 31)) return false;
    memset(&g, 0, sizeof(g));
    g.pg = {geo[0], geo[1], OC, IH, IW, FW, sy, sx, -1, -1, -geo[2], -geo[3],
            magic_of((unsigned)IH * IW), magic_of((unsigned)IW), (unsigned)zbytes};
    g.virt = VIRT_A_ROWS;
    g.A = gz, g.B = w, g.C = (void *)gx;
    g.M = B * IH * IW, g.N = IC, g.K = OC;
    g.ldb = (int)(T * IC), g.sB = IC, g.ldc = IC;
    g.batch = 1, g.red = (int)T, g.splits = 1, g.beta = 1.f;
    return implicit_eligible(dtype, g, 0, 0);
}

// z computed output pixel by output pixel: the sy * sx residue classes of output coordinates are each
// a stride-1 patch product over the taps that reach them (OutClass), all in one launch; nothing
// is staged.  Needs a tap for every class (FH >= sy, FW >= sx) and tile-sized classes.
static bool deconv_implicit_fwd(int dtype, int B, int IH, int IW, int IC, int OC, int FH, int FW, int sy, int sx,
                                const int *geo, const void *x, const void *w, const void *z, GemmArgs &g, bool *untouched) {
    *untouched = false;
    if (getenv("D8_CONV_EXPLICIT") != nullptr) return false;
    const long es = (long)dtype_bytes(dtype), T = (long)FH * FW;
    const int OH = geo[0], OW = geo[1], pt = geo[2], pl = geo[3];
    if (sy * sx > MAX_CLASSES || OH < sy || OW < sx) return false;
    const long xbytes = (long)B * IH * IW * IC * es;
    if (xbytes >= (1L << 31) || (long)B * OH * OW * OC * es >= (1L << 31) || T * IC * OC * es >= (1L << 31)) return false;
    memset(&g, 0, sizeof(g));
    g.pg = {IH, IW, IC, 0, 0, 0, 1, 1, 1, 1, 0, 0, 0, 0, (unsigned)xbytes};
    g.virt = VIRT_A_CLASSES;
    g.A = x, g.B = w, g.C = (void *)z;
    g.N = OC, g.K = IC;
    g.ldb = (int)(T * IC), g.sB = (long)sx * IC, g.sB_row = (long)sy * FW * IC, g.ldc = OC;
    g.batch = 1, g.red = 1, g.splits = 1, g.beta = 0.f;
    g.out_H = OH, g.out_W = OW, g.out_sy = sy, g.out_sx = sx;
    int largest = 0, smallest = 0x7fffffff, most_taps = 0;
    for (int py = 0; py < sy; ++py)
        for (int px = 0; px < sx; ++px) {
            // taps fy with (py - pt + fy) a multiple of sy: fy = f0y + sy * j
            const int f0y = (((pt - py) % sy) + sy) % sy, f0x = (((pl - px) % sx) + sx) % sx;
            if (f0y >= FH || f0x >= FW) {  // a stride larger than the filter: output pixels that no tap writes (zero; the caller fills z)
                *untouched = true;
                continue;
            }
            OutClass &c = g.cls[g.ncls++];
            c.OH = (OH - py + sy - 1) / sy, c.OW = (OW - px + sx - 1) / sx;
            c.M = B * c.OH * c.OW;
            const int nty = (FH - f0y + sy - 1) / sy, ntx = (FW - f0x + sx - 1) / sx;
            c.taps_w = ntx, c.red = nty * ntx;
            c.pt = -((py - pt + f0y) / sy), c.pl = -((px - pl + f0x) / sx);  // input row = y' + j + (py - pt + f0y) / sy
            c.py = py, c.px = px;
            c.b_off = (unsigned)((f0y * FW + f0x) * IC);
            largest = c.M > largest ? c.M : largest;
            smallest = c.M < smallest ? c.M : smallest;
            most_taps = c.red > most_taps ? c.red : most_taps;
        }
    if (g.ncls == 0) return false;
    g.tiles_per_split = most_taps * (IC / (dtype == D8_FLOAT64 ? 16 : gemm_tiled_k_step(dtype)) + 1);  // never the limit: a class walks all its taps
    g.M = smallest;
    const bool ok = implicit_eligible(dtype, g, 0, 1);
    g.M = largest;
    return ok;
}

// dw[oc][tap][ic] += sum over input pixels m of dz gathered for (m, tap)[oc] . x[m][ic], computed as the
// transposed product [IC] x [taps x OC] = x^T . patch(dz) -- the patch matrix of dz read by the tile loader, as
// for Conv2d's filter gradient -- and stored transposed per tap by the reduction.
static bool deconv_implicit_grad_y(int dtype, int B, int IH, int IW, int IC, int OC, int FH, int FW, int sy, int sx,
                                   const int *geo, const void *x, const void *gw, const void *gz, GemmArgs &g) {
    if (getenv("D8_CONV_EXPLICIT") != nullptr) return false;
    const long es = (long)dtype_bytes(dtype), T = (long)FH * FW;
    const long zbytes = (long)B * geo[0] * geo[1] * OC * es;
    if (zbytes >= (1L << 31) || (long)B * IH * IW >= (1L << 31) || T * OC >= (1L << 31)) return false;
    memset(&g, 0, sizeof(g));
    g.pg = {geo[0], geo[1], OC, IH, IW, FW, sy, sx, -1, -1, -geo[2], -geo[3],
            magic_of((unsigned)IH * IW), magic_of((unsigned)IW), (unsigned)zbytes};
    g.virt = VIRT_B_KROWS;
    g.A = x, g.B = gz, g.C = (void *)gw;
    g.M = IC, g.N = (int)(T * OC), g.K = B * IH * IW;
    g.lda = IC, g.ldc = IC;
    g.batch = 1, g.red = 1, g.splits = 1, g.beta = 1.f;
    g.perm_T = (int)T, g.perm_OC = OC;
    return implicit_eligible(dtype, g, 1, 0);
}

// geo = {OH, OW, padTop, padLeft}: Deep8's own (from `covered`) or the caller's (the _ex entry points)
static int check_deconv_geo(const char *who, const int *geo) {
    D8_REQUIRE(geo[0] > 0 && geo[1] > 0 && geo[2] >= 0 && geo[3] >= 0, "%s: output %d x %d, pads %d / %d", who, geo[0], geo[1], geo[2], geo[3]);
    return 0;
}
// ... and the output's pixel count is an int as well
static int check_deconv_out(const char *who, int B, const int *geo) {
    D8_REQUIRE((long)B * geo[0] * geo[1] < (1L << 31), "%s: %d x %d x %d output pixels exceed 2^31 - 1", who, B, geo[0], geo[1]);
    return 0;
}

static size_t deconv2d_scratch_bytes(int dtype, int which, int B, int IH, int IW, int IC,
                                     int OC, int FH, int FW, const int *geo, int sy, int sx) {
    if (which == 3)  // for d8_deconv2d_grad_xy: both gradients' scratch side by side
        return align256(deconv2d_scratch_bytes(dtype, 2, B, IH, IW, IC, OC, FH, FW, geo, sy, sx)) +
               deconv2d_scratch_bytes(dtype, 1, B, IH, IW, IC, OC, FH, FW, geo, sy, sx);
    if (check_deconv_out("d8_deconv2d_scratch_bytes", B, geo)) return 0;
    const int M = B * IH * IW, T = FH * FW;
    GemmArgs ga;
    if (which == 1 && deconv_implicit_grad_x(dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, geo, nullptr, nullptr, nullptr, ga))
        return implicit_workspace(dtype, ga);
    bool untouched = false;
    if (which == 0 && deconv_implicit_fwd(dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, geo, nullptr, nullptr, nullptr, ga, &untouched)) return 0;
    if (which == 2 && deconv_implicit_grad_y(dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, geo, nullptr, nullptr, nullptr, ga))
        return implicit_workspace(dtype, ga);
    const size_t mat = align256((size_t)M * T * OC * dtype_bytes(dtype));
    return mat + gemm_ws(dtype, deconv_plan(which, M, T, OC, IC, nullptr, nullptr, nullptr));
}

size_t d8_deconv2d_scratch_bytes(int dtype, int which, int B, int IH, int IW, int IC,
                                 int OC, int FH, int FW, int covered, int sy, int sx) {
    int geo[4];
    if (check_conv("d8_deconv2d_scratch_bytes", dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, 1, 1)) return 0;
    if (d8_deconv2d_geometry(IH, IW, FH, FW, covered, sy, sx, geo)) return 0;
    return deconv2d_scratch_bytes(dtype, which, B, IH, IW, IC, OC, FH, FW, geo, sy, sx);
}

size_t d8_deconv2d_scratch_bytes_ex(int dtype, int which, int B, int IH, int IW, int IC,
                                    int OC, int FH, int FW, int OH, int OW, int padTop, int padLeft, int sy, int sx) {
    const int geo[4] = {OH, OW, padTop, padLeft};
    if (check_conv("d8_deconv2d_scratch_bytes_ex", dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, 1, 1)) return 0;
    if (check_deconv_geo("d8_deconv2d_scratch_bytes_ex", geo)) return 0;
    return deconv2d_scratch_bytes(dtype, which, B, IH, IW, IC, OC, FH, FW, geo, sy, sx);
}

static int deconv2d_impl(int dtype, const void *x, int B, int IH, int IW, int IC,
                         const void *w, int OC, int FH, int FW, void *z, const int *g, int sy, int sx,
                         void *scratch, size_t scratch_bytes, void *stream) {
    const int M = B * IH * IW, T = FH * FW;
    const size_t mat = align256((size_t)M * T * OC * dtype_bytes(dtype));
    D8_REQUIRE(x && w && z, "d8_deconv2d: null tensor");
    if (int rc = check_deconv_out("d8_deconv2d", B, g)) return rc;
    {
        GemmArgs ga;
        bool untouched = false;
        if (deconv_implicit_fwd(dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, g, x, w, z, ga, &untouched)) {
            if (untouched)  // the pixels between the filter's footprints stay zero
                if (int rc = d8_fill(dtype, z, (size_t)B * g[0] * g[1] * OC, 0.f, stream)) return rc;
            return implicit_run(dtype, ga, 0, 1, nullptr, 0, as_stream(stream));
        }
    }
    if (int rc = need_scratch("d8_deconv2d", scratch, scratch_bytes, (size_t)M * T * OC * dtype_bytes(dtype), x, w, z)) return rc;
    const size_t ws = scratch_bytes > mat ? scratch_bytes - mat : 0;
    if (int rc = run(dtype, deconv_plan(0, M, T, OC, IC, scratch, w, x), ws ? (char *)scratch + mat : nullptr, ws, stream))
        return rc;
    return launch_col2im(dtype, scratch, z, deconv_mirror(B, IH, IW, OC, FH, FW, sy, sx, g), false, as_stream(stream));
}

int d8_deconv2d(int dtype, const void *x, int B, int IH, int IW, int IC,
                const void *w, int OC, int FH, int FW, void *z,
                int covered, int sy, int sx,
                void *scratch, size_t scratch_bytes, void *stream) {
    int g[4];
    if (int rc = check_conv("d8_deconv2d", dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, 1, 1)) return rc;
    if (int rc = d8_deconv2d_geometry(IH, IW, FH, FW, covered, sy, sx, g)) return rc;
    return deconv2d_impl(dtype, x, B, IH, IW, IC, w, OC, FH, FW, z, g, sy, sx, scratch, scratch_bytes, stream);
}

int d8_deconv2d_ex(int dtype, const void *x, int B, int IH, int IW, int IC,
                   const void *w, int OC, int FH, int FW, void *z,
                   int OH, int OW, int padTop, int padLeft, int sy, int sx,
                   void *scratch, size_t scratch_bytes, void *stream) {
    const int g[4] = {OH, OW, padTop, padLeft};
    if (int rc = check_conv("d8_deconv2d_ex", dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, 1, 1)) return rc;
    if (int rc = check_deconv_geo("d8_deconv2d_ex", g)) return rc;
    return deconv2d_impl(dtype, x, B, IH, IW, IC, w, OC, FH, FW, z, g, sy, sx, scratch, scratch_bytes, stream);
}

static int deconv2d_grad_x_geo(int dtype, void *gx, int B, int IH, int IW, int IC,
                       const void *w, int OC, int FH, int FW, const void *gz,
                       const int *g, int sy, int sx,
                       void *scratch, size_t scratch_bytes, void *stream, float beta) {
    const int M = B * IH * IW, T = FH * FW;
    const size_t mat = align256((size_t)M * T * OC * dtype_bytes(dtype));
    D8_REQUIRE(gx && w && gz, "d8_deconv2d_grad_x: null tensor");
    if (int rc = check_deconv_out("d8_deconv2d_grad_x", B, g)) return rc;
    {
        GemmArgs ga;
        if (deconv_implicit_grad_x(dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, g, gx, w, gz, ga)) {
            ga.beta = beta;
            return implicit_run(dtype, ga, 0, 0, scratch, scratch_bytes, as_stream(stream));
        }
    }
    if (int rc = need_scratch("d8_deconv2d_grad_x", scratch, scratch_bytes, (size_t)M * T * OC * dtype_bytes(dtype), gx, w, gz)) return rc;
    if (int rc = launch_im2col(dtype, gz, scratch, deconv_mirror(B, IH, IW, OC, FH, FW, sy, sx, g), as_stream(stream)))
        return rc;
    const size_t ws = scratch_bytes > mat ? scratch_bytes - mat : 0;
    Gemm plan = deconv_plan(1, M, T, OC, IC, scratch, w, gx);
    plan.beta = beta;
    return run(dtype, plan, ws ? (char *)scratch + mat : nullptr, ws, stream);
}

static int d8_deconv2d_grad_x_impl(int dtype, void *gx, int B, int IH, int IW, int IC,
                       const void *w, int OC, int FH, int FW, const void *gz,
                       int covered, int sy, int sx,
                       void *scratch, size_t scratch_bytes, void *stream, float beta) {
    int g[4];
    if (int rc = check_conv("d8_deconv2d_grad_x", dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, 1, 1)) return rc;
    if (int rc = d8_deconv2d_geometry(IH, IW, FH, FW, covered, sy, sx, g)) return rc;
    return deconv2d_grad_x_geo(dtype, gx, B, IH, IW, IC, w, OC, FH, FW, gz, g, sy, sx, scratch, scratch_bytes, stream, beta);
}

int d8_deconv2d_grad_x_ex(int dtype, void *gx, int B, int IH, int IW, int IC,
                          const void *w, int OC, int FH, int FW, const void *gz,
                          int OH, int OW, int padTop, int padLeft, int sy, int sx, int overwrite,
                          void *scratch, size_t scratch_bytes, void *stream) {
    const int g[4] = {OH, OW, padTop, padLeft};
    if (int rc = check_conv("d8_deconv2d_grad_x_ex", dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, 1, 1)) return rc;
    if (int rc = check_deconv_geo("d8_deconv2d_grad_x_ex", g)) return rc;
    return deconv2d_grad_x_geo(dtype, gx, B, IH, IW, IC, w, OC, FH, FW, gz, g, sy, sx, scratch, scratch_bytes, stream, overwrite ? 0.f : 1.f);
}

static int deconv2d_grad_y_geo(int dtype, const void *x, int B, int IH, int IW, int IC,
                       void *gw, int OC, int FH, int FW, const void *gz,
                       const int *g, int sy, int sx,
                       void *scratch, size_t scratch_bytes, void *stream, float beta) {
    const int M = B * IH * IW, T = FH * FW;
    const size_t mat = align256((size_t)M * T * OC * dtype_bytes(dtype));
    D8_REQUIRE(x && gw && gz, "d8_deconv2d_grad_y: null tensor");
    if (int rc = check_deconv_out("d8_deconv2d_grad_y", B, g)) return rc;
    {
        GemmArgs ga;
        if (deconv_implicit_grad_y(dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, g, x, gw, gz, ga)) {
            ga.beta = beta;
            return implicit_run(dtype, ga, 1, 0, scratch, scratch_bytes, as_stream(stream));
        }
    }
    if (int rc = need_scratch("d8_deconv2d_grad_y", scratch, scratch_bytes, (size_t)M * T * OC * dtype_bytes(dtype), x, gw, gz)) return rc;
    if (int rc = launch_im2col(dtype, gz, scratch, deconv_mirror(B, IH, IW, OC, FH, FW, sy, sx, g), as_stream(stream)))
        return rc;
    const size_t ws = scratch_bytes > mat ? scratch_bytes - mat : 0;
    Gemm plan = deconv_plan(2, M, T, OC, IC, scratch, gw, x);
    plan.beta = beta;
    return run(dtype, plan, ws ? (char *)scratch + mat : nullptr, ws, stream);
}

static int d8_deconv2d_grad_y_impl(int dtype, const void *x, int B, int IH, int IW, int IC,
                       void *gw, int OC, int FH, int FW, const void *gz,
                       int covered, int sy, int sx,
                       void *scratch, size_t scratch_bytes, void *stream, float beta) {
    int g[4];
    if (int rc = check_conv("d8_deconv2d_grad_y", dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, 1, 1)) return rc;
    if (int rc = d8_deconv2d_geometry(IH, IW, FH, FW, covered, sy, sx, g)) return rc;
    return deconv2d_grad_y_geo(dtype, x, B, IH, IW, IC, gw, OC, FH, FW, gz, g, sy, sx, scratch, scratch_bytes, stream, beta);
}

int d8_deconv2d_grad_y_ex(int dtype, const void *x, int B, int IH, int IW, int IC,
                          void *gw, int OC, int FH, int FW, const void *gz,
                          int OH, int OW, int padTop, int padLeft, int sy, int sx, int overwrite,
                          void *scratch, size_t scratch_bytes, void *stream) {
    const int g[4] = {OH, OW, padTop, padLeft};
    if (int rc = check_conv("d8_deconv2d_grad_y_ex", dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, 1, 1)) return rc;
    if (int rc = check_deconv_geo("d8_deconv2d_grad_y_ex", g)) return rc;
    return deconv2d_grad_y_geo(dtype, x, B, IH, IW, IC, gw, OC, FH, FW, gz, g, sy, sx, scratch, scratch_bytes, stream, overwrite ? 0.f : 1.f);
}

#define D8_CONV_GRAD_PAIR(name, first, grad)                                                                      \
    int name(int dtype, first, int B, int IH, int IW, int IC, grad, int OC, int FH, int FW, const void *gz,        \
             int covered, int sy, int sx, int dy, int dx, void *scratch, size_t scratch_bytes, void *stream) {       \
        return name##_impl(dtype, a0, B, IH, IW, IC, a1, OC, FH, FW, gz, covered, sy, sx, dy, dx, scratch,           \
                           scratch_bytes, stream, 1.f);                                                              \
    }                                                                                                                \
    int name##_overwrite(int dtype, first, int B, int IH, int IW, int IC, grad, int OC, int FH, int FW,             \
                         const void *gz, int covered, int sy, int sx, int dy, int dx, void *scratch,                 \
                         size_t scratch_bytes, void *stream) {                                                       \
        return name##_impl(dtype, a0, B, IH, IW, IC, a1, OC, FH, FW, gz, covered, sy, sx, dy, dx, scratch,           \
                           scratch_bytes, stream, 0.f);                                                              \
    }
#define D8_DECONV_GRAD_PAIR(name, first, grad)                                                                    \
    int name(int dtype, first, int B, int IH, int IW, int IC, grad, int OC, int FH, int FW, const void *gz,        \
             int covered, int sy, int sx, void *scratch, size_t scratch_bytes, void *stream) {                       \
        return name##_impl(dtype, a0, B, IH, IW, IC, a1, OC, FH, FW, gz, covered, sy, sx, scratch, scratch_bytes,    \
                           stream, 1.f);                                                                             \
    }                                                                                                                \
    int name##_overwrite(int dtype, first, int B, int IH, int IW, int IC, grad, int OC, int FH, int FW,             \
                         const void *gz, int covered, int sy, int sx, void *scratch, size_t scratch_bytes,           \
                         void *stream) {                                                                             \
        return name##_impl(dtype, a0, B, IH, IW, IC, a1, OC, FH, FW, gz, covered, sy, sx, scratch, scratch_bytes,    \
                           stream, 0.f);                                                                             \
    }

// the accumulating entry points and their overwrite forms (the destination's old contents ignored)
D8_CONV_GRAD_PAIR(d8_conv2d_grad_x, void *a0, const void *a1)
D8_CONV_GRAD_PAIR(d8_conv2d_grad_y, const void *a0, void *a1)
D8_DECONV_GRAD_PAIR(d8_deconv2d_grad_x, void *a0, const void *a1)
D8_DECONV_GRAD_PAIR(d8_deconv2d_grad_y, const void *a0, void *a1)

// Both gradients of a convolution from one call: what the _grad_x call followed by the _grad_y call leave
// (overwrite: bit 0 -- gx is written instead of added to, bit 1 -- gw likewise).  Where both gradients read their
// patch matrices inside the GEMM and each would leave compute units idle, they run as ONE launch
// (gemm_tiled_run_pair); otherwise one after the other.
int d8_conv2d_grad_xy(int dtype, const void *x, void *gx, int B, int IH, int IW, int IC,
                      const void *w, void *gw, int OC, int FH, int FW, const void *gz,
                      int covered, int sy, int sx, int dy, int dx, int overwrite,
                      void *scratch, size_t scratch_bytes, void *stream) {
    const float bx = (overwrite & 1) ? 0.f : 1.f, bw = (overwrite & 2) ? 0.f : 1.f;
    int g[4];
    if (int rc = check_conv("d8_conv2d_grad_xy", dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, dy, dx)) return rc;
    if (int rc = d8_conv2d_geometry(IH, IW, FH, FW, covered, sy, sx, dy, dx, g)) return rc;
    D8_REQUIRE(x && gx && w && gw && gz, "d8_conv2d_grad_xy: null tensor");
    {
        const ConvShape cs = {B, IH, IW, IC, OC, FH, FW, g[0], g[1], sy, sx, dy, dx, g[2], g[3]};
        GemmArgs px, pw;
        int ta, tb;
        if (conv_implicit_plan(dtype, 1, cs, gx, w, gz, px, ta, tb) && conv_implicit_plan(dtype, 2, cs, x, gw, gz, pw, ta, tb)) {
            px.beta = bx, pw.beta = bw;
            int rc = 0;
            if (gemm_tiled_run_pair(dtype, px, pw, scratch, scratch_bytes, as_stream(stream), &rc)) return rc;
        }
    }
    if (int rc = d8_conv2d_grad_x_impl(dtype, gx, B, IH, IW, IC, w, OC, FH, FW, gz, covered, sy, sx, dy, dx, scratch, scratch_bytes, stream, bx))
        return rc;
    return d8_conv2d_grad_y_impl(dtype, x, B, IH, IW, IC, gw, OC, FH, FW, gz, covered, sy, sx, dy, dx, scratch, scratch_bytes, stream, bw);
}

static int deconv2d_grad_xy_geo(int dtype, const void *x, void *gx, int B, int IH, int IW, int IC,
                                const void *w, void *gw, int OC, int FH, int FW, const void *gz,
                                const int *g, int sy, int sx, int overwrite,
                                void *scratch, size_t scratch_bytes, void *stream) {
    const float bx = (overwrite & 1) ? 0.f : 1.f, bw = (overwrite & 2) ? 0.f : 1.f;
    D8_REQUIRE(x && gx && w && gw && gz, "d8_deconv2d_grad_xy: null tensor");
    if (int rc = check_deconv_out("d8_deconv2d_grad_xy", B, g)) return rc;
    {
        GemmArgs px, pw;
        if (deconv_implicit_grad_x(dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, g, gx, w, gz, px) &&
            deconv_implicit_grad_y(dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, g, x, gw, gz, pw)) {
            px.beta = bx, pw.beta = bw;
            int rc = 0;
            if (gemm_tiled_run_pair(dtype, px, pw, scratch, scratch_bytes, as_stream(stream), &rc)) return rc;
        }
    }
    if (int rc = deconv2d_grad_x_geo(dtype, gx, B, IH, IW, IC, w, OC, FH, FW, gz, g, sy, sx, scratch, scratch_bytes, stream, bx)) return rc;
    return deconv2d_grad_y_geo(dtype, x, B, IH, IW, IC, gw, OC, FH, FW, gz, g, sy, sx, scratch, scratch_bytes, stream, bw);
}

int d8_deconv2d_grad_xy(int dtype, const void *x, void *gx, int B, int IH, int IW, int IC,
                        const void *w, void *gw, int OC, int FH, int FW, const void *gz,
                        int covered, int sy, int sx, int overwrite,
                        void *scratch, size_t scratch_bytes, void *stream) {
    int g[4];
    if (int rc = check_conv("d8_deconv2d_grad_xy", dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, 1, 1)) return rc;
    if (int rc = d8_deconv2d_geometry(IH, IW, FH, FW, covered, sy, sx, g)) return rc;
    return deconv2d_grad_xy_geo(dtype, x, gx, B, IH, IW, IC, w, gw, OC, FH, FW, gz, g, sy, sx, overwrite, scratch, scratch_bytes, stream);
}

int d8_deconv2d_grad_xy_ex(int dtype, const void *x, void *gx, int B, int IH, int IW, int IC,
                           const void *w, void *gw, int OC, int FH, int FW, const void *gz,
                           int OH, int OW, int padTop, int padLeft, int sy, int sx, int overwrite,
                           void *scratch, size_t scratch_bytes, void *stream) {
    const int g[4] = {OH, OW, padTop, padLeft};
    if (int rc = check_conv("d8_deconv2d_grad_xy_ex", dtype, B, IH, IW, IC, OC, FH, FW, sy, sx, 1, 1)) return rc;
    if (int rc = check_deconv_geo("d8_deconv2d_grad_xy_ex", g)) return rc;
    return deconv2d_grad_xy_geo(dtype, x, gx, B, IH, IW, IC, w, gw, OC, FH, FW, gz, g, sy, sx, overwrite, scratch, scratch_bytes, stream);
}

}  // extern "C"
