// Host side of the large-output fp16 GEMM (gemm_wide_kernel.h): eligibility, the launch of one product and the
// launch of two products as one (gemm_wide_pair_launch: the two gradients of a MatrixMultiply).
#include "gemm_wide_kernel.h"

// (what the kernels are built from; only diag/gemm_wide_diag.hip, which is not part of the library, sets another)
#ifndef D8_WIDE_POLICY
#define D8_WIDE_POLICY wide::Shipped
#endif

namespace d8 {

bool gemm_wide_eligible(const GemmArgs &g, int transA, int transB) {
    if (g.virt != VIRT_NONE || g.red != 1 || g.splits != 1) return false;
    if (transA && transB) return false;
    if (g.M < 256 || g.N < 256 || g.K < 64 || g.K % 64) return false;
    if (g.lda % 8 || g.ldb % 8 || g.ldc % 8 || g.sA % 8 || g.sB % 8 || g.sC % 8 || g.N % 8) return false;
    if (transA && g.M % 8) return false;
    if (((size_t)g.A | (size_t)g.B | (size_t)g.C | (size_t)g.bias) & 15) return false;
    if (2L * (transA ? g.K : g.M) * g.lda >= (1L << 31) || 2L * (transB ? g.N : g.K) * g.ldb >= (1L << 31)) return false;
    if ((long)ceil_div(g.M, 256) * ceil_div(g.N, 256) * g.batch > 0x3fffffffL) return false;
    return true;
}

size_t gemm_wide_stamp_bytes(const GemmArgs &g) {
    return (size_t)ceil_div(g.M, 256) * ceil_div(g.N, 256) * g.batch * 6 * sizeof(unsigned long long);
}

static wide::Product as_product(const GemmArgs &g, int transA, int transB) {
    wide::Product p;
    p.A = (const f16 *)g.A, p.B = (const f16 *)g.B, p.C = (f16 *)g.C, p.bias = (const f16 *)g.bias;
    p.M = g.M, p.N = g.N, p.K = g.K;
    p.lda = g.lda, p.ldb = g.ldb, p.ldc = g.ldc;
    p.sA = g.sA, p.sB = g.sB, p.sC = g.sC;
    p.tilesM = ceil_div(g.M, 256), p.tilesN = ceil_div(g.N, 256);
    p.tiles = p.tilesM * p.tilesN * g.batch;
    p.form = transA ? wide::FORM_TN : (transB ? wide::FORM_NT : wide::FORM_NN);
    p.beta = g.beta, p.relu = g.relu;
    return p;
}

// One workgroup per compute unit at most, each walking its share of the tiles; the grid is kept a multiple of
// eight (the XCD count: a workgroup's tiles then all fall to its own XCD's share) unless every tile gets its own.
static int grid_for(int total) {
    const int cus = cu_count();
    if (total <= cus) return total;
    return cus >= 8 ? cus - cus % 8 : cus;
}

template <int FORMS>
static int launch_forms(const wide::Launch &L, hipStream_t stream) {
    hipLaunchKernelGGL((gemm_wide_kernel<D8_WIDE_POLICY, FORMS>), dim3(grid_for(L.total)), dim3(256), 0, stream, L);
    D8_LAUNCH_CHECK();
    return 0;
}

static int launch(const wide::Launch &L, hipStream_t stream) {
    int forms = 0;
    for (int i = 0; i < L.n; ++i) forms |= 1 << L.p[i].form;
    switch (forms) {
        case 1: return launch_forms<1>(L, stream);
        case 2: return launch_forms<2>(L, stream);
        case 4: return launch_forms<4>(L, stream);
        case 6: return launch_forms<6>(L, stream);  // dX (NT) and dY (TN) of one MatrixMultiply
        default: return launch_forms<7>(L, stream);
    }
}

// measurement aid: with D8_GEMM_STAMPS in the environment and a workspace that holds them, the tiles write their
// phase records (wide::Launch::rec)
static unsigned long long *stamp_buffer(const GemmArgs &g) {
    static const bool stamps = getenv("D8_GEMM_STAMPS") != nullptr;
    const bool on = stamps && g.ws && ((size_t)g.ws & 7) == 0 && g.ws_bytes >= gemm_wide_stamp_bytes(g);
    return on ? (unsigned long long *)g.ws : nullptr;
}

int gemm_wide_launch(const GemmArgs &g, int transA, int transB, hipStream_t stream) {
    wide::Launch L;
    memset(&L, 0, sizeof(L));
    L.p[0] = as_product(g, transA, transB);
    L.n = 1, L.total = L.p[0].tiles;
    L.rec = stamp_buffer(g);
    return launch(L, stream);
}

int gemm_wide_pair_launch(const GemmArgs &g0, int transA0, int transB0, const GemmArgs &g1, int transA1, int transB1,
                          hipStream_t stream) {
    wide::Launch L;
    memset(&L, 0, sizeof(L));
    L.p[0] = as_product(g0, transA0, transB0);
    L.p[1] = as_product(g1, transA1, transB1);
    L.n = 2, L.total = L.p[0].tiles + L.p[1].tiles;
    // (records of both products in the first one's workspace, when it holds them)
    GemmArgs both = g0;
    both.batch = 1, both.M = 256, both.N = 256 * L.total;
    L.rec = stamp_buffer(both);
    return launch(L, stream);
}

}  // namespace d8
