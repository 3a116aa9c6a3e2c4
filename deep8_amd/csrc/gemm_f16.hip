// Tiled fp16 GEMM for gfx950: fp16 operands, fp32 accumulation on v_mfma_f32_32x32x16_f16.
//
// A workgroup owns a BM x BN tile of C and walks K in steps of 64.  While step t is multiplied
// out of one half of a double-buffered LDS area, the A and B tiles of step t+1 are written from
// registers into the other half and the tiles of step t+2 are fetched from global memory into
// those registers with 16-byte loads.  The loop body is written (and pinned with scheduling
// barriers) in issue order: every MFMA is followed by at most one LDS write, one global load and
// a couple of LDS reads, so the matrix pipe never waits behind a burst of memory instructions.
// The one workgroup barrier per step sits before the last quarter of the step's MFMAs, which
// then cover the latency of the first operand reads of the next step.
//
// Both tiles keep in LDS the layout they have in memory:
//   * an operand that is contiguous along K is stored [row][k] and read back with one 16-byte
//     LDS read per MFMA operand;
//   * an operand that is contiguous along M (A of a TN product) or N (B of an NN / TN product)
//     is stored [k][row] and read back with ds_read_b64_tr_b16, the transposing LDS read, which
//     hands each lane the four consecutive-k values of its row.  No transpose is ever materialised.
// Workgroup ids are remapped so that the workgroups one XCD receives (ids congruent mod 8) cover
// a compact block of tiles and share A / B panels in that XCD's L2.
#include "gemm_args.h"

namespace d8 {

typedef __fp16 f16x4v __attribute__((ext_vector_type(4)));
typedef __fp16 f16x8v __attribute__((ext_vector_type(8)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T *)(p))

// Four k-rows x 16 columns, transposed on the way out of LDS: the lane whose index within its
// group of 16 is i must pass the address of row (i / 4), columns 4 * (i % 4) .. + 3, and receives
// the four rows' values of column i.
__device__ __forceinline__ f16x8 lds_read_transposed(const f16 *p, int row_stride) {
    const f16x4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4f16(LDS_PTR(f16x4v, p));
    const f16x4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4f16(LDS_PTR(f16x4v, p + 4 * row_stride));
    const f16x8v both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(f16x8, both);
}

// instruction classes of __builtin_amdgcn_sched_group_barrier
#define SG_MFMA 0x008
#define SG_VMEM_READ 0x020
#define SG_DS_READ 0x100
#define SG_DS_WRITE 0x200

template <int BM_, int BN_, int WGM_, int WGN_, bool A_KC_, bool B_KC_>
struct F16Tile {
    static constexpr int BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_;
    static constexpr bool A_KC = A_KC_, B_KC = B_KC_;
    static constexpr int BK = 64;
    static constexpr int NT = WGM * WGN * 64;
    static constexpr int TM = BM / WGM / 32, TN = BN / WGN / 32, MT = TM * TN;
    // leading dimensions (in halfs) chosen so that the rows one LDS instruction touches fall into
    // different banks: +16 bytes for [row][k], +64 bytes for [k][row]
    static constexpr int A_LD = A_KC ? BK + 8 : BM + 32;
    static constexpr int B_LD = B_KC ? BK + 8 : BN + 32;
    static constexpr int A_SZ = A_KC ? BM * A_LD : BK * A_LD;
    static constexpr int B_SZ = B_KC ? BN * B_LD : BK * B_LD;
    // 16-byte pieces each thread moves per K step, and the rows one pass of all threads covers
    static constexpr int A_IT = BM * BK / 8 / NT, B_IT = BN * BK / 8 / NT, NP = A_IT + B_IT;
    static constexpr int A_ROWS = A_KC ? NT / 8 : NT / (BM / 8);
    static constexpr int B_ROWS = B_KC ? NT / 8 : NT / (BN / 8);
    // LDS read instructions per operand fragment
    static constexpr int A_RD = A_KC ? 1 : 2, B_RD = B_KC ? 1 : 2;
};

// Pieces [lo(q), lo(q+1)) are written to LDS during quarter q = 0, 1, 2 of a step and re-fetched
// from global memory during quarter q + 1.
template <int NP>
__device__ __host__ constexpr int piece_lo(int q) { return q * NP / 3; }
// The t-th of n events of a quarter goes right after MFMA number (t * MT) / n.
__device__ __host__ constexpr int slot_of(int t, int n, int MT) { return t * MT / n; }

// One K step.  Ar/Br: this lane's operand addresses in the LDS half being multiplied; An/Bn: the
// same in the other half (next step); Aw/Bw: where this thread's pieces of the next step go;
// ra/rb: buffer descriptors of the A and B matrices; ga/gb: wave-uniform byte offset (tile origin +
// K step) of the pieces of the step after that, a_off/b_off: this thread's byte offset in a piece.
// Uniform parts stay in scalar registers, so a piece costs one address VGPR per operand.
template <typename T>
__device__ __forceinline__ void k_step(const f16 *Ar, const f16 *Br, const f16 *An, const f16 *Bn, f16 *Aw, f16 *Bw,
                                       __amdgpu_buffer_rsrc_t ra, __amdgpu_buffer_rsrc_t rb, unsigned ga, unsigned gb,
                                       unsigned a_pass, unsigned b_pass, unsigned a_off, unsigned b_off,
                                       u32x4 (&R)[T::NP], f16x8 (&fa)[2][T::TM], f16x8 (&fb)[2][T::TN],
                                       f32x16 (&acc)[T::TM][T::TN]) {
    constexpr int TM = T::TM, TN = T::TN, MT = T::MT, NP = T::NP, A_IT = T::A_IT, NF = TM + TN;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        if (q == 3) __syncthreads();  // every wave has written its pieces and finished reading this half
        const int w_lo = q < 3 ? piece_lo<NP>(q) : 0, w_n = q < 3 ? piece_lo<NP>(q + 1) - w_lo : 0;
        const int g_lo = q > 0 ? piece_lo<NP>(q - 1) : 0, g_n = q > 0 ? piece_lo<NP>(q) - g_lo : 0;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            acc[m / TN][m % TN] =
                __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[q & 1][m / TN], fb[q & 1][m % TN], acc[m / TN][m % TN], 0, 0, 0);
#pragma unroll
            for (int t = 0; t < w_n; ++t)
                if (slot_of(t, w_n, MT) == m) {
                    const int p = w_lo + t;
                    f16 *dst = p < A_IT ? Aw + p * T::A_ROWS * T::A_LD : Bw + (p - A_IT) * T::B_ROWS * T::B_LD;
                    *(u32x4 *)dst = R[p];
                }
#pragma unroll
            for (int t = 0; t < g_n; ++t)
                if (slot_of(t, g_n, MT) == m) {
                    const int p = g_lo + t;
                    R[p] = p < A_IT ? __builtin_amdgcn_raw_buffer_load_b128(ra, a_off, ga + p * a_pass, 0)
                                    : __builtin_amdgcn_raw_buffer_load_b128(rb, b_off, gb + (p - A_IT) * b_pass, 0);
                }
            // operands of the next quarter (of the next step's first quarter when q == 3)
#pragma unroll
            for (int f = 0; f < NF; ++f)
                if (slot_of(f, NF, MT) == m) {
                    const int kk = q < 3 ? (q + 1) * 16 : 0;
                    const f16 *a_base = q < 3 ? Ar : An, *b_base = q < 3 ? Br : Bn;
                    if (f < TM)
                        fa[(q + 1) & 1][f] = T::A_KC ? *(const f16x8 *)(a_base + f * 32 * T::A_LD + kk)
                                                     : lds_read_transposed(a_base + kk * T::A_LD + f * 32, T::A_LD);
                    else
                        fb[(q + 1) & 1][f - TM] = T::B_KC ? *(const f16x8 *)(b_base + (f - TM) * 32 * T::B_LD + kk)
                                                          : lds_read_transposed(b_base + kk * T::B_LD + (f - TM) * 32, T::B_LD);
                }
        }
        // pin the issue order to the program order above
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
#pragma unroll
            for (int t = 0; t < w_n; ++t)
                if (slot_of(t, w_n, MT) == m) __builtin_amdgcn_sched_group_barrier(SG_DS_WRITE, 1, 0);
#pragma unroll
            for (int t = 0; t < g_n; ++t)
                if (slot_of(t, g_n, MT) == m) __builtin_amdgcn_sched_group_barrier(SG_VMEM_READ, 1, 0);
#pragma unroll
            for (int f = 0; f < NF; ++f)
                if (slot_of(f, NF, MT) == m) {
                    if (f < TM) __builtin_amdgcn_sched_group_barrier(SG_DS_READ, T::A_RD, 0);
                    else __builtin_amdgcn_sched_group_barrier(SG_DS_READ, T::B_RD, 0);
                }
        }
    }
}

template <typename T>
__global__ __launch_bounds__(T::NT) void gemm_f16_tiled_kernel(GemmArgs g, int tilesM, int tilesN) {
    constexpr int BM = T::BM, BN = T::BN, BK = T::BK, TM = T::TM, TN = T::TN, A_LD = T::A_LD, B_LD = T::B_LD;
    constexpr int A_IT = T::A_IT, NP = T::NP;
    constexpr bool A_KC = T::A_KC, B_KC = T::B_KC;
    // four separate arrays, so that reads of one half are known not to touch the other
    __shared__ __attribute__((aligned(16))) f16 As0[T::A_SZ];
    __shared__ __attribute__((aligned(16))) f16 As1[T::A_SZ];
    __shared__ __attribute__((aligned(16))) f16 Bs0[T::B_SZ];
    __shared__ __attribute__((aligned(16))) f16 Bs1[T::B_SZ];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / T::WGN, wn = wave % T::WGN;
    const int l32 = lane & 31, l16 = lane & 15, kg = (lane >> 5) * 8;

    // ---- which tile: ids of one XCD (same id mod 8) form a contiguous run, runs are laid out in
    // bands of GM tile rows walked column by column
    int id = blockIdx.x;
    const int total = tilesM * tilesN;
    if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    constexpr int GM = 4;
    const int band = id / (GM * tilesN), first = band * GM;
    const int rows_in_band = min(GM, tilesM - first);
    const int in_band = id - band * GM * tilesN;
    const int tm = first + in_band % rows_in_band, tn = in_band / rows_in_band;
    // A tile that would stick out of the matrix is moved back inside; the rows / columns it then
    // shares with its neighbour are computed twice but stored only by the neighbour.
    const int m_own = tm * BM, n_own = tn * BN;
    const int m0 = min(m_own, g.M - BM), n0 = min(n_own, g.N - BN);

    // ---- the 16-byte pieces this thread moves each K step: piece `it` of an operand lies a fixed
    // number of rows below piece 0, in global memory and in LDS alike.  Global memory is read
    // through buffer descriptors: byte offset = uniform part (tile origin, K step, piece; scalar
    // registers) + per-thread part (one VGPR per operand).
    const int b = blockIdx.z;
    const long a_rows = A_KC ? g.M : g.K, b_rows = B_KC ? g.N : g.K;
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((const f16 *)g.A + (long)b * g.sA), 0, (int)(2 * a_rows * g.lda), 0x00020000);
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((const f16 *)g.B + (long)b * g.sB), 0, (int)(2 * b_rows * g.ldb), 0x00020000);
    const unsigned Au = 2u * (A_KC ? (unsigned)m0 * g.lda : (unsigned)m0);
    const unsigned Bu = 2u * (B_KC ? (unsigned)n0 * g.ldb : (unsigned)n0);
    const int a_r = A_KC ? tid >> 3 : tid / (BM / 8), a_c = A_KC ? tid & 7 : tid % (BM / 8);
    const int b_r = B_KC ? tid >> 3 : tid / (BN / 8), b_c = B_KC ? tid & 7 : tid % (BN / 8);
    const unsigned a_off = 2u * ((unsigned)a_r * (unsigned)g.lda + a_c * 8);
    const unsigned b_off = 2u * ((unsigned)b_r * (unsigned)g.ldb + b_c * 8);
    const int a_dst = a_r * A_LD + a_c * 8, b_dst = b_r * B_LD + b_c * 8;
    const unsigned a_pass = 2u * T::A_ROWS * g.lda, b_pass = 2u * T::B_ROWS * g.ldb;  // bytes
    const unsigned a_step = A_KC ? 2u * BK : 2u * BK * g.lda;
    const unsigned b_step = B_KC ? 2u * BK : 2u * BK * g.ldb;

    // ---- per-lane LDS offsets of its MFMA operands
    const int a_frag = A_KC ? (wm * TM * 32 + l32) * A_LD + kg
                            : (kg + (l16 >> 2)) * A_LD + wm * TM * 32 + 16 * ((lane >> 4) & 1) + 4 * (l16 & 3);
    const int b_frag = B_KC ? (wn * TN * 32 + l32) * B_LD + kg
                            : (kg + (l16 >> 2)) * B_LD + wn * TN * 32 + 16 * ((lane >> 4) & 1) + 4 * (l16 & 3);

    u32x4 R[NP];
    f16x8 fa[2][TM], fb[2][TN];
    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // ---- prologue: step 0 into LDS half 0, step 1 into registers, first operands of step 0
    const int ktiles = g.K / BK;
#pragma unroll
    for (int p = 0; p < NP; ++p)
        R[p] = p < A_IT ? __builtin_amdgcn_raw_buffer_load_b128(ra, a_off, Au + p * a_pass, 0)
                        : __builtin_amdgcn_raw_buffer_load_b128(rb, b_off, Bu + (p - A_IT) * b_pass, 0);
#pragma unroll
    for (int p = 0; p < NP; ++p)
        *(u32x4 *)(p < A_IT ? As0 + a_dst + p * T::A_ROWS * A_LD : Bs0 + b_dst + (p - A_IT) * T::B_ROWS * B_LD) = R[p];
    {
        const int t1 = min(1, ktiles - 1);
        const unsigned pa = Au + t1 * a_step, pb = Bu + t1 * b_step;
#pragma unroll
        for (int p = 0; p < NP; ++p)
            R[p] = p < A_IT ? __builtin_amdgcn_raw_buffer_load_b128(ra, a_off, pa + p * a_pass, 0)
                            : __builtin_amdgcn_raw_buffer_load_b128(rb, b_off, pb + (p - A_IT) * b_pass, 0);
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TM; ++i)
        fa[0][i] = A_KC ? *(const f16x8 *)(As0 + a_frag + i * 32 * A_LD) : lds_read_transposed(As0 + a_frag + i * 32, A_LD);
#pragma unroll
    for (int j = 0; j < TN; ++j)
        fb[0][j] = B_KC ? *(const f16x8 *)(Bs0 + b_frag + j * 32 * B_LD) : lds_read_transposed(Bs0 + b_frag + j * 32, B_LD);

    // ---- main loop, two steps per trip so that the LDS half of every access is known statically;
    // fetches past the last step re-read the last step and are never used
    for (int kt = 0; kt < ktiles; kt += 2) {
        {
            const int t2 = min(kt + 2, ktiles - 1);
            k_step<T>(As0 + a_frag, Bs0 + b_frag, As1 + a_frag, Bs1 + b_frag, As1 + a_dst, Bs1 + b_dst,
                      ra, rb, Au + t2 * a_step, Bu + t2 * b_step, a_pass, b_pass, a_off, b_off, R, fa, fb, acc);
        }
        if (kt + 1 < ktiles) {
            const int t3 = min(kt + 3, ktiles - 1);
            k_step<T>(As1 + a_frag, Bs1 + b_frag, As0 + a_frag, Bs0 + b_frag, As0 + a_dst, Bs0 + b_dst,
                      ra, rb, Au + t3 * a_step, Bu + t3 * b_step, a_pass, b_pass, a_off, b_off, R, fa, fb, acc);
        }
    }

    // ---- epilogue.  Lane holds column l32 of rows 8*(r/4) + 4*(lane/32) + r%4 of each 32x32 block.
    f16 *Cg = (f16 *)g.C + (long)b * g.sC;
    const int lhi = lane >> 5;
    const bool vector_ok = (g.ldc % 8 == 0) && (g.sC % 8 == 0) && (((size_t)g.C & 15) == 0) && (g.N % 8 == 0);
    if (vector_ok) {
        // Each wave turns one 32x32 block at a time around through its own 32 x 36 float patch of
        // LDS (the A half is free once every wave is past the last step), so that a lane ends up
        // with 8 consecutive columns of one row: 16-byte loads of the old C and 16-byte stores.
        static_assert((size_t)T::A_SZ * sizeof(f16) >= (size_t)T::NT / 64 * 32 * 36 * sizeof(float), "patch space");
        __syncthreads();
        float *patch = (float *)As0 + wave * (32 * 36);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
#pragma unroll
                for (int r = 0; r < 16; ++r) patch[((r >> 2) * 8 + lhi * 4 + (r & 3)) * 36 + l32] = acc[i][j][r];
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const int q = lane + 64 * t, row = q >> 2, cc = (q & 3) * 8;
                    const int m = m0 + (wm * TM + i) * 32 + row, n = n0 + (wn * TN + j) * 32 + cc;
                    const f32x4 lo = *(const f32x4 *)(patch + row * 36 + cc), hi = *(const f32x4 *)(patch + row * 36 + cc + 4);
                    if (m >= m_own && n >= n_own) {
                        f16 *c = Cg + (long)m * g.ldc + n;
                        f16x8 o;
                        if (g.beta != 0.f) {
                            const f16x8 old = *(const f16x8 *)c;
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                o[e] = (f16)(lo[e] + (float)old[e]);
                                o[e + 4] = (f16)(hi[e] + (float)old[e + 4]);
                            }
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                o[e] = (f16)lo[e];
                                o[e + 4] = (f16)hi[e];
                            }
                        }
                        *(f16x8 *)c = o;
                    }
                }
            }
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + (wn * TN + j) * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + (wm * TM + i) * 32 + (r >> 2) * 8 + lhi * 4 + (r & 3);
                if (m >= m_own && n >= n_own) {
                    f16 *c = Cg + (long)m * g.ldc + n;
                    float v = acc[i][j][r];
                    if (g.beta != 0.f) v += (float)*c;
                    *c = (f16)v;
                }
            }
        }
}

template <int BM, int BN, int WGM, int WGN, bool A_KC, bool B_KC>
static int launch_tiled(const GemmArgs &g, hipStream_t stream) {
    typedef F16Tile<BM, BN, WGM, WGN, A_KC, B_KC> T;
    const int tilesM = ceil_div(g.M, BM), tilesN = ceil_div(g.N, BN);
    hipLaunchKernelGGL((gemm_f16_tiled_kernel<T>), dim3(tilesM * tilesN, 1, g.batch), dim3(T::NT), 0, stream, g, tilesM, tilesN);
    D8_LAUNCH_CHECK();
    return 0;
}

template <bool A_KC, bool B_KC>
static int pick_tile(const GemmArgs &g, hipStream_t stream) {
    static const char *force = getenv("D8_F16_TILE");  // tuning aid
    const long big_tiles = (long)ceil_div(g.M, 256) * ceil_div(g.N, 256) * g.batch;
    bool big = g.M >= 256 && g.N >= 256 && big_tiles >= (long)cu_count() * 3 / 4;
    if (force && g.M >= 256 && g.N >= 256) {
        switch (atoi(force)) {
        case 2: return launch_tiled<256, 256, 2, 4, A_KC, B_KC>(g, stream);
        case 4: return launch_tiled<256, 256, 2, 2, A_KC, B_KC>(g, stream);
        case 128: big = false; break;
        default: big = true;
        }
    }
    if (big) return launch_tiled<256, 256, 4, 2, A_KC, B_KC>(g, stream);
    return launch_tiled<128, 128, 2, 2, A_KC, B_KC>(g, stream);
}

bool gemm_f16_tiled(const GemmArgs &g, int transA, int transB, hipStream_t stream, int *rc) {
    if (g.red != 1 || g.splits != 1) return false;
    // byte offsets inside one matrix are 32-bit
    if ((long)(transA ? g.K : g.M) * g.lda >= (1L << 30) || (long)(transB ? g.N : g.K) * g.ldb >= (1L << 30)) return false;
    if (g.M < 128 || g.N < 128 || g.K < 64 || g.K % 64 || g.lda % 8 || g.ldb % 8 || g.sA % 8 || g.sB % 8) return false;
    if (((size_t)g.A | (size_t)g.B) & 15) return false;
    if (transA && g.M % 8) return false;
    if (!transB && g.N % 8) return false;
    if ((long)ceil_div(g.M, 128) * ceil_div(g.N, 128) > 0x7fffffffL || g.batch > 65535) return false;
    if (!transA && !transB) *rc = pick_tile<true, false>(g, stream);
    else if (!transA && transB) *rc = pick_tile<true, true>(g, stream);
    else *rc = pick_tile<false, false>(g, stream);
    return true;
}

}  // namespace d8
