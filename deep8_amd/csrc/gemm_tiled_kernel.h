// Tiled GEMM for gfx950, fp16 (v_mfma_f32_32x32x16_f16, fp32 accumulation) and fp32
// (v_mfma_f32_32x32x2_f32, true fp32 operands).
//
// A workgroup owns a BM x BN tile of C and walks K in steps of 128 bytes of a row (64 halfs or
// 32 floats).  While step t is multiplied out of one half of a double-buffered LDS area, the A
// and B tiles of step t+1 are written from registers into the other half and the tiles of step
// t+2 are fetched from global memory into those registers with 16-byte buffer loads (uniform
// address part in scalar registers, one offset VGPR per operand).  The loop body is written, and
// pinned with scheduling barriers, in issue order: every MFMA is followed by at most one LDS
// write, one global load and a couple of LDS reads, so the matrix pipe never waits behind a burst
// of memory instructions.  The one workgroup barrier per step sits before the last quarter of the
// step's MFMAs, which then cover the latency of the first operand reads of the next step.
//
// Both tiles keep in LDS the layout they have in memory; the transposed-operand products differ
// only in how the tiles are read back:
//   * an operand contiguous along K is stored [row][k]; one 16-byte LDS read gives a lane the 8
//     halfs (4 floats) of its row that it feeds to the next MFMA(s);
//   * an operand contiguous along M (A of a TN product) or N (B of an NN / TN product) is stored
//     [k][row]; fp16 reads it back with ds_read_b64_tr_b16, the transposing LDS read, which hands
//     each lane four consecutive-k values of its row; fp32 reads one float per k, consecutive
//     lanes reading consecutive addresses.  No transpose is ever materialised.
// Any pairing of k values with lanes works as long as A and B use the same one, because the MFMA
// sums over k; both element types pair lanes 0-31 with the first half of a k group and lanes
// 32-63 with the second half.
//
// Workgroup ids are remapped so that the workgroups one XCD receives (ids congruent mod 8) cover
// a compact block of tiles and share A / B panels in that XCD's L2.  The epilogue turns each
// 32 x 32 accumulator block around through LDS so that C is read and written 16 bytes per lane.
//
// An operand may be a patch matrix that is never written out (GemmArgs::virt): its loader turns
// row / column numbers into image offsets, and an offset outside the image makes the buffer load
// return zeros, which is the padding.  That carries the convolutions: Conv2d forward and its two
// gradients, DeConv2d's gradient of x and of the filter, and -- one residue class of output
// pixels per grid layer (OutClass) -- DeConv2d forward and Conv2d's gradient of x for strides
// above 1, whose rows of C are then pixels of the output image rather than consecutive rows.
//
// The same device covers ragged reductions and skinny matrices of real operands: in a last K step that is
// partly past K the pieces beyond K are fetched at an offset outside the buffer (zeros), and a matrix with
// fewer rows or columns than the tile is covered by a tile that starts at 0 and reaches past it -- what
// its loads bring in from there only enters results that are not stored.
#ifndef DEEP8_AMD_GEMM_TILED_KERNEL_H
#define DEEP8_AMD_GEMM_TILED_KERNEL_H

#include "gemm_args.h"

namespace d8 {

typedef __fp16 f16x4v __attribute__((ext_vector_type(4)));
typedef __fp16 f16x8v __attribute__((ext_vector_type(8)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T *)(p))

// instruction classes of __builtin_amdgcn_sched_group_barrier
#define SG_MFMA 0x008
#define SG_VMEM_READ 0x020
#define SG_DS_READ 0x100
#define SG_DS_WRITE 0x200

// ---- per element type: operand fragments and how to multiply one k group --------------------
template <typename E>
struct Elem;

template <>
struct Elem<f16> {
    typedef f16x8 Frag;                      // 8 k values of one row
    static constexpr int KG = 16;            // k values one fragment pair covers (2 lane halves x 8)
    static constexpr int MFMA_PER_FRAG = 1;  // MFMAs that consume one fragment pair
    static constexpr int TR_READS = 2;       // LDS instructions per fragment in the [k][row] layout
    static constexpr int TR_PAD = 64;        // bytes added to a [k][row] row: its 4 k-rows x 64 B hit different banks
    static constexpr int KC_HALF = 8;        // [row][k] tile: elements between what the two lane halves read
    // ... and inside a [k][row] tile: the lane whose index within its group of 16 is i addresses
    // k-row (i / 4), columns 4 * (i % 4) .. + 3 of its 16-column group, and receives column i
    __device__ static int tr_offset(int lane, int ld, int row0) {
        return ((lane >> 5) * 8 + ((lane & 15) >> 2)) * ld + row0 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    }
    __device__ static Frag read_kc(const f16 *p) { return *(const f16x8 *)p; }
    __device__ static Frag read_tr(const f16 *p, int ld) {
        const f16x4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4f16(LDS_PTR(f16x4v, p));
        const f16x4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4f16(LDS_PTR(f16x4v, p + 4 * ld));
        const f16x8v both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(f16x8, both);
    }
    __device__ static f32x16 mfma(const Frag &a, const Frag &b, const f32x16 &c, int) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

template <>
struct Elem<float> {
    typedef f32x4 Frag;  // lanes 0-31: k 0..3 of the group of 8, lanes 32-63: k 4..7
    static constexpr int KG = 8;
    static constexpr int MFMA_PER_FRAG = 4;  // MFMA e pairs k = e with k = 4 + e
    static constexpr int TR_READS = 4;
    static constexpr int TR_PAD = 32;  // k-rows 4 apart (the two lane halves) land in different bank halves
    static constexpr int KC_HALF = 4;
    __device__ static int tr_offset(int lane, int ld, int row0) { return (lane >> 5) * 4 * ld + row0 + (lane & 31); }
    __device__ static Frag read_kc(const float *p) { return *(const f32x4 *)p; }
    __device__ static Frag read_tr(const float *p, int ld) {
        Frag v;
        v[0] = p[0];
        v[1] = p[ld];
        v[2] = p[2 * ld];
        v[3] = p[3 * ld];
        return v;
    }
    __device__ static f32x16 mfma(const Frag &a, const Frag &b, const f32x16 &c, int e) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], c, 0, 0, 0);
    }
};

template <typename E_, int BM_, int BN_, int WGM_, int WGN_, bool A_KC_, bool B_KC_, int VIRT_ = VIRT_NONE>
struct Tile {
    typedef E_ E;
    typedef Elem<E> EL;
    static constexpr int BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_;
    static constexpr bool A_KC = A_KC_, B_KC = B_KC_;
    static constexpr int VIRT = VIRT_;  // which operand, if any, is a patch matrix read from its image
    static_assert((VIRT != VIRT_A_ROWS && VIRT != VIRT_A_CLASSES) || A_KC, "patch rows are K-contiguous");
    static_assert(VIRT != VIRT_B_KROWS || !B_KC, "patch k-rows are N-contiguous");
    static constexpr int ES = sizeof(E), EPV = 16 / ES;  // element size, elements per 16-byte piece
    static constexpr int BK = 128 / ES;                  // K step: 128 bytes of a row
    static constexpr int QUARTERS = 4, KQ = BK / QUARTERS;
    static_assert(KQ == EL::KG, "a quarter step is one k group");
    static constexpr int NT = WGM * WGN * 64;
    static constexpr int TM = BM / WGM / 32, TN = BN / WGN / 32;
    static constexpr int MQ = TM * TN * EL::MFMA_PER_FRAG;  // MFMAs per quarter step
    // A [row][k] tile keeps its rows (128 bytes each) in order with 16 bytes of padding after every
    // second row: the 16 rows that one cycle of a 16-byte LDS read touches then start in 16 different
    // groups of four banks, and two workgroup tiles of the 64-wide shapes stay under a third of the
    // CU's LDS.  A [k][row] tile has a leading dimension (A_LD / B_LD) with TR_PAD bytes of padding.
    __device__ __host__ static constexpr int kc_row(int r) { return r * BK + (r >> 1) * EPV; }
    static constexpr int KC_BLK = kc_row(32);  // elements between rows 32 apart (from an even row)
    static constexpr int A_LD = BM + EL::TR_PAD / ES, B_LD = BN + EL::TR_PAD / ES;
    static constexpr int A_SZ = A_KC ? kc_row(BM) : BK * A_LD;
    static constexpr int B_SZ = B_KC ? kc_row(BN) : BK * B_LD;
    // 16-byte pieces each thread moves per K step, and the rows one pass of all threads covers
    static constexpr int A_IT = BM * 8 / NT, B_IT = BN * 8 / NT, NP = A_IT + B_IT;
    static constexpr int A_ROWS = A_KC ? NT / 8 : NT / (BM / EPV);
    // Patch k-rows as B, fp32: the threads' passes walk the tile's columns instead of its rows -- a pass is all BK k-rows
    // x 32 columns, so a thread keeps ONE patch row per K step, decoded once, and its pieces differ by tap and channel
    // (an add and a bounds check each).  Decoding a row per piece cost Conv2d C4's filter gradient 11 of its 74 us.
    static constexpr bool B_COLS = VIRT == VIRT_B_KROWS && ES == 4 && NT / 8 == BK;
    static constexpr int B_ROWS = B_COLS ? BK : B_KC ? NT / 8 : NT / (BN / EPV);
    static_assert(A_ROWS % 2 == 0 && B_ROWS % 2 == 0, "a pass of all threads starts on an even row");
    // elements between the pieces two consecutive passes write, and between a wave's 32-row blocks
    static constexpr int A_PASS = A_KC ? kc_row(A_ROWS) : A_ROWS * A_LD, B_PASS = B_COLS ? 8 * EPV : B_KC ? kc_row(B_ROWS) : B_ROWS * B_LD;
    static constexpr int A_BLK = A_KC ? KC_BLK : 32, B_BLK = B_KC ? KC_BLK : 32;
    static constexpr int A_RD = A_KC ? 1 : EL::TR_READS, B_RD = B_KC ? 1 : EL::TR_READS;
    // the epilogue's transposing patches reuse the two halves of the larger operand area: the first
    // half of the waves turn their blocks around in one, the rest in the other
    static constexpr bool PATCH_IN_A = A_SZ >= B_SZ;
    static constexpr int PATCH_SZ = PATCH_IN_A ? A_SZ : B_SZ;
};

// Pieces [lo(q), lo(q+1)) are written to LDS during quarter q = 0, 1, 2 of a step and re-fetched
// from global memory during quarter q + 1.
template <int NP>
__device__ __host__ constexpr int piece_lo(int q) { return q * NP / 3; }
// The t-th of n events of a quarter goes right after MFMA number (t * MQ) / n.
__device__ __host__ constexpr int slot_of(int t, int n, int MQ) { return t * MQ / n; }

// One K step.  Ar/Br: this lane's operand addresses in the LDS half being multiplied; An/Bn: the
// same in the other half (next step); Aw/Bw: where this thread's pieces of the next step go;
// ra/rb: buffer descriptors of the A and B matrices; ga/gb: wave-uniform byte offset (tile origin +
// K step) of the pieces of the step after that, av/bv: this thread's byte offset for each piece.
template <typename T>
__device__ __forceinline__ void k_step(const typename T::E *Ar, const typename T::E *Br, const typename T::E *An,
                                       const typename T::E *Bn, typename T::E *Aw, typename T::E *Bw,
                                       __amdgpu_buffer_rsrc_t ra, __amdgpu_buffer_rsrc_t rb, unsigned ga, unsigned gb,
                                       unsigned a_pass, unsigned b_pass, const unsigned (&av)[T::A_IT],
                                       const unsigned (&bv)[T::B_IT], u32x4 (&R)[T::NP], typename T::EL::Frag (&fa)[2][T::TM],
                                       typename T::EL::Frag (&fb)[2][T::TN], f32x16 (&acc)[T::TM][T::TN]) {
    typedef typename T::E E;
    typedef typename T::EL EL;
    constexpr int TM = T::TM, TN = T::TN, MQ = T::MQ, NP = T::NP, A_IT = T::A_IT, NF = TM + TN;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        if (q == 3) __syncthreads();  // every wave has written its pieces and finished reading this half
        const int w_lo = q < 3 ? piece_lo<NP>(q) : 0, w_n = q < 3 ? piece_lo<NP>(q + 1) - w_lo : 0;
        const int g_lo = q > 0 ? piece_lo<NP>(q - 1) : 0, g_n = q > 0 ? piece_lo<NP>(q) - g_lo : 0;
#pragma unroll
        for (int m = 0; m < MQ; ++m) {
            {
                const int e = m / (TM * TN), ij = m % (TM * TN), i = ij / TN, j = ij % TN;
                acc[i][j] = EL::mfma(fa[q & 1][i], fb[q & 1][j], acc[i][j], e);
            }
#pragma unroll
            for (int t = 0; t < w_n; ++t)
                if (slot_of(t, w_n, MQ) == m) {
                    const int p = w_lo + t;
                    E *dst = p < A_IT ? Aw + p * T::A_PASS : Bw + (p - A_IT) * T::B_PASS;
                    *(u32x4 *)dst = R[p];
                }
#pragma unroll
            for (int t = 0; t < g_n; ++t)
                if (slot_of(t, g_n, MQ) == m) {
                    const int p = g_lo + t;
                    R[p] = p < A_IT ? __builtin_amdgcn_raw_buffer_load_b128(ra, av[p < A_IT ? p : 0], ga + p * a_pass, 0)
                                    : __builtin_amdgcn_raw_buffer_load_b128(rb, bv[p < A_IT ? 0 : p - A_IT], gb + (p - A_IT) * b_pass, 0);
                }
            // operands of the next quarter (of the next step's first quarter when q == 3)
#pragma unroll
            for (int f = 0; f < NF; ++f)
                if (slot_of(f, NF, MQ) == m) {
                    const int kk = q < 3 ? (q + 1) * T::KQ : 0;
                    const E *a_base = q < 3 ? Ar : An, *b_base = q < 3 ? Br : Bn;
                    if (f < TM)
                        fa[(q + 1) & 1][f] = T::A_KC ? EL::read_kc(a_base + f * T::A_BLK + kk)
                                                     : EL::read_tr(a_base + kk * T::A_LD + f * 32, T::A_LD);
                    else
                        fb[(q + 1) & 1][f - TM] = T::B_KC ? EL::read_kc(b_base + (f - TM) * T::B_BLK + kk)
                                                          : EL::read_tr(b_base + kk * T::B_LD + (f - TM) * 32, T::B_LD);
                }
        }
        // pin the issue order to the program order above
#pragma unroll
        for (int m = 0; m < MQ; ++m) {
            __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
#pragma unroll
            for (int t = 0; t < w_n; ++t)
                if (slot_of(t, w_n, MQ) == m) __builtin_amdgcn_sched_group_barrier(SG_DS_WRITE, 1, 0);
#pragma unroll
            for (int t = 0; t < g_n; ++t)
                if (slot_of(t, g_n, MQ) == m) __builtin_amdgcn_sched_group_barrier(SG_VMEM_READ, 1, 0);
#pragma unroll
            for (int f = 0; f < NF; ++f)
                if (slot_of(f, NF, MQ) == m) {
                    if (f < TM) __builtin_amdgcn_sched_group_barrier(SG_DS_READ, T::A_RD, 0);
                    else __builtin_amdgcn_sched_group_barrier(SG_DS_READ, T::B_RD, 0);
                }
        }
    }
}

__device__ inline float as_f32(float v) { return v; }
__device__ inline float as_f32(f16 v) { return (float)v; }

struct Origin {
    int m0, n0;        // where the computed tile starts (moved inside the matrix)
    int m_own, n_own;  // rows / columns from here on are this workgroup's to store
    int m_end, n_end;  // ... up to the matrix's own (a tile may be larger than a matrix with fewer than BM rows or BN columns)
    int wm0, wn0;      // this wave's offset inside the tile
};

// Store a wave's accumulators.  Lane holds column lane%32 of rows 8*(r/4) + 4*(lane/32) + r%4 of
// each 32x32 block.  Where rows of C can be moved 16 bytes at a time, each block is turned around
// through the wave's own 32 x 36 float patch of LDS, so that a lane ends up with 8 consecutive
// columns of one row: 16-byte loads of the old C and 16-byte stores.
// C row of tile row m: m itself, or the output pixel of row (b, y', x') of a class of a transposed convolution
struct RowMap {
    int plane, OW;                           // 0: identity
    int out_H, out_W, out_sy, out_sx, py, px;
    int perm_T, perm_OC;                     // perm_OC > 0: stored transposed per tap (GemmArgs::perm_OC)
    __device__ long operator()(int m) const {
        if (!plane) return m;
        const int img = m / plane, rem = m - img * plane, y = rem / OW, x = rem - y * OW;
        return ((long)img * out_H + out_sy * y + py) * out_W + out_sx * x + px;
    }
    __device__ long at(int m, int n, int ldc) const {
        if (perm_OC) {
            const int t = n / perm_OC, oc = n - t * perm_OC;
            return ((long)oc * perm_T + t) * ldc + m;
        }
        return (*this)(m) * ldc + n;
    }
};

template <typename T, typename O>
__device__ __forceinline__ void store_tile(f32x16 (&acc)[T::TM][T::TN], float *lds0, float *lds1, O *C, int ldc, float beta,
                                           bool aligned, int N, const Origin &o, const RowMap &crow,
                                           const O *bias = nullptr, bool relu = false) {
    constexpr int TM = T::TM, TN = T::TN, OPV = 16 / sizeof(O);
    typedef O OV __attribute__((ext_vector_type(OPV)));
    constexpr int HALF_WAVES = T::NT / 128;
    static_assert((size_t)T::PATCH_SZ * T::ES >= (size_t)HALF_WAVES * 32 * 36 * sizeof(float), "patch space");
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, lhi = lane >> 5;
    if (aligned && N % 8 == 0 && !crow.perm_OC && ((size_t)bias & 15) == 0) {
        float *patch = (wave < HALF_WAVES ? lds0 + wave * (32 * 36) : lds1 + (wave - HALF_WAVES) * (32 * 36));
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
#pragma unroll
                for (int r = 0; r < 16; ++r) patch[((r >> 2) * 8 + lhi * 4 + (r & 3)) * 36 + l32] = acc[i][j][r];
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const int q = lane + 64 * t, row = q >> 2, cc = (q & 3) * 8;
                    const int m = o.m0 + o.wm0 + i * 32 + row, n = o.n0 + o.wn0 + j * 32 + cc;
                    float v[8];
                    *(f32x4 *)&v[0] = *(const f32x4 *)(patch + row * 36 + cc);
                    *(f32x4 *)&v[4] = *(const f32x4 *)(patch + row * 36 + cc + 4);
                    if (m >= o.m_own && n >= o.n_own && m < o.m_end && n < o.n_end) {
                        O *c = C + crow(m) * ldc + n;
#pragma unroll
                        for (int h = 0; h < 8 / OPV; ++h) {
                            OV out;
                            if (beta != 0.f) {
                                const OV old = *(const OV *)(c + h * OPV);
#pragma unroll
                                for (int e = 0; e < OPV; ++e) v[h * OPV + e] += as_f32(old[e]);
                            }
                            if (bias) {
                                const OV bv = *(const OV *)(bias + n + h * OPV);
#pragma unroll
                                for (int e = 0; e < OPV; ++e) v[h * OPV + e] += as_f32(bv[e]);
                            }
#pragma unroll
                            for (int e = 0; e < OPV; ++e) out[e] = (O)(relu && !(v[h * OPV + e] > 0.f) ? 0.f : v[h * OPV + e]);
                            *(OV *)(c + h * OPV) = out;
                        }
                    }
                }
            }
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = o.n0 + o.wn0 + j * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = o.m0 + o.wm0 + i * 32 + (r >> 2) * 8 + lhi * 4 + (r & 3);
                if (m >= o.m_own && n >= o.n_own && m < o.m_end && n < o.n_end) {
                    O *c = C + crow.at(m, n, ldc);
                    float v = acc[i][j][r];
                    if (beta != 0.f) v += as_f32(*c);
                    if (bias) v += as_f32(bias[n]);
                    *c = (O)(relu && !(v > 0.f) ? 0.f : v);
                }
            }
        }
}

// The work of one workgroup: workgroup (bx, bz) of a grid of nbx x layers (the launch's own blockIdx / gridDim, or what a
// launch of two products makes of them).  As0 .. Bs1: the two halves of both operand areas in LDS.
template <typename T, bool TAIL>
__device__ __forceinline__ void gemm_tiled_body(const GemmArgs &g, int tilesM, const int tilesN, const int bx, const int bz, const int nbx,
                                                typename T::E *As0, typename T::E *As1, typename T::E *Bs0, typename T::E *Bs1) {
    typedef typename T::E E;
    typedef typename T::EL EL;
    typedef E EV __attribute__((ext_vector_type(T::EPV)));
    constexpr int BM = T::BM, BN = T::BN, BK = T::BK, TM = T::TM, TN = T::TN, A_LD = T::A_LD, B_LD = T::B_LD;
    constexpr int A_IT = T::A_IT, NP = T::NP, ES = T::ES, EPV = T::EPV;
    constexpr bool A_KC = T::A_KC, B_KC = T::B_KC;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / T::WGN, wn = wave % T::WGN;
    unsigned long long st_w[4] = {0, 0, 0, 0}, st_c[2] = {0, 0};  // phase record (GemmArgs::phase_rec), a measurement aid
    if (g.phase_rec) st_w[0] = wall_clock64();

    // ---- which tile: ids of one XCD (same id mod 8) form a contiguous run, runs are laid out in
    // bands of GM tile rows walked column by column
    // blockIdx.z = output batch index * splits + piece of the reduction.  The reduction runs over
    // `red` products (1 unless the whole batch is summed into one C) times K, cut into `splits`.
    // The tiles of one piece read the same rows of A and B, so they should meet in one L2: the
    // launch's workgroups (x fastest, then z) go to the XCDs in turn, and the ids one XCD receives
    // are therefore dealt out piece by piece, all tiles of a piece before the next.
    constexpr int VIRT = T::VIRT, B_IT = T::B_IT;
    constexpr bool VA = VIRT == VIRT_A_ROWS || VIRT == VIRT_A_CLASSES;  // A's rows are patch rows
    PatchGeom pg = g.pg;
    int M = g.M, red = g.red;
    unsigned b_cls = 0;
    RowMap crow = {0, 0, 0, 0, 0, 0, 0, 0, g.perm_T, g.perm_OC};
    const RowMap plain = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    if constexpr (VIRT == VIRT_A_CLASSES) {
        const OutClass &c = g.cls[bz];
        M = c.M, red = c.red, b_cls = c.b_off;
        pg.OH = c.OH, pg.OW = c.OW, pg.FW = c.taps_w, pg.pt = c.pt, pg.pl = c.pl;
        crow = {c.OH * c.OW, c.OW, g.out_H, g.out_W, g.out_sy, g.out_sx, c.py, c.px, 0, 0};
        tilesM = (M + BM - 1) / BM;
        if (bx >= tilesM * tilesN) return;  // the grid is sized for the largest class
    }
    int id = bx;
    const int total = tilesM * tilesN;
    int b = VIRT == VIRT_A_CLASSES ? 0 : bz / g.splits;
    int split = VIRT == VIRT_A_CLASSES ? 0 : bz - b * g.splits;
    // a workgroup past the product's own tiles works on the remainder band (GemmArgs::tail_m0)
    const bool in_tail = VIRT != VIRT_A_CLASSES && g.tail_splits > 0 && id >= total;
    int tps = g.tiles_per_split;
    if (in_tail) {
        const int t = id - total;
        split = t % g.tail_splits;
        id = t / g.tail_splits;  // tile of the band, column by column
        tps = g.tail_tps;
    } else {
        // an unsplit batched product is dealt out the same way over its batch index: one XCD takes all
        // tiles of a batch element, whose A and B it then reads once
        const bool by_batch = g.splits == 1;
        int layer = by_batch ? b : split;
        const int layers = by_batch ? g.batch : g.splits;
        const int linear = id + total * layer, whole = total * (layers & ~7);
        if (linear < whole) {
            const int j = linear >> 3, piece = j / total;
            layer = (piece << 3) + (linear & 7);
            id = j - piece * total;
        } else if ((total & 7) == 0) {
            id = (id & 7) * (total >> 3) + (id >> 3);
        }
        if (by_batch) b = layer;
        else split = layer;
    }
    constexpr int GM = 4;
    const int band = id / (GM * tilesN), first = band * GM;
    const int rows_in_band = max(1, min(GM, tilesM - first));
    const int in_band = id - band * GM * tilesN;
    const int tail_tilesM = in_tail ? (M - g.tail_m0 + BM - 1) / BM : 1;
    const int tm = in_tail ? id % tail_tilesM : first + in_band % rows_in_band;
    const int tn = in_tail ? id / tail_tilesM : in_band / rows_in_band;
    // A tile that would stick out of the matrix is moved back inside; the rows / columns it then
    // shares with its neighbour are computed twice but stored only by the neighbour.
    const int m_own = (in_tail ? g.tail_m0 : 0) + tm * BM, n_own = tn * BN;
    // (a matrix with fewer rows or columns than the tile: the tile starts at 0 and reaches past it; what the loads
    // bring in from there -- zeros past the end of the buffer, otherwise whatever follows -- only ever enters
    // results of rows / columns past the matrix, which are not stored)
    const int m0 = max(0, min(m_own, M - BM)), n0 = max(0, min(n_own, g.N - BN));

    // ---- the 16-byte pieces this thread moves each K step: piece `it` of an operand lies a fixed
    // number of rows below piece 0, in global memory and in LDS alike.  Global memory is read
    // through buffer descriptors: byte offset = uniform part (tile origin, K step, piece; scalar
    // registers) + per-thread part (one VGPR per operand).
    const long a_rows = A_KC ? g.M : g.K, b_rows = B_KC ? g.N : g.K;
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((const E *)g.A + (long)b * g.sA), 0,
        VA ? (int)pg.bytes : (int)(ES * ((g.red - 1) * g.sA + a_rows * g.lda)), 0x00020000);
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((const E *)g.B + (long)b * g.sB), 0,
        VIRT == VIRT_B_KROWS ? (int)pg.bytes
                             // (the taps of a filter interleave inside its rows: the filter ends with its last row)
                             : (int)(ES * ((VA ? 0 : (g.red - 1) * g.sB) + b_rows * g.ldb)), 0x00020000);
    const unsigned Au = (unsigned)ES * (A_KC ? (unsigned)m0 * g.lda : (unsigned)m0);
    const unsigned Bu = (unsigned)ES * (B_KC ? (unsigned)n0 * g.ldb : (unsigned)n0);
    const int a_r = A_KC ? tid >> 3 : tid / (BM / EPV), a_c = A_KC ? tid & 7 : tid % (BM / EPV);
    const int b_r = (B_KC || T::B_COLS) ? tid >> 3 : tid / (BN / EPV), b_c = (B_KC || T::B_COLS) ? tid & 7 : tid % (BN / EPV);
    const int a_dst = (A_KC ? T::kc_row(a_r) : a_r * A_LD) + a_c * EPV, b_dst = (B_KC ? T::kc_row(b_r) : b_r * B_LD) + b_c * EPV;
    const unsigned a_pass = VA ? 0u : (unsigned)ES * T::A_ROWS * g.lda;  // bytes
    const unsigned b_pass = VIRT == VIRT_B_KROWS ? 0u : (unsigned)ES * T::B_ROWS * g.ldb;
    const unsigned a_step = A_KC ? 128u : (unsigned)ES * BK * g.lda;
    const unsigned b_step = B_KC ? 128u : (unsigned)ES * BK * g.ldb;
    // per-thread byte offset of each piece: one value for a real matrix, recomputed every step
    // for a patch matrix (an offset beyond the image makes the buffer load return zeros)
    constexpr unsigned OUTSIDE = 0x80000000u;
    unsigned av[A_IT], bv[B_IT];
#pragma unroll
    for (int p = 0; p < A_IT; ++p) av[p] = (unsigned)ES * ((unsigned)a_r * (unsigned)g.lda + a_c * EPV);
#pragma unroll
    for (int p = 0; p < B_IT; ++p) bv[p] = (unsigned)ES * ((unsigned)b_r * (unsigned)g.ldb + b_c * EPV);
    // patch rows as A: this thread's rows never change; a step selects the tap
    int va_base[A_IT], va_iy[A_IT], va_ix[A_IT];
    if constexpr (VA) {
        const int plane = pg.OH * pg.OW;
#pragma unroll
        for (int p = 0; p < A_IT; ++p) {
            const int m = g.m_base + m0 + a_r + p * T::A_ROWS, img = m / plane, rem = m - img * plane;
            const int oy = rem / pg.OW, ox = rem - oy * pg.OW;
            va_iy[p] = oy * pg.sy - pg.pt;
            va_ix[p] = ox * pg.sx - pg.pl;
            va_base[p] = (((img * pg.H + va_iy[p]) * pg.W + va_ix[p]) * pg.C + a_c * EPV) * ES;
        }
    }
    // patch k-rows as B: this thread's tap and channel never change; a step selects the rows
    // (with column passes, Tile::B_COLS: this thread's k-row within the step never changes; piece p has its own tap and channel)
    int vb_dy = 0, vb_dx = 0, vb_c = 0;
    int vb_ty[B_IT], vb_tx[B_IT], vb_off[B_IT];
    if constexpr (T::B_COLS) {
#pragma unroll
        for (int p = 0; p < B_IT; ++p) {
            const int n = n0 + p * T::B_PASS + b_c * EPV, t = n / pg.C, fy = t / pg.FW, fx = t - fy * pg.FW;
            vb_ty[p] = fy * pg.dy;
            vb_tx[p] = fx * pg.dx;
            vb_off[p] = ((vb_ty[p] * pg.W + vb_tx[p]) * pg.C + (n - t * pg.C)) * ES;
        }
    } else if constexpr (VIRT == VIRT_B_KROWS) {
        const int n = n0 + b_c * EPV, t = n / pg.C, fy = t / pg.FW, fx = t - fy * pg.FW;
        vb_c = n - t * pg.C;
        vb_dy = fy * pg.dy - pg.pt;
        vb_dx = fx * pg.dx - pg.pl;
    }

    // ---- per-lane LDS offsets of its MFMA operands
    const int a_frag = A_KC ? T::kc_row(wm * TM * 32 + (lane & 31)) + (lane >> 5) * EL::KC_HALF : EL::tr_offset(lane, A_LD, wm * TM * 32);
    const int b_frag = B_KC ? T::kc_row(wn * TN * 32 + (lane & 31)) + (lane >> 5) * EL::KC_HALF : EL::tr_offset(lane, B_LD, wn * TN * 32);

    u32x4 R[NP];
    typename EL::Frag fa[2][TM], fb[2][TN];
    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // ---- this workgroup's steps x0 .. x0 + nsteps - 1 of the extended reduction; step x reads
    // product x / ktiles at K offset (x % ktiles) * BK (all uniform: scalar arithmetic)
    // K need not be a multiple of the K step for real matrices: the last step of a product is then partly past
    // K, and the pieces that lie past it are fetched at an offset beyond the buffer, i.e. as zeros.
    const int ktiles = (g.K + BK - 1) / BK, tail_len = g.K % BK;
    const unsigned av_plain = (unsigned)ES * ((unsigned)a_r * (unsigned)g.lda + a_c * EPV);
    const unsigned bv_plain = (unsigned)ES * ((unsigned)b_r * (unsigned)g.ldb + b_c * EPV);
    const int x0 = split * tps, nsteps = min(red * ktiles, x0 + tps) - x0;
    const unsigned a_prod = (unsigned)ES * (unsigned)g.sA, b_prod = (unsigned)ES * (unsigned)g.sB;
    const unsigned b_prod_row = (unsigned)ES * (unsigned)g.sB_row, b_first = (unsigned)ES * b_cls;
    auto step_a = [&](int i) -> unsigned {
        const int x = x0 + min(i, nsteps - 1), r = x / ktiles;  // past the end: refetch the last step, never used
        if constexpr (VA) {
            const int fy = r / pg.FW, fx = r - fy * pg.FW, tdy = fy * pg.dy, tdx = fx * pg.dx;
            const int toff = ((tdy * pg.W + tdx) * pg.C + (x - r * ktiles) * BK) * ES;
#pragma unroll
            for (int p = 0; p < A_IT; ++p) {
                const bool inside = (unsigned)(va_iy[p] + tdy) < (unsigned)pg.H && (unsigned)(va_ix[p] + tdx) < (unsigned)pg.W;
                av[p] = inside ? (unsigned)(va_base[p] + toff) : OUTSIDE;
            }
            return 0u;
        } else {
            const int kx = x - r * ktiles;
            if constexpr (VIRT == VIRT_NONE) {
                if constexpr (TAIL) {
                    const bool tail = kx == ktiles - 1;
#pragma unroll
                    for (int p = 0; p < A_IT; ++p) {
                        const bool past = A_KC ? a_c * EPV >= tail_len : a_r + p * T::A_ROWS >= tail_len;
                        av[p] = tail && past ? OUTSIDE : av_plain;
                    }
                }
            }
            return Au + (g.red > 1 ? r * a_prod : 0u) + kx * a_step;
        }
    };
    auto step_b = [&](int i) -> unsigned {
        const int x = x0 + min(i, nsteps - 1), r = x / ktiles;
        if constexpr (T::B_COLS) {
            const unsigned plane = pg.OH * pg.OW, m = (unsigned)x * BK + b_r;
            unsigned img = __umulhi(m, pg.mg_plane), rem = m - img * plane;
            if (rem >= plane) ++img, rem -= plane;
            unsigned oy = __umulhi(rem, pg.mg_ow), ox = rem - oy * pg.OW;
            if (ox >= (unsigned)pg.OW) ++oy, ox -= pg.OW;
            const int iy0 = (int)oy * pg.sy - pg.pt, ix0 = (int)ox * pg.sx - pg.pl;
            const int base = (((int)img * pg.H + iy0) * pg.W + ix0) * pg.C * ES;
#pragma unroll
            for (int p = 0; p < B_IT; ++p) {
                const bool inside = (unsigned)(iy0 + vb_ty[p]) < (unsigned)pg.H && (unsigned)(ix0 + vb_tx[p]) < (unsigned)pg.W;
                bv[p] = inside ? (unsigned)(base + vb_off[p]) : OUTSIDE;
            }
            return 0u;
        } else if constexpr (VIRT == VIRT_B_KROWS) {
            const unsigned plane = pg.OH * pg.OW;
#pragma unroll
            for (int p = 0; p < B_IT; ++p) {
                const unsigned m = (unsigned)x * BK + b_r + p * T::B_ROWS;
                unsigned img = __umulhi(m, pg.mg_plane), rem = m - img * plane;
                if (rem >= plane) ++img, rem -= plane;
                unsigned oy = __umulhi(rem, pg.mg_ow), ox = rem - oy * pg.OW;
                if (ox >= (unsigned)pg.OW) ++oy, ox -= pg.OW;
                const int iy = (int)oy * pg.sy + vb_dy, ix = (int)ox * pg.sx + vb_dx;
                const bool inside = (unsigned)iy < (unsigned)pg.H && (unsigned)ix < (unsigned)pg.W;
                bv[p] = inside ? (unsigned)(((((int)img * pg.H + iy) * pg.W + ix) * pg.C + vb_c) * ES) : OUTSIDE;
            }
            return 0u;
        } else if constexpr (VIRT == VIRT_A_CLASSES) {
            const int fy = r / pg.FW, fx = r - fy * pg.FW;
            return Bu + b_first + fy * b_prod_row + fx * b_prod + (x - r * ktiles) * b_step;
        } else {
            const int kx = x - r * ktiles;
            if constexpr (VIRT == VIRT_NONE) {
                if constexpr (TAIL) {
                    const bool tail = kx == ktiles - 1;
#pragma unroll
                    for (int p = 0; p < B_IT; ++p) {
                        const bool past = B_KC ? b_c * EPV >= tail_len : b_r + p * T::B_ROWS >= tail_len;
                        bv[p] = tail && past ? OUTSIDE : bv_plain;
                    }
                }
            }
            return Bu + (g.red > 1 ? r * b_prod : 0u) + kx * b_step;
        }
    };

    // ---- prologue: step 0 into LDS half 0, step 1 into registers, first operands of step 0
    {
        const unsigned pa = step_a(0), pb = step_b(0);
#pragma unroll
        for (int p = 0; p < NP; ++p)
            R[p] = p < A_IT ? __builtin_amdgcn_raw_buffer_load_b128(ra, av[p < A_IT ? p : 0], pa + p * a_pass, 0)
                            : __builtin_amdgcn_raw_buffer_load_b128(rb, bv[p < A_IT ? 0 : p - A_IT], pb + (p - A_IT) * b_pass, 0);
    }
#pragma unroll
    for (int p = 0; p < NP; ++p)
        *(u32x4 *)(p < A_IT ? As0 + a_dst + p * T::A_PASS : Bs0 + b_dst + (p - A_IT) * T::B_PASS) = R[p];
    {
        const unsigned pa = step_a(1), pb = step_b(1);
#pragma unroll
        for (int p = 0; p < NP; ++p)
            R[p] = p < A_IT ? __builtin_amdgcn_raw_buffer_load_b128(ra, av[p < A_IT ? p : 0], pa + p * a_pass, 0)
                            : __builtin_amdgcn_raw_buffer_load_b128(rb, bv[p < A_IT ? 0 : p - A_IT], pb + (p - A_IT) * b_pass, 0);
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TM; ++i)
        fa[0][i] = A_KC ? EL::read_kc(As0 + a_frag + i * T::A_BLK) : EL::read_tr(As0 + a_frag + i * 32, A_LD);
#pragma unroll
    for (int j = 0; j < TN; ++j)
        fb[0][j] = B_KC ? EL::read_kc(Bs0 + b_frag + j * T::B_BLK) : EL::read_tr(Bs0 + b_frag + j * 32, B_LD);

    if (g.phase_rec) st_w[1] = wall_clock64(), st_c[0] = __builtin_readcyclecounter();
    // ---- main loop, two steps per trip so that the LDS half of every access is known statically;
    for (int i = 0; i < nsteps; i += 2) {
        {
            const unsigned pa = step_a(i + 2), pb = step_b(i + 2);
            k_step<T>(As0 + a_frag, Bs0 + b_frag, As1 + a_frag, Bs1 + b_frag, As1 + a_dst, Bs1 + b_dst, ra, rb, pa, pb,
                      a_pass, b_pass, av, bv, R, fa, fb, acc);
        }
        if (i + 1 < nsteps) {
            const unsigned pa = step_a(i + 3), pb = step_b(i + 3);
            k_step<T>(As1 + a_frag, Bs1 + b_frag, As0 + a_frag, Bs0 + b_frag, As0 + a_dst, Bs0 + b_dst, ra, rb, pa, pb,
                      a_pass, b_pass, av, bv, R, fa, fb, acc);
        }
    }

    if (g.phase_rec) st_w[2] = wall_clock64(), st_c[1] = __builtin_readcyclecounter();
    // ---- epilogue: the result itself, or this piece's fp32 partial sums when the reduction is split
    __syncthreads();  // every wave is past the last step: the operand areas are free
    const Origin o = {m0, n0, m_own, n_own, M, g.N, (wm * TM) * 32, (wn * TN) * 32};
    float *patches = (float *)(T::PATCH_IN_A ? As0 : Bs0), *patches1 = (float *)(T::PATCH_IN_A ? As1 : Bs1);
    if (in_tail) {  // partial sums of the band, rows counted from its first
        const int tail_M = M - g.tail_m0;
        const Origin ot = {m0 - g.tail_m0, n0, m_own - g.tail_m0, n_own, tail_M, g.N, (wm * TM) * 32, (wn * TN) * 32};
        store_tile<T, float>(acc, patches, patches1, g.ws + ((long)split * tail_M) * g.N, g.N, 0.f, true, g.N, ot, plain);
    } else if (g.splits > 1)
        store_tile<T, float>(acc, patches, patches1, g.ws + ((long)(b * g.splits + split) * g.M) * g.N, g.N, 0.f, true, g.N, o, plain);
    else
        store_tile<T, E>(acc, patches, patches1, (E *)g.C + (long)b * g.sC, g.ldc, g.beta,
                         g.ldc % EPV == 0 && g.sC % EPV == 0 && ((size_t)g.C & 15) == 0, g.N, o, crow, (const E *)g.bias, g.relu != 0);
    if (g.phase_rec) {
        __builtin_amdgcn_s_waitcnt(0x0f70);  // this wave's stores have been acknowledged
        st_w[3] = wall_clock64();
        if (tid == 0) {
            unsigned long long *rec = g.phase_rec + 8 * (bx + (unsigned long long)nbx * bz);
            rec[0] = st_w[0], rec[1] = st_w[1], rec[2] = st_w[2], rec[3] = st_w[3], rec[4] = st_c[0], rec[5] = st_c[1];
            // s_getreg_b32 of all 32 bits of hardware registers 20 (XCC_ID) and 4 (HW_ID: wave, SIMD, CU, SH, SE)
            rec[6] = ((unsigned long long)__builtin_amdgcn_s_getreg((31 << 11) | 20) << 32) | __builtin_amdgcn_s_getreg((31 << 11) | 4);
            rec[7] = (in_tail ? 1 : 0) | (g.stamps << 1);  // (stamps: which product of a launch of two)
        }
    }
}

// TAIL: K is not a multiple of the K step (an instantiation of its own, so that the per-piece offsets of the
// ordinary case stay constants)
template <typename T, bool TAIL = false>
__global__ __launch_bounds__(T::NT) void gemm_tiled_kernel(GemmArgs g, int tilesM, int tilesN) {
    typedef typename T::E E;
    // four separate arrays, so that reads of one half are known not to touch the other
    __shared__ __attribute__((aligned(16))) E As0[T::A_SZ];
    __shared__ __attribute__((aligned(16))) E As1[T::A_SZ];
    __shared__ __attribute__((aligned(16))) E Bs0[T::B_SZ];
    __shared__ __attribute__((aligned(16))) E Bs1[T::B_SZ];
    gemm_tiled_body<T, TAIL>(g, tilesM, tilesN, (int)blockIdx.x, (int)blockIdx.z, (int)gridDim.x, As0, As1, Bs0, Bs1);
}

// Two products in one launch: the first nx0 * nz0 workgroups are the first product's grid (x fastest), the rest the
// second's.  Built for the two gradients of a convolution on a small layer, which are independent of each other and
// each leave the chip half empty: their workgroups are short (a dozen K steps between a prologue and an epilogue
// that nothing hides when a compute unit holds one workgroup), and side by side on a compute unit one's waits are
// the other's issue slots.  The operand areas are as large as the larger tile needs.
template <typename T0, typename T1>
__global__ __launch_bounds__(T0::NT) void gemm_tiled_pair_kernel(GemmArgs g0, GemmArgs g1, int tilesM0, int tilesN0, int nx0, int nz0,
                                                                 int tilesM1, int tilesN1, int nx1) {
    typedef typename T0::E E;
    static_assert(T0::NT == T1::NT && sizeof(typename T0::E) == sizeof(typename T1::E), "one workgroup shape, one element type");
    constexpr int A_SZ = T0::A_SZ > T1::A_SZ ? T0::A_SZ : T1::A_SZ, B_SZ = T0::B_SZ > T1::B_SZ ? T0::B_SZ : T1::B_SZ;
    __shared__ __attribute__((aligned(16))) E As0[A_SZ];
    __shared__ __attribute__((aligned(16))) E As1[A_SZ];
    __shared__ __attribute__((aligned(16))) E Bs0[B_SZ];
    __shared__ __attribute__((aligned(16))) E Bs1[B_SZ];
    const int id = (int)blockIdx.x, first = nx0 * nz0;
    if (id < first) {
        gemm_tiled_body<T0, false>(g0, tilesM0, tilesN0, id % nx0, id / nx0, nx0, As0, As1, Bs0, Bs1);
    } else {
        const int j = id - first;
        gemm_tiled_body<T1, false>(g1, tilesM1, tilesN1, j % nx1, j / nx1, nx1, As0, As1, Bs0, Bs1);
    }
}

// where d8_gemm_phase_record asked the next launches to write their records (process-wide; null: no records; defined in
// gemm_tiled.hip)
extern unsigned long long *phase_rec_buf;
extern size_t phase_rec_bytes;

// Which tile a product runs on.
enum TileId { TILE_WIDE, TILE_256, TILE_128x64, TILE_64x64, TILE_64x128, TILE_128x128 };

template <typename E, bool A_KC, bool B_KC, int VIRT = VIRT_NONE>
static TileId choose_tile(const GemmArgs &g) {
    static const char *force = getenv("D8_GEMM_TILE");  // tuning aid
    const long big_tiles = (long)ceil_div(g.M, 256) * ceil_div(g.N, 256) * g.batch * g.splits;
    bool big = g.M >= 256 && g.N >= 256 && big_tiles >= (long)cu_count() * 3 / 4;
    if (force && g.M >= 256 && g.N >= 256) big = atoi(force) != 128;
    // fp32 runs 64-cycle MFMAs on a quarter of the bytes per flop: the 128 x 128 tile already
    // keeps the matrix pipe fed, and the compiler cannot hold the 256 x 256 variant in registers
    if constexpr (sizeof(E) == 2) {
        static const char *wide = getenv("D8_GEMM_WIDE");  // tuning aid: 0 keeps the 32x32x16 kernel
        if (big && VIRT == VIRT_NONE && !(wide && atoi(wide) == 0) && gemm_wide_eligible(g, !A_KC, B_KC)) return TILE_WIDE;
        if (big) return TILE_256;
    }
    // a 64-wide side gets a tile of that width (im2col products with 64 output channels)
    if (g.N < 128) return TILE_128x64;
    // a patch-matrix product whose last 128-column tile would be at most half full: 64 x 64 tiles, no padding
    // multiplied (C4's filter gradient, N = 576: 83.7 -> 73.8 us)
    if (gemm_tiled_krows_64(VIRT, g.M, g.N)) return TILE_64x64;
    if (g.M < 128) return TILE_64x128;
    if (g.splits == 1 && gemm_tiled_half_tiles(g.M, g.N, g.batch, (long)g.red * ceil_div(g.K, 128 / (int)sizeof(E)), 128 / (int)sizeof(E)))
        return TILE_64x128;
    return TILE_128x128;
}

// ---- two products in one launch (gemm_tiled_pair_kernel): the tile grid of a product, and the launch of gy's workgroups
// followed by gx's
static void grid_of(TileId t, const GemmArgs &g, int &tilesM, int &tilesN) {
    const int bm = (t == TILE_64x64 || t == TILE_64x128) ? 64 : 128, bn = (t == TILE_64x64 || t == TILE_128x64) ? 64 : 128;
    tilesM = ceil_div(g.M, bm), tilesN = ceil_div(g.N, bn);
}

template <typename TX, typename TY>
static int launch_pair_tiles(const GemmArgs &gx0, const GemmArgs &gy0, hipStream_t stream) {
    GemmArgs gx = gx0, gy = gy0;
    // (gx may carry its remainder band as pieces of the same launch: GemmArgs::tail_m0; then it has one layer)
    const bool tail = gx.tail_splits > 0;
    const int tMx = ceil_div(tail ? gx.tail_m0 : gx.M, TX::BM), tNx = ceil_div(gx.N, TX::BN), tMy = ceil_div(gy.M, TY::BM), tNy = ceil_div(gy.N, TY::BN);
    const int extra = tail ? ceil_div(gx.M - gx.tail_m0, TX::BM) * tNx * gx.tail_splits : 0;
    // the longer-running product first: gy's pieces, then gx's tiles
    const int ny = tMy * tNy, nzy = gy.batch * gy.splits, nx = tMx * tNx + extra, nzx = tail ? 1 : gx.batch * gx.splits;
    // phase records (a measurement aid): gy's workgroups first, then gx's, tagged 0 and 1
    const bool rec = (size_t)(ny * nzy + nx * nzx) * 64 <= phase_rec_bytes;
    gy.phase_rec = rec ? phase_rec_buf : nullptr, gy.stamps = 0;
    gx.phase_rec = rec && phase_rec_buf ? phase_rec_buf + 8L * ny * nzy : nullptr, gx.stamps = 1;
    hipLaunchKernelGGL((gemm_tiled_pair_kernel<TY, TX>), dim3(ny * nzy + nx * nzx), dim3(TX::NT), 0, stream, gy, gx, tMy, tNy, ny, nzy, tMx, tNx, nx);
    D8_LAUNCH_CHECK();
    return 0;
}

}  // namespace d8

#endif
