// fp16 GEMM for large outputs on gfx950: 256 x 256 tile of C per workgroup, four waves, each
// owning 128 x 128 of it as 8 x 8 blocks of v_mfma_f32_16x16x32_f16 (fp32 accumulation; the 256
// accumulator registers of a lane are the whole AGPR file, one wave per SIMD).
//
// Why this shape: under matrix load the chip runs at the clock its power limit allows, so the
// rate is set by energy per flop.  Measured on real-valued operands, a stream of 16x16x32 MFMAs
// sustains 10-15 % more flops than a stream of 32x32x16 MFMAs, and a 128 x 128 wave tile reads
// one 1 KB operand fragment from LDS per 4 MFMAs (a 64 x 128 tile of 32x32x16: three per 4).
//
// Data path.  K is walked in steps of 64.  The A and B tiles of a step (32 KB each) go from
// global memory straight into LDS with buffer_load_dwordx4 ... lds (no staging registers, no LDS
// write instructions); two stages of LDS alternate.  A lane's 16 bytes land at a fixed place
// (wave-uniform base + 16 x lane), so bank conflicts are avoided not by padding but by choosing
// WHICH 16 bytes each lane fetches: 16-byte chunk c of row r is kept at chunk position
// c ^ swizzle(r), and the fragment reads apply the same exclusive-or.
//   * operand contiguous along K: LDS holds [row][64 k], 128 B per row, swizzle(r) = (r >> 1) & 7;
//     a fragment (16 rows x 32 k) is one ds_read_b128 per lane;
//   * operand contiguous along M or N: LDS holds [k][256 rows], 512 B per k-row, 32-byte column
//     groups exchanged by ((k & 3) | (k >> 3 & 1) << 2); a fragment is two ds_read_b64_tr_b16
//     (the transposing LDS read).  Transposed operands are never materialised.
//
// Schedule of one step (128 MFMAs per wave, in two halves of 64, one per 32-wide k group):
//   half 0: MFMAs of k group 0; between them the 16 fragment reads of k group 1;
//   half 1: workgroup barrier (every wave's loads of the next step have landed, every wave is
//           done reading this stage), then the MFMAs of k group 1; between them, evenly spread,
//           the 16 loads of the step after next into the stage just released and the 16
//           fragment reads of the next step's k group 0.
// The MFMAs are volatile asm statements (accumulators pinned to AGPRs, updated in place); the
// compiler keeps memory instructions between the two MFMAs they were written between, so the
// issue order is the program order.
//
// One launch, several tiles per workgroup.  A launch carries up to two products (the two gradients of a
// MatrixMultiply, which read the same dz, are the case it is built for) and at most one workgroup per compute
// unit; a workgroup takes tiles idx = blockIdx.x, blockIdx.x + gridDim.x, ... of the products' concatenated
// tile lists.  Between two of its tiles nothing is waited for that need not be: when a tile's K loop ends,
// the first two steps of the NEXT tile are put on their way into the two LDS stages, then the finished tile
// goes through the epilogue (its own 32 KB patch area of LDS, so the stages are free) and its stores are left
// to drain while the next K loop runs.  A launch of one tile per workgroup costs, besides its loop, the first
// operand bytes' way from memory (about 2 us), the write of the whole of C at the very end (4 us at the HBM
// write rate) and the gap to the next launch; with two tiles per workgroup those are paid once for both.
#ifndef DEEP8_AMD_GEMM_WIDE_KERNEL_H
#define DEEP8_AMD_GEMM_WIDE_KERNEL_H

#include <type_traits>

#include "gemm_args.h"

namespace d8 {

typedef __fp16 wf16x4v __attribute__((ext_vector_type(4)));
typedef __fp16 wf16x8v __attribute__((ext_vector_type(8)));
#define WIDE_LDS(T, p) ((__attribute__((address_space(3))) T *)(p))

namespace wide {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int OPERAND_BYTES = 256 * 64 * 2;                   // one operand tile of one step
constexpr int STAGE_BYTES = 2 * OPERAND_BYTES;                // A then B
constexpr int PATCH_BYTES = 4 * 16 * 128 * 4;                 // per wave: 16 rows x 128 floats of the epilogue
constexpr int LDS_BYTES = 2 * STAGE_BYTES + PATCH_BYTES;      // two stages + patches = 160 KB, all of a CU's LDS
enum { FORM_NN = 0, FORM_NT = 1, FORM_TN = 2 };

// One product of a launch (plain matrices, fp16, M and N >= 256, K a multiple of 64).
struct Product {
    const f16 *A, *B;
    f16 *C;
    const f16 *bias;  // fused store: bias[n] added to column n (may be null), then ReLu when relu != 0
    int M, N, K;
    int lda, ldb, ldc;
    long sA, sB, sC;
    int tilesM, tilesN, tiles;  // tiles = tilesM * tilesN * batch
    int form;
    float beta;
    int relu;
};

struct Launch {
    Product p[2];
    int n;      // products
    int total;  // tiles of all products
    // measurement aid: when set, tile idx records six 64-bit words at rec[6 * idx]: the chip's 100 MHz wall clock when
    // the workgroup turned to the tile, when its K loop began and ended and when its epilogue was through (its stores
    // acknowledged, if it is the workgroup's last tile), and the shader clock at both ends of the loop
    unsigned long long *rec;
};

// The parts of the kernel a build may leave out.  The library only ever instantiates Shipped; diag/gemm_wide_diag.hip,
// which is not part of it, builds the others to measure what each part costs.
struct Shipped {
    static constexpr bool LOADS = true;           // false: the K loop without its global -> LDS loads
    static constexpr bool FRAGMENT_READS = true;  // false: ... without its LDS reads (the MFMAs keep the first fragments)
    static constexpr bool BARRIER = true;         // false: ... without its barrier
    static constexpr bool STORES = true;          // false: the epilogue does everything but the stores to C
    static constexpr bool ADVANCE_K = true;       // false: every K step fetches the tile's first step again (all loads hit in cache)
};

typedef unsigned wu32x4 __attribute__((ext_vector_type(4)));

// Buffer descriptor over `bytes` bytes from p (raw buffer, reads beyond the end give zero).
__device__ __forceinline__ wu32x4 make_desc(const void *p, unsigned bytes) {
    const unsigned long a = (unsigned long)p;
    return wu32x4{(unsigned)a, (unsigned)(a >> 32) & 0xffffu, bytes, 0x00020000u};
}

// One 16-byte piece per lane from global memory straight into LDS: lane i's piece lands at LDS
// byte address m0 + 16 * i (m0, `soffset` and the descriptor are wave-uniform).  Written as asm so
// that the compiler does not know LDS is written behind its back by loads that are still in
// flight: it would otherwise hold every later LDS read until all of them have landed.  The barrier
// of each step (with its vmcnt(0)) is what orders these writes against the reads.  m0 must be
// written at least one instruction before the load that uses it (the hardware does not interlock
// that), so the two are separate statements with an MFMA between them; m0 is a reserved register
// that the compiler only ever sets right before a use of its own.
// (the target is `base` + a compile-time constant: one register holds all of a wave's targets)
template <int OFFSET>
__device__ __forceinline__ void set_lds_target(unsigned base) {
    asm volatile("s_add_u32 m0, %0, %1" : : "s"(base), "n"(OFFSET) : "memory", "scc");
}
__device__ __forceinline__ void load_to_lds(const wu32x4 &desc, unsigned voffset, unsigned soffset) {
    asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds" : : "v"(voffset), "s"(desc), "s"(soffset) : "memory");
}

// body(std::integral_constant<int, 0>) ... body(std::integral_constant<int, N - 1>), in order
template <int N, int I = 0, class F>
__device__ __forceinline__ void static_for(F &&body) {
    if constexpr (I < N) {
        body(std::integral_constant<int, I>());
        static_for<N, I + 1>(body);
    }
}

// Per-thread constants of one operand: how it fetches its pieces and where its fragments lie.
template <bool KC>
struct Operand {
    unsigned voff[2];      // byte offset of this thread's piece within a fetch round (even / odd round)
    unsigned round_bytes;  // uniform global-memory distance between rounds
    int frag[KC ? 2 : 8];  // LDS byte offsets: per k group (KC) or per fragment (transposed form)

    // ld: leading dimension in elements; wbase: first of the wave's 128 rows / columns in the tile
    __device__ __forceinline__ void init(int ld, int wave, int lane, int wbase) {
        if constexpr (KC) {
            // round t holds rows t*32 .. t*32+31: wave w the 8 rows from w*8, 8 lanes per row
            const int row = wave * 8 + (lane >> 3), pos = lane & 7;
            const int sw = (row >> 1) & 7;
            voff[0] = voff[1] = 2u * ((unsigned)row * ld + (unsigned)((pos ^ sw) * 8));
            round_bytes = 2u * 32u * ld;
            const int r = lane & 15, j = lane >> 4, s = (r >> 1) & 7;
#pragma unroll
            for (int kg = 0; kg < 2; ++kg) frag[kg] = (wbase + r) * 128 + (((j ^ s) ^ (kg << 2)) * 16);
        } else {
            // round t holds k-rows t*8 .. t*8+7: wave w the 2 k-rows from w*2, 32 lanes per k-row
            const int kr = wave * 2 + (lane >> 5), pos = lane & 31;
#pragma unroll
            for (int par = 0; par < 2; ++par) {
                const int f = (kr & 3) | (par << 2);  // k-row t*8 + kr: bit 3 is the round's parity
                voff[par] = 2u * ((unsigned)kr * ld + (unsigned)((pos ^ (f << 1)) * 8));
            }
            round_bytes = 2u * 8u * ld;
            const int i = lane & 15, j = lane >> 4, f = (i >> 2) | ((j & 1) << 2);
#pragma unroll
            for (int n = 0; n < 8; ++n)
                frag[n] = (j * 8 + (i >> 2)) * 512 + wbase * 2 + ((n ^ f) * 32) + (i & 3) * 8;
        }
    }

    // fetch this operand's tile of one step: 8 rounds of 4 KB, this wave's KB of each
    // wave_base: LDS address of the wave's KB in round 0 of stage 0's A tile; AREA: byte offset of the operand tile
    template <int AREA, int T>
    __device__ __forceinline__ void aim_round(unsigned wave_base) const {
        set_lds_target<AREA + T * 4096>(wave_base);
    }
    __device__ __forceinline__ void fetch_round(const wu32x4 &rsrc, unsigned sbase, int t) const {
        load_to_lds(rsrc, voff[t & 1], sbase + t * round_bytes);
    }

    // fragment n (16 rows or columns) of k group kg
    __device__ __forceinline__ f16x8 read(const char *stage, int kg, int n) const {
        if constexpr (KC) {
            return *(const f16x8 *)(stage + frag[kg] + n * 2048);
        } else {
            const char *p = stage + frag[n] + kg * 16384;
            const wf16x4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4f16(WIDE_LDS(wf16x4v, p));
            const wf16x4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4f16(WIDE_LDS(wf16x4v, p + 2048));
            const wf16x8v both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            return __builtin_bit_cast(f16x8, both);
        }
    }
};

// Order of a k group's 64 MFMAs over the wave's 8 x 8 blocks: row by row, every other row backwards, so that each MFMA
// differs from the one before it in ONE operand (the A fragment stays for a row, the B fragment at a row's end).  The
// kernel is power-limited, and the order is measurable: forward 4096^3 102.3 us row by row, 101.6 this way, 105.0
// with both operands changing every time.  (Each block still sums its k values in the same order.)
#define WIDE_BI(m) ((m) >> 3)
#define WIDE_BJ(m) ((((m) >> 3) & 1) ? 7 - ((m) & 7) : ((m) & 7))
__device__ __forceinline__ void mfma(f32x4 &acc, const f16x8 &a, const f16x8 &b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
// a tile's first MFMA into a block: the sum starts at zero (no pass over the accumulators to clear them)
__device__ __forceinline__ void mfma_first(f32x4 &acc, const f16x8 &a, const f16x8 &b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(acc) : "v"(a), "v"(b));
}

// Where a tile lies: which product and batch element, the rows / columns it owns and those it computes (a tile that
// would stick out of the matrix is moved back inside; it stores only what it owns).
struct Where {
    int p, b, m_own, n_own, m0, n0;
};

// Tile `idx` of the launch.  The workgroups of one XCD (ids congruent mod 8; the grid is a multiple of 8 or one
// workgroup per tile) take a contiguous run of a product's tiles, runs laid out in bands of 4 tile rows walked
// column by column, so that the A and B panels an XCD re-reads stay in its L2.
__device__ __forceinline__ Where locate(const Launch &L, int idx) {
    Where w;
    w.p = (L.n > 1 && idx >= L.p[0].tiles) ? 1 : 0;
    const Product &P = L.p[w.p];
    int id = idx - (w.p ? L.p[0].tiles : 0);
    const int per = P.tilesM * P.tilesN;
    w.b = id / per;
    id -= w.b * per;
    if ((per & 7) == 0) id = (id & 7) * (per >> 3) + (id >> 3);
    constexpr int GM = 4;
    const int band = id / (GM * P.tilesN), first = band * GM;
    const int rows_in_band = min(GM, P.tilesM - first);
    const int in_band = id - band * GM * P.tilesN;
    const int tm = first + in_band % rows_in_band, tn = in_band / rows_in_band;
    w.m_own = tm * BM, w.n_own = tn * BN;
    w.m0 = min(w.m_own, P.M - BM), w.n0 = min(w.n_own, P.N - BN);
    return w;
}

// Everything a wave needs to fetch and read the operands of one tile.
template <bool A_KC, bool B_KC>
struct TileOperands {
    Operand<A_KC> oa;
    Operand<B_KC> ob;
    wu32x4 ra, rb;
    unsigned a_org, b_org, a_step, b_step;  // uniform byte offset of the tile at step 0, and from one step to the next
    int nsteps;

    template <class Policy>
    __device__ __forceinline__ void init(const Product &P, const Where &w, int wave, int lane) {
        asm volatile("" : "+v"(lane));  // per tile, not once per kernel and kept across the other tiles' loops
        const long a_rows = A_KC ? P.M : P.K, b_rows = B_KC ? P.N : P.K;
        ra = make_desc(P.A + (long)w.b * P.sA, (unsigned)(2 * a_rows * P.lda));
        rb = make_desc(P.B + (long)w.b * P.sB, (unsigned)(2 * b_rows * P.ldb));
        oa.init(P.lda, wave, lane, (wave >> 1) * 128);
        ob.init(P.ldb, wave, lane, (wave & 1) * 128);
        a_org = 2u * (A_KC ? (unsigned)w.m0 * P.lda : (unsigned)w.m0);
        b_org = 2u * (B_KC ? (unsigned)w.n0 * P.ldb : (unsigned)w.n0);
        a_step = Policy::ADVANCE_K ? (A_KC ? 128u : 2u * BK * P.lda) : 0u;
        b_step = Policy::ADVANCE_K ? (B_KC ? 128u : 2u * BK * P.ldb) : 0u;
        nsteps = P.K / BK;
    }

    // steps 0 and 1 of the tile into the two stages (32 loads per wave, not waited for)
    __device__ __forceinline__ void issue_first_steps(unsigned wave_base) const {
        issue_step<0>(wave_base, 0);
        issue_step<1>(wave_base, min(1, nsteps - 1));
    }
    template <int S>
    __device__ __forceinline__ void issue_step(unsigned wave_base, int step) const {
        issue_rounds<S, 0>(wave_base, step);
    }
    template <int S, int T>
    __device__ __forceinline__ void issue_rounds(unsigned wave_base, int step) const {
        if constexpr (T < 8) {
            oa.template aim_round<S * STAGE_BYTES, T>(wave_base);
            asm volatile("s_nop 0");
            oa.fetch_round(ra, a_org + step * a_step, T);
            ob.template aim_round<S * STAGE_BYTES + OPERAND_BYTES, T>(wave_base);
            asm volatile("s_nop 0");
            ob.fetch_round(rb, b_org + step * b_step, T);
            issue_rounds<S, T + 1>(wave_base, step);
        }
    }
};

// The K loop of one tile.  On entry the tile's first two steps are in the two stages (every wave's loads landed,
// barrier passed); on exit every wave is past its last LDS read and no load of the tile is on its way (barrier).
template <class Policy, bool A_KC, bool B_KC>
__device__ __forceinline__ void k_loop(const TileOperands<A_KC, B_KC> &T, char *lds, unsigned wave_base, f32x4 (&acc)[8][8]) {
    const Operand<A_KC> &oa = T.oa;
    const Operand<B_KC> &ob = T.ob;
    const int nsteps = T.nsteps;
    f16x8 fa[2][8], fb[2][8];
#pragma unroll
    for (int n = 0; n < 8; ++n) {
        fb[0][n] = ob.read(lds + OPERAND_BYTES, 0, n);
        fa[0][n] = oa.read(lds, 0, n);
    }

    // ---- one step out of stage `cur`; `fetch_step` is the step whose tiles are fetched into it (a step beyond
    // the last fetches nothing: its loads run against an empty descriptor and write zeros to a stage that is
    // not read again)
    auto do_step = [&](auto cur_tag, auto first_tag, int fetch_step) {
        constexpr int cur = decltype(cur_tag)::value;
        constexpr bool first = decltype(first_tag)::value;
        char *As = lds + cur * STAGE_BYTES, *Bs = As + OPERAND_BYTES;
        char *An = lds + (cur ^ 1) * STAGE_BYTES, *Bn = An + OPERAND_BYTES;
        const bool live = fetch_step < nsteps;
        wu32x4 ra = T.ra, rb = T.rb;
        ra[2] = live ? ra[2] : 0u, rb[2] = live ? rb[2] : 0u;
        const unsigned a_src = T.a_org + fetch_step * T.a_step, b_src = T.b_org + fetch_step * T.b_step;
        // half 0
#pragma unroll
        for (int m = 0; m < 64; ++m) {
            if constexpr (first) mfma_first(acc[WIDE_BI(m)][WIDE_BJ(m)], fa[0][WIDE_BI(m)], fb[0][WIDE_BJ(m)]);
            else mfma(acc[WIDE_BI(m)][WIDE_BJ(m)], fa[0][WIDE_BI(m)], fb[0][WIDE_BJ(m)]);
            if constexpr (Policy::FRAGMENT_READS) {
                if (m % 3 == 0 && m < 48) {
                    const int e = m / 3;  // 16 reads: the B fragments first (all needed by the first row)
                    if (e < 8) fb[1][e] = ob.read(Bs, 1, e);
                    else fa[1][e - 8] = oa.read(As, 1, e - 8);
                }
            }
        }
        // half 1
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): my pieces of the next step have landed
        if constexpr (Policy::BARRIER) __syncthreads();
        static_for<64>([&](auto m_tag) {
            constexpr int m = decltype(m_tag)::value;
            if constexpr (Policy::LOADS) {
                if constexpr ((m & 3) == 0) {
                    if constexpr ((m >> 2) < 8) oa.template aim_round<cur * STAGE_BYTES, (m >> 2)>(wave_base);
                    else ob.template aim_round<cur * STAGE_BYTES + OPERAND_BYTES, (m >> 2) - 8>(wave_base);
                }
            }
            mfma(acc[WIDE_BI(m)][WIDE_BJ(m)], fa[1][WIDE_BI(m)], fb[1][WIDE_BJ(m)]);
            if constexpr (Policy::LOADS) {
                if constexpr ((m & 3) == 0) {
                    // 16 loads into the stage every wave has finished with, one per 4 MFMAs: a load
                    // keeps the CU's address path busy for 16 cycles, as long as an MFMA runs, and all
                    // four waves issue theirs in the same window; issued closer together they hold up
                    // instruction issue (2600 cycles per step at one per 2 MFMAs, 2330 at one per 4)
                    constexpr int d = m >> 2;
                    if constexpr (d < 8) oa.fetch_round(ra, a_src, d);
                    else ob.fetch_round(rb, b_src, d - 8);
                }
            }
            if constexpr (Policy::FRAGMENT_READS) {
                // fragments of the next step's k group 0, in the order of their first use (A fragment 0, the
                // eight B fragments of the first row of blocks, then the other A fragments), on MFMA slots the
                // loads do not use
                if constexpr (((m & 3) == 2 && m < 56) || m == 1 || m == 5) {
                    constexpr int e = m == 1 ? 0 : m == 2 ? 1 : m == 5 ? 2 : m == 6 ? 3 : (m >> 2) + 2;
                    if constexpr (e == 0) fa[0][0] = oa.read(An, 0, 0);
                    else if constexpr (e <= 8) fb[0][e - 1] = ob.read(Bn, 0, e - 1);
                    else fa[0][e - 8] = oa.read(An, 0, e - 8);
                }
            }
        });
    };

    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    using No = std::false_type;
    using Yes = std::true_type;
    // The first two steps apart (the first starts the sums), then four steps per trip: a taken branch costs a
    // wave that is alone on its SIMD some 80 cycles in which the matrix pipe runs dry.
    do_step(S0(), Yes(), 2);
    if (nsteps > 1) do_step(S1(), No(), 3);
    int s = 2;
    for (; s + 4 <= nsteps; s += 4) {
        do_step(S0(), No(), s + 2);
        do_step(S1(), No(), s + 3);
        do_step(S0(), No(), s + 4);
        do_step(S1(), No(), s + 5);
    }
    for (; s < nsteps; s += 2) {
        do_step(S0(), No(), s + 2);
        if (s + 1 < nsteps) do_step(S1(), No(), s + 3);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();  // no load is still on its way into LDS, every wave is past its last read
}

// One 16-row slab of a wave's accumulators into its patch: element r of block column J at wr[J & 3] + a constant.
template <int IDX>
__device__ __forceinline__ void write_slab(const unsigned (&wr)[4], const f32x4 (&row)[8]) {
    if constexpr (IDX < 32) {
        constexpr int J = IDX >> 2, R = IDX & 3;
        asm volatile("ds_write_b32 %0, %1 offset:%2" : : "v"(wr[J & 3]), "a"(row[J][R]), "n"(R * 512 + (J >> 2) * 256) : "memory");
        write_slab<IDX + 1>(wr, row);
    }
}

// A finished tile on its way out: 16 rows of the wave's 128 x 128 at a time through the wave's patch of LDS, so
// that C is read (beta = 1) and written 16 bytes per lane, 256 contiguous bytes per 16 lanes.  Element (row, col) of
// a slab sits at float row * 128 + (col ^ (row >> 2) * 16): the accumulators' four rows per lane group meet four
// different bank groups.
// INTERIOR: the tile lies wholly inside C, so every lane stores all its 32 pieces, unconditionally: the caller
// counts on at least that many vector-memory instructions after the loads it issued before (see the kernel's wait
// for the next tile's first steps).
template <class Policy, bool INTERIOR>
__device__ __forceinline__ void store_tile(const Product &P, const Where &w, float *patch, int wave, int lane, f32x4 (&acc)[8][8]) {
    const int wm = wave >> 1, wn = wave & 1;
    f16 *C = P.C + (long)w.b * P.sC;
    // (the lane id as a value the compiler cannot see through: everything derived from it is computed here, per tile,
    // instead of once per kernel and kept -- or spilled -- across the K loops)
    asm volatile("" : "+v"(lane));
    const int l15 = lane & 15, l4 = lane >> 4;
    const int n = w.n0 + wn * 128 + l15 * 8;  // this lane's eight columns, the same in every slab
    const bool beta = P.beta != 0.f;
    // beta = 1: the old C of a 16-row slab is fetched while the slab before it goes through the patch, so that
    // only the first slab's read is waited for
    f16x8 oldc[2][4];
    auto fetch_old = [&](int i, f16x8(&dst)[4]) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int m = w.m0 + wm * 128 + i * 16 + t * 4 + l4;
            if (INTERIOR || (m >= w.m_own && n >= w.n_own)) dst[t] = *(const f16x8 *)(C + (long)m * P.ldc + n);
        }
    };
    // fused store: the lane's eight bias values, read once, before any store (a load waited for after a store
    // would wait for that store's acknowledgement as well)
    float bias[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (P.bias) {
        const f16x8 bv = *(const f16x8 *)(P.bias + n);
#pragma unroll
        for (int e = 0; e < 8; ++e) bias[e] = (float)bv[e];
    }
    // LDS byte addresses of the lane's patch writes: block column j goes to 16-float group j ^ l4 of rows 4 * l4 + r
    unsigned wr[4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
        wr[q] = (unsigned)(size_t)WIDE_LDS(float, patch) + 4u * ((4 * l4) * 128 + ((q ^ l4) * 16 + l15));
    if (beta) fetch_old(0, oldc[0]);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        if (beta && i + 1 < 8) fetch_old(i + 1, oldc[(i + 1) & 1]);
        // (written straight from the accumulator registers, in program order: LDS serves a wave's instructions in
        // the order it issued them, so the reads below see these writes)
        write_slab<0>(wr, acc[i]);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int row = t * 4 + l4, cc = (l15 * 8) ^ (t * 16);
            const int m = w.m0 + wm * 128 + i * 16 + row;
            float v[8];
            *(f32x4 *)&v[0] = *(const f32x4 *)(patch + row * 128 + cc);
            *(f32x4 *)&v[4] = *(const f32x4 *)(patch + row * 128 + cc + 4);
            if ((INTERIOR || (m >= w.m_own && n >= w.n_own)) && Policy::STORES) {
                f16 *c = C + (long)m * P.ldc + n;
                if (beta) {
                    const f16x8 old = oldc[i & 1][t];
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] += (float)old[e];
                }
                if (P.bias) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] += bias[e];
                }
                if (P.relu) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] = v[e] > 0.f ? v[e] : 0.f;
                }
                // (two values per conversion instruction, round to nearest even as the single conversion does)
                f16x2 o2[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) o2[e] = __builtin_convertvector((f32x2){v[2 * e], v[2 * e + 1]}, f16x2);
                const f16x8 out = __builtin_shufflevector(__builtin_shufflevector(o2[0], o2[1], 0, 1, 2, 3),
                                                          __builtin_shufflevector(o2[2], o2[3], 0, 1, 2, 3), 0, 1, 2, 3, 4, 5, 6, 7);
                // streamed past the L2: the whole output leaves the chip during the kernel's last microseconds
                // either way, and lines left dirty in L2 are written back only after the last wave has ended
                // (a tile with another one after it gains nothing from ordinary stores either: measured, the time
                // between a workgroup's two K loops is the same)
                __builtin_nontemporal_store(out, (f16x8 *)c);
            }
        }
    }
}

}  // namespace wide

// FORMS: bit f set = products of form f (wide::FORM_*) may occur in the launch (the others' loops are left out).
template <class Policy, int FORMS>
__global__ __launch_bounds__(256) void gemm_wide_kernel(wide::Launch L) {
    using namespace wide;
    __shared__ __attribute__((aligned(1024))) char lds[LDS_BYTES];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    float *patch = (float *)(lds + 2 * STAGE_BYTES) + wave * (16 * 128);
    const unsigned wave_base = (unsigned)(size_t)WIDE_LDS(const char, lds) + wave * 1024;
    f32x4 acc[8][8];
    unsigned long long wall[4] = {0, 0, 0, 0}, clk[2] = {0, 0};
    if (L.rec) wall[0] = wall_clock64();

    // run f<A_KC, B_KC> for the form of product p (uniform)
#define WIDE_FOR_FORM(form, ...)                                                                   \
    do {                                                                                           \
        if ((FORMS & 1) && ((FORMS == 1) || (form) == FORM_NN)) {                                  \
            constexpr bool A_KC = true, B_KC = false;                                              \
            __VA_ARGS__                                                                            \
        } else if ((FORMS & 2) && ((FORMS & 4) == 0 || (form) == FORM_NT)) {                       \
            constexpr bool A_KC = true, B_KC = true;                                               \
            __VA_ARGS__                                                                            \
        } else if (FORMS & 4) {                                                                    \
            constexpr bool A_KC = false, B_KC = false;                                             \
            __VA_ARGS__                                                                            \
        }                                                                                          \
    } while (0)

    int idx = blockIdx.x;
    Where cur = locate(L, idx);
    WIDE_FOR_FORM(L.p[cur.p].form, {
        TileOperands<A_KC, B_KC> T;
        T.template init<Policy>(L.p[cur.p], cur, wave, lane);
        T.issue_first_steps(wave_base);
    });
    // vmcnt(16): this wave's pieces of the first stage are in LDS (the 16 loads of the second stage may still be on
    // their way: the first step's own wait, before its barrier, covers them)
    __builtin_amdgcn_s_waitcnt(0x4f70);
    __syncthreads();

    for (;;) {
        const int nidx = idx + gridDim.x;
        const bool more = nidx < L.total;
        const Where nxt = more ? locate(L, nidx) : cur;
        if (L.rec) wall[1] = wall_clock64(), clk[0] = __builtin_readcyclecounter();
        WIDE_FOR_FORM(L.p[cur.p].form, {
            TileOperands<A_KC, B_KC> T;
            T.template init<Policy>(L.p[cur.p], cur, wave, lane);
            k_loop<Policy, A_KC, B_KC>(T, lds, wave_base, acc);
        });
        if (L.rec) wall[2] = wall_clock64(), clk[1] = __builtin_readcyclecounter();
        // The next tile's first two steps set out before this tile's epilogue (32 loads per wave).
        if (more) {
            WIDE_FOR_FORM(L.p[nxt.p].form, {
                TileOperands<A_KC, B_KC> T;
                T.template init<Policy>(L.p[nxt.p], nxt, wave, lane);
                T.issue_first_steps(wave_base);
            });
        }
        const Product &P = L.p[cur.p];
        const bool interior = cur.m0 == cur.m_own && cur.n0 == cur.n_own;
        if (interior) store_tile<Policy, true>(P, cur, patch, wave, lane, acc);
        else store_tile<Policy, false>(P, cur, patch, wave, lane, acc);
        if (L.rec) {
            if (!more) __builtin_amdgcn_s_waitcnt(0x0f70);  // this wave's stores have been acknowledged
            wall[3] = wall_clock64();
            if (tid == 0) {
                unsigned long long *rec = L.rec + 6 * (long)idx;
                rec[0] = wall[0], rec[1] = wall[1], rec[2] = wall[2], rec[3] = wall[3], rec[4] = clk[0], rec[5] = clk[1];
            }
            wall[0] = wall[2];  // the next tile's record starts where this tile's loop ended
        }
        if (!more) break;
        // Vector-memory instructions complete in the order they were issued.  The epilogue of an interior tile issues
        // at least 32 of them (its stores), so "at most 32 outstanding" means: the 32 loads issued before them have
        // landed, whatever the stores do -- they drain while the next K loop runs.  Any other epilogue may issue
        // fewer: wait for all.
        if (interior && Policy::STORES) __builtin_amdgcn_s_waitcnt(0x8f70);  // vmcnt(32)
        else __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        cur = nxt, idx = nidx;
    }
#undef WIDE_FOR_FORM
}

}  // namespace d8

#endif
