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
// Diagnostic builds (never defined in the shipped library; `python bench.py --phases --wide-diagnostic NAME`
// compiles this file with one of them into a scratch copy of the library and prints the kernel's phase
// record).  Each answers one question about where a launch's time goes; all but BARRIER_CLOCKS and DIRECT_STORE give
// wrong results (none of them reads or writes outside the operands):
//   D8_WIDE_DIAG_SAME_K          every K step fetches the tile's first step again, so all loads after the first
//                                hit in cache: what the loop costs when no load ever waits for HBM
//   D8_WIDE_DIAG_BARRIER_CLOCKS  reads the shader clock around the step's wait for its own loads and around its
//                                barrier; the record's first three fields become the summed cycles of a pair of
//                                back-to-back clock reads, of the wait and of the barrier
//   D8_WIDE_DIAG_NO_STORE        the epilogue does everything but the stores to C: its cost without HBM writes
//   D8_WIDE_DIAG_NO_FRAGMENT_READS  the K loop without its LDS reads (the MFMAs keep the first fragments)
//   D8_WIDE_DIAG_NO_LOADS        ... without its global -> LDS loads (the MFMAs see the first two steps again and again)
//   D8_WIDE_DIAG_NO_BARRIER      ... without its barrier
//                                (the three combine: what each part of the loop costs in cycles -- on all-zero operands,
//                                `--operands zeros` -- and in energy, i.e. in clock, on the config's data)
//   D8_WIDE_DIAG_DIRECT_STORE    accumulates the blocks transposed (MFMA operands exchanged) so that a lane owns
//                                four consecutive columns, and stores them straight from registers, 8 bytes per
//                                lane, without the LDS patch (correct results)
#include <type_traits>

#include "gemm_args.h"

namespace d8 {

typedef __fp16 wf16x4v __attribute__((ext_vector_type(4)));
typedef __fp16 wf16x8v __attribute__((ext_vector_type(8)));
#define WIDE_LDS(T, p) ((__attribute__((address_space(3))) T *)(p))

namespace wide {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int OPERAND_BYTES = 256 * 64 * 2;         // one operand tile of one step
constexpr int STAGE_BYTES = 2 * OPERAND_BYTES;      // A then B
constexpr int LDS_BYTES = 2 * STAGE_BYTES;          // two stages
constexpr int PATCH_LD = 132;                       // floats per row of an epilogue patch

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
__device__ __forceinline__ void set_lds_target(unsigned lds) { asm volatile("s_mov_b32 m0, %0" : : "s"(lds) : "memory"); }
__device__ __forceinline__ void load_to_lds(const wu32x4 &desc, unsigned voffset, unsigned soffset) {
    asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds" : : "v"(voffset), "s"(desc), "s"(soffset) : "memory");
}

// Per-thread constants of one operand: how it fetches its pieces and where its fragments lie.
template <bool KC>
struct Operand {
    unsigned voff[2];      // byte offset of this thread's piece within a fetch round (even / odd round)
    unsigned round_bytes;  // uniform global-memory distance between rounds
    int frag[KC ? 2 : 8];  // LDS byte offsets: per k group (KC) or per fragment (transposed form)

    // ld: leading dimension in elements; wbase: first of the wave's 128 rows / columns in the tile
    __device__ void init(int ld, int wave, int lane, int wbase) {
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
    __device__ __forceinline__ void aim_round(const char *stage, int wave, int t) const {
        set_lds_target((unsigned)(size_t)WIDE_LDS(const char, stage) + (t * 4 + wave) * 1024);
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
#define BI(m) ((m) >> 3)
#define BJ(m) ((((m) >> 3) & 1) ? 7 - ((m) & 7) : ((m) & 7))
__device__ __forceinline__ void mfma(f32x4 &acc, const f16x8 &a, const f16x8 &b) {
#ifdef D8_WIDE_DIAG_DIRECT_STORE
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %2, %1, %0" : "+a"(acc) : "v"(a), "v"(b));
#else
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
#endif
}

}  // namespace wide

template <bool A_KC, bool B_KC>
__global__ __launch_bounds__(256) void gemm_wide_kernel(GemmArgs g, int tilesM, int tilesN) {
    using namespace wide;
    __shared__ __attribute__((aligned(1024))) char lds[LDS_BYTES];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // optional phase record: wall clock (100 MHz, the same on every CU) and shader clock
    unsigned long long wall[4] = {0, 0, 0, 0}, clk[2] = {0, 0};
    if (g.stamps) wall[0] = wall_clock64();
    const int wm = wave >> 1, wn = wave & 1;

    // ---- which tile: the workgroups of one XCD (ids congruent mod 8) take a contiguous run of
    // tiles, runs laid out in bands of 4 tile rows walked column by column
    int id = blockIdx.x;
    const int total = tilesM * tilesN;
    if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    constexpr int GM = 4;
    const int band = id / (GM * tilesN), first = band * GM;
    const int rows_in_band = min(GM, tilesM - first);
    const int in_band = id - band * GM * tilesN;
    const int tm = first + in_band % rows_in_band, tn = in_band / rows_in_band;
    // a tile that would stick out of the matrix is moved back inside; it stores only what it owns
    const int m_own = tm * BM, n_own = tn * BN;
    const int m0 = min(m_own, g.M - BM), n0 = min(n_own, g.N - BN);

    const int b = blockIdx.z;
    const long a_rows = A_KC ? g.M : g.K, b_rows = B_KC ? g.N : g.K;
    const wu32x4 ra = make_desc((const f16 *)g.A + (long)b * g.sA, (unsigned)(2 * a_rows * g.lda));
    const wu32x4 rb = make_desc((const f16 *)g.B + (long)b * g.sB, (unsigned)(2 * b_rows * g.ldb));

    Operand<A_KC> oa;
    Operand<B_KC> ob;
    oa.init(g.lda, wave, lane, wm * 128);
    ob.init(g.ldb, wave, lane, wn * 128);
    // uniform byte offset of the tile at step 0, and from one step to the next
    const unsigned a_org = 2u * (A_KC ? (unsigned)m0 * g.lda : (unsigned)m0), a_step_ = A_KC ? 128u : 2u * BK * g.lda;
    const unsigned b_org = 2u * (B_KC ? (unsigned)n0 * g.ldb : (unsigned)n0), b_step_ = B_KC ? 128u : 2u * BK * g.ldb;
#ifndef D8_WIDE_DIAG_SAME_K
    const unsigned a_step = a_step_, b_step = b_step_;
#else
    const unsigned a_step = 0u * a_step_, b_step = 0u * b_step_;
#endif
    const int nsteps = g.K / BK;

    f32x4 acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
            asm volatile("" : "+a"(acc[i][j]));  // from here on the value lives in AGPRs
        }
    f16x8 fa[2][8], fb[2][8];
#ifdef D8_WIDE_DIAG_BARRIER_CLOCKS
    unsigned long long bar_cal = 0, bar_vm = 0, bar_sync = 0;
#endif

    // ---- prologue: steps 0 and 1 into the two stages, fragments of step 0's k group 0
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        const int step = min(s, nsteps - 1);
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            oa.aim_round(lds + s * STAGE_BYTES, wave, t);
            asm volatile("s_nop 0");
            oa.fetch_round(ra, a_org + step * a_step, t);
            ob.aim_round(lds + s * STAGE_BYTES + OPERAND_BYTES, wave, t);
            asm volatile("s_nop 0");
            ob.fetch_round(rb, b_org + step * b_step, t);
        }
    }
    // vmcnt(16): this wave's pieces of the first stage are in LDS (the 16 loads of the second stage may still be on
    // their way: the first step's own wait, before its barrier, covers them)
    __builtin_amdgcn_s_waitcnt(0x4f70);
    __syncthreads();
    if (g.stamps) wall[1] = wall_clock64(), clk[0] = __builtin_readcyclecounter();
#pragma unroll
    for (int n = 0; n < 8; ++n) {
        fb[0][n] = ob.read(lds + OPERAND_BYTES, 0, n);
        fa[0][n] = oa.read(lds, 0, n);
    }

    // ---- one step out of stage `cur`; `fetch_step` is the step whose tiles are fetched into it
    auto do_step = [&](auto cur_tag, int fetch_step) {
        constexpr int cur = decltype(cur_tag)::value;
        char *As = lds + cur * STAGE_BYTES, *Bs = As + OPERAND_BYTES;
        char *An = lds + (cur ^ 1) * STAGE_BYTES, *Bn = An + OPERAND_BYTES;
        const unsigned a_src = a_org + fetch_step * a_step, b_src = b_org + fetch_step * b_step;
        // half 0
#pragma unroll
        for (int m = 0; m < 64; ++m) {
            mfma(acc[BI(m)][BJ(m)], fa[0][BI(m)], fb[0][BJ(m)]);
#ifndef D8_WIDE_DIAG_NO_FRAGMENT_READS
            if (m % 3 == 0 && m < 48) {
                const int e = m / 3;  // 16 reads: the B fragments first (all needed by the first row)
                if (e < 8) fb[1][e] = ob.read(Bs, 1, e);
                else fa[1][e - 8] = oa.read(As, 1, e - 8);
            }
#endif
        }
        // half 1
#ifdef D8_WIDE_DIAG_BARRIER_CLOCKS
        const unsigned long long tb0 = __builtin_readcyclecounter();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        const unsigned long long tb1 = __builtin_readcyclecounter();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#endif
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): my pieces of the next step have landed
#ifdef D8_WIDE_DIAG_BARRIER_CLOCKS
        const unsigned long long tb2 = __builtin_readcyclecounter();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#endif
#ifndef D8_WIDE_DIAG_NO_BARRIER
        __syncthreads();
#endif
#ifdef D8_WIDE_DIAG_BARRIER_CLOCKS
        const unsigned long long tb3 = __builtin_readcyclecounter();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        bar_cal += tb1 - tb0, bar_vm += tb2 - tb1, bar_sync += tb3 - tb2;
#endif
#pragma unroll
        for (int m = 0; m < 64; ++m) {
#ifndef D8_WIDE_DIAG_NO_LOADS
            if ((m & 3) == 0) {
                if ((m >> 2) < 8) oa.aim_round(As, wave, m >> 2);
                else ob.aim_round(Bs, wave, (m >> 2) - 8);
            }
#endif
            mfma(acc[BI(m)][BJ(m)], fa[1][BI(m)], fb[1][BJ(m)]);
            if ((m & 3) == 0) {
                // 16 loads into the stage every wave has finished with, one per 4 MFMAs: a load
                // keeps the CU's address path busy for 16 cycles, as long as an MFMA runs, and all
                // four waves issue theirs in the same window; issued closer together they hold up
                // instruction issue (2600 cycles per step at one per 2 MFMAs, 2330 at one per 4)
#ifndef D8_WIDE_DIAG_NO_LOADS
                const int d = m >> 2;
                if (d < 8) oa.fetch_round(ra, a_src, d);
                else ob.fetch_round(rb, b_src, d - 8);
#endif
            }
#ifndef D8_WIDE_DIAG_NO_FRAGMENT_READS
            if (m % 3 == 1 && m < 48) {
                const int e = m / 3;  // fragments of the next step's k group 0
                if (e < 8) fb[0][e] = ob.read(Bn, 0, e);
                else fa[0][e - 8] = oa.read(An, 0, e - 8);
            }
#endif
        }
    };

    for (int s = 0; s < nsteps; s += 2) {
        do_step(std::integral_constant<int, 0>(), min(s + 2, nsteps - 1));
        if (s + 1 < nsteps) do_step(std::integral_constant<int, 1>(), min(s + 3, nsteps - 1));
    }

    // ---- epilogue: 16 rows of the wave's 128 x 128 at a time through a patch of LDS, so that C
    // is read (beta = 1) and written 16 bytes per lane, 256 contiguous bytes per 16 lanes
    if (g.stamps) wall[2] = wall_clock64(), clk[1] = __builtin_readcyclecounter();
#ifdef D8_WIDE_DIAG_DIRECT_STORE
    {
        // the blocks were accumulated transposed (operands exchanged): lane holds C[i*16 + (lane & 15)][j*16 + 4*(lane >> 4) + 0..3]
        f16 *C = (f16 *)g.C + (long)b * g.sC;
        const int l15 = lane & 15, l4 = lane >> 4;
        typedef __fp16 h4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int m = m0 + wm * 128 + i * 16 + l15;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int n = n0 + wn * 128 + j * 16 + 4 * l4;
                if (m >= m_own && n >= n_own) {
                    f16 *c = C + (long)m * g.ldc + n;
                    h4 out;
                    if (g.beta != 0.f) {
                        const h4 old = *(const h4 *)c;
#pragma unroll
                        for (int e = 0; e < 4; ++e) out[e] = (__fp16)(acc[i][j][e] + (float)old[e]);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) out[e] = (__fp16)acc[i][j][e];
                    }
                    __builtin_nontemporal_store(out, (h4 *)c);
                }
            }
        }
    }
#else
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();  // no load is still on its way into LDS, every wave is past its last read
    float *patch = (float *)lds + wave * (16 * PATCH_LD);
    f16 *C = (f16 *)g.C + (long)b * g.sC;
    const int l15 = lane & 15, l4 = lane >> 4;
    // beta = 1: the old C of a 16-row slab is fetched while the slab before it goes through the patch, so that
    // only the first slab's read is waited for
    f16x8 oldc[2][4];
    auto fetch_old = [&](int i, f16x8(&dst)[4]) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int m = m0 + wm * 128 + i * 16 + t * 4 + l4, n = n0 + wn * 128 + l15 * 8;
            if (m >= m_own && n >= n_own) dst[t] = *(const f16x8 *)(C + (long)m * g.ldc + n);
        }
    };
    if (g.beta != 0.f) fetch_old(0, oldc[0]);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        if (g.beta != 0.f && i + 1 < 8) fetch_old(i + 1, oldc[(i + 1) & 1]);
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) patch[(4 * l4 + r) * PATCH_LD + j * 16 + l15] = acc[i][j][r];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int row = t * 4 + l4, cc = l15 * 8;
            const int m = m0 + wm * 128 + i * 16 + row, n = n0 + wn * 128 + cc;
            float v[8];
            *(f32x4 *)&v[0] = *(const f32x4 *)(patch + row * PATCH_LD + cc);
            *(f32x4 *)&v[4] = *(const f32x4 *)(patch + row * PATCH_LD + cc + 4);
#ifdef D8_WIDE_DIAG_NO_STORE
            if (m >= m_own && n >= n_own && g.K < 0) {
#else
            if (m >= m_own && n >= n_own) {
#endif
                f16 *c = C + (long)m * g.ldc + n;
                f16x8 out;
                if (g.beta != 0.f) {
                    const f16x8 old = oldc[i & 1][t];
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] += (float)old[e];
                }
                if (g.bias) {  // fused store: per-column bias, then ReLu (see GemmArgs::bias)
                    const f16x8 bv = *(const f16x8 *)((const f16 *)g.bias + n);
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] += (float)bv[e];
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) out[e] = (f16)(g.relu && !(v[e] > 0.f) ? 0.f : v[e]);
                // streamed past the L2: the whole output leaves the chip during the kernel's last microseconds
                // either way, and lines left dirty in L2 are written back only after the last wave has ended
                __builtin_nontemporal_store(out, (f16x8 *)c);
            }
        }
    }
#endif
    if (g.stamps) {
        __builtin_amdgcn_s_waitcnt(0x0f70);  // this wave's stores have been acknowledged
        wall[3] = wall_clock64();
        if (tid == 0) {
            unsigned long long *rec = (unsigned long long *)g.ws + 6 * (blockIdx.x + gridDim.x * blockIdx.z);
            rec[0] = wall[0], rec[1] = wall[1], rec[2] = wall[2], rec[3] = wall[3], rec[4] = clk[0], rec[5] = clk[1];
#ifdef D8_WIDE_DIAG_BARRIER_CLOCKS
            rec[0] = bar_cal, rec[1] = bar_vm, rec[2] = bar_sync;
#endif
        }
    }
}

bool gemm_wide_eligible(const GemmArgs &g, int transA, int transB) {
    if (g.virt != VIRT_NONE || g.red != 1 || g.splits != 1) return false;
    if (g.M < 256 || g.N < 256 || g.K < 64 || g.K % 64) return false;
    if (g.lda % 8 || g.ldb % 8 || g.ldc % 8 || g.sA % 8 || g.sB % 8 || g.sC % 8 || g.N % 8) return false;
    if (transA && g.M % 8) return false;
    if (((size_t)g.A | (size_t)g.B | (size_t)g.C | (size_t)g.bias) & 15) return false;
    if (2L * (transA ? g.K : g.M) * g.lda >= (1L << 31) || 2L * (transB ? g.N : g.K) * g.ldb >= (1L << 31)) return false;
    if ((long)ceil_div(g.M, 256) * ceil_div(g.N, 256) > 0x7fffffffL || g.batch > 65535) return false;
    return true;
}

size_t gemm_wide_stamp_bytes(const GemmArgs &g) {
    return (size_t)ceil_div(g.M, 256) * ceil_div(g.N, 256) * g.batch * 6 * sizeof(unsigned long long);
}

int gemm_wide_launch(const GemmArgs &g0, int transA, int transB, hipStream_t stream) {
    static const bool stamps = getenv("D8_GEMM_STAMPS") != nullptr;  // measurement aid, see GemmArgs::stamps
    GemmArgs g = g0;
    g.stamps = stamps && g.ws && ((size_t)g.ws & 7) == 0 && g.ws_bytes >= gemm_wide_stamp_bytes(g);
    const int tilesM = ceil_div(g.M, 256), tilesN = ceil_div(g.N, 256);
    const dim3 grid(tilesM * tilesN, 1, g.batch), block(256);
    if (!transA && !transB) hipLaunchKernelGGL((gemm_wide_kernel<true, false>), grid, block, 0, stream, g, tilesM, tilesN);
    else if (!transA && transB) hipLaunchKernelGGL((gemm_wide_kernel<true, true>), grid, block, 0, stream, g, tilesM, tilesN);
    else hipLaunchKernelGGL((gemm_wide_kernel<false, false>), grid, block, 0, stream, g, tilesM, tilesN);
    D8_LAUNCH_CHECK();
    return 0;
}

}  // namespace d8
