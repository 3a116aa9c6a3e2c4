// Host side of the tiled GEMM kernels (gemm_tiled_kernel.h): the launch of one product on the tile its shape asks for,
// eligibility, the phase-record switch.
#include "gemm_tiled_kernel.h"

namespace d8 {

unsigned long long *phase_rec_buf = nullptr;
size_t phase_rec_bytes = 0;


void gemm_tiled_phase_record(void *records, size_t bytes) {
    phase_rec_buf = (unsigned long long *)records;
    phase_rec_bytes = records ? bytes : 0;
}

template <typename E, int BM, int BN, int WGM, int WGN, bool A_KC, bool B_KC, int VIRT>
static int launch_tiled(const GemmArgs &g0, hipStream_t stream) {
    GemmArgs g = g0;
    typedef Tile<E, BM, BN, WGM, WGN, A_KC, B_KC, VIRT> T;
    const bool tail = g.tail_splits > 0;  // (gemm_tiled_run sets it only for 128-row tiles and a tail_m0 that is a multiple of them)
    const int tilesM = ceil_div(tail ? g.tail_m0 : g.M, BM), tilesN = ceil_div(g.N, BN);
    const int extra = tail ? ceil_div(g.M - g.tail_m0, BM) * tilesN * g.tail_splits : 0;
    // A launch of at most two workgroups per CU is spread evenly only if a CU cannot take a third:
    // where the tile's own LDS would let three in, unused dynamic LDS is requested on top.
    constexpr long lds = 2L * (T::A_SZ + T::B_SZ) * T::ES, third = 160 * 1024 / 3;
    const int layers = VIRT == VIRT_A_CLASSES ? g.ncls : g.batch * g.splits;  // for classes g.M is the largest one's
    const long wgs = (long)tilesM * tilesN * layers, cus = cu_count();
    const unsigned pad = (lds <= third && wgs > cus && wgs <= 2 * cus) ? (unsigned)(third + 512 - lds) : 0u;
    // a launch whose records would not fit the caller's buffer writes none
    g.phase_rec = (size_t)(tilesM * tilesN + extra) * layers * 64 <= phase_rec_bytes ? phase_rec_buf : nullptr;
    if (VIRT == VIRT_NONE && g.K % T::BK)
        hipLaunchKernelGGL((gemm_tiled_kernel<T, VIRT == VIRT_NONE>), dim3(tilesM * tilesN + extra, 1, layers), dim3(T::NT), pad, stream, g, tilesM, tilesN);
    else
        hipLaunchKernelGGL((gemm_tiled_kernel<T, false>), dim3(tilesM * tilesN + extra, 1, layers), dim3(T::NT), pad, stream, g, tilesM, tilesN);
    D8_LAUNCH_CHECK();
    return 0;
}

template <typename E, bool A_KC, bool B_KC, int VIRT = VIRT_NONE>
static int pick_tile(const GemmArgs &g, hipStream_t stream) {
    switch (choose_tile<E, A_KC, B_KC, VIRT>(g)) {
        case TILE_WIDE: return gemm_wide_launch(g, !A_KC, B_KC, stream);
        case TILE_256:
            if constexpr (sizeof(E) == 2) return launch_tiled<E, 256, 256, 4, 2, A_KC, B_KC, VIRT>(g, stream);
            break;
        case TILE_128x64: return launch_tiled<E, 128, 64, 2, 2, A_KC, B_KC, VIRT>(g, stream);
        case TILE_64x64:
            if constexpr (VIRT == VIRT_B_KROWS) return launch_tiled<E, 64, 64, 2, 2, A_KC, B_KC, VIRT>(g, stream);
            break;
        case TILE_64x128: return launch_tiled<E, 64, 128, 2, 2, A_KC, B_KC, VIRT>(g, stream);
        default: break;
    }
    return launch_tiled<E, 128, 128, 2, 2, A_KC, B_KC, VIRT>(g, stream);
}

template <typename E>
static bool eligible(const GemmArgs &g, int transA, int transB) {
    constexpr long ES = sizeof(E), EPV = 16 / ES, BK = 128 / ES;
    const bool va = g.virt == VIRT_A_ROWS || g.virt == VIRT_A_CLASSES, vb = g.virt == VIRT_B_KROWS;
    if (g.virt == VIRT_A_CLASSES && (g.splits > 1 || g.ncls < 1 || g.ncls > MAX_CLASSES || g.M < 128)) return false;
    if (va && (transA || g.K != g.pg.C)) return false;                       // a K step stays inside one tap
    if (vb && (!transA || transB || g.red != 1 || g.pg.C % EPV || g.N % g.pg.C)) return false;  // a piece stays inside one tap
    if ((va || vb) && (g.pg.bytes >= (1u << 31) || g.batch != 1)) return false;
    // byte offsets inside one operand (all summed products of it included) are 32-bit
    if (!va && ((g.red - 1) * g.sA + (long)(transA ? g.K : g.M) * g.lda) * ES >= (1L << 31)) return false;
    if (!vb && ((g.red - 1) * g.sB + (long)(transB ? g.N : g.K) * g.ldb) * ES >= (1L << 31)) return false;
    // one side may be shorter than any tile (a few rows against a wide matrix: the 64 x 128 / 128 x 64 tile
    // then reaches past it) when the other side fills a tile
    if ((g.M < 128 && g.N < 128) || g.K < 1) return false;  // (a K below one K step is a lone partial step)
    // (patch rows as A: a filter with few output channels is fine, its rows past the last read as zeros)
    if (g.virt != VIRT_NONE && (g.M < 64 || (g.N < 64 && g.virt == VIRT_B_KROWS))) return false;
    // a last K step that is partly past K: real matrices only, and a 16-byte piece of an operand stored along K
    // must lie wholly on one side of K
    if (g.K % BK && (g.virt != VIRT_NONE || ((!transA || transB) && g.K % EPV))) return false;
    if (!va && (g.lda % EPV || g.sA % EPV)) return false;
    if (!vb && (g.ldb % EPV || g.sB % EPV)) return false;
    if (((size_t)g.A | (size_t)g.B) & 15) return false;
    if (transA && g.M % EPV) return false;
    if (!transB && g.N % EPV) return false;
    if ((long)ceil_div(g.M, 128) * ceil_div(g.N, 128) > 0x7fffffffL || (long)g.batch * 128 > 65535) return false;
    return true;
}

template <typename E>
static int launch_any(const GemmArgs &g, int transA, int transB, hipStream_t stream) {
    if (g.virt == VIRT_A_CLASSES) {  // every class has at least 128 rows (checked by eligible)
        if (transB) {
            if (g.N < 128) return launch_tiled<E, 128, 64, 2, 2, true, true, VIRT_A_CLASSES>(g, stream);
            return launch_tiled<E, 128, 128, 2, 2, true, true, VIRT_A_CLASSES>(g, stream);
        }
        if (g.N < 128) return launch_tiled<E, 128, 64, 2, 2, true, false, VIRT_A_CLASSES>(g, stream);
        return launch_tiled<E, 128, 128, 2, 2, true, false, VIRT_A_CLASSES>(g, stream);
    }
    if (g.virt == VIRT_A_ROWS) return transB ? pick_tile<E, true, true, VIRT_A_ROWS>(g, stream) : pick_tile<E, true, false, VIRT_A_ROWS>(g, stream);
    if (g.virt == VIRT_B_KROWS) return pick_tile<E, false, false, VIRT_B_KROWS>(g, stream);
    if (!transA && !transB) return pick_tile<E, true, false>(g, stream);
    if (!transA && transB) return pick_tile<E, true, true>(g, stream);
    return pick_tile<E, false, false>(g, stream);
}

int gemm_tiled_k_step(int dtype) { return dtype == D8_FLOAT16 ? 64 : 32; }

bool gemm_tiled_eligible(int dtype, const GemmArgs &g, int transA, int transB) {
    if (dtype == D8_FLOAT64) return false;
    return dtype == D8_FLOAT16 ? eligible<f16>(g, transA, transB) : eligible<float>(g, transA, transB);
}

int gemm_tiled_launch(int dtype, const GemmArgs &g, int transA, int transB, hipStream_t stream) {
    return dtype == D8_FLOAT16 ? launch_any<f16>(g, transA, transB, stream) : launch_any<float>(g, transA, transB, stream);
}

}  // namespace d8
