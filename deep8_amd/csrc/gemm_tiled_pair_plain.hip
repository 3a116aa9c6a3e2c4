// Two real products as one launch of the tiled kernel (gemm_tiled_pair_kernel, gemm_tiled_kernel.h): the two gradients of a
// mid-size MatrixMultiply.
#include "gemm_tiled_kernel.h"

namespace d8 {

// g0 is NT (a MatrixMultiply's gradient of its first input),
// g1 is TN (the gradient of its second); either may be batched or split along its reduction (the caller reduces).
template <typename E>
static bool plain_pair_tiles(const GemmArgs &g0, const GemmArgs &g1, TileId &t0, TileId &t1) {
    t0 = choose_tile<E, true, true>(g0), t1 = choose_tile<E, false, false>(g1);
    const bool ok0 = t0 == TILE_64x128 || t0 == TILE_128x128 || t0 == TILE_128x64;
    const bool ok1 = t1 == TILE_64x128 || t1 == TILE_128x128 || t1 == TILE_128x64;
    constexpr int BK = 128 / (int)sizeof(E);
    return ok0 && ok1 && g0.K % BK == 0 && g1.K % BK == 0;
}

template <typename E>
static int launch_plain_pair(const GemmArgs &g0, const GemmArgs &g1, hipStream_t stream) {
    TileId t0, t1;
    if (!plain_pair_tiles<E>(g0, g1, t0, t1)) return fail(D8_ERR_ARGUMENT, "gemm_tiled_plain_pair_launch: no kernel for this pair of tiles");
#define D8_PAIR_1(T0T)                                                                                              \
    switch (t1) {                                                                                                   \
        case TILE_128x128: return launch_pair_tiles<T0T, Tile<E, 128, 128, 2, 2, false, false>>(g0, g1, stream);    \
        case TILE_64x128: return launch_pair_tiles<T0T, Tile<E, 64, 128, 2, 2, false, false>>(g0, g1, stream);      \
        default: return launch_pair_tiles<T0T, Tile<E, 128, 64, 2, 2, false, false>>(g0, g1, stream);               \
    }
    typedef Tile<E, 64, 128, 2, 2, true, true> A0;
    typedef Tile<E, 128, 128, 2, 2, true, true> A1;
    typedef Tile<E, 128, 64, 2, 2, true, true> A2;
    if (t0 == TILE_64x128) { D8_PAIR_1(A0) }
    if (t0 == TILE_128x128) { D8_PAIR_1(A1) }
    D8_PAIR_1(A2)
#undef D8_PAIR_1
}

long gemm_tiled_plain_pair_workgroups(int dtype, const GemmArgs &g0, const GemmArgs &g1) {
    TileId t0, t1;
    if (g0.virt != VIRT_NONE || g1.virt != VIRT_NONE || g0.tail_splits || g1.tail_splits) return 0;
    if (!(dtype == D8_FLOAT16 ? plain_pair_tiles<f16>(g0, g1, t0, t1) : plain_pair_tiles<float>(g0, g1, t0, t1))) return 0;
    int m0, n0, m1, n1;
    grid_of(t0, g0, m0, n0);
    grid_of(t1, g1, m1, n1);
    return (long)m0 * n0 * g0.batch * g0.splits + (long)m1 * n1 * g1.batch * g1.splits;
}

int gemm_tiled_plain_pair_launch(int dtype, const GemmArgs &g0, const GemmArgs &g1, hipStream_t stream) {
    return dtype == D8_FLOAT16 ? launch_plain_pair<f16>(g0, g1, stream) : launch_plain_pair<float>(g0, g1, stream);
}

}  // namespace d8
