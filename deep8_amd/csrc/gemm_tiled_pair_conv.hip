// Two patch-matrix products as one launch of the tiled kernel (gemm_tiled_pair_kernel, gemm_tiled_kernel.h): gx has patch
// rows as A (NN), gy patch k-rows as B (TN) -- the gradients of a convolution's input and filter.  gx may carry its
// remainder band; gy may be split along its reduction (the caller reduces).
#include "gemm_tiled_kernel.h"

namespace d8 {

template <typename E>
static bool pair_tiles(const GemmArgs &gx, const GemmArgs &gy, TileId &tx, TileId &ty) {
    tx = choose_tile<E, true, false, VIRT_A_ROWS>(gx), ty = choose_tile<E, false, false, VIRT_B_KROWS>(gy);
    const bool x_ok = tx == TILE_64x128 || tx == TILE_128x128 || tx == TILE_128x64;
    const bool y_ok = ty == TILE_128x128 || ty == TILE_64x128 || ty == TILE_64x64;
    return x_ok && y_ok;
}

template <typename E>
static int launch_pair(const GemmArgs &gx, const GemmArgs &gy, hipStream_t stream) {
    TileId tx, ty;
    if (!pair_tiles<E>(gx, gy, tx, ty)) return fail(D8_ERR_ARGUMENT, "gemm_tiled_pair_launch: no kernel for this pair of tiles");
#define D8_PAIR_Y(TXT)                                                                                                  \
    switch (ty) {                                                                                                       \
        case TILE_128x128: return launch_pair_tiles<TXT, Tile<E, 128, 128, 2, 2, false, false, VIRT_B_KROWS>>(gx, gy, stream); \
        case TILE_64x128: return launch_pair_tiles<TXT, Tile<E, 64, 128, 2, 2, false, false, VIRT_B_KROWS>>(gx, gy, stream);   \
        default: return launch_pair_tiles<TXT, Tile<E, 64, 64, 2, 2, false, false, VIRT_B_KROWS>>(gx, gy, stream);            \
    }
    typedef Tile<E, 64, 128, 2, 2, true, false, VIRT_A_ROWS> X0;
    typedef Tile<E, 128, 128, 2, 2, true, false, VIRT_A_ROWS> X1;
    typedef Tile<E, 128, 64, 2, 2, true, false, VIRT_A_ROWS> X2;
    if (tx == TILE_64x128) { D8_PAIR_Y(X0) }
    if (tx == TILE_128x128) { D8_PAIR_Y(X1) }
    D8_PAIR_Y(X2)
#undef D8_PAIR_Y
}

long gemm_tiled_pair_workgroups(int dtype, const GemmArgs &gx, const GemmArgs &gy) {
    TileId tx, ty;
    if (gx.virt != VIRT_A_ROWS || gy.virt != VIRT_B_KROWS || gy.tail_splits || gx.splits != 1 || gx.batch != 1 || gy.batch != 1)
        return 0;
    if (!(dtype == D8_FLOAT16 ? pair_tiles<f16>(gx, gy, tx, ty) : pair_tiles<float>(gx, gy, tx, ty))) return 0;
    int mx, nx, my, ny;
    grid_of(tx, gx, mx, nx);
    grid_of(ty, gy, my, ny);
    if (gx.tail_splits && tx != TILE_128x64) return 0;  // (a band is cut for 128-row tiles of a narrow output only)
    return (long)mx * nx + (long)my * ny * gy.splits;
}

int gemm_tiled_pair_launch(int dtype, const GemmArgs &gx, const GemmArgs &gy, hipStream_t stream) {
    return dtype == D8_FLOAT16 ? launch_pair<f16>(gx, gy, stream) : launch_pair<float>(gx, gy, stream);
}

}  // namespace d8
