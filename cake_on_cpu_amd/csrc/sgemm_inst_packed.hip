// Macro-tile GEMM instantiations that read A and/or B from the reference's
// packed layouts through bilinear index tables.  Row-major partners use the
// any-alignment loader.
#include "sgemm_tile.hpp"

namespace cake {

template <class T>
static hipError_t by_mode(int a_mode, int b_mode, const GemmArgs& a, int grid, hipStream_t s)
{
    if (a_mode == LOAD_PACKED && b_mode == LOAD_PACKED) return launch_tile<T, LOAD_PACKED, LOAD_PACKED>(a, grid, s);
    if (a_mode == LOAD_PACKED) return launch_tile<T, LOAD_PACKED, LOAD_SCALAR>(a, grid, s);
    if (b_mode == LOAD_PACKED) return launch_tile<T, LOAD_SCALAR, LOAD_PACKED>(a, grid, s);
    return hipErrorInvalidValue;
}

hipError_t launch_sgemm_packed(int tile_id, int a_mode, int b_mode, const GemmArgs& a, int grid,
                               hipStream_t s)
{
    switch (tile_id) {
        case TILE_256x256x32_W128x64: return by_mode<Tile256x256x32>(a_mode, b_mode, a, grid, s);
        case TILE_128x128x32_W64x64: return by_mode<Tile128x128x32>(a_mode, b_mode, a, grid, s);
        case TILE_64x64x32_W32x32: return by_mode<Tile64x64x32>(a_mode, b_mode, a, grid, s);
        case TILE_64x64x64_W32x32: return by_mode<Tile64x64x64>(a_mode, b_mode, a, grid, s);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace cake
