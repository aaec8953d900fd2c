// Macro-tile GEMM instantiations: row-major operands, 16-byte global loads.
#include "sgemm_tile.hpp"

namespace cake {

hipError_t launch_sgemm_vec(int tile_id, const GemmArgs& a, int grid, hipStream_t s)
{
    switch (tile_id) {
        case TILE_256x256x32_W128x64: return launch_tile<Tile256x256x32, LOAD_VEC4, LOAD_VEC4>(a, grid, s);
        case TILE_256x128x32_W64x64: return launch_tile<Tile256x128x32, LOAD_VEC4, LOAD_VEC4>(a, grid, s);
        case TILE_128x256x32_W64x64: return launch_tile<Tile128x256x32, LOAD_VEC4, LOAD_VEC4>(a, grid, s);
        case TILE_128x128x32_W64x64: return launch_tile<Tile128x128x32, LOAD_VEC4, LOAD_VEC4>(a, grid, s);
        case TILE_64x64x32_W32x32: return launch_tile<Tile64x64x32, LOAD_VEC4, LOAD_VEC4>(a, grid, s);
        case TILE_64x64x64_W32x32: return launch_tile<Tile64x64x64, LOAD_VEC4, LOAD_VEC4>(a, grid, s);
        case TILE_96x128x32_W96x32: return launch_tile<Tile96x128x32, LOAD_VEC4, LOAD_VEC4>(a, grid, s);
        case TILE_128x32x32_W32x32: return launch_tile<Tile128x32x32, LOAD_VEC4, LOAD_VEC4>(a, grid, s);
        case TILE_32x128x32_W32x32: return launch_tile<Tile32x128x32, LOAD_VEC4, LOAD_VEC4>(a, grid, s);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace cake
