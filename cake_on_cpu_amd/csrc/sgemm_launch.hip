// GEMM launch dispatch, tile table and the split-K reduction.
#include "sgemm_tile.hpp"

namespace cake {

hipError_t launch_sgemm_vec(int tile_id, const GemmArgs& a, int grid, hipStream_t s);
hipError_t launch_sgemm_vec_nchw(int tile_id, const GemmArgs& a, int grid, hipStream_t s);
hipError_t launch_sgemm_scalar(int tile_id, const GemmArgs& a, int grid, hipStream_t s);
hipError_t launch_sgemm_convrow(int tile_id, const GemmArgs& a, int grid, hipStream_t s);
hipError_t launch_sgemm_vec_nt(int tile_id, const GemmArgs& a, int grid, hipStream_t s);
hipError_t launch_sgemm_conv1x1(int tile_id, const GemmArgs& a, int grid, hipStream_t s);

template <class T>
static constexpr TileInfo info_of()
{
    return TileInfo{T::BM, T::BN, T::BK, T::WM, T::WN, T::THREADS, T::LDS_BYTES};
}

const TileInfo& tile_info(int tile_id)
{
    static const TileInfo table[TILE_COUNT] = {
        info_of<Tile256x256x32>(), info_of<Tile256x128x32>(),
        info_of<Tile128x256x32>(), info_of<Tile128x128x32>(), info_of<Tile64x64x32>(),
        info_of<Tile64x64x64>(), info_of<Tile96x128x32>(), info_of<Tile128x32x32>(), info_of<Tile32x128x32>(),
    };
    return table[tile_id < 0 || tile_id >= TILE_COUNT ? TILE_64x64x32_W32x32 : tile_id];
}

hipError_t launch_sgemm(int tile_id, int a_mode, int b_mode, const GemmArgs& args, int grid,
                        hipStream_t stream)
{
    if (grid <= 0) return hipSuccess;
    if (b_mode == LOAD_IM2COL_1X1) {
        if (a_mode != LOAD_VEC4) return hipErrorInvalidValue;
        return launch_sgemm_conv1x1(tile_id, args, grid, stream);
    }
    if (b_mode == LOAD_IM2COL_ROW) {
        if (a_mode != LOAD_VEC4) return hipErrorInvalidValue;
        return launch_sgemm_convrow(tile_id, args, grid, stream);
    }
    if (b_mode == LOAD_VEC4_T) {
        if (a_mode != LOAD_VEC4) return hipErrorInvalidValue;
        return launch_sgemm_vec_nt(tile_id, args, grid, stream);
    }
    if (b_mode == LOAD_VEC4_NCHW) {
        if (a_mode != LOAD_VEC4 || !args.conv.in) return hipErrorInvalidValue;
        return launch_sgemm_vec_nchw(tile_id, args, grid, stream);
    }
    if (a_mode == LOAD_VEC4 && b_mode == LOAD_VEC4) return launch_sgemm_vec(tile_id, args, grid, stream);
    return launch_sgemm_scalar(tile_id, args, grid, stream);
}

hipError_t launch_tail_reduce(int tile_id, const GemmArgs& a, hipStream_t stream)
{
    if (a.tail_tiles <= 0) return hipSuccess;
    const TileInfo& t = tile_info(tile_id);
    const dim3 grid(a.tail_tiles, t.bm * t.bn / 1024), block(256);
    switch (tile_id) {
        case TILE_256x256x32_W128x64: hipLaunchKernelGGL(tail_reduce_kernel<Tile256x256x32>, grid, block, 0, stream, a); break;
        case TILE_256x128x32_W64x64: hipLaunchKernelGGL(tail_reduce_kernel<Tile256x128x32>, grid, block, 0, stream, a); break;
        case TILE_128x256x32_W64x64: hipLaunchKernelGGL(tail_reduce_kernel<Tile128x256x32>, grid, block, 0, stream, a); break;
        case TILE_128x128x32_W64x64: hipLaunchKernelGGL(tail_reduce_kernel<Tile128x128x32>, grid, block, 0, stream, a); break;
        case TILE_64x64x32_W32x32: hipLaunchKernelGGL(tail_reduce_kernel<Tile64x64x32>, grid, block, 0, stream, a); break;
        case TILE_64x64x64_W32x32: hipLaunchKernelGGL(tail_reduce_kernel<Tile64x64x64>, grid, block, 0, stream, a); break;
        case TILE_96x128x32_W96x32: hipLaunchKernelGGL(tail_reduce_kernel<Tile96x128x32>, grid, block, 0, stream, a); break;
        case TILE_128x32x32_W32x32: hipLaunchKernelGGL(tail_reduce_kernel<Tile128x32x32>, grid, block, 0, stream, a); break;
        case TILE_32x128x32_W32x32: hipLaunchKernelGGL(tail_reduce_kernel<Tile32x128x32>, grid, block, 0, stream, a); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// C = (accumulate ? C : 0) + sum over slices in ascending order: a fixed
// summation order, so the split-K path is run-to-run deterministic like the
// reference (one accumulation chain per element, no atomics).
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float* __restrict__ partial,
                                                            float* __restrict__ C, int M, int N,
                                                            int ldc, int splits, int accumulate,
                                                            ConvGeom conv,
                                                            const float* __restrict__ col_bias)
{
    const size_t total = (size_t)M * N;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        const int row = (int)(i / N), col = (int)(i - (size_t)row * N);
        float* dst = C + (size_t)row * ldc + col;
        if (conv.in) {  // a convolution's column: see conv_out_map
            size_t off, row_stride;
            if (conv_out_map(conv, M, ldc, col, 1, off, row_stride) < 1) continue;
            dst = C + (size_t)row * row_stride + off;
        }
        float acc = accumulate ? *dst : 0.f;
        // (unrolled: the loads of several slices are in flight together, the additions keep their order)
#pragma unroll 8
        for (int s = 0; s < splits; ++s) acc += partial[(size_t)s * total + i];
        if (col_bias) acc += col_bias[col];
        *dst = acc;
    }
}

hipError_t launch_splitk_reduce(const float* partial, float* C, int M, int N, int ldc, int splits,
                                int accumulate, hipStream_t stream, const ConvGeom* conv, const float* col_bias)
{
    const size_t total = (size_t)M * N;
    if (total == 0) return hipSuccess;
    size_t blocks = (total + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, partial, C,
                       M, N, ldc, splits, accumulate, conv ? *conv : ConvGeom{}, col_bias);
    return hipGetLastError();
}

}  // namespace cake
