// kernels.hpp -- launch interface between the host side of the library and the
// gfx950 kernels.  Every launcher only enqueues on `stream` and returns the
// hipError_t of the launch.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "blockdims.hpp"

namespace cake {

// One row (or column) of a packed operand's bilinear index map:
//   offset(row, col) = R.x + C.x + R.y*C.y + R.z*C.z + R.w*C.w
// which is the form every packed layout of the reference reduces to.
struct IndexTables {
    const int4* row;
    const int4* col;
};

// Geometry of a convolution whose column matrix B[k][n] is gathered on the fly from a staged
// copy of the input (conv_stage_input_kernel in misc_kernels.hip: padding written out, rows split
// into column phases when the stride is above 1):
// n / d for n < 2^31 as one 32 x 32 -> 64 bit multiply and a shift (division by an invariant
// integer): with s = ceil(log2 d) and m = floor(2^(31+s) / d) + 1 the error m d - 2^(31+s) is at
// most d <= 2^s, so n (m d - 2^(31+s)) < 2^(31+s) for every n < 2^31 and the quotient is exact.
// A hardware division costs tens of vector instructions (a 64-bit one well over a hundred), enough
// to make a write-bound copy compute-bound -- or, two dozen of them per lane, to put microseconds
// in front of a tile's first load.
struct FastDiv {
    unsigned d, m, sh;
    __host__ static FastDiv make(unsigned d)
    {
        if (d == 0) d = 1;
        unsigned s = 0;
        while ((1ull << s) < d) ++s;
        FastDiv f;
        f.d = d;
        f.m = (unsigned)((1ull << (31 + s)) / d + 1);
        f.sh = 31 + s;
        return f;
    }
    __device__ __forceinline__ unsigned div(unsigned n) const { return (unsigned)(((unsigned long long)n * m) >> sh); }
};

// Tail tiles of the patch kernel: K slices of whole channel blocks, or no slices in memory at
// all: 16 workgroups per tile, each computing 64 rows x 32 pixels over the whole K with the K
// quarters of every block dealt to its waves and summed through LDS (3 x 3 taps only).
enum { CONV_TAIL_BLOCKS = 0, CONV_TAIL_SUBTILES = 2 };
enum { CONV_TAIL_SUBTILES_PER_TILE = 16 };

// k = c*Hf*Wf + h*Wf + w, n = (b*Hout + ho)*row_n + wo,
// B[k][n] = in[((b*Cin*plane_rows + ho*row_step)*pitch + wo) + tap_table[k] / 4].
struct ConvGeom {
    const float* in;        // the staged input (the input itself for stride 1 without padding)
    unsigned in_bytes;      // its size: loads past it read as zero
    int Cin;
    int plane_rows;         // stored rows per (image, channel) plane
    int pitch;              // floats per stored row
    int row_step;           // stored rows per output row
    int Hout, Wout;
    int row_n;              // columns of the product per output row (a multiple of 4)
    const int* tap_table;   // byte offset of tap k = (c, h, w) inside one image, K + CONV_TAP_TABLE_EXTRA entries
    int tap_stride;         // 1 x 1 filters (LOAD_IM2COL_1X1): bytes from channel to channel, instead of the table
    int out_nchw;           // epilogue writes C as [batch][M][Hout*Wout] instead of [M][N]
    // sgemm_conv_patch.hip only (the input read where it lies, `in` = the NCHW input itself):
    int batch, Hin, Win, pad, Hf, Wf;
    int patch_rows, patch_pitch;   // rows and floats per row of the input patch a workgroup keeps in LDS
    // divisions by row_n, Hout, rows of a padded image (Hin + 2 pad), 16-byte chunks per patch
    // channel (patch_rows * ceil(Win / 4)) and chunks per input row
    FastDiv by_row_n, by_hout, by_vrows, by_channel_chunks, by_row_chunks;
    // the 16-byte chunks of a patch row that no load ever writes (one left of the image's columns,
    // the rest right of them): how many per row, and divisions by that and by the count per channel
    int margin_chunks;
    FastDiv by_margin_chunks, by_channel_margin_chunks;
    int stream_out;                // sgemm_conv_patch.hip: the output's rows are whole 128-byte lines, so it may leave
                                   // with non-temporal stores (partial lines written that way cost 35-45 %)
    int tail_mode;                 // sgemm_conv_patch.hip, how the tiles of a thin last round are cut (CONV_TAIL_*)
};

struct GemmArgs {
    const float* A;
    const float* B;
    float* C;
    float* partial;  // split-K slices [split][M][N], or nullptr
    int M, N, K;
    int lda, ldb, ldc;
    int tiles_m, tiles_n;
    int split_k, k_per_split;  // k_per_split is a multiple of the tile's BK
    int group, group_along_n;  // CB-block raster
    int accumulate;
    const float* col_bias;  // added to every row of the finished product (after accumulate), or nullptr
    // Tail splitting: the last `tail_tiles` tiles of the raster (the ones that
    // would run as a thin final round) are cut into `tail_split` K slices each,
    // written to tail_partial[slice][tail tile][BM x BN] and summed by
    // launch_tail_reduce.  0 tail_tiles = off.  Not combined with split_k > 1.
    int tail_tiles, tail_split, tail_k_per_split;
    float* tail_partial;
    ConvGeom conv;             // used by the implicit-im2col loader only
    // A batch of products with one A (sgemm_shortk.hip only): image b reads B + b * b_batch_stride
    // as a K x N matrix and writes C + b * c_batch_stride; tiles_n then counts the column tiles of
    // all images, tiles_n_per_image of them per image.  0 = a single product.
    int tiles_n_per_image;
    size_t b_batch_stride, c_batch_stride;
    // The same batch with its column tiles running across image borders (the kernel for K above 64
    // only): column n of the product is pixel n % batch_cols of image n / batch_cols, N counts the
    // columns of all images, tiles_n their tiles and tiles_n_per_image is 0.  Planes whose pixels
    // do not fill whole tiles then cost no padding.  batch_cols is a multiple of 4 and all of B
    // stays below 2^31 bytes.  0 = off.
    int batch_cols;
    // sgemm_shortk.hip: divisions of the tile walk as multiplications (filled in by its launcher):
    // by tiles per band, by tile rows of a whole band, by those of the last band, by column tiles per image
    FastDiv by_band, by_group, by_last_group, by_image_tiles, by_batch_cols;
};

// Macro-tile shapes the planner can choose from.
enum TileId {
    TILE_256x256x32_W128x64 = 0,  // 8 waves, 2 per SIMD: large compute-bound shapes
    TILE_256x128x32_W64x64,       // 8 waves: N around 128 (tall-skinny)
    TILE_128x256x32_W64x64,       // 8 waves: M around 128
    TILE_128x128x32_W64x64,       // 4 waves: mid-size shapes, 2 workgroups per CU
    TILE_64x64x32_W32x32,         // 4 waves: small shapes with several workgroups per CU
    TILE_64x64x64_W32x32,         // 8 waves, two per 32x32 block of C (one per K half): small shapes, one workgroup per CU
    TILE_96x128x32_W96x32,        // 4 waves side by side, each 96 rows tall: products with 65..96 (or 129..192) rows
    TILE_128x32x32_W32x32,        // 4 waves on top of each other: products with up to 32 columns (or 65..96), which wider tiles would pad
    TILE_32x128x32_W32x32,        // 4 waves side by side: products with up to 32 rows, which taller tiles would pad
    TILE_COUNT
};

struct TileInfo {
    int bm, bn, bk, wm, wn, threads, lds_bytes;
};
const TileInfo& tile_info(int tile_id);

// Operand addressing of the macro-tile loaders.
enum LoadMode {
    LOAD_VEC4 = 0,   // row-major, 16-byte loads (ld % 4 == 0, 16-byte aligned bases)
    LOAD_SCALAR = 1, // row-major, any size/alignment
    LOAD_VEC4_T = 2, // B only: B handed over as its transpose Bt[N][K] (rows ldb apart), 16-byte loads along k
    LOAD_IM2COL_ROW = 4, // B only: column matrix of a convolution gathered from the staged NCHW input,
                         // one 16-byte load per 4 columns
    LOAD_IM2COL_1X1 = 5, // the same for a 1 x 1 filter: row k is channel k, tap_stride bytes after row k - 1,
                         // so no tap table is read
    LOAD_VEC4_NCHW = 6   // B only: loaded as LOAD_VEC4 (an explicit column matrix), C's columns placed as a
                         // convolution's output (GemmArgs::conv describes it).  A mode of its own so that
                         // the plain product's epilogue carries none of that placement.
};

hipError_t launch_sgemm(int tile_id, int a_mode, int b_mode, const GemmArgs& args, int grid,
                        hipStream_t stream);
hipError_t launch_tail_reduce(int tile_id, const GemmArgs& args, hipStream_t stream);
// Products with a short K and many 64 x 64 tiles: workgroups that walk over tiles with the next
// tile's operands in flight (sgemm_shortk.hip).  Both operands row-major and 16-byte-loadable.
// K up to 64 of any kind; K from 65 to SHORTK_MAX_K (a batch of products with one A, i.e. a 1 x 1
// convolution: to SHORTK_MAX_K_BATCH) when it is a multiple of 4 and C is overwritten without a
// bias (launch_sgemm_shortk refuses the rest).
// shortk_tile_n: 0 when the kernel does not apply, else the width of its tiles (64)
enum { SHORTK_MAX_K = 160, SHORTK_MAX_K_BATCH = 256 };
// tile rows per band of the short-K kernel's tile sequence (group of the launch arguments)
int shortk_band_rows(int tiles_m, int N);
// A product that is all stores (K up to 32) into a C of more than the memory-side cache holds,
// with rows that are no whole cache lines apart: every row of a tile then ends in pieces of
// lines, which this memory writes far more slowly than whole ones, and what counts is how the
// pieces of neighbouring tiles meet in the L2.  Measured, us, short-K kernel / macro-tile kernel
// on 64 x 64 / on 96 x 128 / on 256 x 128 tiles: 8548 x 24 x 13421 161 / 144 / 140 / 149,
// 16384 x 16 x 16383 390 / 308 / 278 / 400, 8192 x 24 x 13420 147 / 154 / 122 / 175, 16384 x 16 x 16400
// 297 / 365 / 280 / 395, 9000 x 12 x 9001 102 / 92 / 91 / 103 (with rows 128 bytes apart, 8548 x 24 x 13440,
// the short-K kernel takes 96).  Such products run on the macro-tile kernel's 96 x 128 x 32 tile,
// the best or within 3 % of it on 14 shapes.
inline bool stores_in_pieces_of_lines(int M, int N, int K)
{
    return K <= 32 && N % 32 != 0 && (double)M * N * 4.0 > 256e6;
}
// batch >= 1 with shared_a: `batch` products M x K x N with one A (launched with tiles_n_per_image set)
int shortk_tile_n(int M, int N, int K, int cus, int batch = 1, bool shared_a = false);
inline bool shortk_applies(int M, int N, int K, int cus, int batch = 1, bool shared_a = false)
{
    return shortk_tile_n(M, N, K, cus, batch, shared_a) != 0;
}
hipError_t launch_sgemm_shortk(const GemmArgs& args, int tile_n, int cus, hipStream_t stream);
// sgemm_resident.hip: 256 x 128 tiles of a plain product walked by one resident workgroup per CU
enum { RESIDENT_MAX_K = 1024 };   // from here on the macro-tile kernel
bool resident_applies(int M, int N, int K, int cus, bool plain, bool forced);
bool resident_beats_shortk(int M, int N, int K, int cus);   // where sgemm_shortk.hip applies as well
int resident_lds_bytes();
hipError_t launch_sgemm_resident(const GemmArgs& args, int cus, hipStream_t stream);
void shortk_launch_shape(long tiles, int tile_n, int K, int cus, int* grid, int* lds_bytes);
// conv != nullptr: the columns are those of a convolution's product and go where conv_out_map says
hipError_t launch_splitk_reduce(const float* partial, float* C, int M, int N, int ldc, int splits,
                                int accumulate, hipStream_t stream, const ConvGeom* conv = nullptr,
                                const float* col_bias = nullptr);

// scratch: at least sgemv_rowmajor_scratch_floats(M, K, cus) floats (0 for most shapes), or nullptr
size_t sgemv_rowmajor_scratch_floats(int M, int K, int cus);
// Products in which one operand has few rows or columns (up to 112 rows of A, up to 32 columns
// of B), which stream the other one once: see sgemm_fewrows.hip.
bool fewrows_applies(int M, int N, int K, int lda, int ldb);
int fewrows_slices(int M, int N, int K, int cus);
hipError_t launch_sgemm_fewrows(const float* A, const float* B, float* C, float* partial, int M, int N,
                                int K, int lda, int ldb, int ldc, int accumulate, const float* col_bias,
                                int cus, hipStream_t stream);
bool fewrows_nt_applies(int M, int N, int K, int ldx, int ldw, bool x_kmajor);
int fewrows_nt_slices(int M, int N, int K, int ldw, bool x_kmajor, int cus);
bool fewrows_nt_turn_pays(int cols, int rows, int K, int lda, int cus);
hipError_t launch_sgemm_fewrows_nt(const float* X, const float* W, float* C, float* partial, int M, int N,
                                   int K, int ldx, int ldw, int ldc, bool x_kmajor, bool c_is_n_by_m,
                                   int accumulate, const float* bias, int cus, hipStream_t stream);

hipError_t launch_sgemv_rowmajor(const float* A, const float* x, float* y, int M, int K,
                                 int accumulate, float* scratch, int cus, hipStream_t stream);
// Y[v][m] = bias[m] + sum_k A[m][k] * X[v][k] for 2 vectors (rows of X, ldx apart; rows of Y,
// ldy apart) in one pass over the row-major A; bias may be nullptr
bool sgemv_rowmajor_multi_applies(int M, int K, int vectors, int ldx, const float* A, const float* X, int cus);
hipError_t launch_sgemv_rowmajor_multi(const float* A, const float* X, float* Y, const float* bias, int M,
                                       int K, int vectors, int ldx, int ldy, hipStream_t stream);
// scratch: at least sgemv_colmajor_scratch_floats(M, K) floats
size_t sgemv_colmajor_scratch_floats(int M, int K, int cus);
hipError_t launch_sgemv_colmajor(const float* A, const float* x, float* y, int M, int K,
                                 int accumulate, float* scratch, int cus, hipStream_t stream);

hipError_t launch_im2col(const float* in, float* cols, int batch, int Cin, int Hin, int Win,
                         int Hf, int Wf, int Hout, int Wout, int stride, int pad,
                         hipStream_t stream);
// The input of a convolution staged for the gather: see conv_stage_input_kernel.  `out` holds
// planes * Hs * PW * Wq floats (Wq % 4 == 0, 16-byte aligned).
// `table` (may be nullptr) is filled in the same launch: launch_conv_tap_table's K + extra entries.
hipError_t launch_conv_stage_input(const float* in, float* out, size_t planes, int Hin, int Win, int pad,
                                   int stride, int RH, int PW, int Hs, int Wq, int* table, int K, int extra,
                                   int Hf, int Wf, hipStream_t stream);
// out[plane][ho][wo] = in[plane][ho * stride][wo * stride], out dense and 16-byte aligned,
// planes * Hout * Wout < 2^31
hipError_t launch_subsample_planes(const float* in, float* out, size_t planes, int Hin, int Win, int Hout, int Wout,
                                   int stride, hipStream_t stream);
// table[k] = byte offset of filter tap k inside one staged image; `extra` zero entries follow
enum { CONV_TAP_TABLE_EXTRA = 256 };
hipError_t launch_conv_tap_table(int* table, int K, int extra, int Hs, int pitch, int Wq, int Hf, int Wf,
                                 int stride, int RH, hipStream_t stream);
// [Cout][batch*HW] -> [batch][Cout][HW]
hipError_t launch_cn_to_nchw(const float* src, float* dst, int batch, int Cout, int HW,
                             hipStream_t stream);

// Stride-1 convolutions that read the input where it lies (sgemm_conv_patch.hip).  The product is
// out[Cout][n] = Wt[Cout][K'] . B with K' = conv_patch_k(...) walked as (half block of 16
// channels, tap, channel); Wt is the filters re-laid to that order by launch_conv_filter_relayout.
// conv_patch_geometry: false when the kernel does not take the geometry, else the patch's shape.
enum { CONV_PATCH_PLANE = 512 };   // floats per channel of the LDS patch: rows x pitch must fit
bool conv_patch_geometry(int batch, int Cin, int Hin, int Win, int Hf, int Wf, int stride, int pad, int Hout,
                         int Wout, int* rows, int* pitch);
int conv_patch_k(int Cin, int Hf, int Wf);
int conv_patch_lda(int Cin, int Hf, int Wf);   // floats between rows of Wt (>= K')
bool conv_patch_reads_filters_in_place(int Hf, int Wf);   // no re-laying: A is the filters themselves, lda = K'
hipError_t launch_conv_filter_relayout(const float* W, float* Wt, int Cout, int Cin, int Hf, int Wf, hipStream_t stream);
// args as for launch_sgemm with the 256 x 128 x 32 tile; K slices (tail tiles) must be whole channel
// blocks of 32 * Hf * Wf
hipError_t launch_sgemm_conv_patch(const GemmArgs& args, int grid, hipStream_t stream);

hipError_t launch_fill_uniform(float* dst, size_t n, uint64_t seed, hipStream_t stream);
hipError_t launch_fill_value(float* dst, size_t n, float value, hipStream_t stream);
// dst[c][r] = src[r][c], src rows x cols row-major; rows <= 64 * 65535
hipError_t launch_transpose(const float* src, float* dst, int rows, int cols, hipStream_t stream);

// Packed layouts.  which: 0 = A, 1 = B, 2 = C.
hipError_t launch_build_index_tables(int which, const PackGeom& g, int4* row_tab, int4* col_tab,
                                     hipStream_t stream);
// dst_packed[offset(r,c)] = (r,c) inside the matrix ? src[r*ld + c] : 0   over the padded extent.
// fast / rows_fast: the short axis of a micro-panel (A: mr rows, rows_fast; B and C: nr columns),
// which the packed layout stores fastest; 0 selects the element-wise kernel.
// filters between [Cout][Cin][taps] and the reference's pack_filters layout (g.d from init_block_dims_conv, g.K = Cin)
hipError_t launch_filter_layout(const float* src, float* dst, const PackGeom& g, int Cout, int Cin, int taps,
                                int to_packed, hipStream_t stream);
hipError_t launch_pack(const float* src, float* dst_packed, int rows, int cols, int ld,
                       int rows_padded, int cols_padded, IndexTables tab, int fast, bool rows_fast,
                       hipStream_t stream);
// dst[r*ld + c] = src_packed[offset(r,c)] over the real extent
hipError_t launch_unpack(const float* src_packed, float* dst, int rows, int cols, int ld,
                         IndexTables tab, int fast, bool rows_fast, hipStream_t stream);

}  // namespace cake
