// misc_kernels.hip -- transpose, im2col, layout change, fills, and the reference's
// packed layouts (index tables, pack, unpack).  All HBM-bound copies: one
// thread per output element (or per 4), coalesced along the fastest dimension
// of whichever side is written.
#include <hip/hip_runtime.h>

#include "kernels.hpp"

namespace cake {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4_u __attribute__((ext_vector_type(4), aligned(4)));  // 16 bytes at any 4-byte address



// ---------------------------------------------------------------------------
// transpose: dst[c][r] = src[r][c] for a rows x cols row-major matrix
// (transpose_mat of src/transpose.cpp:5-29).  64x64 tiles through LDS so both
// the read and the write run along the contiguous dimension; the +1 padding
// keeps the transposed LDS reads conflict-free.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256) transpose_kernel(const float* __restrict__ src,
                                                        float* __restrict__ dst, int rows, int cols)
{
    __shared__ float tile[64][65];
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int r = r0 + ty + 4 * i, c = c0 + tx;
        if (r < rows && c < cols) tile[ty + 4 * i][tx] = src[(size_t)r * cols + c];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int c = c0 + ty + 4 * i, r = r0 + tx;
        if (r < rows && c < cols) dst[(size_t)c * rows + r] = tile[tx][ty + 4 * i];
    }
}

// The same with 16-byte global loads and stores (rows and cols multiples of 4, both pointers
// 16-byte aligned): a thread reads 4 pieces of 4 consecutive c, scatters them into the transposed
// tile (pitch 65: the 64 lanes of a store hit 64 banks) and gathers 4 consecutive r per piece on
// the way out (again 64 banks).  A quarter of the global memory instructions of the kernel above.
__global__ void __launch_bounds__(256) transpose_vec_kernel(const float* __restrict__ src,
                                                            float* __restrict__ dst, int rows, int cols)
{
    __shared__ float tile[64 * 65];   // tile[c][r]
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const int q = threadIdx.x & 15, p = threadIdx.x >> 4;   // piece of 4 along the fast axis, line
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = p + 16 * i, c = 4 * q;
        if (r0 + r < rows && c0 + c < cols) {
            const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(src + (size_t)(r0 + r) * cols + c0 + c));
#pragma unroll
            for (int j = 0; j < 4; ++j) tile[(c + j) * 65 + r] = v[j];
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = p + 16 * i, r = 4 * q;
        if (c0 + c < cols && r0 + r < rows) {
            f32x4 v;
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = tile[c * 65 + r + j];
            __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(dst + (size_t)(c0 + c) * rows + r0 + r));
        }
    }
}

hipError_t launch_transpose(const float* src, float* dst, int rows, int cols, hipStream_t stream)
{
    if (rows <= 0 || cols <= 0) return hipSuccess;
    const unsigned gx = (cols + 63) / 64, gy = (rows + 63) / 64;
    if (gy > 65535) return hipErrorInvalidValue;
    if (rows % 4 == 0 && cols % 4 == 0 &&
        (reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) % 16 == 0) {
        hipLaunchKernelGGL(transpose_vec_kernel, dim3(gx, gy), dim3(256), 0, stream, src, dst, rows, cols);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(transpose_kernel, dim3(gx, gy), dim3(256), 0, stream, src, dst, rows, cols);
    return hipGetLastError();
}

__global__ void __launch_bounds__(256) fill_value_kernel(float* __restrict__ dst, size_t n, float v)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
        dst[i] = v;
}

hipError_t launch_fill_value(float* dst, size_t n, float value, hipStream_t stream)
{
    if (n == 0) return hipSuccess;
    size_t blocks = (n + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(fill_value_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, dst, n, value);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Filters in the layout of the reference's pack_filters (examples/cake_conv.cpp:536-610) and
// back.  A thread owns one (padded row, channel) pair and walks its taps: on the plain side those
// are `taps` consecutive floats, on the packed side they lie m_r * k_c floats apart.  Filters are a
// few megabytes at most, so this is a plain index-map kernel.
//   to_packed != 0: packed[off(r, c, t)] = r < Cout ? plain[r][c][t] : 0   for r < padded rows
//   to_packed == 0: plain[r][c][t] = packed[off(r, c, t)]                  for r < Cout
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256) filter_layout_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                            PackGeom g, int Cout, int Cin, int taps, int rows,
                                                            int to_packed)
{
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)rows * Cin) return;
    const int r = (int)(idx / Cin), c = (int)(idx - (size_t)r * Cin);
    const size_t plain = ((size_t)r * Cin + c) * taps;
    for (int t = 0; t < taps; ++t) {
        const int64_t off = packed_filter_offset(g, r, c, t, taps);
        if (to_packed) dst[off] = r < Cout ? src[plain + t] : 0.f;
        else dst[plain + t] = src[off];
    }
}

hipError_t launch_filter_layout(const float* src, float* dst, const PackGeom& g, int Cout, int Cin, int taps,
                                int to_packed, hipStream_t stream)
{
    const int rows = to_packed ? g.d.M_padded : Cout;
    const size_t threads = (size_t)rows * Cin;
    if (threads == 0) return hipSuccess;
    hipLaunchKernelGGL(filter_layout_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream, src, dst, g,
                       Cout, Cin, taps, rows, to_packed);
    return hipGetLastError();
}

// Every stride-th pixel of every stride-th row of each plane, densely: the input of a 1 x 1
// convolution at that stride.  A thread per 4 consecutive outputs (one 16-byte store), their
// (plane, row, column) carried from one to the next.
__global__ void __launch_bounds__(256) subsample_planes_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                               unsigned total, int Hin, int Win, int Hout, int Wout,
                                                               int stride, FastDiv by_hw, FastDiv by_wout)
{
    for (unsigned j = (blockIdx.x * 256 + threadIdx.x) * 4; j < total; j += gridDim.x * 1024) {
        unsigned plane = by_hw.div(j);
        const unsigned r = j - plane * by_hw.d;
        int ho = (int)by_wout.div(r);
        int wo = (int)(r - ho * Wout);
        const int valid = (int)min(4u, total - j);
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        if (stride == 2 && valid == 4 && wo + 3 < Wout && 2 * wo + 7 < Win) {
            // four outputs of one row under stride 2: eight consecutive input values, two 16-byte loads
            const float* src = in + ((size_t)plane * Hin + (size_t)ho * 2) * Win + 2 * wo;
            const f32x4_u a = *reinterpret_cast<const f32x4_u*>(src), b = *reinterpret_cast<const f32x4_u*>(src + 4);
            v = f32x4{a[0], a[2], b[0], b[2]};
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (e < valid) v[e] = in[((size_t)plane * Hin + (size_t)ho * stride) * Win + (size_t)wo * stride];
                if (++wo == Wout) {
                    wo = 0;
                    if (++ho == Hout) { ho = 0; ++plane; }
                }
            }
        }
        if (valid == 4) {
            *reinterpret_cast<f32x4*>(out + j) = v;
        } else {
            for (int e = 0; e < valid; ++e) out[j + e] = v[e];
        }
    }
}

hipError_t launch_subsample_planes(const float* in, float* out, size_t planes, int Hin, int Win, int Hout, int Wout,
                                   int stride, hipStream_t stream)
{
    const size_t total = planes * Hout * Wout;
    if (total == 0) return hipSuccess;
    if (total >= (1ull << 31) || (reinterpret_cast<uintptr_t>(out) & 15) || (Hout - 1) * (long)stride >= Hin ||
        (Wout - 1) * (long)stride >= Win)
        return hipErrorInvalidValue;
    size_t blocks = (total + 1023) / 1024;
    if (blocks > (1u << 20)) blocks = 1u << 20;
    hipLaunchKernelGGL(subsample_planes_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, in, out, (unsigned)total,
                       Hin, Win, Hout, Wout, stride, FastDiv::make((unsigned)(Hout * Wout)), FastDiv::make((unsigned)Wout));
    return hipGetLastError();
}

__device__ __forceinline__ int conv_tap_offset(int k, int Hs, int pitch, int Wq, int Hf, int Wf, int stride, int RH)
{
    const int c = k / (Hf * Wf), tap = k - c * (Hf * Wf);
    const int h = tap / Wf, w = tap - h * Wf;
    const int row = (h / stride) * RH + h % stride;
    return ((c * Hs + row) * pitch + (w % stride) * Wq + w / stride) * 4;
}

// The input of a strided convolution, staged so that the gather reads consecutive floats: a row
// of the zero-padded image is split into its `stride` column phases (wi = wq * stride + phase), of
// which only the PW = min(Wf, stride) phases that a filter tap can reach are kept, each Wq floats
// long (Wq a multiple of 4); of every `stride` rows only the RH = min(Hf, stride) reachable ones
// are kept.  Stored row of padded row hi: (hi / stride) * RH + hi % stride.  Output pixel (ho, wo)
// under tap (h, w) then reads
//     plane[(ho + h / s) * RH + h % s][w % s][wo + w / s]
// whose address splits into a pixel part (ho * RH * pitch + wo, pitch = PW * Wq) and a tap part,
// and 4 consecutive wo are 4 consecutive floats.  stride 1 is the plain zero-padded copy.
// One thread per float4 of the staged image; at stride 1 the four values are one 16-byte load
// wherever they lie inside a row of the image (any 4-byte alignment).  The workgroups past
// `stage_blocks` write the table of tap offsets (conv_tap_table_kernel below) in the same launch,
// so a convolution has one launch in front of its product, not two (table == nullptr: none).
__global__ void __launch_bounds__(256) conv_stage_input_kernel(const float* __restrict__ in,
                                                               float* __restrict__ out, unsigned total4,
                                                               int Hin, int Win, int pad, int stride, int RH,
                                                               int PW, int Hs, int Wq, FastDiv by_wq4,
                                                               FastDiv by_pw, FastDiv by_hs, FastDiv by_rh,
                                                               unsigned stage_blocks, int* __restrict__ table, int K,
                                                               int extra, int Hf, int Wf)
{
    if (blockIdx.x >= stage_blocks) {
        const int k = (blockIdx.x - stage_blocks) * 256 + threadIdx.x;
        if (k < K + extra) table[k] = k < K ? conv_tap_offset(k, Hs, PW * Wq, Wq, Hf, Wf, stride, RH) : 0;
        return;
    }
    for (unsigned i = blockIdx.x * 256 + threadIdx.x; i < total4; i += stage_blocks * 256) {
        unsigned t = by_wq4.div(i);
        const int wq = (int)(i - t * by_wq4.d) * 4;
        unsigned u = by_pw.div(t);
        const int ph = (int)(t - u * PW);
        const unsigned plane = by_hs.div(u);
        const int sr = (int)(u - plane * Hs);
        const int grp = (int)by_rh.div((unsigned)sr);
        const int yi = grp * stride + (sr - grp * RH) - pad;
        const float* src = in + ((size_t)plane * Hin + yi) * Win;
        const bool row_in = (unsigned)yi < (unsigned)Hin;
        f32x4 v;
        const int x0 = wq - pad;
        if (stride == 1 && row_in && x0 >= 0 && x0 + 3 < Win) {
            v = *reinterpret_cast<const f32x4_u*>(src + x0);
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int xi = (wq + e) * stride + ph - pad;
                v[e] = (row_in && (unsigned)xi < (unsigned)Win) ? src[xi] : 0.f;
            }
        }
        *reinterpret_cast<f32x4*>(out + (size_t)i * 4) = v;
    }
}

hipError_t launch_conv_stage_input(const float* in, float* out, size_t planes, int Hin, int Win, int pad,
                                   int stride, int RH, int PW, int Hs, int Wq, int* table, int K, int extra,
                                   int Hf, int Wf, hipStream_t stream)
{
    const size_t total4 = planes * Hs * PW * (Wq / 4);
    if (total4 == 0) return hipSuccess;
    if (Wq % 4 != 0 || total4 >= (1ull << 31)) return hipErrorInvalidValue;
    size_t blocks = (total4 + 255) / 256;
    if (blocks > (1u << 20)) blocks = 1u << 20;
    const unsigned table_blocks = table ? (unsigned)((K + extra + 255) / 256) : 0u;
    hipLaunchKernelGGL(conv_stage_input_kernel, dim3((unsigned)blocks + table_blocks), dim3(256), 0, stream, in, out,
                       (unsigned)total4, Hin, Win, pad, stride, RH, PW, Hs, Wq, FastDiv::make((unsigned)(Wq / 4)),
                       FastDiv::make((unsigned)PW), FastDiv::make((unsigned)Hs), FastDiv::make((unsigned)RH),
                       (unsigned)blocks, table, K, extra, Hf, Wf);
    return hipGetLastError();
}

// Byte offset of filter tap k = (c, h, w) inside one staged image (see above):
// table[k] = (c * Hs * pitch + ((h / s) * RH + h % s) * pitch + (w % s) * Wq + w / s) * 4 for
// k < K, 0 for the `extra` entries after it (the gather prefetches a few stages past the end).
__global__ void __launch_bounds__(256) conv_tap_table_kernel(int* __restrict__ table, int K, int extra,
                                                             int Hs, int pitch, int Wq, int Hf, int Wf,
                                                             int stride, int RH)
{
    const int k = blockIdx.x * 256 + threadIdx.x;
    if (k >= K + extra) return;
    table[k] = k < K ? conv_tap_offset(k, Hs, pitch, Wq, Hf, Wf, stride, RH) : 0;
}

hipError_t launch_conv_tap_table(int* table, int K, int extra, int Hs, int pitch, int Wq, int Hf, int Wf,
                                 int stride, int RH, hipStream_t stream)
{
    hipLaunchKernelGGL(conv_tap_table_kernel, dim3((K + extra + 255) / 256), dim3(256), 0, stream, table, K,
                       extra, Hs, pitch, Wq, Hf, Wf, stride, RH);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// im2col: im_2_col of examples/cake_conv.cpp:1178-1213 with batch, padding and
// stride.  grid.y = input channel c; threads run along n = (b, ho, wo), and every
// thread writes its 4 consecutive n (16 bytes at any 4-byte alignment) into all
// Hf * Wf rows k = (c, h, w) of that channel: the position arithmetic is done once
// for them, and a thread has a filter row's worth of loads and stores in flight.
// (With a thread per 16 bytes of output, one store each, the kernel wrote 2.9 TB/s
// where this memory takes 5.5 to 6.5 TB/s from threads that write several pieces.)
// The 4 elements may run over the end of an output row or image, so their positions
// are carried from element to element.  ncols < 2^31.
// WF: the filter width when it is one of the instantiated ones (the loop over a
// filter row is then unrolled), 0 = any.
// ---------------------------------------------------------------------------
static constexpr int IM2COL_BLOCK = 1024;            // n per workgroup of the kernel that stages input rows in LDS
static constexpr int IM2COL_LDS_BYTES = 48 << 10;    // up to this much of them

template <int WF>
__global__ void __launch_bounds__(256) im2col_kernel(const float* __restrict__ in,
                                                     float* __restrict__ cols, unsigned ncols, int Cin,
                                                     int Hin, int Win, int Hf, int Wf_, int Hout,
                                                     int Wout, int stride, int pad, FastDiv by_hw,
                                                     FastDiv by_wout)
{
    const int Wf = WF ? WF : Wf_;
    const unsigned c = blockIdx.y;
    float* rows = cols + (size_t)c * (Hf * Wf) * ncols;   // row (c, 0, 0)

    for (unsigned n = (blockIdx.x * 256 + threadIdx.x) * 4; n < ncols; n += gridDim.x * 1024) {
        unsigned b = by_hw.div(n);
        const unsigned r = n - b * by_hw.d;
        int ho = (int)by_wout.div(r);
        int wo = (int)(r - ho * Wout);
        // top-left input position of each element's window, and its (image, channel) plane
        int hi0[4], wi0[4];
        const float* plane[4];
        // at stride 1 the 4 elements of a thread that lie in one output row read 4 neighbouring
        // input values: one 16-byte load where the window is inside the image
        const bool one_row = stride == 1 && wo + 3 < Wout && n + 4 <= ncols;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            hi0[e] = ho * stride - pad;
            wi0[e] = wo * stride - pad;
            plane[e] = in + ((size_t)b * Cin + c) * Hin * Win;
            if (++wo == Wout) {
                wo = 0;
                if (++ho == Hout) { ho = 0; ++b; }
            }
        }
        const int valid = (int)min(4u, ncols - n);   // elements that exist
        float* dst = rows + n;
        for (int h = 0; h < Hf; ++h) {
#pragma unroll
            for (int w = 0; w < (WF ? WF : 1); ++w) {
                // WF == 0: this loop runs once per pass of the `wr` loop below
                for (int wr = WF ? w : 0; wr < Wf; wr += WF ? Wf : 1) {
                    float v[4];
                    const int hi_a = hi0[0] + h, wi_a = wi0[0] + wr;
                    if (one_row && hi_a >= 0 && hi_a < Hin && wi_a >= 0 && wi_a + 3 < Win) {
                        const f32x4_u q = *reinterpret_cast<const f32x4_u*>(plane[0] + hi_a * Win + wi_a);
                        v[0] = q[0]; v[1] = q[1]; v[2] = q[2]; v[3] = q[3];
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int hi = hi0[e] + h, wi = wi0[e] + wr;
                            const bool ok = e < valid && hi >= 0 && hi < Hin && wi >= 0 && wi < Win;
                            v[e] = ok ? plane[e][hi * Win + wi] : 0.f;
                        }
                    }
                    float* out = dst + (size_t)(h * Wf + wr) * ncols;
                    if (valid == 4) {
                        const f32x4_u o = {v[0], v[1], v[2], v[3]};
                        __builtin_nontemporal_store(o, reinterpret_cast<f32x4_u*>(out));
                    } else {
                        for (int e = 0; e < valid; ++e) out[e] = v[e];
                    }
                }
            }
        }
    }
}

// The same through LDS.  A workgroup owns 1024 consecutive n of one channel; the input rows under
// their windows -- consecutive rows of the images' planes with the zero padding written out,
// "virtual" row v = b * (Hin + 2 pad) + pad + hi -- are brought into LDS once, each input value by
// one coalesced load, and every thread then builds its 4 consecutive n of all Hf * Wf rows from
// there.  (With the window values loaded from memory per tap, the kernel above, a thread has Hf * Wf
// 16-byte loads at odd addresses in front of as many stores: 925 MB of columns took 207 us between
// other kernels, 155 us with the loads taken out and 127 us as a plain fill.)
// (Stores with and without the non-temporal hint measured the same here, alone and with the product
// behind them, at 29 to 925 MB of columns.)
template <int WF>
__global__ void __launch_bounds__(256) im2col_rows_kernel(const float* __restrict__ in, float* __restrict__ cols,
                                                          unsigned ncols, int Cin, int Hin, int Win, int Hf, int Wf_,
                                                          int Hout, int Wout, int stride, int pad, FastDiv by_hw,
                                                          FastDiv by_wout, FastDiv by_hv, FastDiv by_pitch, int lds_rows)
{
    extern __shared__ float staged[];
    const int Wf = WF ? WF : Wf_;
    const unsigned c = blockIdx.y;
    const int tid = threadIdx.x;
    const int Hv = Hin + 2 * pad, P = (int)by_pitch.d;
    const unsigned first = blockIdx.x * IM2COL_BLOCK;
    const unsigned last = min(first + IM2COL_BLOCK, ncols) - 1;
    auto window_row = [&](unsigned n, int& wo) {   // virtual row of the top of n's window
        const unsigned b = by_hw.div(n), r = n - b * by_hw.d;
        const int ho = (int)by_wout.div(r);
        wo = (int)r - ho * Wout;
        return (int)b * Hv + ho * stride;
    };
    int unused;
    const int v0 = window_row(first, unused);
    const int nv = min(window_row(last, unused) + Hf - v0, lds_rows);   // (the host sized LDS for the longest run)

    // stage: nv rows of P = Win + 2 pad floats, four values per thread in flight
    const int total = nv * P;
    for (int i0 = tid; i0 < total; i0 += 4 * 256) {
        float val[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = i0 + u * 256;
            const int lr = (int)by_pitch.div((unsigned)i), wi = i - lr * P - pad;
            const int v = v0 + lr;
            const int b = (int)by_hv.div((unsigned)v), hi = v - b * Hv - pad;
            val[u] = (i < total && hi >= 0 && hi < Hin && wi >= 0 && wi < Win)
                         ? in[(((size_t)b * Cin + c) * Hin + hi) * Win + wi] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (i0 + u * 256 < total) staged[i0 + u * 256] = val[u];
    }
    __syncthreads();

    const unsigned n = first + tid * 4;
    if (n >= ncols) return;
    int at[4];   // the window's top-left corner of each of the thread's 4 elements, in LDS
    {
        unsigned b = by_hw.div(n);
        const unsigned r = n - b * by_hw.d;
        int ho = (int)by_wout.div(r);
        int wo = (int)(r - ho * Wout);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            at[e] = ((int)b * Hv + ho * stride - v0) * P + wo * stride;
            if (++wo == Wout) {
                wo = 0;
                if (++ho == Hout) { ho = 0; ++b; }
            }
        }
    }
    const int valid = (int)min(4u, ncols - n);
#pragma unroll
    for (int e = 1; e < 4; ++e)
        if (e >= valid) at[e] = at[0];   // elements past the end are never stored; keep their reads inside LDS
    float* dst = cols + (size_t)c * (Hf * Wf) * ncols + n;
    for (int h = 0; h < Hf; ++h) {
#pragma unroll
        for (int w = 0; w < (WF ? WF : 1); ++w) {
            for (int wr = WF ? w : 0; wr < Wf; wr += WF ? Wf : 1) {
                const int tap = h * P + wr;
                const f32x4_u o = {staged[at[0] + tap], staged[at[1] + tap], staged[at[2] + tap], staged[at[3] + tap]};
                float* out = dst + (size_t)(h * Wf + wr) * ncols;
                if (valid == 4) {
                    __builtin_nontemporal_store(o, reinterpret_cast<f32x4_u*>(out));
                } else {
                    for (int e = 0; e < valid; ++e) out[e] = o[e];
                }
            }
        }
    }
}

// Rows of LDS the longest run of IM2COL_BLOCK consecutive n can need: its output rows, at
// `stride` virtual rows each, the rows an image border adds, the window's height.
static int im2col_rows_bound(int Hin, int Hf, int Hout, int Wout, int stride, int pad)
{
    const int Hv = Hin + 2 * pad;
    const int out_rows = (IM2COL_BLOCK - 1) / Wout + 2;
    const int borders = (out_rows - 2) / Hout + 1;
    const int per_border = Hv - Hout * stride > 0 ? Hv - Hout * stride : 0;
    return (out_rows - 1) * stride + borders * per_border + Hf;
}

hipError_t launch_im2col(const float* in, float* cols, int batch, int Cin, int Hin, int Win, int Hf,
                         int Wf, int Hout, int Wout, int stride, int pad, hipStream_t stream)
{
    const int krows = Cin * Hf * Wf;
    const size_t ncols = (size_t)batch * Hout * Wout;
    if (krows <= 0 || ncols == 0) return hipSuccess;
    if (Cin > 65535 || ncols >= (1ull << 31)) return hipErrorInvalidValue;
    const FastDiv by_hw = FastDiv::make((unsigned)(Hout * Wout)), by_wout = FastDiv::make((unsigned)Wout);
    // input rows through LDS where the rows under 1024 consecutive windows fit
    const int pitch = Win + 2 * pad, lds_rows = im2col_rows_bound(Hin, Hf, Hout, Wout, stride, pad);
    const size_t lds_bytes = (size_t)lds_rows * pitch * sizeof(float);
    if (lds_bytes <= (size_t)IM2COL_LDS_BYTES && (double)batch * (Hin + 2 * pad) < 2147483647.0) {
        const dim3 grid((unsigned)((ncols + IM2COL_BLOCK - 1) / IM2COL_BLOCK), Cin);
        const FastDiv by_hv = FastDiv::make((unsigned)(Hin + 2 * pad)), by_pitch = FastDiv::make((unsigned)pitch);
#define CAKE_IM2COL_ROWS(W)                                                                                          \
    hipLaunchKernelGGL(im2col_rows_kernel<W>, grid, dim3(256), lds_bytes, stream, in, cols, (unsigned)ncols, Cin, Hin, \
                       Win, Hf, Wf, Hout, Wout, stride, pad, by_hw, by_wout, by_hv, by_pitch, lds_rows)
        switch (Wf) {
            case 1: CAKE_IM2COL_ROWS(1); break;
            case 3: CAKE_IM2COL_ROWS(3); break;
            case 5: CAKE_IM2COL_ROWS(5); break;
            case 7: CAKE_IM2COL_ROWS(7); break;
            default: CAKE_IM2COL_ROWS(0); break;
        }
#undef CAKE_IM2COL_ROWS
        return hipGetLastError();
    }
    size_t bx = (ncols + 1023) / 1024;
    if (bx > 4096) bx = 4096;
    const dim3 grid((unsigned)bx, Cin);
#define CAKE_IM2COL(W)                                                                                             \
    hipLaunchKernelGGL(im2col_kernel<W>, grid, dim3(256), 0, stream, in, cols, (unsigned)ncols, Cin, Hin, Win, Hf, \
                       Wf, Hout, Wout, stride, pad, by_hw, by_wout)
    switch (Wf) {
        case 1: CAKE_IM2COL(1); break;
        case 3: CAKE_IM2COL(3); break;
        case 5: CAKE_IM2COL(5); break;
        case 7: CAKE_IM2COL(7); break;
        default: CAKE_IM2COL(0); break;
    }
#undef CAKE_IM2COL
    return hipGetLastError();
}

// [Cout][batch][HW] -> [batch][Cout][HW]
__global__ void __launch_bounds__(256) cn_to_nchw_kernel(const float* __restrict__ src,
                                                         float* __restrict__ dst, int batch,
                                                         int Cout, int HW)
{
    const size_t total = (size_t)batch * Cout * HW;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const int hw = (int)(i % HW);
        const size_t t = i / HW;
        const int co = (int)(t % Cout);
        const int b = (int)(t / Cout);
        dst[i] = src[((size_t)co * batch + b) * HW + hw];
    }
}

// the same in 16-byte pieces (HW a multiple of 4, both pointers 16-byte aligned); hw4 = HW / 4
__global__ void __launch_bounds__(256) cn_to_nchw_vec_kernel(const f32x4* __restrict__ src,
                                                             f32x4* __restrict__ dst, int batch,
                                                             int Cout, FastDiv by_hw4, FastDiv by_cout)
{
    const unsigned hw4 = by_hw4.d;
    const size_t total = (size_t)batch * Cout * hw4;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        // total < 2^31 elements / 4
        const unsigned t = by_hw4.div((unsigned)i), q = (unsigned)i - t * hw4;
        const unsigned b = by_cout.div(t), co = t - b * (unsigned)Cout;
        dst[i] = __builtin_nontemporal_load(src + ((size_t)co * batch + b) * hw4 + q);
    }
}

hipError_t launch_cn_to_nchw(const float* src, float* dst, int batch, int Cout, int HW,
                             hipStream_t stream)
{
    const size_t total = (size_t)batch * Cout * HW;
    if (total == 0) return hipSuccess;
    if (HW % 4 == 0 && total < (1ull << 31) &&
        (reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) % 16 == 0) {
        size_t blocks = (total / 4 + 255) / 256;
        if (blocks > 16384) blocks = 16384;
        hipLaunchKernelGGL(cn_to_nchw_vec_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                           reinterpret_cast<const f32x4*>(src), reinterpret_cast<f32x4*>(dst), batch, Cout,
                           FastDiv::make((unsigned)(HW / 4)), FastDiv::make((unsigned)Cout));
        return hipGetLastError();
    }
    size_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(cn_to_nchw_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, src, dst, batch, Cout, HW);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Seeded uniform[-1,1): element i = 24 top bits of splitmix64(seed + (i+1)*G).
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256) fill_uniform_kernel(float* __restrict__ dst, size_t n,
                                                           uint64_t seed)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        uint64_t z = seed + (i + 1) * 0x9E3779B97F4A7C15ull;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        z ^= z >> 31;
        dst[i] = (float)(uint32_t)(z >> 40) * 0x1p-23f - 1.0f;
    }
}

hipError_t launch_fill_uniform(float* dst, size_t n, uint64_t seed, hipStream_t stream)
{
    if (n == 0) return hipSuccess;
    size_t blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(fill_uniform_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, dst, n, seed);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Packed layouts as bilinear index tables.
//
// Every packed layout of the reference places element (r, c) at
//     R[r].x + C[c].x + R[r].y*C[c].y + R[r].z*C[c].z + R[r].w*C[c].w
// where R depends only on the row and C only on the column: the CB-block walk
// contributes (block start) x (block extent of the other dimension) products
// and the m_r / n_r panels contribute (panel start) x (panel depth) products.
// Building the two tables costs a handful of integer divisions per row and
// per column; packing, unpacking and the GEMM loaders then address packed
// data with two table reads and three multiply-adds per element.
// ---------------------------------------------------------------------------
__device__ __forceinline__ SplitPos split_m(const PackGeom& g, int row)
{
    return split_pos(row, g.p, g.d.m_c, g.d.Mb, g.d.m_pad, g.mr * g.d.mr_rem, g.d.m_c1, g.d.p_l,
                     g.d.m_c1_last_core);
}

__device__ __forceinline__ SplitPos split_k(const PackGeom& g, int k)
{
    return split_pos(k, g.p, g.d.k_c, g.d.Kb, g.d.k_pad, g.d.k_rem, g.d.k_c1, g.d.p_l,
                     g.d.k_c1_last_core);
}

// Row of C or A inside an M block of the K-split schedules.
struct MPos { int mb, rows, panel, j; };

__device__ __forceinline__ MPos m_block_pos(const PackGeom& g, int row)
{
    const int mspan = (g.sch == CAKE_HIP_MKN) ? g.d.m_c : g.p * g.d.m_c;
    MPos r;
    r.mb = row / mspan;
    const int in = row - r.mb * mspan;
    r.rows = (g.d.m_pad && r.mb == g.d.Mb - 1) ? g.d.m_c1 : mspan;
    r.panel = in / g.mr;
    r.j = in - r.panel * g.mr;
    return r;
}

struct NPos { int nb, cols, panel, j; };

__device__ __forceinline__ NPos n_block_pos(const PackGeom& g, int col)
{
    NPos r;
    r.nb = col / g.d.n_c;
    const int in = col - r.nb * g.d.n_c;
    r.cols = (g.d.n_pad && r.nb == g.d.Nb - 1) ? g.d.n_c1 : g.d.n_c;
    r.panel = in / g.nr;
    r.j = in - r.panel * g.nr;
    return r;
}

// K position of the K-first schedule (K not split over cores).
struct KPos { int kb, kk, kc; };

__device__ __forceinline__ KPos k_block_pos(const PackGeom& g, int k)
{
    KPos r;
    r.kb = k / g.d.k_c;
    r.kk = k - r.kb * g.d.k_c;
    r.kc = (g.d.k_pad && r.kb == g.d.Kb - 1) ? g.d.k_c1 : g.d.k_c;
    return r;
}

__global__ void __launch_bounds__(256) build_tables_kernel(int which, PackGeom g, int4* row_tab,
                                                           int nrows, int4* col_tab, int ncols)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    const int mr = g.mr, nr = g.nr;
    const int Mp = padded_rows(g), Np = padded_cols(g);
    const int mspan = g.p * g.d.m_c, kspan = g.p * g.d.k_c;

    if (i < nrows) {
        int4 R = make_int4(0, 0, 0, 0);
        if (which == 0) {  // A: rows are m
            if (g.sch == CAKE_HIP_KMN) {
                const SplitPos m = split_m(g, i);
                const int panel = m.inner / mr, j = m.inner - panel * mr;
                R = make_int4(m.block * mspan * g.K + j, m.span, m.core * m.slice + panel * mr, 0);
            } else {
                const MPos m = m_block_pos(g, i);
                if (g.sch == CAKE_HIP_MKN) R = make_int4(m.j, m.mb * g.d.m_c, m.rows, m.panel * mr);
                else R = make_int4(m.mb * mspan * g.K + m.j, m.rows, m.panel * mr, 0);
            }
        } else if (which == 1) {  // B: rows are k
            if (g.sch == CAKE_HIP_KMN) {
                const KPos k = k_block_pos(g, i);
                R = make_int4(k.kk * nr, k.kb * g.d.k_c, k.kc, 0);
            } else {
                const SplitPos k = split_k(g, i);
                if (g.sch == CAKE_HIP_MKN)
                    R = make_int4(k.inner * nr, k.block * kspan + k.core * k.slice, k.length, 0);
                else
                    R = make_int4(k.block * kspan * Np + k.inner * nr, k.span, k.core * k.slice, k.length);
            }
        } else {  // C: rows are m
            if (g.sch == CAKE_HIP_KMN) {
                const SplitPos m = split_m(g, i);
                const int pm = m.inner / mr, ii = m.inner - pm * mr;
                R = make_int4(pm * mr * nr + ii * nr, m.block * mspan + m.core * m.slice, m.length, 0);
            } else {
                const MPos m = m_block_pos(g, i);
                const int in = m.panel * mr * nr + m.j * nr;
                if (g.sch == CAKE_HIP_MKN) R = make_int4(in, m.mb * g.d.m_c, m.rows, 0);
                else R = make_int4(Np * m.mb * mspan + in, m.rows, 0, 0);
            }
        }
        row_tab[i] = R;
    }

    if (i < ncols) {
        int4 Cc = make_int4(0, 0, 0, 0);
        if (which == 0) {  // A: columns are k
            if (g.sch == CAKE_HIP_KMN) {
                const KPos k = k_block_pos(g, i);
                Cc = make_int4(k.kk * mr, k.kb * g.d.k_c, k.kc, 0);
            } else {
                const SplitPos k = split_k(g, i);
                if (g.sch == CAKE_HIP_MKN)
                    Cc = make_int4(k.block * Mp * kspan + k.inner * mr, k.span, k.core * k.slice, k.length);
                else
                    Cc = make_int4(k.inner * mr, k.block * kspan + k.core * k.slice, k.length, 0);
            }
        } else {  // B and C: columns are n
            const NPos n = n_block_pos(g, i);
            if (which == 1) {
                if (g.sch == CAKE_HIP_NKM) Cc = make_int4(n.j, n.nb * g.d.n_c, n.cols, n.panel * nr);
                else Cc = make_int4(n.nb * g.K * g.d.n_c + n.j, n.cols, n.panel * nr, 0);
            } else {
                if (g.sch == CAKE_HIP_KMN) Cc = make_int4(n.nb * g.d.n_c * Mp + n.j, n.cols, n.panel * nr, 0);
                else if (g.sch == CAKE_HIP_MKN) Cc = make_int4(Mp * n.nb * g.d.n_c + n.j, n.cols, n.panel * nr, 0);
                else Cc = make_int4(n.j, n.nb * g.d.n_c + n.panel * nr, 0, 0);
            }
        }
        col_tab[i] = Cc;
    }
}

hipError_t launch_build_index_tables(int which, const PackGeom& g, int4* row_tab, int4* col_tab,
                                     hipStream_t stream)
{
    const int Mp = padded_rows(g), Np = padded_cols(g);
    const int nrows = (which == 1) ? g.K : Mp;
    const int ncols = (which == 0) ? g.K : Np;
    const int n = nrows > ncols ? nrows : ncols;
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(build_tables_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, which, g,
                       row_tab, nrows, col_tab, ncols);
    return hipGetLastError();
}

__device__ __forceinline__ size_t table_offset(const int4 R, const int4 Cc)
{
    return (size_t)(R.x + Cc.x + R.y * Cc.y + R.z * Cc.z + R.w * Cc.w);
}

// pack_A / pack_B / pack_C (src/pack_helper.cpp:92-160): row-major -> packed,
// zero in the padding (src/pack_ob.cpp:46-50).
__global__ void __launch_bounds__(256) pack_kernel(const float* __restrict__ src,
                                                   float* __restrict__ dst, int rows, int cols,
                                                   int ld, int rows_p, int cols_p, IndexTables tab)
{
    const int r = blockIdx.y;
    const int4 R = tab.row[r];
    for (int c = blockIdx.x * 256 + threadIdx.x; c < cols_p; c += gridDim.x * 256) {
        const float v = (r < rows && c < cols) ? src[(size_t)r * ld + c] : 0.f;
        dst[table_offset(R, tab.col[c])] = v;
    }
}

// unpack_C (src/pack_helper.cpp:163-184, src/pack_ob.cpp:393-411): packed ->
// row-major, real extent only, assignment.
__global__ void __launch_bounds__(256) unpack_kernel(const float* __restrict__ src,
                                                     float* __restrict__ dst, int rows, int cols,
                                                     int ld, IndexTables tab)
{
    const int r = blockIdx.y;
    const int4 R = tab.row[r];
    for (int c = blockIdx.x * 256 + threadIdx.x; c < cols; c += gridDim.x * 256)
        dst[(size_t)r * ld + c] = src[table_offset(R, tab.col[c])];
}

static dim3 rowwise_grid(int rows, int cols)
{
    int bx = (cols + 255) / 256;
    if (bx > 1024) bx = 1024;
    return dim3(bx, rows);
}

// The same two copies through an LDS tile, so that BOTH sides move in contiguous runs.  In the
// packed layouts a micro-panel is stored with its short axis fastest: A as [k][mr rows], B and C
// as [k or row][nr columns].  A thread per row-major element therefore scatters 4-byte stores
// `fast` floats apart (A) or writes 64-byte pieces (B, C).  Here a workgroup takes a tile of up
// to TR x TC elements whose short-axis extent is a whole number of panels, moves it between the
// row-major side and LDS in rows of TC floats, and walks the packed side in packed order
// (short axis fastest, then the long axis, then the next panel), which is ascending addresses
// wherever the tile lies inside one block of the schedule.  Offsets still come from the index
// tables, so a tile that straddles blocks or starts off a panel boundary is only slower.
// Tiles of 16 to 32 rows of 512 bytes: with 64 x 64 tiles (256-byte rows) 8192 x 8192 took 115-130 us,
// with these 96-110 us, where a plain copy of as many bytes takes 99 us; 32 x 256 and 64 x 128
// (twice the elements per thread) were 10 % slower than 64 x 64, 16-byte accesses on either
// side changed nothing.  STREAM: both sides bypass the caches' keep-for-later policy; it pays from
// about 100 MB per side on (8192 x 8192: 104 -> 96 us) and costs 10 % where both sides fit the
// memory-side cache (4096 x 4096: 28 -> 31 us).
template <bool STREAM>
__device__ __forceinline__ float pack_load(const float* p)
{
    return STREAM ? __builtin_nontemporal_load(p) : *p;
}

template <bool STREAM>
__device__ __forceinline__ void pack_store(float v, float* p)
{
    if (STREAM) __builtin_nontemporal_store(v, p);
    else *p = v;
}

// TC and the long axis of the packed walk (TC when rows are the fast axis, else TR) are powers of two.
template <bool UNPACK, int TR, int TC, bool STREAM>
__global__ void __launch_bounds__(256) pack_tile_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                        int rows, int cols, int ld, int rows_p, int cols_p,
                                                        IndexTables tab, int fast, int rows_fast, int tr, int tc,
                                                        int pitch, int lshift)
{
    constexpr int N = TR * TC / 256;      // elements per thread
    constexpr int RPP = 256 / TC;         // rows per pass of the row-major side
    static_assert(TR * TC % 256 == 0 && 256 % TC == 0, "a pass of the row-major side covers whole rows");
    __shared__ float tile[TR * (TC + 64)];
    __shared__ int4 Rt[TR], Ct[TC];
    const int tid = threadIdx.x;
    const int r0 = blockIdx.y * tr, c0 = blockIdx.x * tc;
    for (int i = tid; i < TR + TC; i += 256) {
        if (i < TR) {
            if (i < tr && r0 + i < rows_p) Rt[i] = tab.row[r0 + i];
        } else {
            const int c = i - TR;
            if (c < tc && c0 + c < cols_p) Ct[c] = tab.col[c0 + c];
        }
    }
    const int lim_r = UNPACK ? rows : rows_p, lim_c = UNPACK ? cols : cols_p;  // extent of the packed-side walk
    const int dc_rm = tid % TC, dr_rm = tid / TC;
    const float inv_fast = 1.0f / (float)fast;
    const int count = tr * tc;
    const int lmask = (1 << lshift) - 1;

    // Fixed trip counts and full unrolling: all N loads of a thread are in flight together
    // (with a run-time bound the compiler keeps one load per thread in flight, and the kernel
    // runs at the speed of N memory latencies per tile).
    if (!UNPACK) {
        float v[N];
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int dr = dr_rm + RPP * i;
            const int r = r0 + dr, c = c0 + dc_rm;
            v[i] = (dr < tr && dc_rm < tc && r < rows && c < cols) ? pack_load<STREAM>(src + (size_t)r * ld + c) : 0.f;
        }
#pragma unroll
        for (int i = 0; i < N; ++i) tile[(dr_rm + RPP * i) * pitch + dc_rm] = v[i];
    }
    __syncthreads();
    {
        float v[N];
        size_t off[N];
        int at[N];
        bool live[N];
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int e = tid + 256 * i;
            // e = (panel * long + l) * fast + j; exact for e < 2^22: (e + 0.5) / fast is at least
            // 0.5 / fast away from an integer
            const int q = (int)(((float)e + 0.5f) * inv_fast);
            const int j = e - q * fast;
            const int panel = q >> lshift, l = q & lmask;
            const int dr = rows_fast ? panel * fast + j : l;
            const int dc = rows_fast ? l : panel * fast + j;
            const int r = r0 + dr, c = c0 + dc;
            live[i] = e < count && dr < tr && dc < tc && r < lim_r && c < lim_c;
            off[i] = live[i] ? table_offset(Rt[dr], Ct[dc]) : 0;
            at[i] = dr * pitch + dc;
            if (UNPACK) v[i] = live[i] ? pack_load<STREAM>(src + off[i]) : 0.f;
            else v[i] = live[i] ? tile[at[i]] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < N; ++i) {
            if (!live[i]) continue;
            if (UNPACK) tile[at[i]] = v[i];
            else pack_store<STREAM>(v[i], dst + off[i]);
        }
    }
    if (UNPACK) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int dr = dr_rm + RPP * i;
            const int r = r0 + dr, c = c0 + dc_rm;
            if (dr < tr && dc_rm < tc && r < rows && c < cols)
                pack_store<STREAM>(tile[dr * pitch + dc_rm], dst + (size_t)r * ld + c);
        }
    }
}

static constexpr int PACK_TC = 128;        // floats per row of a tile
static constexpr int PACK_STREAM_BYTES = 100 << 20;

template <bool UNPACK, int TR, int TC, bool STREAM>
static hipError_t launch_pack_tiles_as(const float* src, float* dst, int rows, int cols, int ld, int rows_p,
                                       int cols_p, IndexTables tab, int fast, bool rows_fast, hipStream_t stream)
{
    const int tr = rows_fast ? fast * (TR / fast) : TR, tc = rows_fast ? TC : fast * (TC / fast);
    // LDS pitch: a wave walking the packed order touches `fast` short-axis positions times 64 / fast
    // long-axis positions; with rows fast, consecutive rows are ceil(64 / fast) banks apart, with
    // columns fast, consecutive rows are `fast` banks apart
    const int pitch = rows_fast ? TC + (64 + fast - 1) / fast : TC + (fast & 63);
    int lshift = 0;
    while ((1 << lshift) < (rows_fast ? TC : TR)) ++lshift;
    const int ext_r = UNPACK ? rows : rows_p, ext_c = UNPACK ? cols : cols_p;
    const int tiles_c = (ext_c + tc - 1) / tc;
    const int tiles_r = (ext_r + tr - 1) / tr;
    for (int t0 = 0; t0 < tiles_r; t0 += 65535) {   // grid.y is limited to 65535
        const int nt = tiles_r - t0 < 65535 ? tiles_r - t0 : 65535;
        const int r0 = t0 * tr;
        IndexTables t = {tab.row + r0, tab.col};
        const float* s = UNPACK ? src : src + (size_t)r0 * ld;
        float* d = UNPACK ? dst + (size_t)r0 * ld : dst;
        const int live = rows - r0 < 0 ? 0 : rows - r0;
        hipLaunchKernelGGL((pack_tile_kernel<UNPACK, TR, TC, STREAM>), dim3(tiles_c, nt), dim3(256), 0, stream, s, d,
                           live, cols, ld, rows_p - r0, cols_p, t, fast, rows_fast ? 1 : 0, tr, tc, pitch, lshift);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// Largest short-axis extent a tile kernel takes: rows of a micro-panel of A up to 64, columns of one of B or C up to 128.
static bool pack_tiles_take(int fast, bool rows_fast)
{
    return fast >= 1 && fast <= (rows_fast ? 64 : PACK_TC);
}

// fast = rows (rows_fast) or columns of a micro-panel.  Tile height: 16 rows, or with rows fast the one of
// 16, 24 and 32 that whole panels fill best (m_r = 6: 24), 64 x 64 tiles for panels of more than 32 rows.
template <bool UNPACK>
static hipError_t launch_pack_tiles(const float* src, float* dst, int rows, int cols, int ld, int rows_p,
                                    int cols_p, IndexTables tab, int fast, bool rows_fast, hipStream_t stream)
{
    const bool big = (size_t)rows * (size_t)cols * sizeof(float) >= (size_t)PACK_STREAM_BYTES;
    int tr = 16;
    if (rows_fast) {
        if (fast > 32) tr = 64;
        else {
            int best = 0;
            for (int cand : {16, 24, 32}) {
                const int used = 1000 * (fast * (cand / fast)) / cand;
                if (used > best) { best = used; tr = cand; }
            }
        }
    }
#define CAKE_PACK_TILES(TR, TC) \
    return big ? launch_pack_tiles_as<UNPACK, TR, TC, true>(src, dst, rows, cols, ld, rows_p, cols_p, tab, fast, rows_fast, stream) \
               : launch_pack_tiles_as<UNPACK, TR, TC, false>(src, dst, rows, cols, ld, rows_p, cols_p, tab, fast, rows_fast, stream)
    switch (tr) {
        case 16: CAKE_PACK_TILES(16, PACK_TC);
        case 24: CAKE_PACK_TILES(24, PACK_TC);
        case 32: CAKE_PACK_TILES(32, PACK_TC);
        default: CAKE_PACK_TILES(64, 64);
    }
#undef CAKE_PACK_TILES
}

hipError_t launch_pack(const float* src, float* dst, int rows, int cols, int ld, int rows_p,
                       int cols_p, IndexTables tab, int fast, bool rows_fast, hipStream_t stream)
{
    if (rows_p <= 0 || cols_p <= 0) return hipSuccess;
    if (pack_tiles_take(fast, rows_fast))
        return launch_pack_tiles<false>(src, dst, rows, cols, ld, rows_p, cols_p, tab, fast, rows_fast, stream);
    // grid.y is limited to 65535 rows per launch
    for (int r0 = 0; r0 < rows_p; r0 += 65535) {
        const int nr = rows_p - r0 < 65535 ? rows_p - r0 : 65535;
        IndexTables t = {tab.row + r0, tab.col};
        const int live = rows - r0 < 0 ? 0 : rows - r0;
        hipLaunchKernelGGL(pack_kernel, rowwise_grid(nr, cols_p), dim3(256), 0, stream,
                           src + (size_t)r0 * ld, dst, live, cols, ld, nr, cols_p, t);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

hipError_t launch_unpack(const float* src, float* dst, int rows, int cols, int ld, IndexTables tab,
                         int fast, bool rows_fast, hipStream_t stream)
{
    if (rows <= 0 || cols <= 0) return hipSuccess;
    if (pack_tiles_take(fast, rows_fast))
        return launch_pack_tiles<true>(src, dst, rows, cols, ld, rows, cols, tab, fast, rows_fast, stream);
    for (int r0 = 0; r0 < rows; r0 += 65535) {
        const int nr = rows - r0 < 65535 ? rows - r0 : 65535;
        IndexTables t = {tab.row + r0, tab.col};
        hipLaunchKernelGGL(unpack_kernel, rowwise_grid(nr, cols), dim3(256), 0, stream, src,
                           dst + (size_t)r0 * ld, nr, cols, ld, t);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

}  // namespace cake
