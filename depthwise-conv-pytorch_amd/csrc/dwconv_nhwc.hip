// Depthwise conv2d on channels-last tensors: input (N,H,W,C), taps (C,1,KH,KW) as everywhere else, output (N,OH,OW,C).
//
// The reference makes every tensor NCHW-contiguous before its kernels run (torch_dwconv/dwconv_kernel.cu:741,
// :855, :1023), which costs a layout-conversion pass either side of the op for a channels-last network.  These
// kernels read and write channels-last directly.  Channels are the fastest dimension, so lanes run along C:
//   * a lane owns CV consecutive channels (one vector access per pixel) and a BH x TW block of output pixels;
//     it walks the input rows of its block once, keeps one row of the window in registers and feeds every
//     output row that the input row touches; neighbouring lanes (next channels) read neighbouring addresses;
//   * taps are transposed once per workgroup into LDS as [tap][channel], so a lane reads the taps of its
//     channels as one vector;
//   * grad-weight keeps K*K*CV sums per lane over a chunk of pixel blocks, adds the lanes of a workgroup that
//     share channels through LDS in a fixed order, and leaves partial[chunk][tap][C] for a second kernel that
//     adds the chunks in a fixed order: bit-identical from run to run, no atomics.
// Geometries outside the fast kernels (C not a multiple of 4, filters other than 3/5/7, fp64) take the
// one-lane-per-element kernels at the end of the file.
#include "dwconv_tile_common.hpp"

#include <algorithm>
#include <type_traits>

namespace dwconv {

namespace {

constexpr int kNhwcThreads = 256;
constexpr int kNhwcTapLds = 48 * 1024;

struct NhwcPlan {
    const void *in;    // element type IO of the kernel template
    const void *in2;   // grad-weight: out_grad
    const void *taps;
    void *out;
    float *partial;
    int batch, channel;
    int in_h, in_w, out_h, out_w;
    int pad_h, pad_w;        // leading zeros (down kernels); floor(pad / 2) for the stride-2 transposed kernel
    int lanes_c;             // channel lanes per workgroup (each CV channels wide)
    unsigned lanes_c_magic;
    int blocks_per_wg;       // pixel blocks per workgroup = 256 / lanes_c
    int blocks_x, blocks_y;  // pixel blocks per image
    long blocks_total;       // batch * blocks_y * blocks_x
    int groups;              // grad-weight: workgroups along the pixel-block axis (= chunks)
    Epilogue epi;            // forward kernel: applied to every sum before it is stored
    int cgroups;             // workgroups along the channel axis
    int wgs;                 // forward / grad-input: workgroups in all (1-D grid)
    int xcd_chunks;          // backward: chunks are dealt to the XCDs in contiguous runs
};

// ---- window loads through a buffer view (nhwc_view / view_load, dwconv_tile_common.hpp) -----------------------
// The lanes of a workgroup read their windows through a raw buffer view that starts at the first image the
// workgroup touches.  A tap that falls outside the image costs no address clamp and no select: its row or
// column offset is replaced by kOob once (per row / per block), and the saturating sum of the two stays out
// of range, where loads return zeros.
// Column part of a lane's window offsets, computed once per pixel block: byte offset of this lane's channels
// in each of the COLS columns (lane_off = image and channel part), kOob for columns outside the image.
template <int COLS>
struct NhwcCols {
    unsigned off[COLS];
};
template <int COLS>
__device__ __forceinline__ void nhwc_cols(int ix0, int in_w, unsigned pixel_bytes, unsigned lane_off, NhwcCols<COLS> &c)
{
#pragma unroll
    for (int j = 0; j < COLS; ++j) {
        const int ix = ix0 + j;
        c.off[j] = static_cast<unsigned>(ix) < static_cast<unsigned>(in_w) ? lane_off + ix * pixel_bytes : kOob;
    }
}

// One row of a lane's window: COLS pixels x CV channels of row iy (zeros outside the image).
template <typename IO, int COLS, int CV = 4>
__device__ __forceinline__ void nhwc_load_row(__amdgpu_buffer_rsrc_t view, int iy, int in_h, unsigned row_bytes,
                                              const NhwcCols<COLS> &cols, float (&row)[COLS * CV])
{
    const unsigned roff = static_cast<unsigned>(iy) < static_cast<unsigned>(in_h) ? iy * row_bytes : kOob;
#pragma unroll
    for (int j = 0; j < COLS; ++j) {
        float t[CV];
        view_load<IO, CV>(view, __builtin_elementwise_add_sat(roff, cols.off[j]), t);
#pragma unroll
        for (int v = 0; v < CV; ++v) row[CV * j + v] = t[v];
    }
}

// Transposes the taps of channels [c0, c0 + nch) into LDS as [tap][channel] (rotated by 180 degrees when FLIP).
template <typename IO, int KK, bool FLIP>
__device__ __forceinline__ void nhwc_stage_taps(const IO *__restrict__ taps, float *lds, int c0, int nch)
{
    for (int i = threadIdx.x; i < nch * KK; i += blockDim.x) {
        const int cl = i / KK, t = i - cl * KK;
        lds[(FLIP ? KK - 1 - t : t) * nch + cl] = Io<IO>::in(taps[static_cast<long>(c0) * KK + i]);
    }
}

// out[n,oy,ox,c] = sum_{ty,tx} in[n, oy*S - pad_h + ty, ox*S - pad_w + tx, c] * f[c,ty,tx]
// CV channels per lane (4: one 128-bit access per pixel for fp32; 1: 32 lanes per 128-byte line of a pixel).
template <typename IO, int K, int S, bool FLIP, int BH, int TW, int CV = 4>
__global__ __launch_bounds__(kNhwcThreads) void nhwc_down_kernel(const NhwcPlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int KK = K * K;
    constexpr int ROWS = (BH - 1) * S + K, COLS = (TW - 1) * S + K;
    const int C = p.channel;
    // 1-D grid, channel group fastest; every XCD (own L2) gets a contiguous run of workgroups, so that pixel
    // groups that share halo rows, and the channel groups of one pixel group (neighbouring addresses), meet there
    const int wg = xcd_contiguous_tile(blockIdx.x, p.wgs);
    const int pg = wg / p.cgroups;
    const int c0 = (wg - pg * p.cgroups) * p.lanes_c * CV;
    const int nch = min(p.lanes_c * CV, C - c0);
    nhwc_stage_taps<IO, KK, FLIP>(static_cast<const IO *>(p.taps), lds, c0, nch);
    __syncthreads();

    const int pb_local = fast_div(threadIdx.x, p.lanes_c_magic);
    const int lane_c = threadIdx.x - pb_local * p.lanes_c;
    const long pb = static_cast<long>(pg) * p.blocks_per_wg + pb_local;
    if (pb_local >= p.blocks_per_wg || pb >= p.blocks_total || CV * lane_c >= nch) return;
    const int per_image = p.blocks_x * p.blocks_y;
    const int n = static_cast<int>(pb / per_image);
    const int rem = static_cast<int>(pb - static_cast<long>(n) * per_image);
    const int by = rem / p.blocks_x, bx = rem - by * p.blocks_x;
    const int oy0 = by * BH, ox0 = bx * TW;
    const int iy0 = oy0 * S - p.pad_h, ix0 = ox0 * S - p.pad_w;
    const int c = c0 + CV * lane_c;
    const float *wl = lds + CV * lane_c;
    // view of the input from the first image this workgroup touches (uniform); this lane's image and channels
    // are part of its column offsets
    const int n0 = static_cast<int>(static_cast<long>(pg) * p.blocks_per_wg / per_image);
    const unsigned pixel_bytes = C * sizeof(IO), row_bytes = p.in_w * pixel_bytes;
    const __amdgpu_buffer_rsrc_t view =
        buffer_view(static_cast<const IO *>(p.in) + static_cast<long>(n0) * p.in_h * p.in_w * C,
                    static_cast<long>(p.batch - n0) * p.in_h * row_bytes);
    const unsigned lane_off = (n - n0) * (p.in_h * row_bytes) + c * static_cast<unsigned>(sizeof(IO));

    float acc[BH][TW * CV];
#pragma unroll
    for (int b = 0; b < BH; ++b)
#pragma unroll
        for (int o = 0; o < TW * CV; ++o) acc[b][o] = 0.f;

    // Rows are loaded one ahead of their use (two row buffers, alternating) and the sums pinned after every
    // row: otherwise the compiler hoists the loads of the whole window to the top and keeps all of it in registers.
    float rows[2][COLS * CV];
    NhwcCols<COLS> cols;
    nhwc_cols<COLS>(ix0, p.in_w, pixel_bytes, lane_off, cols);
    nhwc_load_row<IO, COLS, CV>(view, iy0, p.in_h, row_bytes, cols, rows[0]);
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        float(&cur)[COLS * CV] = rows[r & 1];
        if (r + 1 < ROWS) nhwc_load_row<IO, COLS, CV>(view, iy0 + r + 1, p.in_h, row_bytes, cols, rows[(r + 1) & 1]);
#pragma unroll
        for (int b = 0; b < BH; ++b) {
            const int ty = r - b * S;
            if (ty < 0 || ty >= K) continue;
#pragma unroll
            for (int tx = 0; tx < K; ++tx) {
                float w[CV];
#pragma unroll
                for (int q = 0; q < CV; ++q) w[q] = wl[(ty * K + tx) * nch + q];
#pragma unroll
                for (int o = 0; o < TW; ++o)
#pragma unroll
                    for (int q = 0; q < CV; ++q)
                        acc[b][CV * o + q] = fmaf(cur[CV * (o * S + tx) + q], w[q], acc[b][CV * o + q]);
            }
        }
        pin_registers(acc);
    }

    if constexpr (!FLIP) {
        if (p.epi.enabled()) epilogue_apply_block<CV>(acc, p.epi, c);
    }
    // branch-free stores through a view of the output: pixels past the edge of the image store out of range
    const unsigned out_row_bytes = p.out_w * pixel_bytes;
    const __amdgpu_buffer_rsrc_t out_view =
        buffer_view(static_cast<IO *>(p.out) + static_cast<long>(n0) * p.out_h * p.out_w * C,
                    static_cast<long>(p.batch - n0) * p.out_h * out_row_bytes);
    NhwcCols<TW> ocols;
    nhwc_cols<TW>(ox0, p.out_w, pixel_bytes, (n - n0) * (p.out_h * out_row_bytes) + c * static_cast<unsigned>(sizeof(IO)), ocols);
#pragma unroll
    for (int b = 0; b < BH; ++b) {
        const int oy = oy0 + b;
        const unsigned roff = oy < p.out_h ? oy * out_row_bytes : kOob;
#pragma unroll
        for (int o = 0; o < TW; ++o) {
            const unsigned off = __builtin_elementwise_add_sat(roff, ocols.off[o]);
            if constexpr (CV == 4)
                view_store4<IO>(out_view, off, acc[b][4 * o], acc[b][4 * o + 1], acc[b][4 * o + 2], acc[b][4 * o + 3]);
            else if constexpr (CV == 2)
                view_store2<IO>(out_view, off, acc[b][2 * o], acc[b][2 * o + 1]);
            else
                view_store1<IO>(out_view, off, acc[b][o]);
        }
    }
}

// Grad-input of a stride-2 convolution with padding 2*p.pad_h + PE (same for both axes), taps as stored:
//   gx[iy,ix] = sum over (ty,tx) with iy + pad - ty and ix + pad - tx even of gy[(iy+pad-ty)/2, (ix+pad-tx)/2] * w[ty,tx].
// A lane owns a BH x TW block of gx that starts on even coordinates, so which taps meet which gy sample is
// known at compile time: row b of the block and gy row d (relative to iy0/2 + floor(pad/2)) meet in tap
// ty = b + PE - 2d.  The zero-stuffed intermediate of the reference (torch_dwconv/dwconv_kernel.cu:822-832) never exists.
template <typename IO, int K, int PE, int BH, int TW>
__global__ __launch_bounds__(kNhwcThreads) void nhwc_up2_kernel(const NhwcPlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int KK = K * K;
    static_assert(BH % 2 == 0 && TW % 2 == 0, "blocks start on even coordinates");
    constexpr int DMIN = -((K - 1 - PE) / 2);
    constexpr int GROWS = (BH - 1 + PE) / 2 - DMIN + 1, GCOLS = (TW - 1 + PE) / 2 - DMIN + 1;
    const int C = p.channel;
    // 1-D grid, channel group fastest; every XCD (own L2) gets a contiguous run of workgroups, so that pixel
    // groups that share halo rows, and the channel groups of one pixel group (neighbouring addresses), meet there
    const int wg = xcd_contiguous_tile(blockIdx.x, p.wgs);
    const int pg = wg / p.cgroups;
    const int c0 = (wg - pg * p.cgroups) * p.lanes_c * 4;
    const int nch = min(p.lanes_c * 4, C - c0);
    nhwc_stage_taps<IO, KK, false>(static_cast<const IO *>(p.taps), lds, c0, nch);
    __syncthreads();

    const int pb_local = fast_div(threadIdx.x, p.lanes_c_magic);
    const int lane_c = threadIdx.x - pb_local * p.lanes_c;
    const long pb = static_cast<long>(pg) * p.blocks_per_wg + pb_local;
    if (pb_local >= p.blocks_per_wg || pb >= p.blocks_total || 4 * lane_c >= nch) return;
    const int per_image = p.blocks_x * p.blocks_y;
    const int n = static_cast<int>(pb / per_image);
    const int rem = static_cast<int>(pb - static_cast<long>(n) * per_image);
    const int by = rem / p.blocks_x, bx = rem - by * p.blocks_x;
    // here "out" is gx (extent out_h x out_w) and "in" is gy (extent in_h x in_w)
    const int iy0 = by * BH, ix0 = bx * TW;
    const int gy0 = iy0 / 2 + p.pad_h + DMIN, gx0 = ix0 / 2 + p.pad_w + DMIN;
    const int c = c0 + 4 * lane_c;
    const float *wl = lds + 4 * lane_c;
    const int n0 = static_cast<int>(static_cast<long>(pg) * p.blocks_per_wg / per_image);
    const unsigned pixel_bytes = C * sizeof(IO), row_bytes = p.in_w * pixel_bytes;
    const __amdgpu_buffer_rsrc_t view =
        buffer_view(static_cast<const IO *>(p.in) + static_cast<long>(n0) * p.in_h * p.in_w * C,
                    static_cast<long>(p.batch - n0) * p.in_h * row_bytes);
    const unsigned lane_off = (n - n0) * (p.in_h * row_bytes) + c * static_cast<unsigned>(sizeof(IO));

    float acc[BH][TW * 4];
#pragma unroll
    for (int b = 0; b < BH; ++b)
#pragma unroll
        for (int o = 0; o < TW * 4; ++o) acc[b][o] = 0.f;

    float rows[2][GCOLS * 4];
    NhwcCols<GCOLS> cols;
    nhwc_cols<GCOLS>(gx0, p.in_w, pixel_bytes, lane_off, cols);
    nhwc_load_row<IO, GCOLS>(view, gy0, p.in_h, row_bytes, cols, rows[0]);
#pragma unroll
    for (int g = 0; g < GROWS; ++g) {
        float(&cur)[GCOLS * 4] = rows[g & 1];
        if (g + 1 < GROWS) nhwc_load_row<IO, GCOLS>(view, gy0 + g + 1, p.in_h, row_bytes, cols, rows[(g + 1) & 1]);
#pragma unroll
        for (int b = 0; b < BH; ++b) {
            const int ty = b + PE - 2 * (DMIN + g);
            if (ty < 0 || ty >= K) continue;
#pragma unroll
            for (int o = 0; o < TW; ++o) {
#pragma unroll
                for (int j = 0; j < GCOLS; ++j) {
                    const int tx = o + PE - 2 * (DMIN + j);
                    if (tx < 0 || tx >= K) continue;
                    const float4 w = *reinterpret_cast<const float4 *>(wl + (ty * K + tx) * nch);
                    acc[b][4 * o + 0] = fmaf(cur[4 * j + 0], w.x, acc[b][4 * o + 0]);
                    acc[b][4 * o + 1] = fmaf(cur[4 * j + 1], w.y, acc[b][4 * o + 1]);
                    acc[b][4 * o + 2] = fmaf(cur[4 * j + 2], w.z, acc[b][4 * o + 2]);
                    acc[b][4 * o + 3] = fmaf(cur[4 * j + 3], w.w, acc[b][4 * o + 3]);
                }
            }
        }
        pin_registers(acc);
    }

    const unsigned out_row_bytes = p.out_w * pixel_bytes;
    const __amdgpu_buffer_rsrc_t out_view =
        buffer_view(static_cast<IO *>(p.out) + static_cast<long>(n0) * p.out_h * p.out_w * C,
                    static_cast<long>(p.batch - n0) * p.out_h * out_row_bytes);
    NhwcCols<TW> ocols;
    nhwc_cols<TW>(ix0, p.out_w, pixel_bytes, (n - n0) * (p.out_h * out_row_bytes) + c * static_cast<unsigned>(sizeof(IO)), ocols);
#pragma unroll
    for (int b = 0; b < BH; ++b) {
        const int iy = iy0 + b;
        const unsigned roff = iy < p.out_h ? iy * out_row_bytes : kOob;
#pragma unroll
        for (int o = 0; o < TW; ++o)
            view_store4<IO>(out_view, __builtin_elementwise_add_sat(roff, ocols.off[o]), acc[b][4 * o], acc[b][4 * o + 1],
                            acc[b][4 * o + 2], acc[b][4 * o + 3]);
    }
}

// Grad-weight, pass 1.  in = x (in_h x in_w), in2 = gy (out_h x out_w).  Workgroup (chunk, channel group):
// the lane walks the pixel blocks chunk, chunk + groups, ... with its K*K*CV sums in registers.
template <typename IO, int K, int S, int CV, int BH, int TW>
__global__ __launch_bounds__(kNhwcThreads) void nhwc_wgrad_kernel(const NhwcPlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int KK = K * K;
    constexpr int ROWS = (BH - 1) * S + K, COLS = (TW - 1) * S + K;
    const int C = p.channel;
    // (grid: chunk x channel group, dealt to the XCDs round-robin; giving every XCD a contiguous run of chunks,
    // as the forward kernel does with its pixel groups, measured 2 % slower here)
    // 1-D grid, channel group fastest; with xcd_chunks every XCD (own L2) takes a contiguous run of chunks
    const int wg = p.xcd_chunks ? xcd_contiguous_tile(blockIdx.x, p.groups * p.cgroups) : static_cast<int>(blockIdx.x);
    const int chunk = wg / p.cgroups;
    const int c0 = (wg - chunk * p.cgroups) * p.lanes_c * CV;
    const int nch = min(p.lanes_c * CV, C - c0);
    const int pb_local = fast_div(threadIdx.x, p.lanes_c_magic);
    const int lane_c = threadIdx.x - pb_local * p.lanes_c;
    const bool lane_ok = pb_local < p.blocks_per_wg && CV * lane_c < nch;
    const int c = c0 + (lane_ok ? CV * lane_c : 0);
    const int per_image = p.blocks_x * p.blocks_y;

    float acc[KK][CV];
#pragma unroll
    for (int t = 0; t < KK; ++t)
#pragma unroll
        for (int v = 0; v < CV; ++v) acc[t][v] = 0.f;

    for (long grp = chunk; grp * p.blocks_per_wg < p.blocks_total; grp += p.groups) {
        const long pb = grp * p.blocks_per_wg + pb_local;
        if (!lane_ok || pb >= p.blocks_total) continue;
        const int n = static_cast<int>(pb / per_image);
        const int rem = static_cast<int>(pb - static_cast<long>(n) * per_image);
        const int by = rem / p.blocks_x, bx = rem - by * p.blocks_x;
        const int oy0 = by * BH, ox0 = bx * TW;
        const int iy0 = oy0 * S - p.pad_h, ix0 = ox0 * S - p.pad_w;
        // views of x and gy from the first image of this group of pixel blocks (uniform)
        const int n0 = static_cast<int>(grp * p.blocks_per_wg / per_image);
        const unsigned pixel_bytes = C * sizeof(IO), row_bytes = p.in_w * pixel_bytes, grow_bytes = p.out_w * pixel_bytes;
        const __amdgpu_buffer_rsrc_t xview =
            buffer_view(static_cast<const IO *>(p.in) + static_cast<long>(n0) * p.in_h * p.in_w * C,
                    static_cast<long>(p.batch - n0) * p.in_h * row_bytes);
        const __amdgpu_buffer_rsrc_t gview =
            buffer_view(static_cast<const IO *>(p.in2) + static_cast<long>(n0) * p.out_h * p.out_w * C,
                    static_cast<long>(p.batch - n0) * p.out_h * grow_bytes);
        const unsigned chan_off = c * static_cast<unsigned>(sizeof(IO));

        // out_grad rows are fetched one window row before their first use (row b meets window rows b*S ... b*S+K-1),
        // so a tall block keeps only the rows in use in registers (the loop is unrolled: a row's registers are
        // free again after its last use)
        float g[BH][TW * CV];
        NhwcCols<TW> gcols;
        nhwc_cols<TW>(ox0, p.out_w, pixel_bytes, (n - n0) * (p.out_h * grow_bytes) + chan_off, gcols);
        nhwc_load_row<IO, TW, CV>(gview, oy0, p.out_h, grow_bytes, gcols, g[0]);
        float rows[2][COLS * CV];
        NhwcCols<COLS> cols;
        nhwc_cols<COLS>(ix0, p.in_w, pixel_bytes, (n - n0) * (p.in_h * row_bytes) + chan_off, cols);
        nhwc_load_row<IO, COLS, CV>(xview, iy0, p.in_h, row_bytes, cols, rows[0]);
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            float(&cur)[COLS * CV] = rows[r & 1];
            if (r + 1 < ROWS) nhwc_load_row<IO, COLS, CV>(xview, iy0 + r + 1, p.in_h, row_bytes, cols, rows[(r + 1) & 1]);
            if ((r + 1) % S == 0 && (r + 1) / S < BH)
                nhwc_load_row<IO, TW, CV>(gview, oy0 + (r + 1) / S, p.out_h, grow_bytes, gcols, g[(r + 1) / S]);
            // window row r meets out_grad row b in tap row ty = r - b*S (looping over ty keeps the body small
            // enough for the unroller whatever BH is)
#pragma unroll
            for (int ty = 0; ty < K; ++ty) {
                const int bs = r - ty;
                if (bs < 0 || bs % S != 0 || bs / S >= BH) continue;
                const int b = bs / S;
#pragma unroll
                for (int tx = 0; tx < K; ++tx)
#pragma unroll
                    for (int o = 0; o < TW; ++o)
#pragma unroll
                        for (int v = 0; v < CV; ++v)
                            acc[ty * K + tx][v] = fmaf(g[b][CV * o + v], cur[CV * (o * S + tx) + v], acc[ty * K + tx][v]);
            }
            pin_registers(acc);
        }
    }

    // Lanes that share channels (same lane_c, different pixel block) are added front to back, one tap row at a time.
    const int width = p.lanes_c * CV;  // floats per (pixel block, tap) line in LDS
    float *out = p.partial + static_cast<long>(chunk) * KK * C;
#pragma unroll
    for (int ty = 0; ty < K; ++ty) {
        if (ty) __syncthreads();
        if (pb_local < p.blocks_per_wg) {
#pragma unroll
            for (int tx = 0; tx < K; ++tx)
#pragma unroll
                for (int v = 0; v < CV; ++v) lds[(pb_local * K + tx) * width + CV * lane_c + v] = lane_ok ? acc[ty * K + tx][v] : 0.f;
        }
        __syncthreads();
        for (int e = threadIdx.x; e < K * nch; e += blockDim.x) {
            const int tx = e / nch, cl = e - tx * nch;
            float s = 0.f;
            for (int q = 0; q < p.blocks_per_wg; ++q) s += lds[(q * K + tx) * width + cl];
            out[static_cast<long>(ty * K + tx) * C + c0 + cl] = s;
        }
    }
}

// Grad-input and grad-weight of a stride-1 layer whose output has the extent of its input (pad = K / 2) in one
// sweep: in = x, in2 = out_grad, out = in_grad, all H x W.  The lane owns a BH x TW block of pixels and CV channels.
// It walks the window rows of out_grad (block + K/2 halo either side, fetched once) and, K/2 rows behind, those of
// x.  A row of out_grad feeds the K rows of in_grad it touches (rotated taps from LDS; a row of in_grad is stored
// as soon as its last window row has passed) and its centre pixels are kept for the K rows of x they meet in the
// grad-weight sums.  The loop is unrolled, so only the rows in use are live.  out_grad is read once instead of
// twice and the separate grad-input kernel goes away.  The end of the kernel is that of nhwc_wgrad_kernel.
template <typename IO, int K, int CV, int BH, int TW>
__global__ __launch_bounds__(kNhwcThreads) void nhwc_bwd_fused_kernel(const NhwcPlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int KK = K * K, P = K / 2;
    constexpr int ROWS = BH + K - 1, COLS = TW + K - 1;
    const int C = p.channel;
    // 1-D grid, channel group fastest; with xcd_chunks every XCD (own L2) takes a contiguous run of chunks
    const int wg = p.xcd_chunks ? xcd_contiguous_tile(blockIdx.x, p.groups * p.cgroups) : static_cast<int>(blockIdx.x);
    const int chunk = wg / p.cgroups;
    const int c0 = (wg - chunk * p.cgroups) * p.lanes_c * CV;
    const int nch = min(p.lanes_c * CV, C - c0);
    const int pb_local = fast_div(threadIdx.x, p.lanes_c_magic);
    const int lane_c = threadIdx.x - pb_local * p.lanes_c;
    const bool lane_ok = pb_local < p.blocks_per_wg && CV * lane_c < nch;
    const int c = c0 + (lane_ok ? CV * lane_c : 0);
    const int per_image = p.blocks_x * p.blocks_y;
    nhwc_stage_taps<IO, KK, true>(static_cast<const IO *>(p.taps), lds, c0, nch);
    __syncthreads();
    const float *wl = lds + (lane_ok ? CV * lane_c : 0);

    float acc[KK][CV];
#pragma unroll
    for (int t = 0; t < KK; ++t)
#pragma unroll
        for (int v = 0; v < CV; ++v) acc[t][v] = 0.f;

    for (long grp = chunk; grp * p.blocks_per_wg < p.blocks_total; grp += p.groups) {
        const long pb = grp * p.blocks_per_wg + pb_local;
        if (!lane_ok || pb >= p.blocks_total) continue;
        const int n = static_cast<int>(pb / per_image);
        const int rem = static_cast<int>(pb - static_cast<long>(n) * per_image);
        const int by = rem / p.blocks_x, bx = rem - by * p.blocks_x;
        const int oy0 = by * BH, ox0 = bx * TW;
        const int iy0 = oy0 - P, ix0 = ox0 - P;
        // views of x, out_grad and in_grad from the first image of this group of pixel blocks (uniform); the three
        // tensors have the same extent, so one set of column offsets serves all of them
        const int n0 = static_cast<int>(grp * p.blocks_per_wg / per_image);
        const unsigned pixel_bytes = C * sizeof(IO), row_bytes = p.in_w * pixel_bytes;
        const long image0 = static_cast<long>(n0) * p.in_h * p.in_w * C;
        const long span = static_cast<long>(p.batch - n0) * p.in_h * row_bytes;  // to the end of the tensor
        const __amdgpu_buffer_rsrc_t xview = buffer_view(static_cast<const IO *>(p.in) + image0, span);
        const __amdgpu_buffer_rsrc_t gview = buffer_view(static_cast<const IO *>(p.in2) + image0, span);
        const __amdgpu_buffer_rsrc_t oview = buffer_view(static_cast<IO *>(p.out) + image0, span);
        const unsigned lane_off = (n - n0) * (p.in_h * row_bytes) + c * static_cast<unsigned>(sizeof(IO));
        NhwcCols<COLS> cols;
        nhwc_cols<COLS>(ix0, p.in_w, pixel_bytes, lane_off, cols);

        float gxs[BH][TW * CV];  // in_grad sums
        float gb[BH][TW * CV];   // centre pixels of the out_grad rows (the block itself)
#pragma unroll
        for (int b = 0; b < BH; ++b)
#pragma unroll
            for (int o = 0; o < TW * CV; ++o) gxs[b][o] = 0.f;
        float xr[2][COLS * CV], gr[2][COLS * CV];
        nhwc_load_row<IO, COLS, CV>(gview, iy0, p.in_h, row_bytes, cols, gr[0]);
#pragma unroll
        for (int t = 0; t < ROWS + P; ++t) {
            const int r = t - P;  // window row of x in this step (out_grad runs P rows ahead)
            if (t + 1 < ROWS) nhwc_load_row<IO, COLS, CV>(gview, iy0 + t + 1, p.in_h, row_bytes, cols, gr[(t + 1) & 1]);
            if (r + 1 >= 0 && r + 1 < ROWS)
                nhwc_load_row<IO, COLS, CV>(xview, iy0 + r + 1, p.in_h, row_bytes, cols, xr[(r + 1) & 1]);
            if (t < ROWS) {
                float(&gcur)[COLS * CV] = gr[t & 1];
                // in_grad row b meets this row in rotated tap row u = t - b
#pragma unroll
                for (int u = 0; u < K; ++u) {
                    const int b = t - u;
                    if (b < 0 || b >= BH) continue;
#pragma unroll
                    for (int v = 0; v < K; ++v) {
                        float w[CV];
#pragma unroll
                        for (int q = 0; q < CV; ++q) w[q] = wl[(u * K + v) * nch + q];
#pragma unroll
                        for (int o = 0; o < TW; ++o)
#pragma unroll
                            for (int q = 0; q < CV; ++q)
                                gxs[b][CV * o + q] = fmaf(gcur[CV * (o + v) + q], w[q], gxs[b][CV * o + q]);
                    }
                }
                if (t - P >= 0 && t - P < BH) {
#pragma unroll
                    for (int o = 0; o < TW * CV; ++o) gb[t - P][o] = gcur[CV * P + o];
                }
                if (t - (K - 1) >= 0 && t - (K - 1) < BH) {
                    const int b = t - (K - 1);
                    const unsigned roff = oy0 + b < p.in_h ? (oy0 + b) * row_bytes : kOob;
#pragma unroll
                    for (int o = 0; o < TW; ++o) {
                        const unsigned off = __builtin_elementwise_add_sat(roff, cols.off[o + P]);
                        if constexpr (CV == 4)
                            view_store4<IO>(oview, off, gxs[b][4 * o], gxs[b][4 * o + 1], gxs[b][4 * o + 2], gxs[b][4 * o + 3]);
                        else if constexpr (CV == 2)
                            view_store2<IO>(oview, off, gxs[b][2 * o], gxs[b][2 * o + 1]);
                        else
                            view_store1<IO>(oview, off, gxs[b][o]);
                    }
                }
            }
            if (r >= 0 && r < ROWS) {
                float(&xcur)[COLS * CV] = xr[r & 1];
                // window row r of x meets out_grad row b in tap row ty = r - b
#pragma unroll
                for (int ty = 0; ty < K; ++ty) {
                    const int b = r - ty;
                    if (b < 0 || b >= BH) continue;
#pragma unroll
                    for (int tx = 0; tx < K; ++tx)
#pragma unroll
                        for (int o = 0; o < TW; ++o)
#pragma unroll
                            for (int q = 0; q < CV; ++q)
                                acc[ty * K + tx][q] = fmaf(gb[b][CV * o + q], xcur[CV * (o + tx) + q], acc[ty * K + tx][q]);
                }
            }
            pin_registers(acc);
        }
    }
    __syncthreads();  // the taps in LDS are done with: the sums of the lanes go through the same memory

    const int width = p.lanes_c * CV;
    float *out = p.partial + static_cast<long>(chunk) * KK * C;
#pragma unroll
    for (int ty = 0; ty < K; ++ty) {
        if (ty) __syncthreads();
        if (pb_local < p.blocks_per_wg) {
#pragma unroll
            for (int tx = 0; tx < K; ++tx)
#pragma unroll
                for (int v = 0; v < CV; ++v) lds[(pb_local * K + tx) * width + CV * lane_c + v] = lane_ok ? acc[ty * K + tx][v] : 0.f;
        }
        __syncthreads();
        for (int e = threadIdx.x; e < K * nch; e += blockDim.x) {
            const int tx = e / nch, cl = e - tx * nch;
            float s = 0.f;
            for (int q = 0; q < p.blocks_per_wg; ++q) s += lds[(q * K + tx) * width + cl];
            out[static_cast<long>(ty * K + tx) * C + c0 + cl] = s;
        }
    }
}

// Grad-input and grad-weight of a stride-2 layer with pad K / 2 and even input extents (out = in / 2) in one sweep:
// in = x (in_h x in_w), in2 = out_grad (out_h x out_w), out = in_grad.  The lane owns a BQH x BQW block of out_grad
// pixels and CV channels, i.e. a 2 BQH x 2 BQW block of in_grad and the (2 BQH + K - 2) x (2 BQW + K - 2) window of
// x its sums need.  With q0 the block's first out_grad row and d = q - q0:
//   in_grad row 2 q0 + b   += out_grad row q0 + d  *  tap row ty = b + P - 2 d        (P = K / 2; 0 <= ty < K)
//   sum[ty][tx]            += out_grad row q0 + j  *  x window row r = 2 j + ty        (x row 2 q0 - P + r)
// and the same along columns.  The lane walks the P/2 + BQH + (P + 1)/2 window rows of out_grad once: each feeds the
// rows of in_grad it touches (a row is stored as soon as no later out_grad row reaches it) and, where it belongs to
// the lane's own block, is kept for the x rows it meets; two x rows are consumed per out_grad row, right behind it.
// The loop is unrolled, so only the rows in use are live.  out_grad is read once instead of twice and the separate
// grad-input kernel (nhwc_up2_kernel) goes away.  The end of the kernel is that of nhwc_wgrad_kernel.
template <typename IO, int K, int CV, int BQH, int BQW>
__global__ __launch_bounds__(kNhwcThreads) void nhwc_bwd_s2_fused_kernel(const NhwcPlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int KK = K * K, P = K / 2;
    constexpr int DMIN = -(P / 2);                        // first out_grad row / column of the window, relative to the block
    constexpr int GROWS = BQH + P, GCOLS = BQW + P;       // out_grad window
    constexpr int XROWS = 2 * (BQH - 1) + K, XCOLS = 2 * (BQW - 1) + K;  // x window
    constexpr int GXH = 2 * BQH, GXW = 2 * BQW;           // in_grad block
    constexpr int STEPS = GROWS + P / 2;                  // x rows 2 (t - P/2), 2 (t - P/2) + 1 are consumed in step t
    static_assert(2 * (STEPS - 1 - P / 2) + 1 >= XROWS - 1, "every x row has its step");
    const int C = p.channel;
    // 1-D grid, channel group fastest; with xcd_chunks every XCD (own L2) takes a contiguous run of chunks
    const int wg = p.xcd_chunks ? xcd_contiguous_tile(blockIdx.x, p.groups * p.cgroups) : static_cast<int>(blockIdx.x);
    const int chunk = wg / p.cgroups;
    const int c0 = (wg - chunk * p.cgroups) * p.lanes_c * CV;
    const int nch = min(p.lanes_c * CV, C - c0);
    const int pb_local = fast_div(threadIdx.x, p.lanes_c_magic);
    const int lane_c = threadIdx.x - pb_local * p.lanes_c;
    const bool lane_ok = pb_local < p.blocks_per_wg && CV * lane_c < nch;
    const int c = c0 + (lane_ok ? CV * lane_c : 0);
    const int per_image = p.blocks_x * p.blocks_y;
    nhwc_stage_taps<IO, KK, false>(static_cast<const IO *>(p.taps), lds, c0, nch);
    __syncthreads();
    const float *wl = lds + (lane_ok ? CV * lane_c : 0);

    float acc[KK][CV];
#pragma unroll
    for (int t = 0; t < KK; ++t)
#pragma unroll
        for (int v = 0; v < CV; ++v) acc[t][v] = 0.f;

    for (long grp = chunk; grp * p.blocks_per_wg < p.blocks_total; grp += p.groups) {
        const long pb = grp * p.blocks_per_wg + pb_local;
        if (!lane_ok || pb >= p.blocks_total) continue;
        const int n = static_cast<int>(pb / per_image);
        const int rem = static_cast<int>(pb - static_cast<long>(n) * per_image);
        const int by = rem / p.blocks_x, bx = rem - by * p.blocks_x;
        const int q0 = by * BQH, qx0 = bx * BQW;          // the block in out_grad
        const int xr0 = 2 * q0 - P, xc0 = 2 * qx0 - P;    // first row / column of the x window
        // views from the first image of this group of pixel blocks (uniform): x and in_grad share an extent
        const int n0 = static_cast<int>(grp * p.blocks_per_wg / per_image);
        const unsigned pixel_bytes = C * sizeof(IO);
        const unsigned xrow_bytes = p.in_w * pixel_bytes, grow_bytes = p.out_w * pixel_bytes;
        const long ximage0 = static_cast<long>(n0) * p.in_h * p.in_w * C, gimage0 = static_cast<long>(n0) * p.out_h * p.out_w * C;
        const long xspan = static_cast<long>(p.batch - n0) * p.in_h * xrow_bytes;
        const long gspan = static_cast<long>(p.batch - n0) * p.out_h * grow_bytes;
        const __amdgpu_buffer_rsrc_t xview = buffer_view(static_cast<const IO *>(p.in) + ximage0, xspan);
        const __amdgpu_buffer_rsrc_t gview = buffer_view(static_cast<const IO *>(p.in2) + gimage0, gspan);
        const __amdgpu_buffer_rsrc_t oview = buffer_view(static_cast<IO *>(p.out) + ximage0, xspan);
        NhwcCols<XCOLS> xcols;
        nhwc_cols<XCOLS>(xc0, p.in_w, pixel_bytes, (n - n0) * (p.in_h * xrow_bytes) + c * static_cast<unsigned>(sizeof(IO)), xcols);
        NhwcCols<GCOLS> gcols;
        nhwc_cols<GCOLS>(qx0 + DMIN, p.out_w, pixel_bytes, (n - n0) * (p.out_h * grow_bytes) + c * static_cast<unsigned>(sizeof(IO)), gcols);

        float gxs[GXH][GXW * CV];   // in_grad sums
        float gb[BQH][BQW * CV];    // the lane's own rows of out_grad
#pragma unroll
        for (int b = 0; b < GXH; ++b)
#pragma unroll
            for (int o = 0; o < GXW * CV; ++o) gxs[b][o] = 0.f;
        float gr[2][GCOLS * CV], xr[2][XCOLS * CV];
        nhwc_load_row<IO, GCOLS, CV>(gview, q0 + DMIN, p.out_h, grow_bytes, gcols, gr[0]);
        nhwc_load_row<IO, XCOLS, CV>(xview, xr0, p.in_h, xrow_bytes, xcols, xr[0]);
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
            if (t + 1 < GROWS) nhwc_load_row<IO, GCOLS, CV>(gview, q0 + DMIN + t + 1, p.out_h, grow_bytes, gcols, gr[(t + 1) & 1]);
            if (t < GROWS) {
                float(&gcur)[GCOLS * CV] = gr[t & 1];
                const int d = DMIN + t;
                // in_grad row b meets this row in tap row ty = b + P - 2 d, in_grad column o meets window column j
                // in tap column tx = o + P - 2 (DMIN + j)
#pragma unroll
                for (int b = 0; b < GXH; ++b) {
                    const int ty = b + P - 2 * d;
                    if (ty < 0 || ty >= K) continue;
#pragma unroll
                    for (int o = 0; o < GXW; ++o)
#pragma unroll
                        for (int j = 0; j < GCOLS; ++j) {
                            const int tx = o + P - 2 * (DMIN + j);
                            if (tx < 0 || tx >= K) continue;
#pragma unroll
                            for (int q = 0; q < CV; ++q)
                                gxs[b][CV * o + q] = fmaf(gcur[CV * j + q], wl[(ty * K + tx) * nch + q], gxs[b][CV * o + q]);
                        }
                }
                if (d >= 0 && d < BQH) {
#pragma unroll
                    for (int o = 0; o < BQW * CV; ++o) gb[d >= 0 && d < BQH ? d : 0][o] = gcur[CV * (-DMIN) + o];
                }
                // rows no later out_grad row reaches: b < 2 (d + 1) - P; those finished before this step were stored then
#pragma unroll
                for (int b = 0; b < GXH; ++b) {
                    const bool done_now = b < 2 * (d + 1) - P || t == GROWS - 1;
                    const bool done_before = t > 0 && b < 2 * d - P;
                    if (!done_now || done_before) continue;
                    const unsigned roff = 2 * q0 + b < p.in_h ? (2 * q0 + b) * xrow_bytes : kOob;
#pragma unroll
                    for (int o = 0; o < GXW; ++o) {
                        const unsigned off = __builtin_elementwise_add_sat(roff, xcols.off[o + P]);
                        if constexpr (CV == 4)
                            view_store4<IO>(oview, off, gxs[b][4 * o], gxs[b][4 * o + 1], gxs[b][4 * o + 2], gxs[b][4 * o + 3]);
                        else if constexpr (CV == 2)
                            view_store2<IO>(oview, off, gxs[b][2 * o], gxs[b][2 * o + 1]);
                        else
                            view_store1<IO>(oview, off, gxs[b][o]);
                    }
                }
            }
            // the x rows whose out_grad rows (own rows up to t - P/2) have all passed
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int r = 2 * (t - P / 2) + h;
                if (r < 0 || r >= XROWS) continue;
                if (r + 1 < XROWS) nhwc_load_row<IO, XCOLS, CV>(xview, xr0 + r + 1, p.in_h, xrow_bytes, xcols, xr[(r + 1) & 1]);
                float(&xcur)[XCOLS * CV] = xr[r & 1];
#pragma unroll
                for (int ty = 0; ty < K; ++ty) {
                    if ((r - ty) % 2 != 0) continue;
                    const int j = (r - ty) / 2;
                    if (r - ty < 0 || j >= BQH) continue;
#pragma unroll
                    for (int tx = 0; tx < K; ++tx)
#pragma unroll
                        for (int i = 0; i < BQW; ++i)
#pragma unroll
                            for (int q = 0; q < CV; ++q)
                                acc[ty * K + tx][q] = fmaf(gb[j][CV * i + q], xcur[CV * (2 * i + tx) + q], acc[ty * K + tx][q]);
                }
            }
            pin_registers(acc);
        }
    }
    __syncthreads();  // the taps in LDS are done with: the sums of the lanes go through the same memory

    const int width = p.lanes_c * CV;
    float *out = p.partial + static_cast<long>(chunk) * KK * C;
#pragma unroll
    for (int ty = 0; ty < K; ++ty) {
        if (ty) __syncthreads();
        if (pb_local < p.blocks_per_wg) {
#pragma unroll
            for (int tx = 0; tx < K; ++tx)
#pragma unroll
                for (int v = 0; v < CV; ++v) lds[(pb_local * K + tx) * width + CV * lane_c + v] = lane_ok ? acc[ty * K + tx][v] : 0.f;
        }
        __syncthreads();
        for (int e = threadIdx.x; e < K * nch; e += blockDim.x) {
            const int tx = e / nch, cl = e - tx * nch;
            float sum = 0.f;
            for (int q = 0; q < p.blocks_per_wg; ++q) sum += lds[(q * K + tx) * width + cl];
            out[static_cast<long>(ty * K + tx) * C + c0 + cl] = sum;
        }
    }
}

// Grad-weight, pass 2: gw[c][t] = sum over chunks of partial[chunk][t][c].  16 lanes per output add contiguous
// sixteenths of the chunks in fp64; the sixteen sums are then added in order: bit-identical from run to run.
constexpr int kNhwcFinalParts = 16;
template <typename T>
__global__ __launch_bounds__(256) void nhwc_wgrad_final_kernel(const float *__restrict__ partial, T *__restrict__ gw,
                                                               const int channel, const int taps, const int chunks)
{
    __shared__ double red[kNhwcFinalParts][16];
    const int el = threadIdx.x & 15, part = threadIdx.x >> 4;
    const int e = blockIdx.x * 16 + el;  // e = t * C + c: neighbouring lanes read neighbouring floats
    const bool live = e < channel * taps;
    const long stride = static_cast<long>(channel) * taps;
    const int per = (chunks + kNhwcFinalParts - 1) / kNhwcFinalParts;
    const int k0 = part * per, k1 = min(chunks, k0 + per);
    const float *src = partial + (live ? e : 0);
    double s = 0.0;
    // eight loads at a time, the ones past this lane's share replaced by zero (never a one-by-one tail)
    for (int k = k0; k < k1; k += 8) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = src[min(k + j, k1 - 1) * stride];
#pragma unroll
        for (int j = 0; j < 8; ++j) s += static_cast<double>(k + j < k1 ? v[j] : 0.f);
    }
    red[part][el] = s;
    __syncthreads();
    if (part == 0 && live) {
        double total = 0.0;
#pragma unroll
        for (int q = 0; q < kNhwcFinalParts; ++q) total += red[q][el];
        const int t = e / channel, c = e - t * channel;
        gw[static_cast<long>(c) * taps + t] = Io<T>::out(static_cast<typename Io<T>::acc_t>(total));
    }
}

// ---- one lane per element: any geometry, any element type ------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void nhwc_fwd_direct_kernel(const T *__restrict__ in, const T *__restrict__ taps,
                                                              T *__restrict__ out, const NhwcGeometry g, const long total)
{
    using acc_t = typename Io<T>::acc_t;
    const long e = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (e >= total) return;
    const int c = static_cast<int>(e % g.channel);
    long r = e / g.channel;
    const int ox = static_cast<int>(r % g.out_w);
    r /= g.out_w;
    const int oy = static_cast<int>(r % g.out_h);
    const long n = r / g.out_h;
    acc_t s = 0;
    for (int ty = 0; ty < g.kernel_h; ++ty) {
        const int iy = oy * g.stride_h - g.pad_h + ty;
        if (iy < 0 || iy >= g.in_h) continue;
        for (int tx = 0; tx < g.kernel_w; ++tx) {
            const int ix = ox * g.stride_w - g.pad_w + tx;
            if (ix < 0 || ix >= g.in_w) continue;
            s += static_cast<acc_t>(Io<T>::in(in[((n * g.in_h + iy) * g.in_w + ix) * g.channel + c])) *
                 static_cast<acc_t>(Io<T>::in(taps[(static_cast<long>(c) * g.kernel_h + ty) * g.kernel_w + tx]));
        }
    }
    if (g.epi.enabled()) s = epilogue_apply(s, g.epi, c);
    out[e] = Io<T>::out(s);
}

template <typename T>
__global__ __launch_bounds__(256) void nhwc_gx_direct_kernel(const T *__restrict__ gy, const T *__restrict__ taps,
                                                             T *__restrict__ gx, const NhwcGeometry g, const long total)
{
    using acc_t = typename Io<T>::acc_t;
    const long e = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (e >= total) return;
    const int c = static_cast<int>(e % g.channel);
    long r = e / g.channel;
    const int ix = static_cast<int>(r % g.in_w);
    r /= g.in_w;
    const int iy = static_cast<int>(r % g.in_h);
    const long n = r / g.in_h;
    acc_t s = 0;
    for (int ty = 0; ty < g.kernel_h; ++ty) {
        const int ny = iy + g.pad_h - ty;
        if (ny < 0 || ny % g.stride_h != 0) continue;
        const int oy = ny / g.stride_h;
        if (oy >= g.out_h) continue;
        for (int tx = 0; tx < g.kernel_w; ++tx) {
            const int nx = ix + g.pad_w - tx;
            if (nx < 0 || nx % g.stride_w != 0) continue;
            const int ox = nx / g.stride_w;
            if (ox >= g.out_w) continue;
            s += static_cast<acc_t>(Io<T>::in(gy[((n * g.out_h + oy) * g.out_w + ox) * g.channel + c])) *
                 static_cast<acc_t>(Io<T>::in(taps[(static_cast<long>(c) * g.kernel_h + ty) * g.kernel_w + tx]));
        }
    }
    gx[e] = Io<T>::out(s);
}

// partial[chunk][t][c]: lane = (t, c) with c fastest, loops over the output pixels of its chunk.
template <typename T>
__global__ __launch_bounds__(256) void nhwc_gw_direct_kernel(const T *__restrict__ x, const T *__restrict__ gy,
                                                             float *__restrict__ partial_f, const NhwcGeometry g,
                                                             const long pixels, const int chunks)
{
    using acc_t = typename Io<T>::acc_t;
    acc_t *partial = reinterpret_cast<acc_t *>(partial_f);
    const int taps = g.kernel_h * g.kernel_w;
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= taps * g.channel) return;
    const int t = e / g.channel, c = e - t * g.channel;
    const int ty = t / g.kernel_w, tx = t - ty * g.kernel_w;
    const int chunk = blockIdx.y;
    const long per = (pixels + chunks - 1) / chunks;
    const long p0 = chunk * per, p1 = min(pixels, p0 + per);
    acc_t s = 0;
    for (long q = p0; q < p1; ++q) {
        const int ox = static_cast<int>(q % g.out_w);
        const long r = q / g.out_w;
        const int oy = static_cast<int>(r % g.out_h);
        const long n = r / g.out_h;
        const int iy = oy * g.stride_h - g.pad_h + ty, ix = ox * g.stride_w - g.pad_w + tx;
        if (iy < 0 || iy >= g.in_h || ix < 0 || ix >= g.in_w) continue;
        s += static_cast<acc_t>(Io<T>::in(gy[q * g.channel + c])) *
             static_cast<acc_t>(Io<T>::in(x[((n * g.in_h + iy) * g.in_w + ix) * g.channel + c]));
    }
    partial[static_cast<long>(chunk) * taps * g.channel + e] = s;
}

template <typename T>
__global__ __launch_bounds__(256) void nhwc_gw_direct_final_kernel(const float *__restrict__ partial_f, T *__restrict__ gw,
                                                                   const int channel, const int taps, const int chunks)
{
    using acc_t = typename Io<T>::acc_t;
    const acc_t *partial = reinterpret_cast<const acc_t *>(partial_f);
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= channel * taps) return;
    const int t = e / channel, c = e - t * channel;
    double s = 0.0;
    for (int k = 0; k < chunks; ++k) s += static_cast<double>(partial[static_cast<long>(k) * channel * taps + e]);
    gw[static_cast<long>(c) * taps + t] = Io<T>::out(static_cast<acc_t>(s));
}

// ---- planning -------------------------------------------------------------------------------------------
// Channel lanes per workgroup, at most `cap`.  All of C when it fits (then the pixels of a row are one contiguous
// run).  Otherwise a multiple of `line` lanes (= one 128-byte line of fp32 channels), so that every pixel's
// segment starts and ends on a line: the count under the cap that leaves the fewest lanes of the last channel
// group idle (none when it divides `lanes` = C / CV).  A segment that is not whole lines makes
// every load fetch the lines at its ends in full (C = 240 in groups of 60 channels: 240-byte segments cost
// 384 bytes of L1-to-L2 requests each, and the 28x28 layers ran 1.3-1.6 x slower than with 128-byte ones).
int pick_lanes_c(int lanes, int cap, int line)
{
    if (lanes <= cap) return lanes;
    if (line > 1 && cap >= line) {
        // the count that leaves the fewest idle lanes in the last group; the larger one on a tie
        int best = line, best_padded = (lanes + line - 1) / line * line;
        for (int d = 2 * line; d <= cap; d += line) {
            const int padded = (lanes + d - 1) / d * d;
            if (padded <= best_padded) {
                best = d;
                best_padded = padded;
            }
        }
        return best;
    }
    int best = 1;
    for (int d = cap; d >= 1; --d)
        if (lanes % d == 0) {
            best = d;
            break;
        }
    return best >= 8 ? best : cap;
}

template <int K, int CV>
bool plan_nhwc(NhwcPlan &p, const NhwcGeometry &g, int bh, int tw, int blocks_h, int blocks_w, int min_lanes = 1,
               const char *lanes_env = "DWCONV_NHWC_LANES", int exact_lanes = 0)
{
    p.batch = g.batch;
    p.channel = g.channel;
    // Few channel lanes per workgroup make its pixel blocks cover a compact patch of the image (or whole small
    // images), so halo pixels are shared inside the workgroup's L1 instead of between workgroups.  Measured on
    // the EfficientNet-B0 layers: 8 lanes win on 7x7 and 14x14 maps, 16 on 28x28, 64 on larger ones.
    const long pixels = static_cast<long>(g.in_h) * g.in_w;
    // (large maps: all of C when a workgroup still holds two pixel blocks of it, e.g. C = 144 with two channels
    // per lane: whole-C workgroups of 72 lanes beat 16-lane groups by 8-15 % on the 56x56 grad-weight kernels)
    int cap = pixels <= 256 ? 8 : pixels <= 1024 ? 16 : 256 / CV;
    cap = env_int(lanes_env, std::max(cap, min_lanes));
    cap = std::max(1, std::min(cap, 128));
    while (cap > 1 && static_cast<size_t>(cap) * CV * K * K * 4 > static_cast<size_t>(kNhwcTapLds)) --cap;
    p.lanes_c = pick_lanes_c(g.channel / CV, cap, env_int("DWCONV_NHWC_ALIGN", 1) ? 32 / CV : 1);
    if (exact_lanes > 0 && !env_set(lanes_env) && (g.channel / CV) % exact_lanes == 0) p.lanes_c = exact_lanes;
    p.lanes_c_magic = magic_u16(p.lanes_c);
    p.blocks_per_wg = kNhwcThreads / p.lanes_c;
    p.blocks_y = ceil_div(blocks_h, bh);
    p.blocks_x = ceil_div(blocks_w, tw);
    p.blocks_total = static_cast<long>(g.batch) * p.blocks_y * p.blocks_x;
    // every view starts at the first image of a workgroup's pixel blocks and must reach its last one below kOob
    {
        const long per_image = static_cast<long>(p.blocks_y) * p.blocks_x;
        const long span = (p.blocks_per_wg - 1) / per_image + 2;
        const long image = std::max(static_cast<long>(g.in_h) * g.in_w, static_cast<long>(g.out_h) * g.out_w) * g.channel * 4;
        if (image * span >= 0x80000000l) return false;
    }
    p.cgroups = ceil_div(g.channel / CV, p.lanes_c);
    const long wgs = (p.blocks_total + p.blocks_per_wg - 1) / p.blocks_per_wg * p.cgroups;
    if (p.blocks_total <= 0 || p.cgroups > 65535 || wgs > 0x7fffffffL) return false;
    p.wgs = static_cast<int>(wgs);
    return true;
}

bool nhwc_fast_ok(const NhwcGeometry &g)
{
    if (env_int("DWCONV_FORCE_GENERIC", 0) || env_int("DWCONV_NO_NHWC_FAST", 0)) return false;
    const int K = g.kernel_h;
    if (g.kernel_w != K || (K != 3 && K != 5 && K != 7)) return false;
    if (g.stride_h != g.stride_w || (g.stride_h != 1 && g.stride_h != 2)) return false;
    if (g.channel % 4 != 0) return false;
    if (g.pad_h < 0 || g.pad_w < 0 || g.pad_h >= K || g.pad_w >= K) return false;
    if (g.in_h < 1 || g.in_w < 1 || g.out_h < 1 || g.out_w < 1) return false;
    return true;
}

template <typename IO, int K, int S, bool FLIP, int BH = 4, int TW = 4, int CV = 4>
int launch_nhwc_down(const IO *in, const IO *taps, IO *out, const NhwcGeometry &g, int in_h, int in_w, int out_h,
                     int out_w, int pad_h, int pad_w, hipStream_t stream)
{
    if constexpr (BH == 4 && TW == 4 && CV == 4) {
        if constexpr (K == 5 && S == 1 && sizeof(IO) == 4 && !FLIP) {
            // 5x5 stride 1 on maps of 14 or 28 rows: one channel per lane and 7 x 8 blocks fetch 2.4 input pixels per
            // result instead of 4 (14x14 C=480 31.5 -> 27.1 us, 28x28 C=240 60.5 -> 59.2, 14x14 C=672 unchanged; 7x7
            // maps lose 1.5 us, and 7 x 4 or 4 x 8 blocks with one or two channels per lane lose 3-10 us everywhere)
            const bool fits = out_h % 7 == 0 && out_h >= 14 && g.channel % 32 == 0;
            if (env_int("DWCONV_NHWC_K5_7X8", fits))
                return launch_nhwc_down<IO, K, S, FLIP, 7, 8, 1>(in, taps, out, g, in_h, in_w, out_h, out_w, pad_h, pad_w, stream);
        }
        if constexpr (K > 3) {
            // 5x5 stride 2 onto maps of fewer than 28 rows: twice the lanes with 4 x 2 blocks (14x14 C=672 25.7 -> 21.7 us)
            if (env_int("DWCONV_NHWC_TW", !FLIP && K == 5 && S == 2 && out_h < 28 ? 2 : 4) == 2)
                return launch_nhwc_down<IO, K, S, FLIP, 4, 2, 4>(in, taps, out, g, in_h, in_w, out_h, out_w, pad_h, pad_w, stream);
        }
        // Blocks of 7 x 2 pixels (the registers of 4 x 4) halve the halo rows a lane fetches per output row.  Forward
        // fp32, where seven rows divide the map or it is large: 3x3 stride 1 (112x112 C=32 83.0 -> 80.4 us, 14x14 C=480
        // 23.7 -> 21.2, 56x56 C=144 and 7x7 C=1152 unchanged) and 5x5 stride 2 on maps of 28 rows and more (56x56
        // C=144 72.2 -> 66.5; 14x14 C=672 is 2 us slower with them).  One or two channels per lane with 7 x 8, 7 x 4,
        // 4 x 8 or 4 x 4 blocks won on single layers and lost on others (1.68-1.74 ms per step against 1.67).
        if constexpr (!FLIP && ((K == 3 && S == 1) || (K == 5 && S == 2))) {
            // (16-bit elements: 5x5 stride 2 alike, 56x56 C=144 54.2 -> 48.1 us; 3x3 stride 1 only on maps of 14 to 28 rows,
            // 14x14 C=480 19.9 -> 17.1, while 56x56 C=144 and 7x7 C=1152 lose 6 and 1.5 us with them)
            const bool tall = sizeof(IO) == 4 ? (out_h % 7 == 0 || out_h >= 56) && (K == 3 || out_h >= 28)
                                              : (K == 5 ? out_h >= 28 : out_h % 7 == 0 && out_h >= 14 && out_h <= 28);
            if (env_int("DWCONV_NHWC_DOWN_7X2", tall))
                return launch_nhwc_down<IO, K, S, FLIP, 7, 2, 4>(in, taps, out, g, in_h, in_w, out_h, out_w, pad_h, pad_w, stream);
        }
    }
    NhwcPlan p{};
    const int line_lanes = CV == 4 ? 1 : static_cast<int>(128 / (CV * sizeof(IO)));
    if (!plan_nhwc<K, CV>(p, g, BH, TW, out_h, out_w, line_lanes)) return -1;
    p.in = in;
    p.taps = taps;
    p.out = out;
    if (!FLIP) p.epi = g.epi;
    p.in_h = in_h;
    p.in_w = in_w;
    p.out_h = out_h;
    p.out_w = out_w;
    p.pad_h = pad_h;
    p.pad_w = pad_w;
    const dim3 grid(p.wgs);
    const size_t shmem = static_cast<size_t>(p.lanes_c) * CV * K * K * 4;
    hipLaunchKernelGGL((nhwc_down_kernel<IO, K, S, FLIP, BH, TW, CV>), grid, dim3(kNhwcThreads), shmem, stream, p);
    note_variant("nhwc_down%s<k%d,s%d,%s,%dx%d%s> lanes_c%d", sizeof(IO) == 2 ? "16" : "", K, S, FLIP ? "rot" : "fwd", BH, TW,
                 CV == 4 ? "" : (CV == 2 ? ",cv2" : ",cv1"), p.lanes_c);
    return check_launch("nhwc_down_kernel");
}

template <typename IO, int K, int PE>
int launch_nhwc_up2(const IO *gy, const IO *taps, IO *gx, const NhwcGeometry &g, hipStream_t stream)
{
    constexpr int BH = 4, TW = K == 3 ? 4 : 2;
    NhwcPlan p{};
    if (!plan_nhwc<K, 4>(p, g, BH, TW, g.in_h, g.in_w)) return -1;
    p.in = gy;
    p.taps = taps;
    p.out = gx;
    p.in_h = g.out_h;
    p.in_w = g.out_w;
    p.out_h = g.in_h;
    p.out_w = g.in_w;
    p.pad_h = g.pad_h / 2;
    p.pad_w = g.pad_w / 2;
    const dim3 grid(p.wgs);
    const size_t shmem = static_cast<size_t>(p.lanes_c) * 4 * K * K * 4;
    hipLaunchKernelGGL((nhwc_up2_kernel<IO, K, PE, BH, TW>), grid, dim3(kNhwcThreads), shmem, stream, p);
    note_variant("nhwc_up2%s<k%d,e%d,%dx%d> lanes_c%d", sizeof(IO) == 2 ? "16" : "", K, PE, BH, TW, p.lanes_c);
    return check_launch("nhwc_up2_kernel");
}

template <int K>
struct WgradShape {
    // K*K*CV sums live in registers: 36 for 3x3 with four channels per lane, 50 / 98 with two for 5x5 / 7x7
    static constexpr int CV = K == 3 ? 4 : 2;
    // Seven output rows per block for 3x3 and 5x5: the K - 1 halo rows of x are fetched for seven rows instead of
    // four (fewer L1-to-L2 requests, which is what bounds these kernels; -2 % on the EfficientNet-B0 step), and 7
    // divides the map heights of the usual networks.  Only the rows of out_grad in use are live, so the block
    // height costs no registers.  The 7x7 kernel is bound by its arithmetic and runs faster with two rows.
    static constexpr int BH = K == 7 ? 2 : 7;
    static constexpr int TW = 4;
};

// mode 0: workspace bytes; mode 1: launch.  -1 when the fast kernel does not cover g.
template <typename IO, int K, int S>
long nhwc_wgrad_case(int mode, const IO *x, const IO *gy, IO *gw, void *ws, size_t ws_bytes, const NhwcGeometry &g,
                     hipStream_t stream)
{
    constexpr int CV = WgradShape<K>::CV, BH = WgradShape<K>::BH, TW = WgradShape<K>::TW;
    NhwcPlan p{};
    // At least a 128-byte line of every pixel per workgroup: with fewer channel lanes the other part of the line
    // belongs to another workgroup, on another XCD as likely as not, and is fetched from HBM twice (measured on the
    // 5x5 layers, which run two channels per lane: 2.2 x the bytes of x and gy).  The forward and grad-input
    // kernels (four channels per lane) already cover a line in fp32 and did not gain from it with 16-bit elements.
    const int line_lanes = env_int("DWCONV_NHWC_FULL_LINES", 1) ? static_cast<int>(128 / (CV * sizeof(IO))) : 1;
    if (!plan_nhwc<1, CV>(p, g, BH, TW, g.out_h, g.out_w, line_lanes, "DWCONV_NHWC_WGRAD_LANES")) return -1;
    const int cgroups = p.cgroups;
    const long wg_iters = (p.blocks_total + p.blocks_per_wg - 1) / p.blocks_per_wg;
    // One resident round of workgroups: the kernel's 170-250 registers leave two wavefronts per SIMD, i.e. two
    // 256-lane workgroups on each of the 256 CUs (measured: 512 beats 256, 384, 640, 768 and 1024 by 3-10 %).
    // (16-bit elements, 5x5 stride 2: 768 take the 56x56 C=144 backward from 113.6 to 105.8 us and leave 14x14 C=672 alone;
    // every other instance of this kernel loses 3-7 us with 768)
    long groups = env_int("DWCONV_NHWC_WGRAD_WGS", sizeof(IO) == 2 && K == 5 && S == 2 ? 768 : 512) / cgroups;
    groups = std::max(1l, std::min(groups, wg_iters));
    p.groups = static_cast<int>(groups);
    p.xcd_chunks = env_int("DWCONV_NHWC_XCD_CHUNKS", 0);
    const size_t need = static_cast<size_t>(groups) * K * K * g.channel * sizeof(float);
    if (mode == 0) return static_cast<long>(need);
    if (ws == nullptr || ws_bytes < need)
        return fail(DWCONV_ERR_WORKSPACE, "grad-weight needs a workspace of %zu bytes, got %zu", need, ws_bytes);
    p.in = x;
    p.in2 = gy;
    p.partial = static_cast<float *>(ws);
    p.in_h = g.in_h;
    p.in_w = g.in_w;
    p.out_h = g.out_h;
    p.out_w = g.out_w;
    p.pad_h = g.pad_h;
    p.pad_w = g.pad_w;
    const size_t shmem = static_cast<size_t>(p.blocks_per_wg) * K * p.lanes_c * CV * 4;
    hipLaunchKernelGGL((nhwc_wgrad_kernel<IO, K, S, CV, BH, TW>), dim3(p.groups * cgroups), dim3(kNhwcThreads), shmem, stream, p);
    int rc = check_launch("nhwc_wgrad_kernel");
    if (rc != DWCONV_OK) return rc;
    note_variant("nhwc_wgrad%s<k%d,s%d,cv%d,%dx%d> lanes_c%d chunks%d", sizeof(IO) == 2 ? "16" : "", K, S, CV, BH, TW,
                 p.lanes_c, p.groups);
    hipLaunchKernelGGL(nhwc_wgrad_final_kernel<IO>, dim3(ceil_div(g.channel * K * K, 16)), dim3(256), 0, stream,
                       p.partial, gw, g.channel, K * K, p.groups);
    return check_launch("nhwc_wgrad_final_kernel");
}

template <typename IO>
long nhwc_wgrad_fast(int mode, const IO *x, const IO *gy, IO *gw, void *ws, size_t ws_bytes, const NhwcGeometry &g,
                     hipStream_t stream)
{
    if (!nhwc_fast_ok(g)) return -1;
    const int K = g.kernel_h, S = g.stride_h;
#define DWCONV_NHWC_WGRAD(KV, SV) \
    if (K == KV && S == SV) return nhwc_wgrad_case<IO, KV, SV>(mode, x, gy, gw, ws, ws_bytes, g, stream);
    DWCONV_NHWC_WGRAD(3, 1)
    DWCONV_NHWC_WGRAD(3, 2)
    DWCONV_NHWC_WGRAD(5, 1)
    DWCONV_NHWC_WGRAD(5, 2)
    DWCONV_NHWC_WGRAD(7, 1)
    DWCONV_NHWC_WGRAD(7, 2)
#undef DWCONV_NHWC_WGRAD
    return -1;
}

// Fused backward of K x K stride-1 layers with pad K/2: CV channels per lane, BH x TW results per lane.
// mode 0: workspace bytes; mode 1: launch.  -1 when the kernel does not cover g.
template <typename IO, int K, int CV = 2, int BH = 7, int TW = 4>
long nhwc_bwd_fused_case(int mode, const IO *x, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes,
                         const NhwcGeometry &g, hipStream_t stream)
{
    NhwcPlan p{};
    const int line_lanes = static_cast<int>(128 / (CV * sizeof(IO)));
    if (!plan_nhwc<K, CV>(p, g, BH, TW, g.out_h, g.out_w, line_lanes, "DWCONV_NHWC_WGRAD_LANES")) return -1;
    const int cgroups = p.cgroups;
    const long wg_iters = (p.blocks_total + p.blocks_per_wg - 1) / p.blocks_per_wg;
    // Workgroups per chip: a multiple of the 256 compute units (576-704 and 800-896 are 5-25 % slower than 512 or
    // 768).  The 5x5 kernel holds three workgroups per unit and is bound by its own arithmetic, so a third
    // resident workgroup hides more latency (7x7 C=1152 40.4 -> 36.1 us, 14x14 C=672 69.6 -> 61.0, C=480 51.2 ->
    // 49.0, 28x28 C=240 91.9 -> 90.1); the 3x3 kernels wait for memory and lose 3-20 % with more than two.
    // The two-channel 3x3 instance (168 registers, three workgroups per unit; what 16-bit tensors run) takes 768 as well:
    // bf16 7x7 C=1152 23.7 -> 18.6 us, 56x56 C=144 94.2 -> 90.6, 112x112 C=32 72.6 -> 70.3, 14x14 C=480 30.0 -> 31.4.
    long groups = env_int("DWCONV_NHWC_WGRAD_WGS", K == 5 || CV == 2 ? 768 : 512) / cgroups;
    groups = std::max(1l, std::min(groups, wg_iters));
    p.groups = static_cast<int>(groups);
    p.xcd_chunks = env_int("DWCONV_NHWC_XCD_CHUNKS", 0);
    const size_t need = static_cast<size_t>(groups) * K * K * g.channel * sizeof(float);
    if (mode == 0) return static_cast<long>(need);
    if (ws == nullptr || ws_bytes < need)
        return fail(DWCONV_ERR_WORKSPACE, "backward needs a workspace of %zu bytes, got %zu", need, ws_bytes);
    p.in = x;
    p.in2 = gy;
    p.taps = taps;
    p.out = gx;
    p.partial = static_cast<float *>(ws);
    p.in_h = g.in_h;
    p.in_w = g.in_w;
    p.out_h = g.out_h;
    p.out_w = g.out_w;
    p.pad_h = g.pad_h;
    p.pad_w = g.pad_w;
    const size_t shmem = static_cast<size_t>(p.lanes_c) * CV * 4 * std::max(K * K, p.blocks_per_wg * K);
    hipLaunchKernelGGL((nhwc_bwd_fused_kernel<IO, K, CV, BH, TW>), dim3(p.groups * cgroups), dim3(kNhwcThreads), shmem, stream, p);
    int rc = check_launch("nhwc_bwd_fused_kernel");
    if (rc != DWCONV_OK) return rc;
    note_variant("nhwc_bwd%s<k%d,s1,cv%d,%dx%d> lanes_c%d chunks%d", sizeof(IO) == 2 ? "16" : "", K, CV, BH, TW, p.lanes_c, p.groups);
    hipLaunchKernelGGL(nhwc_wgrad_final_kernel<IO>, dim3(ceil_div(g.channel * K * K, 16)), dim3(256), 0, stream,
                       p.partial, gw, g.channel, K * K, p.groups);
    return check_launch("nhwc_wgrad_final_kernel");
}

// Fused backward of K x K stride-2 layers with pad K/2 and even input extents.  mode 0: workspace bytes; mode 1:
// launch.  -1 when the kernel does not cover g.
template <typename IO, int K, int CV, int BQH, int BQW>
long nhwc_bwd_s2_fused_case(int mode, const IO *x, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes,
                            const NhwcGeometry &g, hipStream_t stream)
{
    NhwcPlan p{};
    const int line_lanes = static_cast<int>(128 / (CV * sizeof(IO)));
    // C = 144 (4.5 lines per pixel) with the 5x5 kernel: three groups of 48 channels, 192-byte segments that start on
    // 64-byte boundaries, instead of five groups of 32 whose last is half idle (56x56: 135.8 -> 129.5 us).  The other
    // kernels, and C = 240 in groups of 48 or 80, are 1-4 us slower than with 32.
    const int lanes48 = K == 5 && CV == 1 && g.channel % 32 != 0 && g.channel % 48 == 0 ? 48 : 0;
    if (!plan_nhwc<K, CV>(p, g, BQH, BQW, g.out_h, g.out_w, line_lanes, "DWCONV_NHWC_WGRAD_LANES", lanes48)) return -1;
    const int cgroups = p.cgroups;
    const long wg_iters = (p.blocks_total + p.blocks_per_wg - 1) / p.blocks_per_wg;
    // three workgroups per compute unit for the 5x5 kernel on small maps (14x14 C=672 48.8 -> 43.8 us), two
    // elsewhere (56x56 C=144 is 5 % slower with three)
    const bool small_map = K == 5 && static_cast<long>(g.out_h) * g.out_w <= 196;
    long groups = env_int("DWCONV_NHWC_WGRAD_WGS", small_map ? 768 : 512) / cgroups;
    groups = std::max(1l, std::min(groups, wg_iters));
    p.groups = static_cast<int>(groups);
    // Workgroups whose pixel blocks share halo rows run at the same time.  Dealt round-robin to the XCDs, they fetch
    // those rows into several L2s; in contiguous runs per XCD the 5x5 kernel on large maps fetches less (56x56 C=144
    // 139.3 -> 135.7 us).  Every other backward kernel is 1-4 us slower that way.
    p.xcd_chunks = env_int("DWCONV_NHWC_XCD_CHUNKS", K == 5 && !small_map);
    const size_t need = static_cast<size_t>(groups) * K * K * g.channel * sizeof(float);
    if (mode == 0) return static_cast<long>(need);
    if (ws == nullptr || ws_bytes < need)
        return fail(DWCONV_ERR_WORKSPACE, "backward needs a workspace of %zu bytes, got %zu", need, ws_bytes);
    p.in = x;
    p.in2 = gy;
    p.taps = taps;
    p.out = gx;
    p.partial = static_cast<float *>(ws);
    p.in_h = g.in_h;
    p.in_w = g.in_w;
    p.out_h = g.out_h;
    p.out_w = g.out_w;
    p.pad_h = g.pad_h;
    p.pad_w = g.pad_w;
    const size_t shmem = static_cast<size_t>(p.lanes_c) * CV * 4 * std::max(K * K, p.blocks_per_wg * K);
    hipLaunchKernelGGL((nhwc_bwd_s2_fused_kernel<IO, K, CV, BQH, BQW>), dim3(p.groups * cgroups), dim3(kNhwcThreads), shmem, stream, p);
    int rc = check_launch("nhwc_bwd_s2_fused_kernel");
    if (rc != DWCONV_OK) return rc;
    note_variant("nhwc_bwd%s<k%d,s2,cv%d,%dx%d> lanes_c%d chunks%d", sizeof(IO) == 2 ? "16" : "", K, CV, BQH, BQW, p.lanes_c, p.groups);
    hipLaunchKernelGGL(nhwc_wgrad_final_kernel<IO>, dim3(ceil_div(g.channel * K * K, 16)), dim3(256), 0, stream,
                       p.partial, gw, g.channel, K * K, p.groups);
    return check_launch("nhwc_wgrad_final_kernel");
}

bool nhwc_fused_s2_ok(const NhwcGeometry &g)
{
    if (!env_int("DWCONV_NHWC_FUSED_S2", 1) || !env_int("DWCONV_NHWC_FUSED_BWD", 1) || !nhwc_fast_ok(g)) return false;
    const int K = g.kernel_h;
    return (K == 3 || K == 5) && g.stride_h == 2 && g.pad_h == K / 2 && g.pad_w == K / 2 && g.in_h % 2 == 0 &&
           g.in_w % 2 == 0 && g.out_h == g.in_h / 2 && g.out_w == g.in_w / 2;
}

bool nhwc_fused_ok(const NhwcGeometry &g)
{
    if (!env_int("DWCONV_NHWC_FUSED_BWD", 1) || !nhwc_fast_ok(g)) return false;
    const int K = g.kernel_h;
    return (K == 3 || K == 5) && g.stride_h == 1 && g.pad_h == K / 2 && g.pad_w == K / 2 && g.out_h == g.in_h &&
           g.out_w == g.in_w;
}

template <typename IO>
long nhwc_bwd_fused(int mode, const IO *x, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes,
                    const NhwcGeometry &g, hipStream_t stream)
{
    if (nhwc_fused_s2_ok(g)) {
        // One fp32 channel per lane, as for the 5x5 stride-1 kernel: blocks of 7 x 4 out_grad pixels for 3x3 filters
        // (95 registers; 112x112 C=96: 274 -> 257 us against the two separate kernels, 28x28 C=240: 56 -> 56), 4 x 2 for
        // 5x5 (157 registers; 56x56 C=144: 147 -> 137 us, 14x14 C=672: 49 -> 48).  Measured and left out: two channels
        // per lane with 4 x 2 or 7 x 2 blocks (3x3: 260-268 and 63 us; 5x5: 251 registers, 141 and 53 us), four channels
        // with 2 x 2 blocks (186 registers, 260 and 64 us), 7 x 4 blocks for 5x5 (256 registers: twice the time).
        // 16-bit elements (two channels per 4-byte access) stay on the separate kernels.
        if constexpr (sizeof(IO) == 4) {
            if (g.kernel_h == 3) return nhwc_bwd_s2_fused_case<IO, 3, 1, 7, 4>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
            return nhwc_bwd_s2_fused_case<IO, 5, 1, 4, 2>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
        }
        return -1;
    }
    if (!nhwc_fused_ok(g)) return -1;
    if (g.kernel_h == 5) {
        // 25 sums per channel: with two channels per lane the kernel needs 228 registers (7 x 2 blocks) to 262 (4 x 4)
        // and loses to the two separate kernels; with ONE fp32 channel per lane (dword accesses, 32 lanes per
        // 128-byte line) it fits 167 registers with 7 x 4 blocks, three wavefronts per SIMD, and wins on every 5x5
        // layer of the stack (28x28 C=240: 112 -> 91 us, 14x14 C=672: 75 -> 68, C=480: 59 -> 50, 7x7 C=1152: 42 -> 39).
        // 16-bit elements (two channels per 4-byte access) stay on the separate kernels.
        if constexpr (sizeof(IO) == 4) {
            if (env_int("DWCONV_NHWC_FUSED5", 1))
                return nhwc_bwd_fused_case<IO, 5, 1, 7, 4>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
        }
        return -1;
    }
    if constexpr (sizeof(IO) == 4) {
        // fp32, 3x3: one channel per lane and 7 x 8 pixel blocks where C is whole groups of 32 lanes (a 128-byte line
        // of every pixel per group), four channels per lane and 7 x 2 blocks otherwise (C = 144: 36 lanes).  Against
        // two channels per lane and 7 x 4 blocks: 112x112 C=32 125.5 -> 120.6 us, 14x14 C=480 40.0 -> 35.8, 7x7 C=1152
        // 29.7 -> 27.1, 56x56 C=144 155.7 -> 149.8 (one channel per lane there: 171-173, its fifth group is half empty).
        if (env_int("DWCONV_NHWC_F3_SHAPE", 1)) {
            if (g.channel % 32 == 0)
                return nhwc_bwd_fused_case<IO, 3, 1, 7, 8>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
            return nhwc_bwd_fused_case<IO, 3, 4, 7, 2>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
        }
    }
    return nhwc_bwd_fused_case<IO, 3>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
}

template <typename T>
int direct_chunks(const NhwcGeometry &g)
{
    const long pixels = static_cast<long>(g.batch) * g.out_h * g.out_w;
    return static_cast<int>(std::max(1l, std::min(256l, pixels / 64)));
}

template <typename T>
size_t nhwc_wgrad_direct_bytes(const NhwcGeometry &g)
{
    return static_cast<size_t>(direct_chunks<T>(g)) * g.kernel_h * g.kernel_w * g.channel * sizeof(typename Io<T>::acc_t);
}

}  // namespace

template <typename T>
int nhwc_forward(const T *in, const T *taps, T *out, const NhwcGeometry &g, hipStream_t stream)
{
    const long total = static_cast<long>(g.batch) * g.out_h * g.out_w * g.channel;
    if (total == 0) {
        note_variant("empty");
        return DWCONV_OK;
    }
    if constexpr (!std::is_same<T, double>::value) {
        if (nhwc_fast_ok(g) && aligned4(in) && aligned4(out)) {
            const int K = g.kernel_h, S = g.stride_h;
            int rc = -1;
#define DWCONV_NHWC_DOWN(KV, SV)                                                                                       \
    if (K == KV && S == SV)                                                                                            \
        rc = launch_nhwc_down<T, KV, SV, false>(in, taps, out, g, g.in_h, g.in_w, g.out_h, g.out_w, g.pad_h, g.pad_w, stream);
            DWCONV_NHWC_DOWN(3, 1)
            DWCONV_NHWC_DOWN(3, 2)
            DWCONV_NHWC_DOWN(5, 1)
            DWCONV_NHWC_DOWN(5, 2)
            DWCONV_NHWC_DOWN(7, 1)
            DWCONV_NHWC_DOWN(7, 2)
#undef DWCONV_NHWC_DOWN
            if (rc >= 0) return rc;
        }
    }
    if ((total + 255) / 256 > 0x7fffffffL) return fail(DWCONV_ERR_UNSUPPORTED, "tensor too large");
    hipLaunchKernelGGL(nhwc_fwd_direct_kernel<T>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, stream, in,
                       taps, out, g, total);
    note_variant("nhwc_fwd_direct");
    return check_launch("nhwc_fwd_direct_kernel");
}

template <typename T>
int nhwc_grad_input(const T *gy, const T *taps, T *gx, const NhwcGeometry &g, hipStream_t stream)
{
    const long total = static_cast<long>(g.batch) * g.in_h * g.in_w * g.channel;
    if (total == 0) {
        note_variant("empty");
        return DWCONV_OK;
    }
    if (static_cast<long>(g.batch) * g.out_h * g.out_w == 0) {
        note_variant("zero");
        return launch_fill_zero(gx, static_cast<size_t>(total) * sizeof(T), stream);
    }
    if constexpr (!std::is_same<T, double>::value) {
        if (nhwc_fast_ok(g) && aligned4(gy) && aligned4(gx)) {
            const int K = g.kernel_h, S = g.stride_h;
            int rc = -1;
            if (S == 1) {
                // the transposed problem is a stride-1 correlation with the rotated taps and pad K - 1 - pad
#define DWCONV_NHWC_ROT(KV)                                                                                            \
    if (K == KV)                                                                                                       \
        rc = launch_nhwc_down<T, KV, 1, true>(gy, taps, gx, g, g.out_h, g.out_w, g.in_h, g.in_w, KV - 1 - g.pad_h,     \
                                              KV - 1 - g.pad_w, stream);
                DWCONV_NHWC_ROT(3)
                DWCONV_NHWC_ROT(5)
                DWCONV_NHWC_ROT(7)
#undef DWCONV_NHWC_ROT
            } else if (((g.pad_h ^ g.pad_w) & 1) == 0) {  // one parity class serves both axes
                const int pe = g.pad_h & 1;
#define DWCONV_NHWC_UP2(KV)                                                                                            \
    if (K == KV) rc = pe ? launch_nhwc_up2<T, KV, 1>(gy, taps, gx, g, stream) : launch_nhwc_up2<T, KV, 0>(gy, taps, gx, g, stream);
                DWCONV_NHWC_UP2(3)
                DWCONV_NHWC_UP2(5)
                DWCONV_NHWC_UP2(7)
#undef DWCONV_NHWC_UP2
            }
            if (rc >= 0) return rc;
        }
    }
    if ((total + 255) / 256 > 0x7fffffffL) return fail(DWCONV_ERR_UNSUPPORTED, "tensor too large");
    hipLaunchKernelGGL(nhwc_gx_direct_kernel<T>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, stream, gy,
                       taps, gx, g, total);
    note_variant("nhwc_gx_direct");
    return check_launch("nhwc_gx_direct_kernel");
}

template <typename T>
size_t nhwc_grad_weight_workspace(const NhwcGeometry &g)
{
    size_t need = nhwc_wgrad_direct_bytes<T>(g);
    if constexpr (!std::is_same<T, double>::value) {
        const long fast = nhwc_wgrad_fast<T>(0, nullptr, nullptr, nullptr, nullptr, 0, g, nullptr);
        if (fast > 0 && static_cast<size_t>(fast) > need) need = static_cast<size_t>(fast);
        const long fused = nhwc_bwd_fused<T>(0, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, g, nullptr);
        if (fused > 0 && static_cast<size_t>(fused) > need) need = static_cast<size_t>(fused);
    }
    return need;
}

template <typename T>
int nhwc_grad_weight(const T *x, const T *gy, T *gw, void *ws, size_t ws_bytes, const NhwcGeometry &g, hipStream_t stream)
{
    const int taps = g.kernel_h * g.kernel_w;
    if (static_cast<long>(g.channel) * taps == 0) {
        note_variant("empty");
        return DWCONV_OK;
    }
    const long pixels = static_cast<long>(g.batch) * g.out_h * g.out_w;
    if (pixels == 0 || g.in_h == 0 || g.in_w == 0) {
        note_variant("zero");
        return launch_fill_zero(gw, static_cast<size_t>(g.channel) * taps * sizeof(T), stream);
    }
    if constexpr (!std::is_same<T, double>::value) {
        if (aligned4(x) && aligned4(gy)) {
            const long rc = nhwc_wgrad_fast<T>(1, x, gy, gw, ws, ws_bytes, g, stream);
            if (rc >= 0) return static_cast<int>(rc);
        }
    }
    const size_t need = nhwc_wgrad_direct_bytes<T>(g);
    if (ws == nullptr || ws_bytes < need)
        return fail(DWCONV_ERR_WORKSPACE, "grad-weight needs a workspace of %zu bytes, got %zu", need, ws_bytes);
    const int chunks = direct_chunks<T>(g);
    hipLaunchKernelGGL(nhwc_gw_direct_kernel<T>, dim3(ceil_div(taps * g.channel, 256), chunks), dim3(256), 0, stream, x, gy,
                       static_cast<float *>(ws), g, pixels, chunks);
    int rc = check_launch("nhwc_gw_direct_kernel");
    if (rc != DWCONV_OK) return rc;
    hipLaunchKernelGGL(nhwc_gw_direct_final_kernel<T>, dim3(ceil_div(taps * g.channel, 256)), dim3(256), 0, stream,
                       static_cast<const float *>(ws), gw, g.channel, taps, chunks);
    note_variant("nhwc_gw_direct chunks%d", chunks);
    return check_launch("nhwc_gw_direct_final_kernel");
}

// Both gradients of one layer in one sweep where nhwc_bwd_fused_kernel covers the geometry; -1 otherwise.
template <typename T>
int nhwc_backward_fused(const T *x, const T *gy, const T *taps, T *gx, T *gw, void *ws, size_t ws_bytes,
                        const NhwcGeometry &g, hipStream_t stream)
{
    if constexpr (!std::is_same<T, double>::value) {
        if (static_cast<long>(g.batch) * g.out_h * g.out_w * g.channel > 0 && aligned4(x) && aligned4(gy) && aligned4(gx))
            return static_cast<int>(nhwc_bwd_fused<T>(1, x, gy, taps, gx, gw, ws, ws_bytes, g, stream));
    }
    return -1;
}

#define DWCONV_INSTANTIATE(T)                                                                                          \
    template int nhwc_backward_fused<T>(const T *, const T *, const T *, T *, T *, void *, size_t, const NhwcGeometry &,    \
                                        hipStream_t);                                                                  \
    template int nhwc_forward<T>(const T *, const T *, T *, const NhwcGeometry &, hipStream_t);                        \
    template int nhwc_grad_input<T>(const T *, const T *, T *, const NhwcGeometry &, hipStream_t);                     \
    template size_t nhwc_grad_weight_workspace<T>(const NhwcGeometry &);                                               \
    template int nhwc_grad_weight<T>(const T *, const T *, T *, void *, size_t, const NhwcGeometry &, hipStream_t);
DWCONV_INSTANTIATE(float)
DWCONV_INSTANTIATE(double)
DWCONV_INSTANTIATE(half_t)
DWCONV_INSTANTIATE(bf16_t)
#undef DWCONV_INSTANTIATE

}  // namespace dwconv
