// LDS-tiled kernels for the forward and grad-input passes (element type fp32, fp16 or bf16; LDS and
// arithmetic are fp32).
//
// Work decomposition (one workgroup of 256 lanes = 4 wavefronts per tile):
//   tile  = P consecutive (n,c) planes x a band of output rows x the full width.
//           Large maps use P = 1 and several row bands per plane; maps small
//           enough use whole planes and P > 1, so a wavefront carries several
//           channels.
//   load  = the input band (with its halo rows) is fetched four elements per
//           load and scattered into an LDS image whose zero padding is materialised,
//           so the arithmetic below needs no bounds checks.
//   item  = a register block of BH x 4 outputs (2*BQ x 4 for the stride-2
//           transposed case) owned by one lane: per input row the lane reads
//           aligned float4s from LDS once and reuses them for every tap and
//           every output row that touches it.
// Both directions of the reference's up/FIR/down kernel
// (torch_dwconv/dwconv_kernel.cu:69-181) and its whole-plane kernel (:308-442)
// map onto two kernel templates:
//   fir_down_kernel: up = 1, decimation S in {1,2}; forward pass, and the
//                    grad-input pass of stride-1 layers (taps rotated).
//   fir_up2_kernel : up = 2, no decimation, taps rotated; grad-input of
//                    stride-2 layers, computed as four interleaved stride-1
//                    correlations (one per output parity) without ever
//                    forming the zero-stuffed intermediate.
#include <type_traits>
#include "dwconv_tile_common.hpp"

namespace dwconv {

namespace {

struct TilePlan {
    StageLayout st;
    const void *in;    // element type IO of the kernel template
    const void *taps;
    void *out;
    long planes;
    int channel;
    int out_h, out_w, out_plane;
    int row_shift;             // LDS row r of a tile holds input row (first row of the tile) - row_shift + r
    int rows_per_tile;         // output rows (down) or half-resolution rows (up) per tile
    int row_tiles;             // tiles per plane
    int planes_per_tile;
    int n_tiles;
    int ncb;                   // column blocks per row band
    unsigned ncb_magic;
    int items_per_plane;
    unsigned ipp_magic;
    int tap_base;              // float offset of the tap table in LDS
    int vec_out;               // 128-bit global stores are legal
    int lds_out;               // fir_down: results go back through LDS and out as one linear stream per plane
    int mult;                  // depth multiplier M (one plane per tile when > 1).  Forward: `channel` counts the output's
                               // channels and output plane (n, c) reads input plane (n, c / M); backward (taps rotated):
                               // `channel` counts the result's channels and plane (n, c) adds up the M planes
                               // (n, c * M + m) of the operand, each with the taps of its own channel
    Epilogue epi;              // forward kernels: applied to every sum before it is stored
    // fir_any_kernel: filter extent, decimation and dilation per axis, and whether the taps are rotated
    int kh, kw, sh, sw, dh, dw, flip;
};

// Copies the tap tables of the tile's planes into LDS, rotated by 180 degrees if FLIP.
template <typename IO, int KK, bool FLIP>
__device__ __forceinline__ void stage_taps(const TilePlan &p, float *lds, long plane0, int nplanes, int channels)
{
    for (int i = threadIdx.x; i < nplanes * KK; i += blockDim.x) {
        const int pl = i / KK, t = i - pl * KK;
        const int c = static_cast<int>((plane0 + pl) % channels);
        lds[p.tap_base + i] = Io<IO>::in(static_cast<const IO *>(p.taps)[c * KK + (FLIP ? KK - 1 - t : t)]);
    }
}

// up = 1, decimation S.  out[oy,ox] = sum_{ty,tx} in[oy*S - pad_h0 + ty, ox*S - pad_w0 + tx] * f[ty,tx].
// ANY_WIDTH: the instance for rows that are not whole, aligned groups of four elements (vec_in or vec_out == 3).
template <typename IO, int K, int S, bool FLIP, int BH, bool ANY_WIDTH = false>
__global__ __launch_bounds__(kThreads) void fir_down_kernel(const TilePlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int KK = K * K;
    constexpr int WIN_ROWS = (BH - 1) * S + K;
    constexpr int NV = (3 * S + K + 3) / 4;  // float4s covering the columns 4 outputs touch

    const int tile = xcd_contiguous_tile(blockIdx.x, p.n_tiles);
    const int pg = tile / p.row_tiles, rt = tile - pg * p.row_tiles;
    const long plane0 = static_cast<long>(pg) * p.planes_per_tile;
    const int nplanes = static_cast<int>(min(static_cast<long>(p.planes_per_tile), p.planes - plane0));
    const int oy0 = rt * p.rows_per_tile;

    stage_taps<IO, KK, FLIP>(p, lds, plane0, nplanes, p.channel);
    stage_tile<IO, false, kStageBatch, true, ANY_WIDTH>(p.st, static_cast<const IO *>(p.in), lds, plane0, nplanes, oy0 * S - p.row_shift);
    __syncthreads();

    const int n_items = nplanes * p.items_per_plane;
    // the block of BH x 4 sums of one item
    auto convolve = [&](int pl, int rb, int cb, float(&acc)[BH][4]) {
        float tapv[KK];
#pragma unroll
        for (int t = 0; t < KK; ++t) tapv[t] = lds[p.tap_base + pl * KK + t];

        const float *base = lds + __mul24(pl, p.st.plane_pitch) + __mul24(rb * BH * S, p.st.pitch) + kSlack + 4 * cb * S;
#pragma unroll
        for (int b = 0; b < BH; ++b)
#pragma unroll
            for (int o = 0; o < 4; ++o) acc[b][o] = 0.f;

        // window rows are read one ahead of their use and the sums pinned after every row (see pin_registers)
        float nxt[4 * NV];
        load_window_row<NV>(base, nxt);
#pragma unroll
        for (int wr = 0; wr < WIN_ROWS; ++wr) {
            float win[4 * NV];
#pragma unroll
            for (int i = 0; i < 4 * NV; ++i) win[i] = nxt[i];
            if (wr + 1 < WIN_ROWS) load_window_row<NV>(base + (wr + 1) * p.st.pitch, nxt);
#pragma unroll
            for (int b = 0; b < BH; ++b) {
                const int ty = wr - b * S;
                if (ty < 0 || ty >= K) continue;
#pragma unroll
                for (int tx = 0; tx < K; ++tx)
#pragma unroll
                    for (int o = 0; o < 4; ++o)
                        acc[b][o] = fmaf(win[o * S + tx], tapv[ty * K + tx], acc[b][o]);
            }
            pin_registers(acc);
        }

        if constexpr (!FLIP) {
            if (p.epi.enabled()) {
                epilogue_apply_block<1>(acc, p.epi, static_cast<int>((plane0 + pl) % p.channel));
            }
        }
    };

    if (p.lds_out) {
        // One item per lane (the planner guarantees it).  The sums go back into LDS in the layout the band has in
        // memory, over the input image, and leave as one linear stream per plane: every store instruction of a
        // wavefront then covers 1 KiB of consecutive bytes, where lane-owned blocks write a row segment at a time
        // and leave the 128-byte lines that straddle two rows to two partial writes.
        const bool has_item = static_cast<int>(threadIdx.x) < n_items;
        const int item = has_item ? threadIdx.x : 0;
        const int pl = fast_div(item, p.ipp_magic);
        const int rem = item - __mul24(pl, p.items_per_plane);
        const int rb = fast_div(rem, p.ncb_magic);
        const int cb = rem - __mul24(rb, p.ncb);
        float acc[BH][4];
        convolve(pl, rb, cb, acc);
        const int rows_here = min(p.rows_per_tile, p.out_h - oy0);
        const int run = rows_here * p.out_w;  // elements per plane, a multiple of four
        __syncthreads();  // every window has been read: the image can be overwritten
        if (has_item) {
#pragma unroll
            for (int b = 0; b < BH; ++b)
                if (rb * BH + b < rows_here)
                    *reinterpret_cast<float4 *>(lds + pl * run + (rb * BH + b) * p.out_w + 4 * cb) =
                        make_float4(acc[b][0], acc[b][1], acc[b][2], acc[b][3]);
        }
        __syncthreads();
        const __amdgpu_buffer_rsrc_t view = buffer_view(static_cast<IO *>(p.out) + plane0 * p.out_plane, static_cast<long>(nplanes) * p.out_plane * sizeof(IO));
        const int run4 = run >> 2, total4 = nplanes * run4;
        for (int i = threadIdx.x; i < total4; i += blockDim.x) {
            const int q = nplanes == 1 ? 0 : i / run4;
            const float4 v = reinterpret_cast<const float4 *>(lds)[i];
            const unsigned off = (q * p.out_plane + oy0 * p.out_w + (i - q * run4) * 4) * static_cast<unsigned>(sizeof(IO));
            view_store4<IO>(view, off, v.x, v.y, v.z, v.w);
        }
        return;
    }

    for (int item = threadIdx.x; item < n_items; item += blockDim.x) {
        // (24-bit multiplies: full rate, and every operand here is an LDS-sized quantity)
        const int pl = fast_div(item, p.ipp_magic);
        const int rem = item - __mul24(pl, p.items_per_plane);
        const int rb = fast_div(rem, p.ncb_magic);
        const int cb = rem - __mul24(rb, p.ncb);
        float acc[BH][4];
        convolve(pl, rb, cb, acc);
        const int ox = 4 * cb;
        if (p.vec_out == 2 || (ANY_WIDTH && p.vec_out == 3)) {
            // branch-free: rows past the end of the plane store out of range
            const __amdgpu_buffer_rsrc_t view = buffer_view(static_cast<IO *>(p.out) + plane0 * p.out_plane, static_cast<long>(nplanes) * p.out_plane * sizeof(IO));
            const unsigned o0 = (pl * p.out_plane + ox) * static_cast<unsigned>(sizeof(IO));
            if constexpr (ANY_WIDTH) {
                if (p.vec_out == 3) {  // the block that ends a row may be short
#pragma unroll
                    for (int b = 0; b < BH; ++b) {
                        const int oy = oy0 + rb * BH + b;
                        view_store_first<IO>(view, oy < p.out_h ? o0 + oy * p.out_w * static_cast<unsigned>(sizeof(IO)) : kOob,
                                             p.out_w - ox, p.out_w & 3, acc[b][0], acc[b][1], acc[b][2], acc[b][3]);
                    }
                    continue;
                }
            }
#pragma unroll
            for (int b = 0; b < BH; ++b) {
                const int oy = oy0 + rb * BH + b;
                view_store4<IO>(view, oy < p.out_h ? o0 + oy * p.out_w * static_cast<unsigned>(sizeof(IO)) : kOob, acc[b][0],
                                acc[b][1], acc[b][2], acc[b][3]);
            }
            continue;
        }
        IO *dst = static_cast<IO *>(p.out) + (plane0 + pl) * p.out_plane + ox;
#pragma unroll
        for (int b = 0; b < BH; ++b) {
            const int oy = oy0 + rb * BH + b;
            if (oy >= p.out_h) continue;
            IO *row = dst + static_cast<long>(oy) * p.out_w;
            if (p.vec_out) {
                store4<IO>(row, acc[b][0], acc[b][1], acc[b][2], acc[b][3]);
            } else {
#pragma unroll
                for (int o = 0; o < 4; ++o)
                    if (ox + o < p.out_w) row[o] = Io<IO>::out(acc[b][o]);
            }
        }
    }
}

// fir_down_kernel for a depth multiplier above 1 (TilePlan::mult), one plane per tile: a kernel of its own, so that the
// plain one carries none of this.
template <typename IO, int K, int S, bool FLIP, int BH>
__global__ __launch_bounds__(kThreads) void fir_down_mult_kernel(const TilePlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int KK = K * K;
    constexpr int WIN_ROWS = (BH - 1) * S + K;
    constexpr int NV = (3 * S + K + 3) / 4;  // float4s covering the columns 4 outputs touch

    const int tile = xcd_contiguous_tile(blockIdx.x, p.n_tiles);
    const int pg = tile / p.row_tiles, rt = tile - pg * p.row_tiles;
    const long plane0 = static_cast<long>(pg) * p.planes_per_tile;
    const int nplanes = static_cast<int>(min(static_cast<long>(p.planes_per_tile), p.planes - plane0));
    const int oy0 = rt * p.rows_per_tile;

    // the operand's first plane and the channel count its taps are indexed by (depth multiplier: see TilePlan::mult)
    long src0 = plane0;
    int tap_channels = p.channel;
    {
        if constexpr (FLIP) {
            src0 = plane0 * p.mult;
            tap_channels = p.channel * p.mult;
        } else {
            const int n = pg / p.channel;
            src0 = static_cast<long>(n) * (p.channel / p.mult) + (pg - n * p.channel) / p.mult;
        }
    }
    stage_taps<IO, KK, FLIP>(p, lds, FLIP ? src0 : plane0, nplanes, tap_channels);
    stage_tile<IO, false, kStageBatch, true>(p.st, static_cast<const IO *>(p.in), lds, src0, nplanes, oy0 * S - p.row_shift);
    __syncthreads();

    const int n_items = nplanes * p.items_per_plane;
    // adds the windows of one item to its block of BH x 4 sums
    auto accumulate = [&](int pl, int rb, int cb, float(&acc)[BH][4]) {
        float tapv[KK];
#pragma unroll
        for (int t = 0; t < KK; ++t) tapv[t] = lds[p.tap_base + pl * KK + t];

        const float *base = lds + __mul24(pl, p.st.plane_pitch) + __mul24(rb * BH * S, p.st.pitch) + kSlack + 4 * cb * S;
        // window rows are read one ahead of their use and the sums pinned after every row (see pin_registers)
        float nxt[4 * NV];
        load_window_row<NV>(base, nxt);
#pragma unroll
        for (int wr = 0; wr < WIN_ROWS; ++wr) {
            float win[4 * NV];
#pragma unroll
            for (int i = 0; i < 4 * NV; ++i) win[i] = nxt[i];
            if (wr + 1 < WIN_ROWS) load_window_row<NV>(base + (wr + 1) * p.st.pitch, nxt);
#pragma unroll
            for (int b = 0; b < BH; ++b) {
                const int ty = wr - b * S;
                if (ty < 0 || ty >= K) continue;
#pragma unroll
                for (int tx = 0; tx < K; ++tx)
#pragma unroll
                    for (int o = 0; o < 4; ++o)
                        acc[b][o] = fmaf(win[o * S + tx], tapv[ty * K + tx], acc[b][o]);
            }
            pin_registers(acc);
        }
    };
    // the block of BH x 4 sums of one item
    auto convolve = [&](int pl, int rb, int cb, float(&acc)[BH][4]) {
#pragma unroll
        for (int b = 0; b < BH; ++b)
#pragma unroll
            for (int o = 0; o < 4; ++o) acc[b][o] = 0.f;
        accumulate(pl, rb, cb, acc);
        if constexpr (!FLIP) {
            if (p.epi.enabled()) {
                epilogue_apply_block<1>(acc, p.epi, static_cast<int>((plane0 + pl) % p.channel));
            }
        }
    };
    // a finished block to memory
    auto store_block = [&](int pl, int rb, int cb, const float(&acc)[BH][4]) {
        const int ox = 4 * cb;
        if (p.vec_out >= 2) {
            // branch-free: rows past the end of the plane store out of range
            const __amdgpu_buffer_rsrc_t view = buffer_view(static_cast<IO *>(p.out) + plane0 * p.out_plane, static_cast<long>(nplanes) * p.out_plane * sizeof(IO));
            const unsigned o0 = (pl * p.out_plane + ox) * static_cast<unsigned>(sizeof(IO));
            {
                if (p.vec_out == 3) {  // rows of any width: the block that ends a row may be short
#pragma unroll
                    for (int b = 0; b < BH; ++b) {
                        const int oy = oy0 + rb * BH + b;
                        view_store_first<IO>(view, oy < p.out_h ? o0 + oy * p.out_w * static_cast<unsigned>(sizeof(IO)) : kOob,
                                             p.out_w - ox, p.out_w & 3, acc[b][0], acc[b][1], acc[b][2], acc[b][3]);
                    }
                    return;
                }
            }
#pragma unroll
            for (int b = 0; b < BH; ++b) {
                const int oy = oy0 + rb * BH + b;
                view_store4<IO>(view, oy < p.out_h ? o0 + oy * p.out_w * static_cast<unsigned>(sizeof(IO)) : kOob, acc[b][0],
                                acc[b][1], acc[b][2], acc[b][3]);
            }
            return;
        }
        IO *dst = static_cast<IO *>(p.out) + (plane0 + pl) * p.out_plane + ox;
#pragma unroll
        for (int b = 0; b < BH; ++b) {
            const int oy = oy0 + rb * BH + b;
            if (oy >= p.out_h) continue;
            IO *row = dst + static_cast<long>(oy) * p.out_w;
            if (p.vec_out) {
                store4<IO>(row, acc[b][0], acc[b][1], acc[b][2], acc[b][3]);
            } else {
#pragma unroll
                for (int o = 0; o < 4; ++o)
                    if (ox + o < p.out_w) row[o] = Io<IO>::out(acc[b][o]);
            }
        }
    };

    if constexpr (FLIP) {
        {
            // One plane per tile and one item per lane (the launcher's rule): the lane keeps its sums while the M
            // operand planes of its result plane pass through LDS one after the other.
            const bool has_item = static_cast<int>(threadIdx.x) < n_items;
            const int item = has_item ? threadIdx.x : 0;
            const int rb = fast_div(item, p.ncb_magic);
            const int cb = item - __mul24(rb, p.ncb);
            float acc[BH][4];
#pragma unroll
            for (int b = 0; b < BH; ++b)
#pragma unroll
                for (int o = 0; o < 4; ++o) acc[b][o] = 0.f;
            for (int m = 0;;) {
                accumulate(0, rb, cb, acc);
                if (++m == p.mult) break;
                __syncthreads();
                stage_taps<IO, KK, FLIP>(p, lds, src0 + m, 1, tap_channels);
                stage_tile<IO, false, kStageBatch, true>(p.st, static_cast<const IO *>(p.in), lds, src0 + m, 1, oy0 * S - p.row_shift);
                __syncthreads();
            }
            if (has_item) store_block(0, rb, cb, acc);
            return;
        }
    }

    if (p.lds_out) {
        // One item per lane (the planner guarantees it).  The sums go back into LDS in the layout the band has in
        // memory, over the input image, and leave as one linear stream per plane: every store instruction of a
        // wavefront then covers 1 KiB of consecutive bytes, where lane-owned blocks write a row segment at a time
        // and leave the 128-byte lines that straddle two rows to two partial writes.
        const bool has_item = static_cast<int>(threadIdx.x) < n_items;
        const int item = has_item ? threadIdx.x : 0;
        const int pl = fast_div(item, p.ipp_magic);
        const int rem = item - __mul24(pl, p.items_per_plane);
        const int rb = fast_div(rem, p.ncb_magic);
        const int cb = rem - __mul24(rb, p.ncb);
        float acc[BH][4];
        convolve(pl, rb, cb, acc);
        const int rows_here = min(p.rows_per_tile, p.out_h - oy0);
        const int run = rows_here * p.out_w;  // elements per plane, a multiple of four
        __syncthreads();  // every window has been read: the image can be overwritten
        if (has_item) {
#pragma unroll
            for (int b = 0; b < BH; ++b)
                if (rb * BH + b < rows_here)
                    *reinterpret_cast<float4 *>(lds + pl * run + (rb * BH + b) * p.out_w + 4 * cb) =
                        make_float4(acc[b][0], acc[b][1], acc[b][2], acc[b][3]);
        }
        __syncthreads();
        const __amdgpu_buffer_rsrc_t view = buffer_view(static_cast<IO *>(p.out) + plane0 * p.out_plane, static_cast<long>(nplanes) * p.out_plane * sizeof(IO));
        const int run4 = run >> 2, total4 = nplanes * run4;
        for (int i = threadIdx.x; i < total4; i += blockDim.x) {
            const int q = nplanes == 1 ? 0 : i / run4;
            const float4 v = reinterpret_cast<const float4 *>(lds)[i];
            const unsigned off = (q * p.out_plane + oy0 * p.out_w + (i - q * run4) * 4) * static_cast<unsigned>(sizeof(IO));
            view_store4<IO>(view, off, v.x, v.y, v.z, v.w);
        }
        return;
    }

    for (int item = threadIdx.x; item < n_items; item += blockDim.x) {
        // (24-bit multiplies: full rate, and every operand here is an LDS-sized quantity)
        const int pl = fast_div(item, p.ipp_magic);
        const int rem = item - __mul24(pl, p.items_per_plane);
        const int rb = fast_div(rem, p.ncb_magic);
        const int cb = rem - __mul24(rb, p.ncb);
        float acc[BH][4];
        convolve(pl, rb, cb, acc);
        store_block(pl, rb, cb, acc);
    }
}

// up = 2, no decimation, taps rotated.  With pad0 = 2m - E (E = pad0 & 1, m = (pad0+E)/2) and the
// rotated filter g shifted by E (g'[t] = g[t-E]):
//   out[2q + r] = sum_a in[q - m + r + a] * g'[r + 2a]      along each axis,
// i.e. a stride-1 correlation per output parity r with every other tap.
// A lane owns 2*BQ output rows x 4 output columns (BQ x 2 half-resolution positions), so that the
// 128-bit stores of consecutive lanes are contiguous in memory.
template <typename IO, int K, int EY, int EX, int BQ>
__global__ __launch_bounds__(kThreads) void fir_up2_kernel(const TilePlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int KK = K * K;
    constexpr int KAY = (K + EY + 1) / 2, KAX = (K + EX + 1) / 2;
    constexpr int WIN_ROWS = BQ + KAY;
    constexpr int NW = 2 * ((KAX + 2 + 1) / 2);  // floats of a row two half-resolution positions touch, as float2s

    const int tile = xcd_contiguous_tile(blockIdx.x, p.n_tiles);
    const int pg = tile / p.row_tiles, rt = tile - pg * p.row_tiles;
    const long plane0 = static_cast<long>(pg) * p.planes_per_tile;
    const int nplanes = static_cast<int>(min(static_cast<long>(p.planes_per_tile), p.planes - plane0));
    const int qy0 = rt * p.rows_per_tile;

    // depth multiplier (see TilePlan::mult): result plane (n, c) adds up the operand's planes (n, c * M + m)
    const long src0 = p.mult > 1 ? plane0 * p.mult : plane0;
    const int tap_channels = p.mult > 1 ? p.channel * p.mult : p.channel;
    stage_taps<IO, KK, true>(p, lds, src0, nplanes, tap_channels);
    stage_tile<IO, false, kStageBatch, true>(p.st, static_cast<const IO *>(p.in), lds, src0, nplanes, qy0 - p.row_shift);
    __syncthreads();

    const int n_items = nplanes * p.items_per_plane;
    // adds the windows of one item to its block of 2*BQ x 4 sums
    auto accumulate = [&](int pl, int rb, int cb, float(&acc)[2 * BQ][4]) {
        float tapv[KK];
#pragma unroll
        for (int t = 0; t < KK; ++t) tapv[t] = lds[p.tap_base + pl * KK + t];

        const float *base = lds + pl * p.st.plane_pitch + (rb * BQ) * p.st.pitch + kSlack + 2 * cb;
        float nxt[NW];
        load_window_row2<NW / 2>(base, nxt);
#pragma unroll
        for (int wr = 0; wr < WIN_ROWS; ++wr) {
            float win[NW];
#pragma unroll
            for (int i = 0; i < NW; ++i) win[i] = nxt[i];
            if (wr + 1 < WIN_ROWS) load_window_row2<NW / 2>(base + (wr + 1) * p.st.pitch, nxt);
#pragma unroll
            for (int bq = 0; bq < BQ; ++bq)
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    const int a = wr - bq - r;
                    if (a < 0 || a >= KAY) continue;
                    const int fy = r + 2 * a - EY;
                    if (fy < 0 || fy >= K) continue;
#pragma unroll
                    for (int xq = 0; xq < 2; ++xq)
#pragma unroll
                        for (int rx = 0; rx < 2; ++rx)
#pragma unroll
                            for (int ax = 0; ax < KAX; ++ax) {
                                const int fx = rx + 2 * ax - EX;
                                if (fx < 0 || fx >= K) continue;
                                acc[2 * bq + r][2 * xq + rx] =
                                    fmaf(win[xq + rx + ax], tapv[fy * K + fx], acc[2 * bq + r][2 * xq + rx]);
                            }
                }
            pin_registers(acc);
        }
    };
    // a finished block to memory
    auto store_block = [&](int pl, int rb, int cb, const float(&acc)[2 * BQ][4]) {
        const int ox = 4 * cb;
        if (p.vec_out >= 2) {
            // branch-free: rows past the end of the plane store out of range
            const __amdgpu_buffer_rsrc_t view = buffer_view(static_cast<IO *>(p.out) + plane0 * p.out_plane, static_cast<long>(nplanes) * p.out_plane * sizeof(IO));
            const unsigned o0 = (pl * p.out_plane + ox) * static_cast<unsigned>(sizeof(IO));
            {
                if (p.vec_out == 3) {  // rows of any width: the block that ends a row may be short
#pragma unroll
                    for (int b = 0; b < 2 * BQ; ++b) {
                        const int oy = 2 * (qy0 + rb * BQ) + b;
                        view_store_first<IO>(view, oy < p.out_h ? o0 + oy * p.out_w * static_cast<unsigned>(sizeof(IO)) : kOob,
                                             p.out_w - ox, p.out_w & 3, acc[b][0], acc[b][1], acc[b][2], acc[b][3]);
                    }
                    return;
                }
            }
#pragma unroll
            for (int b = 0; b < 2 * BQ; ++b) {
                const int oy = 2 * (qy0 + rb * BQ) + b;
                view_store4<IO>(view, oy < p.out_h ? o0 + oy * p.out_w * static_cast<unsigned>(sizeof(IO)) : kOob, acc[b][0],
                                acc[b][1], acc[b][2], acc[b][3]);
            }
            return;
        }
        IO *dst = static_cast<IO *>(p.out) + (plane0 + pl) * p.out_plane + ox;
#pragma unroll
        for (int b = 0; b < 2 * BQ; ++b) {
            const int oy = 2 * (qy0 + rb * BQ) + b;
            if (oy >= p.out_h) continue;
            IO *row = dst + static_cast<long>(oy) * p.out_w;
            if (p.vec_out) {
                store4<IO>(row, acc[b][0], acc[b][1], acc[b][2], acc[b][3]);
            } else {
#pragma unroll
                for (int o = 0; o < 4; ++o)
                    if (ox + o < p.out_w) row[o] = Io<IO>::out(acc[b][o]);
            }
        }
    };

    if (p.mult > 1) {
        // one plane per tile and one item per lane (the launcher's rule), as in fir_down_kernel
        const bool has_item = static_cast<int>(threadIdx.x) < n_items;
        const int item = has_item ? threadIdx.x : 0;
        const int rb = fast_div(item, p.ncb_magic);
        const int cb = item - rb * p.ncb;
        float acc[2 * BQ][4];
#pragma unroll
        for (int b = 0; b < 2 * BQ; ++b)
#pragma unroll
            for (int o = 0; o < 4; ++o) acc[b][o] = 0.f;
        for (int m = 0;;) {
            accumulate(0, rb, cb, acc);
            if (++m == p.mult) break;
            __syncthreads();
            stage_taps<IO, KK, true>(p, lds, src0 + m, 1, tap_channels);
            stage_tile<IO, false, kStageBatch, true>(p.st, static_cast<const IO *>(p.in), lds, src0 + m, 1, qy0 - p.row_shift);
            __syncthreads();
        }
        if (has_item) store_block(0, rb, cb, acc);
        return;
    }

    for (int item = threadIdx.x; item < n_items; item += blockDim.x) {
        const int pl = fast_div(item, p.ipp_magic);
        const int rem = item - pl * p.items_per_plane;
        const int rb = fast_div(rem, p.ncb_magic);
        const int cb = rem - rb * p.ncb;
        float acc[2 * BQ][4];
#pragma unroll
        for (int b = 0; b < 2 * BQ; ++b)
#pragma unroll
            for (int o = 0; o < 4; ++o) acc[b][o] = 0.f;
        accumulate(pl, rb, cb, acc);
        store_block(pl, rb, cb, acc);
    }
}

// Any filter extent, stride and dilation (up = 1): what has no kernel of its own above (rectangular and even-sized
// filters, strip filters such as 1 x 7 or 21 x 1, 15 x 15 and larger, strides above 2, dilations above 2).  The same
// tiles and the same LDS image; the taps are looped over at run time, so a lane reads its BH x 4 inputs from LDS for
// every tap instead of keeping window rows in registers: one LDS read per multiply-add, which still leaves filters of
// few taps bound by HBM.  Replaces the generic instantiation of torch_dwconv/dwconv_kernel.cu:69-181 (kernel sizes of
// -1) for these shapes.
// SW: the column stride when it is 1 or 2 (the four inputs of a row then sit at immediate offsets), 0 = any.
// KHM x KWM (0: none): at stride 1 and dilation 1, filters of at most that extent walk a register window as the
// kernels above do (a window row of 3 + kw inputs is read once and used by every tap and output row that meets it),
// with the loops unrolled to the maxima under uniform bounds: 3 + kw LDS reads for 4 * kw multiply-adds.
// KHM < 0: column stride 1 and undilated columns, any extent, row stride and row dilation: filter rows are walked
// four taps at a time (see there), which is what keeps 15 x 15 and larger filters off the LDS read rate.
template <typename IO, int BH, int SW, int KHM = 0, int KWM = 0>
__global__ __launch_bounds__(kThreads) void fir_any_kernel(const TilePlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    const int KK = p.kh * p.kw;
    const int sw = SW ? SW : p.sw;

    const int tile = xcd_contiguous_tile(blockIdx.x, p.n_tiles);
    const int pg = tile / p.row_tiles, rt = tile - pg * p.row_tiles;
    const long plane0 = static_cast<long>(pg) * p.planes_per_tile;
    const int nplanes = static_cast<int>(min(static_cast<long>(p.planes_per_tile), p.planes - plane0));
    const int oy0 = rt * p.rows_per_tile;

    for (int i = threadIdx.x; i < nplanes * KK; i += blockDim.x) {
        const int pl = i / KK, t = i - pl * KK;
        const int c = static_cast<int>((plane0 + pl) % p.channel);
        lds[p.tap_base + i] = Io<IO>::in(static_cast<const IO *>(p.taps)[c * KK + (p.flip ? KK - 1 - t : t)]);
    }
    stage_tile<IO, false, kStageBatch, true>(p.st, static_cast<const IO *>(p.in), lds, plane0, nplanes, oy0 * p.sh - p.row_shift);
    __syncthreads();

    const int n_items = nplanes * p.items_per_plane;
    const int row_step = p.sh * p.st.pitch;
    for (int item = threadIdx.x; item < n_items; item += blockDim.x) {
        const int pl = fast_div(item, p.ipp_magic);
        const int rem = item - __mul24(pl, p.items_per_plane);
        const int rb = fast_div(rem, p.ncb_magic);
        const int cb = rem - __mul24(rb, p.ncb);
        float acc[BH][4];
#pragma unroll
        for (int b = 0; b < BH; ++b)
#pragma unroll
            for (int o = 0; o < 4; ++o) acc[b][o] = 0.f;
        const float *base = lds + __mul24(pl, p.st.plane_pitch) + __mul24(rb * BH, row_step) + kSlack + 4 * cb * sw;
        const float *tp = lds + p.tap_base + pl * KK;
        if constexpr (KHM > 0) {
            static_assert(SW == 1, "the register window is the stride-1 case");
            float tapr[KHM][KWM];
#pragma unroll
            for (int ty = 0; ty < KHM; ++ty)
#pragma unroll
                for (int tx = 0; tx < KWM; ++tx) tapr[ty][tx] = (ty < p.kh && tx < p.kw) ? tp[ty * p.kw + tx] : 0.f;
#pragma unroll
            for (int wr = 0; wr < BH - 1 + KHM; ++wr) {
                if (wr < BH - 1 + p.kh) {  // (uniform)
                    const float *r = base + wr * p.st.pitch;
                    // (16-byte LDS reads: consecutive lanes then read consecutive banks; the last may reach into the
                    // slack of the row)
                    float win[4 * ((3 + KWM + 3) / 4)];
#pragma unroll
                    for (int v = 0; v < (3 + KWM + 3) / 4; ++v) {
                        float4 q = make_float4(0.f, 0.f, 0.f, 0.f);
                        if (4 * v < 3 + p.kw) q = *reinterpret_cast<const float4 *>(r + 4 * v);
                        win[4 * v] = q.x, win[4 * v + 1] = q.y, win[4 * v + 2] = q.z, win[4 * v + 3] = q.w;
                    }
#pragma unroll
                    for (int b = 0; b < BH; ++b) {
                        const int ty = wr - b;
                        if (ty < 0 || ty >= KHM) continue;
                        if (ty < p.kh) {
#pragma unroll
                            for (int tx = 0; tx < KWM; ++tx) {
                                if (tx < p.kw) {
#pragma unroll
                                    for (int o = 0; o < 4; ++o) acc[b][o] = fmaf(win[o + tx], tapr[ty][tx], acc[b][o]);
                                }
                            }
                        }
                    }
                    pin_registers(acc);
                }
            }
        } else if constexpr (KHM < 0) {
            static_assert(SW == 1, "rows are walked four inputs at a time at column stride 1");
            // undilated columns: a filter row takes four taps at a time from eight inputs per output row (the four
            // read for the taps before, and the next four), one 16-byte LDS read per sixteen multiply-adds
            for (int ty = 0; ty < p.kh; ++ty) {
                const float *trow = base + __mul24(ty * p.dh, p.st.pitch);
                const float *tr = tp + ty * p.kw;
                float w[BH][8];
#pragma unroll
                for (int b = 0; b < BH; ++b) {
                    const float4 v = *reinterpret_cast<const float4 *>(trow + b * row_step);
                    w[b][4] = v.x, w[b][5] = v.y, w[b][6] = v.z, w[b][7] = v.w;
                }
                for (int tx0 = 0; tx0 < p.kw; tx0 += 4) {
#pragma unroll
                    for (int b = 0; b < BH; ++b) {
                        const float4 v = *reinterpret_cast<const float4 *>(trow + b * row_step + tx0 + 4);
#pragma unroll
                        for (int i = 0; i < 4; ++i) w[b][i] = w[b][4 + i];
                        w[b][4] = v.x, w[b][5] = v.y, w[b][6] = v.z, w[b][7] = v.w;
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if (tx0 + j < p.kw) {  // (uniform)
                            const float t = tr[tx0 + j];
#pragma unroll
                            for (int b = 0; b < BH; ++b)
#pragma unroll
                                for (int o = 0; o < 4; ++o) acc[b][o] = fmaf(w[b][j + o], t, acc[b][o]);
                        }
                    }
                }
            }
        } else {
            for (int ty = 0; ty < p.kh; ++ty) {
                const float *trow = base + __mul24(ty * p.dh, p.st.pitch);
                for (int tx = 0; tx < p.kw; ++tx) {
                    const float t = tp[ty * p.kw + tx];
                    if constexpr (SW == 1 || SW == 2) {
                        // The four inputs of a row sit within twelve floats.  Lanes are four or eight floats apart, so
                        // reading them one float at a time would meet the same LDS banks four or eight times over:
                        // 16-byte reads from the 16-byte boundary before the tap's offset on (the last may reach into
                        // the slack of the row) and a uniform choice among what they hold.
                        const int off = tx * p.dw;
                        const float *r = trow + (off & ~3);
                        auto rows = [&](auto shift) {
                            constexpr int S = decltype(shift)::value;
#pragma unroll
                            for (int b = 0; b < BH; ++b) {
                                constexpr int NR = (S + 3 * SW + 4) / 4;  // 16-byte reads that hold inputs S, S + SW .. S + 3 SW
                                float w8[4 * NR];
#pragma unroll
                                for (int v = 0; v < NR; ++v) {
                                    const float4 q = *reinterpret_cast<const float4 *>(r + b * row_step + 4 * v);
                                    w8[4 * v] = q.x, w8[4 * v + 1] = q.y, w8[4 * v + 2] = q.z, w8[4 * v + 3] = q.w;
                                }
#pragma unroll
                                for (int o = 0; o < 4; ++o) acc[b][o] = fmaf(w8[S + o * SW], t, acc[b][o]);
                            }
                        };
                        switch (off & 3) {
                        case 0: rows(std::integral_constant<int, 0>{}); break;
                        case 1: rows(std::integral_constant<int, 1>{}); break;
                        case 2: rows(std::integral_constant<int, 2>{}); break;
                        default: rows(std::integral_constant<int, 3>{}); break;
                        }
                    } else {
                        const float *r = trow + tx * p.dw;
#pragma unroll
                        for (int b = 0; b < BH; ++b)
#pragma unroll
                            for (int o = 0; o < 4; ++o) acc[b][o] = fmaf(r[b * row_step + o * sw], t, acc[b][o]);
                    }
                }
            }
        }
        if (!p.flip && p.epi.enabled()) epilogue_apply_block<1>(acc, p.epi, static_cast<int>((plane0 + pl) % p.channel));

        const int ox = 4 * cb;
        if (p.vec_out >= 2) {
            // branch-free: rows past the end of the plane store out of range
            const __amdgpu_buffer_rsrc_t view = buffer_view(static_cast<IO *>(p.out) + plane0 * p.out_plane, static_cast<long>(nplanes) * p.out_plane * sizeof(IO));
            const unsigned o0 = (pl * p.out_plane + ox) * static_cast<unsigned>(sizeof(IO));
#pragma unroll
            for (int b = 0; b < BH; ++b) {
                const int oy = oy0 + rb * BH + b;
                const unsigned off = oy < p.out_h ? o0 + oy * p.out_w * static_cast<unsigned>(sizeof(IO)) : kOob;
                if (p.vec_out == 3) view_store_first<IO>(view, off, p.out_w - ox, p.out_w & 3, acc[b][0], acc[b][1], acc[b][2], acc[b][3]);
                else view_store4<IO>(view, off, acc[b][0], acc[b][1], acc[b][2], acc[b][3]);
            }
            continue;
        }
        IO *dst = static_cast<IO *>(p.out) + (plane0 + pl) * p.out_plane + ox;
#pragma unroll
        for (int b = 0; b < BH; ++b) {
            const int oy = oy0 + rb * BH + b;
            if (oy >= p.out_h) continue;
            IO *row = dst + static_cast<long>(oy) * p.out_w;
            if (p.vec_out) {
                store4<IO>(row, acc[b][0], acc[b][1], acc[b][2], acc[b][3]);
            } else {
#pragma unroll
                for (int o = 0; o < 4; ++o)
                    if (ox + o < p.out_w) row[o] = Io<IO>::out(acc[b][o]);
            }
        }
    }
}

// Fills in the tiling of `p` for a plane whose output is split into `row_units`
// units of rows (BH output rows or BQ half-resolution rows each) and `ncb` column
// blocks.  `rows_for(units)` gives the LDS rows a band of that many units needs.
// Returns false when even the smallest tile exceeds the LDS budget.
template <typename RowsFor>
bool plan_tiles(TilePlan &p, int row_units, int unit_rows, int used_cols, int taps_per_plane, RowsFor rows_for,
                int lds_budget = dwconv::kLdsBudget)
{
    const int threads = kThreads;
    const int target_items = env_int("DWCONV_TILE_ITEMS", threads);
    const int kLdsBudget = env_int("DWCONV_TILE_LDS", lds_budget);
    layout_columns(p.st, used_cols);

    auto bytes = [&](int units, int planes) {
        return static_cast<long>(planes) * (static_cast<long>(rows_for(units)) * p.st.pitch + taps_per_plane) * 4;
    };

    const int ipp_full = row_units * p.ncb;
    int units_per_tile, planes_per_tile;
    if (2 * ipp_full <= target_items) {
        // whole planes, several per tile
        units_per_tile = row_units;
        planes_per_tile = target_items / ipp_full;
        while (planes_per_tile > 1 && bytes(units_per_tile, planes_per_tile) > kLdsBudget) --planes_per_tile;
        if (static_cast<long>(planes_per_tile) > p.planes) planes_per_tile = static_cast<int>(p.planes);
        if (bytes(units_per_tile, planes_per_tile) > kLdsBudget) planes_per_tile = 0;  // fall through to bands
    } else {
        planes_per_tile = 0;
    }
    if (planes_per_tile == 0) {
        planes_per_tile = 1;
        units_per_tile = target_items / p.ncb;
        if (units_per_tile < 1) units_per_tile = 1;
        if (units_per_tile > row_units) units_per_tile = row_units;
        while (units_per_tile > 1 && bytes(units_per_tile, 1) > kLdsBudget) --units_per_tile;
        if (bytes(units_per_tile, 1) > kLdsBudget) return false;
        // even out the bands
        const int bands = ceil_div(row_units, units_per_tile);
        units_per_tile = ceil_div(row_units, bands);
    }
    p.planes_per_tile = planes_per_tile;
    p.rows_per_tile = units_per_tile * unit_rows;
    p.row_tiles = ceil_div(row_units, units_per_tile);
    if (!layout_rows(p.st, rows_for(units_per_tile), planes_per_tile)) return false;
    p.items_per_plane = units_per_tile * p.ncb;
    p.tap_base = planes_per_tile * p.st.plane_pitch;
    const long groups = (p.planes + planes_per_tile - 1) / planes_per_tile;
    const long tiles = groups * p.row_tiles;
    if (tiles > 0x7fffffffL) return false;
    p.n_tiles = static_cast<int>(tiles);
    // the in-kernel divisions use a 16-bit reciprocal
    if (planes_per_tile * p.items_per_plane >= 65536) return false;
    p.ncb_magic = magic_u16(p.ncb);
    p.ipp_magic = magic_u16(p.items_per_plane);
    return true;
}

// The tile is known: whether its planes fit a buffer view decides between modes 1 and 2, and whether rows of any
// width (mode 3) can be served at all.
template <typename IO>
void settle_vector_modes(TilePlan &p)
{
    const int in_view = stage_vector_mode(p.st, p.planes_per_tile, sizeof(IO));
    const int out_view = vector_mode(p.planes_per_tile, p.out_plane, sizeof(IO));
    if (p.st.vec_in == 1) p.st.vec_in = in_view;
    else if (p.st.vec_in == 3 && in_view != 2) p.st.vec_in = 0;
    if (p.vec_out == 1) p.vec_out = out_view;
    else if (p.vec_out == 3 && out_view != 2) p.vec_out = 0;
}

size_t lds_bytes(const TilePlan &p, int taps_per_plane)
{
    return static_cast<size_t>(p.planes_per_tile) * (p.st.plane_pitch + taps_per_plane) * 4;
}

template <typename IO, int K, int S, bool FLIP, int BH>
int launch_down(TilePlan &p, hipStream_t stream)
{
    constexpr int NV = (3 * S + K + 3) / 4;
    p.ncb = ceil_div(p.out_w, 4);
    const int used_cols = 4 * (p.ncb - 1) * S + 4 * NV;
    auto rows_for = [](int units) { return (units * BH - 1) * S + K; };
    // A stride-2 layer reads four times what it writes: smaller tiles (more workgroups per CU, more loads in flight)
    // beat the halo rows they add: -17 % on a 56x56 5x5 layer, -3 % on a 112x112 3x3 one, -6 % on 128x96 5x5.
    // (16-bit elements land in an fp32 image, so the same bytes in flight need twice the LDS: 28 KiB measured best
    // on the 112x112 3x3 layer, -12 %.)  With four rows per lane 16 KiB is another 1-3 % better on 3x3 layers 112-128
    // wide (bands of 12 rows instead of 16-20) and changes nothing for 5x5 ones; with seven rows per lane it would halve
    // the band (150 -> 75: 248 -> 305 us) and 20 KiB stays.  Those 16 KiB are for 3x3 layers on wide maps: planes of
    // 36-40 columns fit one to a tile in them, 25 items for 256 lanes, and two with 20 KiB (38x38 3x3: 71 -> 54 us,
    // 40x40: 58 -> 45, 36x36 5x5: 69 -> 52; a 64x64 5x5 layer takes bands of 32 rows instead of 16: 76 -> 71).
    const int budget = S == 2 ? (sizeof(IO) == 2 ? 28 : (BH == 7 || K != 3 || p.st.in_w < 96 ? 20 : 16)) * 1024 : dwconv::kLdsBudget;
    if (!plan_tiles(p, ceil_div(p.out_h, BH), BH, used_cols, K * K, rows_for, budget)) return -1;
    // a depth multiplier is served where a tile is one plane (and, backward, a lane has one item): larger maps
    if (p.mult > 1 && (p.planes_per_tile != 1 || p.items_per_plane > kThreads)) return -1;
    settle_vector_modes<IO>(p);
    // Results through LDS: measured to pay where a workgroup owns a whole fp32 plane of a 3x3 stride-1 layer whose
    // rows are not whole 128-byte lines (56x56: -10 %); neutral or worse elsewhere (+2 % with 16-bit elements, +9 %
    // on a 5x5 stride-2 layer).
    const bool lds_out_pays = sizeof(IO) == 4 && K == 3 && S == 1 && p.row_tiles == 1 && (p.out_w * sizeof(IO)) % 128 != 0;
    p.lds_out = env_int("DWCONV_TILE_LDS_OUT", lds_out_pays) && p.vec_out == 2 && p.mult == 1 &&
                p.planes_per_tile * p.items_per_plane <= kThreads;
    if (p.mult > 1)
        hipLaunchKernelGGL((fir_down_mult_kernel<IO, K, S, FLIP, BH>), dim3(p.n_tiles), dim3(kThreads), lds_bytes(p, K * K),
                           stream, p);
    else if (p.st.vec_in == 3 || p.vec_out == 3)
        hipLaunchKernelGGL((fir_down_kernel<IO, K, S, FLIP, BH, true>), dim3(p.n_tiles), dim3(kThreads), lds_bytes(p, K * K),
                           stream, p);
    else
        hipLaunchKernelGGL((fir_down_kernel<IO, K, S, FLIP, BH>), dim3(p.n_tiles), dim3(kThreads), lds_bytes(p, K * K),
                           stream, p);
    char mult[16] = "";
    if (p.mult > 1) std::snprintf(mult, sizeof(mult), " m%d", p.mult);
    note_variant("tile_down%s<k%d,s%d,%s,bh%d> P%d rows%d vin%d vout%d%s%s", sizeof(IO) == 2 ? "16" : "", K, S, FLIP ? "rot" : "fwd", BH,
                 p.planes_per_tile, p.rows_per_tile, p.st.vec_in, p.vec_out, p.lds_out ? " ldsout" : "", mult);
    return check_launch("fir_down_kernel");
}

template <typename IO, int K, int S, bool FLIP>
int launch_down_bh(TilePlan &p, hipStream_t stream)
{
    const int forced = env_int("DWCONV_TILE_BH", 0);
    // Seven rows per lane where four would leave rows over and seven would not, and (stride 2) on tall planes that
    // four does not divide; stride-1 layers measured better with four there (150x150 3x3: 159 -> 152 us, 75x75: 221
    // -> 206; stride 2, 150 -> 75: 254 against 259 with four).
    const bool seven = forced ? forced == 7 : (p.out_h % 7 == 0 || (S == 2 && p.out_h > 64)) && p.out_h % 4 != 0;
    return seven ? launch_down<IO, K, S, FLIP, 7>(p, stream) : launch_down<IO, K, S, FLIP, 4>(p, stream);
}

template <typename IO, int K, int EY, int EX>
int launch_up2(TilePlan &p, hipStream_t stream)
{
    constexpr int BQ = 4;
    constexpr int KAY = (K + EY + 1) / 2, KAX = (K + EX + 1) / 2;
    constexpr int NW = 2 * ((KAX + 2 + 1) / 2);
    p.ncb = ceil_div(p.out_w, 4);
    const int used_cols = 2 * (p.ncb - 1) + NW;
    auto rows_for = [](int units) { return units * BQ + KAY; };
    if (!plan_tiles(p, ceil_div(ceil_div(p.out_h, 2), BQ), BQ, used_cols, K * K, rows_for)) return -1;
    if (p.mult > 1 && (p.planes_per_tile != 1 || p.items_per_plane > kThreads)) return -1;
    settle_vector_modes<IO>(p);
    hipLaunchKernelGGL((fir_up2_kernel<IO, K, EY, EX, BQ>), dim3(p.n_tiles), dim3(kThreads), lds_bytes(p, K * K), stream,
                       p);
    char mult[16] = "";
    if (p.mult > 1) std::snprintf(mult, sizeof(mult), " m%d", p.mult);
    note_variant("tile_up2%s<k%d,e%d%d,bq%d> P%d rows%d vin%d vout%d%s", sizeof(IO) == 2 ? "16" : "", K, EY, EX, BQ, p.planes_per_tile,
                 p.rows_per_tile, p.st.vec_in, p.vec_out, mult);
    return check_launch("fir_up2_kernel");
}

template <typename IO, int K>
int launch_up2_parity(TilePlan &p, int ey, int ex, hipStream_t stream)
{
    if (ey == 0 && ex == 0) return launch_up2<IO, K, 0, 0>(p, stream);
    if (ey == 0 && ex == 1) return launch_up2<IO, K, 0, 1>(p, stream);
    if (ey == 1 && ex == 0) return launch_up2<IO, K, 1, 0>(p, stream);
    return launch_up2<IO, K, 1, 1>(p, stream);
}

}  // namespace

template <typename IO>
int try_launch_fir_any(const IO *in, const IO *taps, IO *out, const Geometry &g, hipStream_t stream)
{
    if (!env_int("DWCONV_FIR_ANY", 1)) return -1;
    if (g.up_h != 1 || g.up_w != 1 || g.mult != 1) return -1;
    if (g.kernel_h < 1 || g.kernel_w < 1 || g.down_h < 1 || g.down_w < 1 || g.dil_h < 1 || g.dil_w < 1) return -1;
    if (g.pad_h0 < 0 || g.pad_w0 < 0 || g.in_h < 1 || g.in_w < 1) return -1;
    if (static_cast<long>(g.kernel_h) * g.kernel_w > 4096) return -1;
    if (static_cast<long>(g.in_h) * g.in_w >= (1l << 30) || static_cast<long>(g.out_h) * g.out_w >= (1l << 30)) return -1;
    // (everything the staging multiplies must stay far below 2^23)
    const long span_h = static_cast<long>(g.kernel_h - 1) * g.dil_h, span_w = static_cast<long>(g.kernel_w - 1) * g.dil_w;
    if (span_h > 4096 || span_w > 4096 || g.down_h > 64 || g.down_w > 64 || g.pad_h0 > 4096 || g.pad_w0 > 4096) return -1;

    constexpr int BH = 4;
    TilePlan p{};
    p.in = in;
    p.taps = taps;
    p.out = out;
    p.planes = g.planes();
    p.channel = g.channel;
    p.mult = 1;
    p.epi = g.epi;
    p.st.in_h = g.in_h;
    p.st.in_w = g.in_w;
    p.out_h = g.out_h;
    p.out_w = g.out_w;
    p.st.in_plane = g.in_h * g.in_w;
    p.out_plane = g.out_h * g.out_w;
    p.st.vec_in = row_vector_mode(g.in_w, in);
    p.vec_out = row_vector_mode(g.out_w, out, false);
    p.row_shift = g.pad_h0;
    p.st.col_shift = g.pad_w0;
    p.kh = g.kernel_h;
    p.kw = g.kernel_w;
    p.sh = g.down_h;
    p.sw = g.down_w;
    p.dh = g.dil_h;
    p.dw = g.dil_w;
    p.flip = !g.forward;
    p.ncb = ceil_div(p.out_w, 4);
    // stride 1, dilation 1, small extents: the register-window instances (the smallest maxima that hold the filter)
    const bool plain = p.sh == 1 && p.sw == 1 && p.dh == 1 && p.dw == 1 && env_int("DWCONV_ANY_WINDOW", 1);
    const bool windowed = plain && ((p.kh == 1 && p.kw <= 24) || (p.kw == 1 && p.kh <= 24) || (p.kh <= 8 && p.kw <= 8));
    // otherwise rows of three taps and more, next to each other, are walked four taps at a time
    const bool walk = !windowed && p.sw == 1 && p.dw == 1 && p.kw >= 3 && env_int("DWCONV_ANY_WALK", 1);
    // (the walk reads whole groups of four inputs past the last tap)
    const long used_cols = walk ? 4l * p.ncb + round_up(p.kw, 4) : static_cast<long>(4 * p.ncb - 1) * p.sw + span_w + 1;
    if (used_cols > (1 << 16)) return -1;
    const int sh = p.sh, span = static_cast<int>(span_h);
    auto rows_for = [sh, span](int units) { return (units * BH - 1) * sh + span + 1; };
    if (!plan_tiles(p, ceil_div(p.out_h, BH), BH, static_cast<int>(used_cols), p.kh * p.kw, rows_for)) return -1;
    settle_vector_modes<IO>(p);
    const dim3 grid(p.n_tiles), block(kThreads);
    const size_t shmem = lds_bytes(p, p.kh * p.kw);
    const char *window = "";
    if (walk) {
        hipLaunchKernelGGL((fir_any_kernel<IO, BH, 1, -1>), grid, block, shmem, stream, p);
        window = " walk4";
    } else if (plain && p.kh == 1 && p.kw <= 8) {
        hipLaunchKernelGGL((fir_any_kernel<IO, BH, 1, 1, 8>), grid, block, shmem, stream, p);
        window = " win1x8";
    } else if (plain && p.kh <= 8 && p.kw == 1) {
        hipLaunchKernelGGL((fir_any_kernel<IO, BH, 1, 8, 1>), grid, block, shmem, stream, p);
        window = " win8x1";
    } else if (plain && p.kh <= 4 && p.kw <= 4) {
        hipLaunchKernelGGL((fir_any_kernel<IO, BH, 1, 4, 4>), grid, block, shmem, stream, p);
        window = " win4x4";
    } else if (plain && p.kh == 1 && p.kw <= 24) {
        hipLaunchKernelGGL((fir_any_kernel<IO, BH, 1, 1, 24>), grid, block, shmem, stream, p);
        window = " win1x24";
    } else if (plain && p.kh <= 24 && p.kw == 1) {
        hipLaunchKernelGGL((fir_any_kernel<IO, BH, 1, 24, 1>), grid, block, shmem, stream, p);
        window = " win24x1";
    } else if (plain && p.kh <= 8 && p.kw <= 8) {
        hipLaunchKernelGGL((fir_any_kernel<IO, BH, 1, 8, 8>), grid, block, shmem, stream, p);
        window = " win8x8";
    } else if (p.sw == 1) hipLaunchKernelGGL((fir_any_kernel<IO, BH, 1>), grid, block, shmem, stream, p);
    else if (p.sw == 2) hipLaunchKernelGGL((fir_any_kernel<IO, BH, 2>), grid, block, shmem, stream, p);
    else hipLaunchKernelGGL((fir_any_kernel<IO, BH, 0>), grid, block, shmem, stream, p);
    note_variant("tile_any%s<k%dx%d,s%dx%d,d%dx%d,%s> P%d rows%d vin%d vout%d%s", sizeof(IO) == 2 ? "16" : "", p.kh, p.kw, p.sh, p.sw,
                 p.dh, p.dw, p.flip ? "rot" : "fwd", p.planes_per_tile, p.rows_per_tile, p.st.vec_in, p.vec_out, window);
    return check_launch("fir_any_kernel");
}

template int try_launch_fir_any<float>(const float *, const float *, float *, const Geometry &, hipStream_t);
template int try_launch_fir_any<half_t>(const half_t *, const half_t *, half_t *, const Geometry &, hipStream_t);
template int try_launch_fir_any<bf16_t>(const bf16_t *, const bf16_t *, bf16_t *, const Geometry &, hipStream_t);

template <typename IO>
int try_launch_fir_tiled(const IO *in, const IO *taps, IO *out, const Geometry &g, hipStream_t stream)
{
    const int K = g.kernel_h;
    if (g.kernel_w != K || (K != 3 && K != 5 && K != 7)) return -1;
    // leading pads beyond 7 would let the staged columns start right of the first window
    if (g.pad_h0 < 0 || g.pad_w0 < 0 || g.pad_h0 > 7 || g.pad_w0 > 7) return -1;
    if (g.in_h < 1 || g.in_w < 1) return -1;
    if (static_cast<long>(g.in_h) * g.in_w >= (1l << 30) || static_cast<long>(g.out_h) * g.out_w >= (1l << 30))
        return -1;

    TilePlan p{};
    p.in = in;
    p.taps = taps;
    p.out = out;
    p.planes = g.planes();
    p.channel = g.channel;
    p.mult = g.mult;
    if (g.mult > 1 && g.forward && g.channel % g.mult != 0) return -1;
    p.epi = g.epi;
    p.st.in_h = g.in_h;
    p.st.in_w = g.in_w;
    p.out_h = g.out_h;
    p.out_w = g.out_w;
    p.st.in_plane = g.in_h * g.in_w;
    p.out_plane = g.out_h * g.out_w;
    p.st.vec_in = row_vector_mode(g.in_w, in);
    p.vec_out = row_vector_mode(g.out_w, out, false);

    if (g.up_h == 1 && g.up_w == 1 && g.down_h == g.down_w && (g.down_h == 1 || g.down_h == 2)) {
        p.row_shift = g.pad_h0;
        p.st.col_shift = g.pad_w0;
        const bool rot = !g.forward;
        if (g.down_h == 1) {
            if (K == 3) return rot ? launch_down_bh<IO, 3, 1, true>(p, stream) : launch_down_bh<IO, 3, 1, false>(p, stream);
            if (K == 5) return rot ? launch_down_bh<IO, 5, 1, true>(p, stream) : launch_down_bh<IO, 5, 1, false>(p, stream);
            return rot ? launch_down_bh<IO, 7, 1, true>(p, stream) : launch_down_bh<IO, 7, 1, false>(p, stream);
        }
        if (rot) return -1;
        if (K == 3) return launch_down_bh<IO, 3, 2, false>(p, stream);
        if (K == 5) return launch_down_bh<IO, 5, 2, false>(p, stream);
        return launch_down_bh<IO, 7, 2, false>(p, stream);
    }
    if (g.up_h == 2 && g.up_w == 2 && g.down_h == 1 && g.down_w == 1 && !g.forward) {
        const int ey = g.pad_h0 & 1, ex = g.pad_w0 & 1;
        p.row_shift = (g.pad_h0 + ey) / 2;
        p.st.col_shift = (g.pad_w0 + ex) / 2;
        if (K == 3) return launch_up2_parity<IO, 3>(p, ey, ex, stream);
        if (K == 5) return launch_up2_parity<IO, 5>(p, ey, ex, stream);
        return launch_up2_parity<IO, 7>(p, ey, ex, stream);
    }
    return -1;
}

template int try_launch_fir_tiled<float>(const float *, const float *, float *, const Geometry &, hipStream_t);
template int try_launch_fir_tiled<half_t>(const half_t *, const half_t *, half_t *, const Geometry &, hipStream_t);
template int try_launch_fir_tiled<bf16_t>(const bf16_t *, const bf16_t *, bf16_t *, const Geometry &, hipStream_t);

}  // namespace dwconv
