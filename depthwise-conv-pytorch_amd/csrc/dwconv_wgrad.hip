// Grad-weight with LDS tiles and a fixed-order two-pass reduction (fp32, fp16 or bf16 tensors; fp32 sums).
//
//   gw[c,i,j] = sum_{n,oy,ox} gy[n,c,oy,ox] * x[n,c, oy*S - pad_h + i, ox*S - pad_w + j]
//
// Pass 1: workgroup (channel group g, chunk k) walks the tiles (image n, band of
// rows) of its chunk.  Per tile the band of x (with halo) is staged in LDS exactly
// as in the forward kernel; each lane owns a BH x 4 block of gy, read straight
// from global memory, and accumulates all K*K taps in registers from one pass
// over the LDS window.  So x and gy are read once, not K*K times as in the
// reference's one-block-per-tap kernel (torch_dwconv/dwconv_kernel.cu:260-306),
// and nothing is accumulated with atomics.  At the end the lanes' K*K sums are
// reduced in a fixed order (DPP within a wavefront, LDS across wavefronts) and
// stored as partial[c][k][tap].
// Pass 2: one lane per (c, tap) adds the chunk partials front to back in double.
//
// Large maps use one channel per workgroup (all 256 lanes reduce into one tap
// table); small maps put P channels of one image side by side, each lane staying
// with its channel for the whole chunk.
#include <type_traits>
#include "dwconv_tile_common.hpp"

namespace dwconv {

namespace {

struct WgradPlan {
    StageLayout st;
    const void *x;    // element type IO of the kernel template
    const void *gy;
    float *partial;
    int batch, channel;
    int out_h, out_w, out_plane;
    int pad_h;
    int rows_per_tile, row_tiles;
    int planes_per_tile;   // channels a workgroup carries
    int groups;            // channel groups = ceil(C / planes_per_tile)
    int chunks;            // chunks per channel group
    int tiles_per_group;   // batch * row_tiles
    int tiles_per_chunk;
    int ncb;
    unsigned ncb_magic;
    int items_per_plane;
    unsigned ipp_magic;
    int vec_gy;
    // fused grad-input (stride 1, "same" padding): taps, destination, and where the gy image sits in LDS
    const void *taps;
    void *gx;
    int g_base;            // float offset of the gy image (same layout as the x image)
    int vec_gx;
    int strided;           // chunk k takes tiles k, k+chunks, ... instead of a contiguous range
    int lds_gx;            // fused: grad-input goes back through LDS and leaves as one linear stream (one plane per tile)
    int mult;              // depth multiplier M (grad-weight alone, one plane per tile): `channel` counts the channels of
                           // gy and of the taps; plane (n, c) of gy meets plane (n, c / M) of an x with channel / M channels
};

// GX (stride 1, pad = K/2 only): the band of gy is staged in LDS next to the band of x, with the same
// layout.  The lane first walks its gy window: that gives its block of grad-input (gy against the
// rotated taps, stored straight to memory) and, from the window's centre, its block of gy for the
// grad-weight sums.  gy is read from HBM once for both gradients.

// ANY_WIDTH: the instance for rows that are not whole, aligned groups of four elements (a mode 3 among st.vec_in,
// vec_gy, vec_gx); the other instance carries none of it.
template <typename IO, int K, int S, int BH, bool GX, bool ANY_WIDTH = false>
__global__ __launch_bounds__(kThreads) void wgrad_tile_kernel(const WgradPlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int KK = K * K;
    constexpr int WIN_ROWS = (BH - 1) * S + K;
    constexpr int NV = (3 * S + K + 3) / 4;
    static_assert(!GX || S == 1, "the fused variant is the stride-1 one");
    const IO *const x = static_cast<const IO *>(p.x);
    const IO *const gy = static_cast<const IO *>(p.gy);

    const int group = blockIdx.x / p.chunks;
    const int chunk = blockIdx.x - group * p.chunks;
    const int c0 = group * p.planes_per_tile;
    const int nplanes = min(p.planes_per_tile, p.channel - c0);
    // Chunk k takes tiles k, k + chunks, k + 2*chunks, ...: at any moment the workgroups of the grid
    // work on a narrow window of images, which keeps the DRAM pages they stream from open.
    const int t_begin = p.strided ? chunk : chunk * p.tiles_per_chunk;
    const int t_end = p.strided ? p.tiles_per_group : min(p.tiles_per_group, t_begin + p.tiles_per_chunk);
    const int t_step = p.strided ? p.chunks : 1;
    const int n_items = nplanes * p.items_per_plane;

    float acc[KK];
#pragma unroll
    for (int t = 0; t < KK; ++t) acc[t] = 0.f;

    // One item per lane (the planner guarantees n_items <= blockDim.x): its place in the tile is fixed.
    const bool has_item = static_cast<int>(threadIdx.x) < n_items;
    const int item = has_item ? threadIdx.x : 0;
    const int pl = fast_div(item, p.ipp_magic);
    const int rem = item - pl * p.items_per_plane;
    const int rb = fast_div(rem, p.ncb_magic);
    const int cb = rem - rb * p.ncb;
    const int ox = 4 * cb;
    const float *base = lds + pl * p.st.plane_pitch + (rb * BH * S) * p.st.pitch + kSlack + 4 * cb * S;

    float rot[GX ? KK : 1];
    if constexpr (GX) {
#pragma unroll
        for (int t = 0; t < KK; ++t) rot[t] = Io<IO>::in(static_cast<const IO *>(p.taps)[(c0 + pl) * KK + KK - 1 - t]);
    }

    for (int tile = t_begin; tile < t_end; tile += t_step) {
        const int n = tile / p.row_tiles, rt = tile - n * p.row_tiles;
        const long plane0 = static_cast<long>(n) * p.channel + c0;
        const int oy0 = rt * p.rows_per_tile;

        // this lane's block of gy (zero where it hangs over the edge of the plane); issued before the
        // x band is staged so that both sets of loads are in flight together
        float g[BH][4];
        const IO *gsrc = gy + (plane0 + pl) * p.out_plane + ox;
#pragma unroll
        for (int b = 0; b < BH; ++b) {
            if constexpr (GX) break;
            const int oy = oy0 + rb * BH + b;
            const IO *row = gsrc + static_cast<long>(oy) * p.out_w;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (p.vec_gy == 2 || (ANY_WIDTH && p.vec_gy == 3)) {
                // branch-free: rows past the plane (and lanes without an item) read zeros through the view
                const unsigned off = ((pl * p.out_plane + ox) + oy * p.out_w) * static_cast<unsigned>(sizeof(IO));
                if (ANY_WIDTH && p.vec_gy == 3 && mixed_row_starts(gy + plane0 * p.out_plane, p.out_w)) {
                    // (16-bit rows that do not all start on 32-bit boundaries)
                    v = any_width_load4<IO>(any_width_view(gy + plane0 * p.out_plane, static_cast<long>(nplanes) * p.out_plane * sizeof(IO)),
                                            has_item && oy < p.out_h ? off : kOob);
                    keep_first(v, p.out_w - ox);
                } else if (ANY_WIDTH && p.vec_gy == 3) {  // rows of any width: the block that ends a row is cut short
                    v = view_load4<IO>(buffer_view(gy + plane0 * p.out_plane, static_cast<long>(nplanes) * p.out_plane * sizeof(IO)), has_item && oy < p.out_h ? off : kOob);
                    keep_first(v, p.out_w - ox);
                } else {
                    v = view_load4<IO>(buffer_view(gy + plane0 * p.out_plane, static_cast<long>(nplanes) * p.out_plane * sizeof(IO)), has_item && oy < p.out_h ? off : kOob);
                }
            } else if (has_item && oy < p.out_h) {
                if (p.vec_gy) {
                    v = load4<IO>(row);
                } else {
                    if (ox + 0 < p.out_w) v.x = Io<IO>::in(row[0]);
                    if (ox + 1 < p.out_w) v.y = Io<IO>::in(row[1]);
                    if (ox + 2 < p.out_w) v.z = Io<IO>::in(row[2]);
                    if (ox + 3 < p.out_w) v.w = Io<IO>::in(row[3]);
                }
            }
            g[b][0] = v.x;
            g[b][1] = v.y;
            g[b][2] = v.z;
            g[b][3] = v.w;
        }

        if (tile != t_begin) __syncthreads();  // the previous tile's window reads are done
        stage_tile<IO, false, kStageBatch, false, ANY_WIDTH>(p.st, x, lds, p.mult > 1 ? static_cast<long>(n) * (p.channel / p.mult) + c0 / p.mult : plane0,
                                                             nplanes, oy0 * S - p.pad_h);
        if constexpr (GX) stage_tile<IO, false, kStageBatch, false, ANY_WIDTH>(p.st, gy, lds + p.g_base, plane0, nplanes, oy0 - p.pad_h);
        __syncthreads();

        float xacc[GX ? BH : 1][4];  // grad-input block (kept until the tile's window reads are over when it leaves through LDS)
        if constexpr (GX) {
            constexpr int PC = K / 2;  // the lane's own gy block sits PC rows and columns into its window
#pragma unroll
            for (int b = 0; b < BH; ++b)
#pragma unroll
                for (int o = 0; o < 4; ++o) xacc[b][o] = 0.f;
            float nxt[4 * NV];
            load_window_row<NV>(base + p.g_base, nxt);
#pragma unroll
            for (int wr = 0; wr < WIN_ROWS; ++wr) {
                float win[4 * NV];
#pragma unroll
                for (int i = 0; i < 4 * NV; ++i) win[i] = nxt[i];
                if (wr + 1 < WIN_ROWS) load_window_row<NV>(base + p.g_base + (wr + 1) * p.st.pitch, nxt);
                const int gb = wr - PC;
                if (gb >= 0 && gb < BH) {
#pragma unroll
                    for (int o = 0; o < 4; ++o) g[gb >= 0 && gb < BH ? gb : 0][o] = has_item ? win[o + PC] : 0.f;
                }
#pragma unroll
                for (int b = 0; b < BH; ++b) {
                    const int ty = wr - b;
                    if (ty < 0 || ty >= K) continue;
#pragma unroll
                    for (int tx = 0; tx < K; ++tx)
#pragma unroll
                        for (int o = 0; o < 4; ++o) xacc[b][o] = fmaf(win[o + tx], rot[ty * K + tx], xacc[b][o]);
                }
                pin_registers(xacc);
            }
            if (p.lds_gx) {
                // stored after the grad-weight sums, below
            } else if (p.vec_gx == 2 || (ANY_WIDTH && p.vec_gx == 3)) {
                // branch-free: rows past the end of the plane (and lanes without an item) store out of range
                const __amdgpu_buffer_rsrc_t view = buffer_view(static_cast<IO *>(p.gx) + plane0 * p.st.in_plane, static_cast<long>(nplanes) * p.st.in_plane * sizeof(IO));
                const unsigned o0 = (pl * p.st.in_plane + ox) * static_cast<unsigned>(sizeof(IO));
                bool done = false;
                if constexpr (ANY_WIDTH) {
                    if (p.vec_gx == 3) {  // the block that ends a row may be short
#pragma unroll
                        for (int b = 0; b < BH; ++b) {
                            const int oy = oy0 + rb * BH + b;
                            const bool ok = has_item && oy < p.st.in_h;
                            view_store_first<IO>(view, ok ? o0 + oy * p.st.in_w * static_cast<unsigned>(sizeof(IO)) : kOob,
                                                 p.st.in_w - ox, p.st.in_w & 3, xacc[b][0], xacc[b][1], xacc[b][2], xacc[b][3]);
                        }
                        done = true;
                    }
                }
                if (!done) {
#pragma unroll
                    for (int b = 0; b < BH; ++b) {
                        const int oy = oy0 + rb * BH + b;
                        const bool ok = has_item && oy < p.st.in_h;
                        view_store4<IO>(view, ok ? o0 + oy * p.st.in_w * static_cast<unsigned>(sizeof(IO)) : kOob, xacc[b][0],
                                        xacc[b][1], xacc[b][2], xacc[b][3]);
                    }
                }
            } else if (has_item) {
                IO *dst = static_cast<IO *>(p.gx) + (plane0 + pl) * p.st.in_plane + ox;
#pragma unroll
                for (int b = 0; b < BH; ++b) {
                    const int oy = oy0 + rb * BH + b;
                    if (oy >= p.st.in_h) continue;
                    IO *row = dst + static_cast<long>(oy) * p.st.in_w;
                    if (p.vec_gx) {
                        store4<IO>(row, xacc[b][0], xacc[b][1], xacc[b][2], xacc[b][3]);
                    } else {
#pragma unroll
                        for (int o = 0; o < 4; ++o)
                            if (ox + o < p.st.in_w) row[o] = Io<IO>::out(xacc[b][o]);
                    }
                }
            }
        }

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
                        acc[ty * K + tx] = fmaf(g[b][o], win[o * S + tx], acc[ty * K + tx]);
            }
            pin_registers(acc);
        }

        if constexpr (GX) {
            if (p.lds_gx) {
                // One plane per tile (the planner guarantees it).  The grad-input block goes into LDS in the layout the
                // band has in memory, over the x image, and leaves as one linear stream: every store of a wavefront
                // covers 1 KiB of consecutive bytes.  Lane-owned blocks write a row segment per instruction, and rows
                // that are not whole 64-byte bursts (56 floats) leave the bursts that straddle two rows to two writes.
                const int rows_here = min(p.rows_per_tile, p.st.in_h - oy0);
                const int run = rows_here * p.st.in_w;  // floats, a multiple of four
                __syncthreads();                        // every window has been read
                if (has_item) {
#pragma unroll
                    for (int b = 0; b < BH; ++b)
                        if (rb * BH + b < rows_here)
                            *reinterpret_cast<float4 *>(lds + (rb * BH + b) * p.st.in_w + ox) =
                                make_float4(xacc[b][0], xacc[b][1], xacc[b][2], xacc[b][3]);
                }
                __syncthreads();
                const __amdgpu_buffer_rsrc_t view = buffer_view(static_cast<IO *>(p.gx) + plane0 * p.st.in_plane, static_cast<long>(p.st.in_plane) * sizeof(IO));
                const unsigned o0 = oy0 * p.st.in_w * static_cast<unsigned>(sizeof(IO));
                for (int i = threadIdx.x; i < (run >> 2); i += blockDim.x) {
                    const float4 v = reinterpret_cast<const float4 *>(lds)[i];
                    view_store4<IO>(view, o0 + i * 4 * static_cast<unsigned>(sizeof(IO)), v.x, v.y, v.z, v.w);
                }
            }
        }
    }

    __syncthreads();  // the tile image is dead; its LDS is reused for the reduction
    float *out = p.partial + (static_cast<long>(c0) * p.chunks + chunk) * KK;
    if (p.planes_per_tile == 1) {
        // every lane worked on the same channel: wavefront sums, then the four wavefronts in order
#pragma unroll
        for (int t = 0; t < KK; ++t) {
            const float s = wave_sum_to_last_lane(acc[t]);
            if ((threadIdx.x & 63) == 63) lds[(threadIdx.x >> 6) * KK + t] = s;
        }
        __syncthreads();
        if (threadIdx.x < KK) {
            float s = lds[threadIdx.x];
#pragma unroll
            for (int w = 1; w < kThreads / 64; ++w) s += lds[w * KK + threadIdx.x];
            out[threadIdx.x] = s;
        }
    } else {
        // lanes [pl*ipp, (pl+1)*ipp) hold channel c0+pl: transpose through LDS, then add each run front to back
#pragma unroll
        for (int t = 0; t < KK; ++t) lds[t * kRedPitch + threadIdx.x] = acc[t];
        __syncthreads();
        for (int e = threadIdx.x; e < nplanes * KK; e += blockDim.x) {
            const int pl = e / KK, t = e - pl * KK;
            const float *col = lds + t * kRedPitch + pl * p.items_per_plane;
            float s = 0.f;
            for (int i = 0; i < p.items_per_plane; ++i) s += col[i];
            out[static_cast<long>(pl) * p.chunks * KK + t] = s;
        }
    }
}

// Pass 2: gw[c,tap] = sum over chunks of partial[c][chunk][tap], in double and in a fixed order.
// kFinalLanes lanes share one output: each adds a contiguous share of the chunks front to back, then the
// shares are combined by a fixed butterfly.  The loads are issued eight at a time with the ones past the
// lane's share replaced by zero, never one by one: the kernel then costs one or two memory latencies
// whatever the chunk count (a scalar tail loop made it one latency per chunk, 4.6 us for 43 chunks).
constexpr int kFinalLanes = 8;

template <typename IO>
__global__ __launch_bounds__(256) void wgrad_tile_final_kernel(const float *__restrict__ partial,
                                                               IO *__restrict__ gw, const int channel_taps,
                                                               const int taps, const int chunks)
{
    const int gid = blockIdx.x * blockDim.x + threadIdx.x;
    const int e = gid / kFinalLanes, part = gid - e * kFinalLanes;
    const bool live = e < channel_taps;
    const int ee = live ? e : 0;
    const int c = ee / taps, t = ee - c * taps;
    const float *p = partial + static_cast<long>(c) * chunks * taps + t;
    const int per = (chunks + kFinalLanes - 1) / kFinalLanes;
    const int k0 = part * per, k1 = min(chunks, k0 + per);
    double s = 0.0;
    for (int k = k0; k < k1; k += 8) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = p[static_cast<long>(min(k + j, k1 - 1)) * taps];
#pragma unroll
        for (int j = 0; j < 8; ++j) s += static_cast<double>(k + j < k1 ? v[j] : 0.f);
    }
#pragma unroll
    for (int off = 1; off < kFinalLanes; off <<= 1) s += __shfl_xor(s, off, 64);
    if (live && part == 0) gw[e] = Io<IO>::out(static_cast<float>(s));
}

// Grad-weight for any filter extent, stride and dilation (what make_plan's filter sizes do not cover: rectangular,
// even-sized and strip filters, strides above 2, dilated taps): one channel per workgroup, the same chunks and
// partial sums, the taps looped over at run time.  A workgroup keeps up to kAnyTaps sums per lane (the loop over
// them is unrolled under a uniform bound, so the sums stay in registers); larger filters are cut into passes of
// kAnyTaps taps (blockIdx.y), each of which stages the x bands again.  One LDS read per multiply-add.
constexpr int kAnyTaps = 64;

struct AnyTaps {
    int kh, kw, sh, sw, dh, dw;
    int walk;    // rows of taps walked in groups of four (the KHM < 0 instance)
    int passes;  // launches of kAnyTaps sums each (blockIdx.y)
};

constexpr int kWalkGroups = kAnyTaps / 4;  // groups of four taps per pass
constexpr int kRedSums = 32;               // sums that cross LDS at a time where a workgroup carries several channels

// KHM x KWM (0: none): at stride 1 and dilation 1, filters of at most that extent (and at most kAnyTaps taps) walk a
// register window of x rows instead: a row of 3 + kw inputs is read once for every tap and gy row that meets it, the
// loops unrolled to the maxima under uniform bounds; sum (ty, tx) lives in acc[ty * KWM + tx].
// KHM < 0: column stride 1, undilated columns, any extent: every filter row is cut into groups of four taps, a pass
// holds kWalkGroups of them, and a group takes its sums from eight inputs per gy row (two 16-byte LDS reads, the
// first shared with the group before it in the same row).
template <typename IO, int BH, int SW, int KHM = 0, int KWM = 0>
__global__ __launch_bounds__(kThreads) void wgrad_any_kernel(const WgradPlan p, const AnyTaps a)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    const IO *const x = static_cast<const IO *>(p.x);
    const IO *const gy = static_cast<const IO *>(p.gy);
    const int KK = a.kh * a.kw;
    const int sw = SW ? SW : a.sw;
    const int t_first = blockIdx.y * kAnyTaps;
    const int nt = min(kAnyTaps, KK - t_first);

    // a workgroup carries planes_per_tile channels (whole small planes side by side, one block per lane) or one
    const int grp = blockIdx.x / p.chunks;
    const int chunk = blockIdx.x - grp * p.chunks;
    const int c = grp * p.planes_per_tile;
    const int nplanes = min(p.planes_per_tile, p.channel - c);

    constexpr int kSums = KHM > 0 ? KHM * KWM : kAnyTaps;
    float acc[kSums];
#pragma unroll
    for (int t = 0; t < kSums; ++t) acc[t] = 0.f;

    const bool has_item = static_cast<int>(threadIdx.x) < nplanes * p.items_per_plane;
    const int item = has_item ? threadIdx.x : 0;
    const int pl = p.planes_per_tile > 1 ? fast_div(item, p.ipp_magic) : 0;
    const int rem = item - __mul24(pl, p.items_per_plane);
    const int rb = fast_div(rem, p.ncb_magic);
    const int cb = rem - rb * p.ncb;
    const int ox = 4 * cb;
    const int row_step = a.sh * p.st.pitch;
    const float *base = lds + __mul24(pl, p.st.plane_pitch) + __mul24(rb * BH, row_step) + kSlack + 4 * cb * sw;
    const int ty_first = t_first / a.kw, tx_first = t_first - ty_first * a.kw;

    for (int tile = chunk; tile < p.tiles_per_group; tile += p.chunks) {
        const int n = tile / p.row_tiles, rt = tile - n * p.row_tiles;
        const long plane0 = static_cast<long>(n) * p.channel + c;
        const int oy0 = rt * p.rows_per_tile;

        // this lane's block of gy (zero where it hangs over the edge of the plane, and for lanes without an item)
        float g[BH][4];
        const IO *gsrc = gy + (plane0 + pl) * p.out_plane + ox;
        const long gy_bytes = static_cast<long>(nplanes) * p.out_plane * sizeof(IO);
#pragma unroll
        for (int b = 0; b < BH; ++b) {
            const int oy = oy0 + rb * BH + b;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (p.vec_gy >= 2) {
                const unsigned off = (__mul24(pl, p.out_plane) + ox + oy * p.out_w) * static_cast<unsigned>(sizeof(IO));
                const bool ok = has_item && oy < p.out_h;
                if (p.vec_gy == 3 && mixed_row_starts(gy + plane0 * p.out_plane, p.out_w))
                    v = any_width_load4<IO>(any_width_view(gy + plane0 * p.out_plane, gy_bytes), ok ? off : kOob);
                else
                    v = view_load4<IO>(buffer_view(gy + plane0 * p.out_plane, gy_bytes), ok ? off : kOob);
                if (p.vec_gy == 3) keep_first(v, p.out_w - ox);
            } else if (has_item && oy < p.out_h) {
                const IO *row = gsrc + static_cast<long>(oy) * p.out_w;
                if (p.vec_gy) {
                    v = load4<IO>(row);
                } else {
                    if (ox + 0 < p.out_w) v.x = Io<IO>::in(row[0]);
                    if (ox + 1 < p.out_w) v.y = Io<IO>::in(row[1]);
                    if (ox + 2 < p.out_w) v.z = Io<IO>::in(row[2]);
                    if (ox + 3 < p.out_w) v.w = Io<IO>::in(row[3]);
                }
            }
            g[b][0] = v.x;
            g[b][1] = v.y;
            g[b][2] = v.z;
            g[b][3] = v.w;
        }

        if (tile != chunk) __syncthreads();  // the previous tile's window reads are done
        stage_tile(p.st, x, lds, plane0, nplanes, oy0 * a.sh - p.pad_h);
        __syncthreads();

        if constexpr (KHM > 0) {
            static_assert(SW == 1 && KHM * KWM <= kAnyTaps, "the register window is the stride-1 case, one pass");
#pragma unroll
            for (int wr = 0; wr < BH - 1 + KHM; ++wr) {
                if (wr < BH - 1 + a.kh) {  // (uniform)
                    const float *r = base + wr * p.st.pitch;
                    // (16-byte LDS reads: consecutive lanes then read consecutive banks; the last may reach into the
                    // slack of the row)
                    float win[4 * ((3 + KWM + 3) / 4)];
#pragma unroll
                    for (int v = 0; v < (3 + KWM + 3) / 4; ++v) {
                        float4 q = make_float4(0.f, 0.f, 0.f, 0.f);
                        if (4 * v < 3 + a.kw) q = *reinterpret_cast<const float4 *>(r + 4 * v);
                        win[4 * v] = q.x, win[4 * v + 1] = q.y, win[4 * v + 2] = q.z, win[4 * v + 3] = q.w;
                    }
#pragma unroll
                    for (int b = 0; b < BH; ++b) {
                        const int wy = wr - b;
                        if (wy < 0 || wy >= KHM) continue;
                        if (wy < a.kh) {
#pragma unroll
                            for (int wx = 0; wx < KWM; ++wx) {
                                if (wx < a.kw) {
                                    float sum = acc[wy * KWM + wx];
#pragma unroll
                                    for (int o = 0; o < 4; ++o) sum = fmaf(g[b][o], win[o + wx], sum);
                                    acc[wy * KWM + wx] = sum;
                                }
                            }
                        }
                    }
                    pin_registers(acc);
                }
            }
            continue;
        }
        if constexpr (KHM < 0) {
            static_assert(SW == 1, "rows are walked four inputs at a time at column stride 1");
            const int gpr = (a.kw + 3) >> 2, groups = a.kh * gpr;
            const int g_first = blockIdx.y * kWalkGroups;
            int wy = g_first / gpr, wg = g_first - wy * gpr;
            float w[BH][8];
#pragma unroll
            for (int q = 0; q < kWalkGroups; ++q) {
                if (g_first + q < groups) {  // (uniform)
                    const float *r = base + __mul24(wy * a.dh, p.st.pitch) + 4 * wg;
                    if (q == 0 || wg == 0) {
#pragma unroll
                        for (int b = 0; b < BH; ++b) {
                            const float4 v = *reinterpret_cast<const float4 *>(r + b * row_step);
                            w[b][4] = v.x, w[b][5] = v.y, w[b][6] = v.z, w[b][7] = v.w;
                        }
                    }
#pragma unroll
                    for (int b = 0; b < BH; ++b) {
                        const float4 v = *reinterpret_cast<const float4 *>(r + b * row_step + 4);
#pragma unroll
                        for (int i = 0; i < 4; ++i) w[b][i] = w[b][4 + i];
                        w[b][4] = v.x, w[b][5] = v.y, w[b][6] = v.z, w[b][7] = v.w;
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if (4 * wg + j < a.kw) {  // (uniform)
                            float sum = acc[4 * q + j];
#pragma unroll
                            for (int b = 0; b < BH; ++b)
#pragma unroll
                                for (int o = 0; o < 4; ++o) sum = fmaf(g[b][o], w[b][j + o], sum);
                            acc[4 * q + j] = sum;
                        }
                    }
                    if (++wg == gpr) {
                        wg = 0;
                        ++wy;
                    }
                }
            }
            continue;
        }
        int ty = ty_first, tx = tx_first;
#pragma unroll
        for (int t = 0; t < kAnyTaps; ++t) {
            if (t < nt) {  // (uniform)
                float sum = acc[t];
                if constexpr (SW == 1 || SW == 2) {
                    // lanes are four or eight floats apart: 16-byte LDS reads from the boundary before the tap's offset
                    // on (the last may reach into the slack of the row) and a uniform choice among what they hold,
                    // instead of single floats that would meet the same banks four or eight times over
                    const int off = tx * a.dw;
                    const float *r = base + __mul24(ty * a.dh, p.st.pitch) + (off & ~3);
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
                            for (int o = 0; o < 4; ++o) sum = fmaf(g[b][o], w8[S + o * SW], sum);
                        }
                    };
                    switch (off & 3) {
                    case 0: rows(std::integral_constant<int, 0>{}); break;
                    case 1: rows(std::integral_constant<int, 1>{}); break;
                    case 2: rows(std::integral_constant<int, 2>{}); break;
                    default: rows(std::integral_constant<int, 3>{}); break;
                    }
                } else {
                    const float *r = base + __mul24(ty * a.dh, p.st.pitch) + tx * a.dw;
#pragma unroll
                    for (int b = 0; b < BH; ++b)
#pragma unroll
                        for (int o = 0; o < 4; ++o) sum = fmaf(g[b][o], r[b * row_step + o * sw], sum);
                }
                acc[t] = sum;
                if (++tx == a.kw) {
                    tx = 0;
                    ++ty;
                }
            }
        }
    }

    __syncthreads();  // the tile image is dead; its LDS is reused for the reduction
    if (p.planes_per_tile > 1) {
        // lanes [q * ipp, (q + 1) * ipp) hold channel c + q: the sums cross LDS kRedSums at a time, a column per lane,
        // then one lane per (channel, sum) adds its run front to back
#pragma unroll
        for (int s0 = 0; s0 < kSums; s0 += kRedSums) {
            if (s0) __syncthreads();
#pragma unroll
            for (int t = 0; t < kRedSums; ++t)
                if (s0 + t < kSums) lds[t * kRedPitch + threadIdx.x] = acc[s0 + t];
            __syncthreads();
            for (int e = threadIdx.x; e < nplanes * kRedSums; e += blockDim.x) {
                const int q = e / kRedSums, t = e - q * kRedSums, slot = s0 + t;
                int tap = -1;  // the tap that sum `slot` belongs to
                if constexpr (KHM > 0) {
                    const int wy = slot / KWM, wx = slot - wy * KWM;
                    if (slot < kSums && wy < a.kh && wx < a.kw) tap = wy * a.kw + wx;
                } else if constexpr (KHM < 0) {
                    const int gpr = (a.kw + 3) >> 2;
                    const int walk_group = blockIdx.y * kWalkGroups + (slot >> 2);
                    const int wy = walk_group / gpr, wx = 4 * (walk_group - wy * gpr) + (slot & 3);
                    if (wy < a.kh && wx < a.kw) tap = wy * a.kw + wx;
                } else {
                    if (slot < nt) tap = t_first + slot;
                }
                if (tap >= 0) {
                    const float *col = lds + t * kRedPitch + q * p.items_per_plane;
                    float sum = 0.f;
                    for (int i = 0; i < p.items_per_plane; ++i) sum += col[i];
                    p.partial[(static_cast<long>(c + q) * p.chunks + chunk) * KK + tap] = sum;
                }
            }
        }
        return;
    }
    // every lane worked on the same channel: wavefront sums, then the four wavefronts in order
    if constexpr (KHM > 0) {
#pragma unroll
        for (int wy = 0; wy < KHM; ++wy)
#pragma unroll
            for (int wx = 0; wx < KWM; ++wx) {
                if (wy < a.kh && wx < a.kw) {
                    const float sum = wave_sum_to_last_lane(acc[wy * KWM + wx]);
                    if ((threadIdx.x & 63) == 63) lds[(threadIdx.x >> 6) * kAnyTaps + wy * a.kw + wx] = sum;
                }
            }
    } else if constexpr (KHM < 0) {
        const int gpr = (a.kw + 3) >> 2, groups = a.kh * gpr;
        const int g_first = blockIdx.y * kWalkGroups;
#pragma unroll
        for (int t = 0; t < kAnyTaps; ++t) {
            if (g_first + t / 4 < groups) {
                const float sum = wave_sum_to_last_lane(acc[t]);
                if ((threadIdx.x & 63) == 63) lds[(threadIdx.x >> 6) * kAnyTaps + t] = sum;
            }
        }
        __syncthreads();
        const int grp = g_first + static_cast<int>(threadIdx.x >> 2);
        const int wy = grp / gpr, wx = 4 * (grp - wy * gpr) + static_cast<int>(threadIdx.x & 3);
        if (threadIdx.x < kAnyTaps && grp < groups && wx < a.kw) {
            float sum = lds[threadIdx.x];
#pragma unroll
            for (int w = 1; w < kThreads / 64; ++w) sum += lds[w * kAnyTaps + threadIdx.x];
            p.partial[(static_cast<long>(c) * p.chunks + chunk) * KK + wy * a.kw + wx] = sum;
        }
        return;
    } else {
#pragma unroll
        for (int t = 0; t < kAnyTaps; ++t) {
            if (t < nt) {
                const float sum = wave_sum_to_last_lane(acc[t]);
                if ((threadIdx.x & 63) == 63) lds[(threadIdx.x >> 6) * kAnyTaps + t] = sum;
            }
        }
    }
    __syncthreads();
    if (static_cast<int>(threadIdx.x) < nt) {
        float sum = lds[threadIdx.x];
#pragma unroll
        for (int w = 1; w < kThreads / 64; ++w) sum += lds[w * kAnyTaps + threadIdx.x];
        p.partial[(static_cast<long>(c) * p.chunks + chunk) * KK + t_first + threadIdx.x] = sum;
    }
}

// The plan of wgrad_any_kernel for g (dilation dil_h x dil_w), or false.
bool make_any_plan(WgradPlan &p, AnyTaps &a, const WgradGeometry &g, int dil_h, int dil_w)
{
    constexpr int BH = 4;
    if (g.mult != 1 || g.kernel_h < 1 || g.kernel_w < 1 || g.down_h < 1 || g.down_w < 1 || dil_h < 1 || dil_w < 1) return false;
    if (g.pad_h < 0 || g.pad_w < 0 || g.in_h < 1 || g.in_w < 1 || g.out_h < 1 || g.out_w < 1) return false;
    const long KK = static_cast<long>(g.kernel_h) * g.kernel_w;
    if (KK > 4096) return false;
    if (static_cast<long>(g.in_h) * g.in_w >= (1l << 30) || static_cast<long>(g.out_h) * g.out_w >= (1l << 30)) return false;
    const long span_h = static_cast<long>(g.kernel_h - 1) * dil_h, span_w = static_cast<long>(g.kernel_w - 1) * dil_w;
    if (span_h > 4096 || span_w > 4096 || g.down_h > 64 || g.down_w > 64 || g.pad_h > 4096 || g.pad_w > 4096) return false;
    a = AnyTaps{g.kernel_h, g.kernel_w, g.down_h, g.down_w, dil_h, dil_w, 0, 1};
    const bool plain = a.sh == 1 && a.sw == 1 && a.dh == 1 && a.dw == 1 && env_int("DWCONV_ANY_WINDOW", 1);
    const bool windowed = plain && ((a.kh == 1 && a.kw <= 24) || (a.kw == 1 && a.kh <= 24) || (a.kh <= 8 && a.kw <= 8));
    a.walk = !windowed && a.sw == 1 && a.dw == 1 && a.kw >= 3 && env_int("DWCONV_ANY_WALK", 1);
    a.passes = a.walk ? ceil_div(a.kh * ceil_div(a.kw, 4), kWalkGroups) : ceil_div(static_cast<int>(KK), kAnyTaps);
    p.batch = g.batch;
    p.channel = g.channel;
    p.out_h = g.out_h;
    p.out_w = g.out_w;
    p.out_plane = g.out_h * g.out_w;
    p.pad_h = g.pad_h;
    p.st.in_h = g.in_h;
    p.st.in_w = g.in_w;
    p.st.in_plane = g.in_h * g.in_w;
    p.st.col_shift = g.pad_w;
    p.ncb = ceil_div(g.out_w, 4);
    if (p.ncb > kThreads) return false;
    // (the walk reads whole groups of four inputs past the last tap)
    const long used_cols = a.walk ? 4l * p.ncb + round_up(a.kw, 4) : static_cast<long>(4 * p.ncb - 1) * g.down_w + span_w + 1;
    if (used_cols > (1 << 16)) return false;
    layout_columns(p.st, static_cast<int>(used_cols));
    auto rows_for = [&](int units) { return static_cast<long>(units * BH - 1) * g.down_h + span_h + 1; };
    auto bytes = [&](int units) { return rows_for(units) * p.st.pitch * 4; };
    const int row_units = ceil_div(g.out_h, BH);
    int units = std::max(1, std::min(row_units, kThreads / p.ncb));
    while (units > 1 && bytes(units) > dwconv::kLdsBudget) --units;
    if (bytes(units) > dwconv::kLdsBudget) return false;
    units = ceil_div(row_units, ceil_div(row_units, units));  // even out the bands
    // small planes: whole planes of several channels side by side, a block per lane (14x14 with 15x15 taps: 16 of 256
    // lanes would have one otherwise)
    int planes = 1;
    const int ipp_full = row_units * p.ncb;
    if (units == row_units && 2 * ipp_full <= kThreads && g.channel > 1 && env_int("DWCONV_WGRAD_ANY_PLANES", 1)) {
        planes = std::min(kThreads / ipp_full, g.channel);
        while (planes > 1 && planes * bytes(units) > dwconv::kLdsBudget) --planes;
    }
    p.planes_per_tile = planes;
    p.groups = ceil_div(g.channel, planes);
    p.rows_per_tile = units * BH;
    p.row_tiles = ceil_div(row_units, units);
    if (!layout_rows(p.st, static_cast<int>(rows_for(units)), planes)) return false;
    p.items_per_plane = units * p.ncb;
    p.ncb_magic = magic_u16(p.ncb);
    p.ipp_magic = magic_u16(p.items_per_plane);
    const long tiles = static_cast<long>(g.batch) * p.row_tiles;
    if (tiles > 0x7fffffffL) return false;
    p.tiles_per_group = static_cast<int>(tiles);
    // Three workgroups fit a CU (the sums take the registers), and the 64-sum reduction at a workgroup's end is its
    // largest fixed cost: 768 workgroups in all, passes included, every one resident from the start, measured best
    // (atrous 3x3 on 65x65 C=256: 98 -> 83 us; 8x8 on 128x128: 78 -> 68; 10x10, two passes: 141 -> 110; 15x15, four:
    // 268 -> 214; 31x31 on 56x56, sixteen: 401 -> 299; 1024 and 1536 leave a second, part-filled round: 10-20 %
    // slower); channels that fill less than two such rounds on their own get two chunks each.
    const long lanes = static_cast<long>(p.groups) * a.passes;
    const long target = env_int("DWCONV_WGRAD_WGS", 768);
    int chunks = static_cast<int>(std::min<long>(std::max<long>((target + lanes - 1) / lanes, lanes < 1536 ? 2 : 1), 1 << 20));
    if (chunks > p.tiles_per_group) chunks = p.tiles_per_group;
    if (chunks < 1) chunks = 1;
    p.chunks = chunks;
    p.tiles_per_chunk = ceil_div(p.tiles_per_group, chunks);
    p.strided = 1;
    if (static_cast<long>(p.groups) * chunks > 0x7fffffffL) return false;
    return true;
}

template <int K, int S, int BH>
bool make_plan(WgradPlan &p, const WgradGeometry &g, bool fused)
{
    constexpr int NV = (3 * S + K + 3) / 4;
    constexpr int KK = K * K;
    // Workgroups in all: the 3x3 kernels gain 2-3 % from four times as many, shorter chunks; the 5x5 ones, whose
    // per-workgroup reduction of K*K sums weighs more, lose 6-7 %; with 49 sums per lane the 7x7 ones want half as
    // many again (56x56 fused backward: 124 -> 114 us).
    const int target_wgs = env_int(K == 3 ? "DWCONV_WGRAD_WGS_K3" : "DWCONV_WGRAD_WGS", K == 3 ? 12288 : (K == 5 ? 3072 : 1536));
    p.batch = g.batch;
    p.channel = g.channel;
    p.out_h = g.out_h;
    p.out_w = g.out_w;
    p.out_plane = g.out_h * g.out_w;
    p.pad_h = g.pad_h;
    p.st.in_h = g.in_h;
    p.st.in_w = g.in_w;
    p.st.in_plane = g.in_h * g.in_w;
    p.st.col_shift = g.pad_w;
    p.ncb = ceil_div(g.out_w, 4);
    const int used_cols = 4 * (p.ncb - 1) * S + 4 * NV;
    layout_columns(p.st, used_cols);
    auto rows_for = [](int units) { return (units * BH - 1) * S + K; };
    auto tile_bytes = [&](int units, int planes) {
        return static_cast<long>(planes) * rows_for(units) * p.st.pitch * 4 * (fused ? 2 : 1);
    };
    const int kLdsBudget = env_int("DWCONV_WGRAD_LDS", dwconv::kLdsBudget);
    const int row_units = ceil_div(g.out_h, BH);
    const int ipp_full = row_units * p.ncb;
    int units_per_tile, planes_per_tile;
    if (2 * ipp_full <= kThreads && g.channel > 1) {
        // whole planes, P channels side by side, one item per lane
        units_per_tile = row_units;
        planes_per_tile = kThreads / ipp_full;
        if (planes_per_tile > g.channel) planes_per_tile = g.channel;
        while (planes_per_tile > 1 && tile_bytes(units_per_tile, planes_per_tile) > kLdsBudget) --planes_per_tile;
        if (tile_bytes(units_per_tile, planes_per_tile) > kLdsBudget) return false;
    } else {
        planes_per_tile = 1;
        units_per_tile = kThreads / p.ncb;
        if (units_per_tile < 1) units_per_tile = 1;
        if (units_per_tile > row_units) units_per_tile = row_units;
        while (units_per_tile > 1 && tile_bytes(units_per_tile, 1) > kLdsBudget) --units_per_tile;
        if (tile_bytes(units_per_tile, 1) > kLdsBudget) return false;
        const int bands = ceil_div(row_units, units_per_tile);
        units_per_tile = ceil_div(row_units, bands);
    }
    p.planes_per_tile = planes_per_tile;
    p.rows_per_tile = units_per_tile * BH;
    p.row_tiles = ceil_div(row_units, units_per_tile);
    if (!layout_rows(p.st, rows_for(units_per_tile), planes_per_tile)) return false;
    p.g_base = planes_per_tile * p.st.plane_pitch;
    p.items_per_plane = units_per_tile * p.ncb;
    if (planes_per_tile * p.items_per_plane > kThreads) return false;  // one item per lane
    p.ncb_magic = magic_u16(p.ncb);
    p.ipp_magic = magic_u16(p.items_per_plane);
    p.groups = ceil_div(g.channel, planes_per_tile);
    const long tiles_per_group = static_cast<long>(g.batch) * p.row_tiles;
    if (tiles_per_group > 0x7fffffffL) return false;
    p.tiles_per_group = static_cast<int>(tiles_per_group);
    int chunks = ceil_div(target_wgs, p.groups);
    if (chunks > p.tiles_per_group) chunks = p.tiles_per_group;
    if (chunks < 1) chunks = 1;
    p.tiles_per_chunk = ceil_div(p.tiles_per_group, chunks);
    p.chunks = ceil_div(p.tiles_per_group, p.tiles_per_chunk);
    if (static_cast<long>(p.groups) * p.chunks > 0x7fffffffL) return false;
    (void)KK;
    return true;
}

template <int K, int S, int BH>
size_t lds_bytes(const WgradPlan &p, bool fused)
{
    const size_t tile = static_cast<size_t>(p.planes_per_tile) * p.st.plane_pitch * 4 * (fused ? 2 : 1);
    const size_t red = p.planes_per_tile == 1 ? static_cast<size_t>(kThreads / 64) * K * K * 4
                                              : static_cast<size_t>(K) * K * kRedPitch * 4;
    return tile > red ? tile : red;
}

// Calls fn.template operator()<K,S,BH>() for the instance that covers g; false if none does.
template <typename Fn>
bool dispatch(const WgradGeometry &g, Fn &&fn)
{
    const int K = g.kernel_h, S = g.down_h;
    if (g.kernel_w != K || g.down_w != S) return false;
    if (g.pad_h < 0 || g.pad_w < 0 || g.pad_h > 7 || g.pad_w > 7) return false;
    if (g.in_h < 1 || g.in_w < 1 || g.out_h < 1 || g.out_w < 1) return false;
    if (static_cast<long>(g.in_h) * g.in_w >= (1l << 30) || static_cast<long>(g.out_h) * g.out_w >= (1l << 30))
        return false;
    // every gy element must map inside the padded plane the LDS image covers
    if ((g.out_h - 1) * S - g.pad_h + K - 1 > g.in_h - 1 + 7 || (g.out_w - 1) * S - g.pad_w + K - 1 > g.in_w - 1 + 7)
        return false;
    const int forced = env_int("DWCONV_TILE_BH", 0);
    // (as in the forward launcher; the fused stride-1 backward of a 150x150 3x3 layer: 289 -> 270 us with four rows per
    // lane, of a 74x74 5x5 one 289 -> 220)
    const bool seven = forced ? forced == 7 : (g.out_h % 7 == 0 || (S == 2 && g.out_h > 64)) && g.out_h % 4 != 0;
#define DWCONV_WGRAD_CASE(KV, SV)                                                   \
    if (K == KV && S == SV) {                                                       \
        if (seven) fn.template operator()<KV, SV, 7>();                            \
        else fn.template operator()<KV, SV, 4>();                                  \
        return true;                                                                \
    }
    DWCONV_WGRAD_CASE(3, 1)
    DWCONV_WGRAD_CASE(5, 1)
    DWCONV_WGRAD_CASE(7, 1)
    DWCONV_WGRAD_CASE(3, 2)
    DWCONV_WGRAD_CASE(5, 2)
    DWCONV_WGRAD_CASE(7, 2)
#undef DWCONV_WGRAD_CASE
    return false;
}

struct WorkspaceQuery {
    const WgradGeometry &g;
    size_t bytes = 0;
    template <int K, int S, int BH>
    void operator()()
    {
        for (int fused = 0; fused < 2; ++fused) {
            WgradPlan p{};
            if (!make_plan<K, S, BH>(p, g, fused != 0)) continue;
            const size_t need = static_cast<size_t>(p.groups) * p.planes_per_tile * p.chunks * K * K * sizeof(float);
            if (need > bytes) bytes = need;
        }
    }
};

template <typename IO>
struct Launcher {
    const IO *x;
    const IO *gy;
    IO *gw;
    void *ws;
    size_t ws_bytes;
    const WgradGeometry &g;
    hipStream_t stream;
    const IO *taps = nullptr;  // with gx: also produce grad-input (stride 1, "same" padding)
    IO *gx = nullptr;
    int rc = -1;
    template <int K, int S, int BH>
    void operator()()
    {
        const bool fused = gx != nullptr;
        if (fused && S != 1) return;
        if (g.mult > 1 && (fused || g.channel % g.mult != 0)) return;
        WgradPlan p{};
        if (!make_plan<K, S, BH>(p, g, fused)) return;
        if (g.mult > 1 && p.planes_per_tile != 1) return;  // (larger maps only)
        p.mult = g.mult;
        const size_t need = static_cast<size_t>(p.groups) * p.planes_per_tile * p.chunks * K * K * sizeof(float);
        if (ws == nullptr || ws_bytes < need) {
            rc = fail(DWCONV_ERR_WORKSPACE, "grad-weight needs a workspace of %zu bytes, got %zu", need, ws_bytes);
            return;
        }
        p.x = x;
        p.gy = gy;
        p.partial = static_cast<float *>(ws);
        p.st.vec_in = row_vector_mode(g.in_w, x);
        p.vec_gy = row_vector_mode(g.out_w, gy);
        p.strided = env_int("DWCONV_WGRAD_STRIDED", 1);
        p.taps = taps;
        p.gx = gx;
        p.vec_gx = row_vector_mode(g.in_w, gx, false);
        const size_t shmem = lds_bytes<K, S, BH>(p, fused);
        const dim3 grid(p.groups * p.chunks), block(kThreads);
        // gy is staged with the x image's layout and mode
        if (fused && p.st.vec_in != 0) {
            const int gy_mode = row_vector_mode(g.in_w, gy);
            if (gy_mode == 0) p.st.vec_in = 0;
            else if (gy_mode == 3) p.st.vec_in = 3;
        }
        const int in_view = stage_vector_mode(p.st, p.planes_per_tile, sizeof(IO));
        const int gx_view = vector_mode(p.planes_per_tile, p.st.in_plane, sizeof(IO));
        const int gy_view = vector_mode(p.planes_per_tile, p.out_plane, sizeof(IO));
        // (rows of any width, mode 3, need the view; the aligned modes choose between pointer and view)
        p.st.vec_in = p.st.vec_in == 1 ? in_view : (p.st.vec_in == 3 && in_view == 2 ? 3 : 0);
        p.vec_gx = p.vec_gx == 1 ? gx_view : (p.vec_gx == 3 && gx_view == 2 ? 3 : 0);
        p.vec_gy = p.vec_gy == 1 ? gy_view : (p.vec_gy == 3 && gy_view == 2 ? 3 : 0);
        // grad-input through LDS: 3x3 filters on fp32 rows that are not whole 64-byte bursts, one plane per tile
        // (56x56: 148 -> 143 us; rows of 112 or 256 floats: unchanged or 1.5 % slower; 7x7 filters, which are bound
        // by arithmetic, 3 % slower; 16-bit elements 2 % slower)
        const bool lds_gx_pays = sizeof(IO) == 4 && K == 3 && (g.in_w * sizeof(IO)) % 64 != 0;
        p.lds_gx = fused && p.planes_per_tile == 1 && p.vec_gx == 2 && env_int("DWCONV_WGRAD_LDS_GX", lds_gx_pays);
        const bool any_width = p.st.vec_in == 3 || p.vec_gy == 3 || (fused && p.vec_gx == 3);
        if constexpr (S == 1) {
            if (fused && any_width) hipLaunchKernelGGL((wgrad_tile_kernel<IO, K, S, BH, true, true>), grid, block, shmem, stream, p);
        }
        if (!fused && any_width) hipLaunchKernelGGL((wgrad_tile_kernel<IO, K, S, BH, false, true>), grid, block, shmem, stream, p);
        if constexpr (S == 1) {
            if (fused && !any_width) hipLaunchKernelGGL((wgrad_tile_kernel<IO, K, S, BH, true>), grid, block, shmem, stream, p);
        }
        if (!fused && !any_width) hipLaunchKernelGGL((wgrad_tile_kernel<IO, K, S, BH, false>), grid, block, shmem, stream, p);
        rc = check_launch("wgrad_tile_kernel");
        if (rc != DWCONV_OK) return;
        char mult[16] = "";
        if (p.mult > 1) std::snprintf(mult, sizeof(mult), " m%d", p.mult);
        note_variant("%s%s<k%d,s%d,bh%d> P%d rows%d chunks%d vin%d vgy%d%s%s", fused ? "bwd_tile" : "wgrad_tile",
                     sizeof(IO) == 2 ? "16" : "", K, S, BH, p.planes_per_tile, p.rows_per_tile, p.chunks, p.st.vec_in, p.vec_gy,
                     p.lds_gx ? " ldsgx" : "", mult);
        rc = launch_wgrad_final(static_cast<const float *>(ws), gw, g.channel, K * K, p.chunks, stream);
    }
};

}  // namespace

template <typename IO>
int launch_wgrad_final(const float *partial, IO *gw, int channel, int taps, int chunks, hipStream_t stream)
{
    const int total = channel * taps;
    hipLaunchKernelGGL(wgrad_tile_final_kernel<IO>, dim3(ceil_div(total * kFinalLanes, 256)), dim3(256), 0, stream, partial,
                       gw, total, taps, chunks);
    return check_launch("wgrad_tile_final_kernel");
}

size_t wgrad_tiled_workspace(const WgradGeometry &g)
{
    WorkspaceQuery q{g};
    dispatch(g, q);
    return q.bytes;
}

template <typename IO>
int try_launch_wgrad_tiled(const IO *in, const IO *gy, IO *gw, void *ws, size_t ws_bytes, const WgradGeometry &g,
                           hipStream_t stream)
{
    Launcher<IO> l{in, gy, gw, ws, ws_bytes, g, stream};
    if (!dispatch(g, l)) return -1;
    return l.rc;
}

size_t wgrad_any_workspace(const WgradGeometry &g, int dil_h, int dil_w)
{
    if (!env_int("DWCONV_FIR_ANY", 1)) return 0;
    WgradPlan p{};
    AnyTaps a{};
    if (!make_any_plan(p, a, g, dil_h, dil_w)) return 0;
    return static_cast<size_t>(g.channel) * p.chunks * g.kernel_h * g.kernel_w * sizeof(float);
}

template <typename IO>
int try_launch_wgrad_any(const IO *in, const IO *gy, IO *gw, void *ws, size_t ws_bytes, const WgradGeometry &g, int dil_h,
                         int dil_w, hipStream_t stream)
{
    if (!env_int("DWCONV_FIR_ANY", 1)) return -1;
    constexpr int BH = 4;
    WgradPlan p{};
    AnyTaps a{};
    if (!make_any_plan(p, a, g, dil_h, dil_w)) return -1;
    const int KK = g.kernel_h * g.kernel_w;
    const size_t need = static_cast<size_t>(g.channel) * p.chunks * KK * sizeof(float);
    if (ws == nullptr || ws_bytes < need)
        return fail(DWCONV_ERR_WORKSPACE, "grad-weight needs a workspace of %zu bytes, got %zu", need, ws_bytes);
    p.x = in;
    p.gy = gy;
    p.partial = static_cast<float *>(ws);
    p.st.vec_in = row_vector_mode(g.in_w, in);
    p.vec_gy = row_vector_mode(g.out_w, gy);
    const int in_view = stage_vector_mode(p.st, p.planes_per_tile, sizeof(IO)), gy_view = vector_mode(p.planes_per_tile, p.out_plane, sizeof(IO));
    p.st.vec_in = p.st.vec_in == 1 ? in_view : (p.st.vec_in == 3 && in_view == 2 ? 3 : 0);
    p.vec_gy = p.vec_gy == 1 ? gy_view : (p.vec_gy == 3 && gy_view == 2 ? 3 : 0);
    const size_t image = static_cast<size_t>(p.planes_per_tile) * p.st.plane_pitch * 4;
    const size_t red = p.planes_per_tile > 1 ? static_cast<size_t>(kRedSums) * kRedPitch * 4 : static_cast<size_t>(kThreads / 64) * kAnyTaps * 4;
    const size_t shmem = image > red ? image : red;
    const int passes = a.passes;
    const dim3 grid(static_cast<unsigned>(p.groups * p.chunks), static_cast<unsigned>(passes)), block(kThreads);
    const bool plain = a.sh == 1 && a.sw == 1 && a.dh == 1 && a.dw == 1 && env_int("DWCONV_ANY_WINDOW", 1);
    const char *window = "";
    if (a.walk) {
        hipLaunchKernelGGL((wgrad_any_kernel<IO, BH, 1, -1>), grid, block, shmem, stream, p, a);
        window = " walk4";
    } else if (plain && a.kh == 1 && a.kw <= 8) {
        hipLaunchKernelGGL((wgrad_any_kernel<IO, BH, 1, 1, 8>), grid, block, shmem, stream, p, a);
        window = " win1x8";
    } else if (plain && a.kh <= 8 && a.kw == 1) {
        hipLaunchKernelGGL((wgrad_any_kernel<IO, BH, 1, 8, 1>), grid, block, shmem, stream, p, a);
        window = " win8x1";
    } else if (plain && a.kh <= 4 && a.kw <= 4) {
        hipLaunchKernelGGL((wgrad_any_kernel<IO, BH, 1, 4, 4>), grid, block, shmem, stream, p, a);
        window = " win4x4";
    } else if (plain && a.kh == 1 && a.kw <= 24) {
        hipLaunchKernelGGL((wgrad_any_kernel<IO, BH, 1, 1, 24>), grid, block, shmem, stream, p, a);
        window = " win1x24";
    } else if (plain && a.kh <= 24 && a.kw == 1) {
        hipLaunchKernelGGL((wgrad_any_kernel<IO, BH, 1, 24, 1>), grid, block, shmem, stream, p, a);
        window = " win24x1";
    } else if (plain && a.kh <= 8 && a.kw <= 8) {
        hipLaunchKernelGGL((wgrad_any_kernel<IO, BH, 1, 8, 8>), grid, block, shmem, stream, p, a);
        window = " win8x8";
    } else if (a.sw == 1) hipLaunchKernelGGL((wgrad_any_kernel<IO, BH, 1>), grid, block, shmem, stream, p, a);
    else if (a.sw == 2) hipLaunchKernelGGL((wgrad_any_kernel<IO, BH, 2>), grid, block, shmem, stream, p, a);
    else hipLaunchKernelGGL((wgrad_any_kernel<IO, BH, 0>), grid, block, shmem, stream, p, a);
    const int rc = check_launch("wgrad_any_kernel");
    if (rc != DWCONV_OK) return rc;
    note_variant("wgrad_any%s<k%dx%d,s%dx%d,d%dx%d> P%d rows%d chunks%d passes%d vin%d vgy%d%s", sizeof(IO) == 2 ? "16" : "", a.kh, a.kw,
                 a.sh, a.sw, a.dh, a.dw, p.planes_per_tile, p.rows_per_tile, p.chunks, passes, p.st.vec_in, p.vec_gy, window);
    return launch_wgrad_final(static_cast<const float *>(ws), gw, g.channel, KK, p.chunks, stream);
}

template <typename IO>
int try_launch_bwd_tiled(const IO *in, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes,
                         const WgradGeometry &g, hipStream_t stream)
{
    if (env_int("DWCONV_NO_FUSED_TILE", 0)) return -1;
    const int K = g.kernel_h;
    // stride 1 and "same" padding: the gradient planes have the input's extent and the gy band can share
    // the x band's LDS layout
    if (g.down_h != 1 || g.down_w != 1 || g.kernel_w != K || g.pad_h != K / 2 || g.pad_w != K / 2) return -1;
    if (g.out_h != g.in_h || g.out_w != g.in_w) return -1;
    Launcher<IO> l{in, gy, gw, ws, ws_bytes, g, stream, taps, gx};
    if (!dispatch(g, l)) return -1;
    return l.rc;
}

#define DWCONV_INSTANTIATE(IO)                                                                                        \
    template int launch_wgrad_final<IO>(const float *, IO *, int, int, int, hipStream_t);                             \
    template int try_launch_wgrad_any<IO>(const IO *, const IO *, IO *, void *, size_t, const WgradGeometry &, int,   \
                                          int, hipStream_t);                                                          \
    template int try_launch_wgrad_tiled<IO>(const IO *, const IO *, IO *, void *, size_t, const WgradGeometry &,      \
                                            hipStream_t);                                                             \
    template int try_launch_bwd_tiled<IO>(const IO *, const IO *, const IO *, IO *, IO *, void *, size_t,             \
                                          const WgradGeometry &, hipStream_t);
DWCONV_INSTANTIATE(float)
DWCONV_INSTANTIATE(half_t)
DWCONV_INSTANTIATE(bf16_t)
#undef DWCONV_INSTANTIATE

}  // namespace dwconv
