// Stride-1 "same" convolutions with large filters on maps too wide for several planes per workgroup: forward /
// grad-input, and the fused grad-input + grad-weight sweep (element type fp32, fp16 or bf16; LDS and arithmetic fp32).
//
// These shapes (7x7 filters on 56 x 56 maps) are bound by the vector unit, not by HBM, and the general tiled
// kernels (dwconv_tile.hip, dwconv_wgrad.hip) leave it underused there in two ways, both repaired here:
//
//  * Lanes.  A lane owns a 4 x 4 block of outputs and a workgroup a band of one plane: 56 x 56 has 14 x 14 blocks, so
//    196 of 256 lanes work (112 x 112 and 128 x 96 planes lose the same quarter to bands that do not divide).
//    Here a workgroup keeps ONE channel and walks that channel's images as one tall stack: image n's rows sit at
//    stacked rows n * (H + K/2) + K/2 ..., with K/2 rows of zeros between neighbours (the bottom padding of one image
//    is the top padding of the next).  A tile is U = 256 / (W / 4) consecutive 4-row units of the stack, wherever the
//    image boundaries fall: 252 of 256 lanes work on a 56-wide map.
//  * Registers.  All lanes of a workgroup share the channel, so the K*K taps of the grad-input (or forward) pass
//    are wavefront-uniform: they live in scalar registers and enter the FMAs as scalar operands, not in K*K
//    vector registers per lane.  The 7x7 fused instance needs about 130 vector registers instead of 188: three
//    wavefronts per SIMD instead of two.
//
//  * Loads.  The vector unit is the bottleneck only if it never waits: a tile image is fetched into registers while
//    the workgroup computes on the images already in LDS (see stack_kernel), so every load has a whole arithmetic
//    phase to arrive in.
//
// The arithmetic is that of the general kernels: the band (with halo) of x, and of gy in the fused kernel, is
// staged in LDS with the zero padding materialised; per window row a lane reads aligned float4s once and reuses
// them for every tap and output row.  Grad-weight sums stay in registers over all tiles of the workgroup's chunk
// and are reduced in a fixed order (wave64 DPP sum, then the four wavefronts through LDS) into
// partial[c][chunk][tap]; the second pass is launch_wgrad_final.  Replaces torch_dwconv/dwconv_kernel.cu:69-181
// (large kernel, both directions at stride 1) and :260-306 (grad-weight) for these shapes.
//
// One source, several translation units: built as it is, it holds the instances for 5x5 / 7x7 filters and the dilated
// 3x3 / 5x5 ones (and 3x3 for 16-bit tensors); built with DWCONV_STACK_BIGK = 9, 11 or 13 it holds the instances of
// that one filter size and exports them as stack_bigk_* (dwconv_common.hpp), which the first unit calls.
#include "dwconv_tile_common.hpp"

#include <initializer_list>

#ifndef DWCONV_STACK_BIGK
#define DWCONV_STACK_BIGK 0
#endif

namespace dwconv {

namespace {

constexpr int kStackBH = 4;  // rows per unit (the rows of a unit that hangs over the end of an image are masked)

struct StackPlan {
    const void *x;     // forward: the input; fused backward: x.  Element type IO of the kernel template
    const void *gy;    // fused backward only
    const void *taps;
    void *out;         // forward: the output; fused backward: grad-input
    float *partial;    // fused backward: partial[c][chunk][tap]
    int batch, channel;
    int h, w, plane;
    int img_stride;        // elements from one image's plane of a channel to the next image's: channel * plane
    int ru;                // row units per image = ceil(h / 4)
    int vh;                // rows per image in the stack = h + K/2
    int ncb;               // 4-wide column blocks per row
    int units_per_tile;    // U
    int total_units;       // batch * ru
    int tiles, chunks;
    int pitch;             // floats per LDS row
    int spr;               // float4 slots fetched per row (ceil(padding / 4) of zeros on either side)
    int img_floats;        // floats of one staged image (x or gy)
    int rpp;               // rows of an image the workgroup stages per pass: 256 / spr
    int slots_per_lane;    // loads a lane issues per tile image: ceil(rows / rpp) for the tallest tile
    int step_n, step_r;    // chunks * units_per_tile units = step_n images + step_r row units
    unsigned ncb_magic, ru_magic, vh_magic, spr_magic;
};

// n / d through the reciprocal made by magic_u16(d), for 2 <= d (no test for d == 1: the planner rules it out)
__device__ __forceinline__ int div_magic(int n, unsigned magic) { return static_cast<int>(__umulhi(static_cast<unsigned>(n), magic)); }

// What a workgroup needs to know about one tile (all uniform).
struct StackTile {
    int n0, r0;       // image and row unit of the tile's first unit
    int units_here;   // units of the tile (the last tile of a channel may be short)
    int vrel0;        // stacked row, relative to image n0, of LDS row 0
    int rows;         // stacked rows the tile's windows cover
    int n_span;       // images from n0 on that the tile may touch
    long plane0;      // plane index of (image n0, this channel)
};

// The tile whose first unit is row unit r0 of image n0 (n0 * ru + r0 < total_units).
__device__ __forceinline__ StackTile stack_tile(const StackPlan &p, int n0, int r0, int c, int KE)
{
    StackTile t;
    t.n0 = n0;
    t.r0 = r0;
    t.units_here = min(p.units_per_tile, p.total_units - (n0 * p.ru + r0));
    const int ql = r0 + t.units_here - 1;  // last unit of the tile, counted from image n0's first
    const int nl = div_magic(ql, p.ru_magic), rl = ql - nl * p.ru;
    t.vrel0 = r0 * kStackBH;
    t.rows = nl * p.vh + rl * kStackBH + kStackBH + KE - 1 - t.vrel0;
    t.n_span = min(p.batch - n0, nl + 2);
    t.plane0 = static_cast<long>(n0) * p.channel + c;
    return t;
}

// This lane's part in staging, the same for every tile: one float4 column of the image and every rpp-th row.
struct StackLane {
    int jr;        // first LDS row (lanes beyond rpp whole rows stage nothing: jr is then past every image)
    unsigned coff; // byte offset of the column within a row of the tensor
    bool col_ok;   // the column lies inside the plane (else it reads as zeros)
    int dcol;      // float offset of the column within an LDS row
    int left;      // elements of the row from this column on (rows of any width: what a load reads past them is zeroed)
};

template <typename IO, int PADW>
__device__ __forceinline__ StackLane stack_lane(const StackPlan &p)
{
    StackLane l;
    const int jr = div_magic(threadIdx.x, p.spr_magic);
    const int ix = 4 * (static_cast<int>(threadIdx.x) - jr * p.spr - (PADW + 3) / 4);
    l.jr = jr < p.rpp ? jr : (1 << 20);
    l.coff = static_cast<unsigned>(ix) * static_cast<unsigned>(sizeof(IO));
    l.col_ok = static_cast<unsigned>(ix) < static_cast<unsigned>(p.w);
    l.dcol = kSlack + ix + PADW;
    l.left = p.w - ix;
    return l;
}

// A tile image travels in two steps, so that its loads are in flight while the workgroup computes on the images
// already in LDS: fetch_stack issues this lane's NS loads into registers (elements as loaded, not yet widened),
// commit_stack writes them into the LDS image.  LDS row j, column kSlack + ix + K/2 holds column ix of stacked row
// vrel0 + j of the tensor whose (image n0, channel c) plane starts at `src`; zero rows, columns outside the plane
// and images past n_span read zeros through the view.
template <typename IO, int PADW, int NS>
__device__ __forceinline__ void fetch_stack(const StackPlan &p, const StackLane &l, const IO *__restrict__ src, const StackTile &t,
                                            typename Raw4<IO>::type (&v)[NS])
{
    constexpr unsigned ES = sizeof(IO);
    const long extent = (static_cast<long>(t.n_span - 1) * p.img_stride + p.plane) * ES;
    const __amdgpu_buffer_rsrc_t view = buffer_view(src, extent);
#pragma unroll
    for (int u = 0; u < NS; ++u) {
        const int j = l.jr + u * p.rpp;
        const int vr = t.vrel0 + min(j, t.rows);   // (rows past the tile: any row, the load is switched off)
        const int n = div_magic(vr, p.vh_magic);
        const int rr = vr - __mul24(n, p.vh) - PADW;
        const bool ok = j < t.rows && l.col_ok && rr >= 0 && n < t.n_span;
        const unsigned off = (static_cast<unsigned>(n) * static_cast<unsigned>(p.img_stride) + __mul24(rr, p.w)) * ES + l.coff;
        if constexpr (sizeof(IO) == 4) {
            const u32x4 q = __builtin_amdgcn_raw_buffer_load_b128(view, ok ? off : kOob, 0, 0);
            v[u] = make_float4(__uint_as_float(q.x), __uint_as_float(q.y), __uint_as_float(q.z), __uint_as_float(q.w));
        } else {
            const u32x2 q = __builtin_amdgcn_raw_buffer_load_b64(view, ok ? off : kOob, 0, 0);
            v[u] = make_uint2(q.x, q.y);
        }
    }
}

// ANY_WIDTH: rows that are not whole groups of four elements (the last slot of a row has read into the next row).
template <typename IO, int NS, bool ANY_WIDTH>
__device__ __forceinline__ void commit_stack(const StackPlan &p, const StackLane &l, float *lds, const StackTile &t,
                                             const typename Raw4<IO>::type (&v)[NS])
{
    const int dump = p.img_floats - 4;  // right-hand slack of the last row
#pragma unroll
    for (int u = 0; u < NS; ++u) {
        const int j = l.jr + u * p.rpp;
        float *d = lds + (j < t.rows ? __mul24(j, p.pitch) + l.dcol : dump);
        float4 w = widen4<IO>(v[u]);
        if constexpr (ANY_WIDTH) keep_first(w, l.left);
        d[0] = w.x;
        d[1] = w.y;
        d[2] = w.z;
        d[3] = w.w;
    }
}

// FUSED: grad-input (taps rotated) and grad-weight of one channel's images; otherwise the forward pass (FLIP: taps
// rotated, the grad-input pass on its own).  NS: loads a lane issues per tile image (the planner's bound).
//
// Order of a fused tile, two barriers: [gy of this tile is in registers] commit gy | barrier | issue the loads of x |
// slide the taps over the gy windows (grad-input out, own gy block kept) | commit x | barrier | issue the loads of the
// next tile's gy | grad-weight sums over the x windows.  Every image's loads fly during one arithmetic phase.
// D: dilation (both axes); the window then spans KE = (K - 1) * D + 1 rows and columns and the "same" padding is
// D * (K/2).
// ANY_WIDTH: the instance for rows that are not whole, 16-byte-aligned groups of four elements (loads and stores at
// element alignment through the same views, the block that ends a row cut short); the other instance carries none of it.
template <typename IO, int K, int D, bool FUSED, bool FLIP, int NS, bool ANY_WIDTH = false>
__global__ __launch_bounds__(kThreads) void stack_kernel(const StackPlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int BH = kStackBH;
    constexpr int KE = (K - 1) * D + 1;
    constexpr int PW = D * (K / 2);
    constexpr int KK = K * K;
    constexpr int WIN_ROWS = BH - 1 + KE;
    constexpr int NV = (3 + KE + 3) / 4;  // float4s that hold a window row: columns 4*cb - PW ... 4*cb + 3 + PW
    constexpr unsigned ES = sizeof(IO);

    const int c = blockIdx.x / p.chunks;
    const int chunk = blockIdx.x - c * p.chunks;
    const IO *const slide_src = static_cast<const IO *>(FUSED ? p.gy : p.x);  // the tensor the taps slide over
    float *const lds_slide = lds;                   // its image
    float *const lds_x = lds + p.img_floats;        // fused: the image of x

    typename Raw4<IO>::type staged[NS];
    const StackLane lane = stack_lane<IO, PW>(p);
    // chunk k takes tiles k, k + chunks, ...: the first unit of the next tile lies step_n images and step_r row
    // units further on
    const int u_first = chunk * p.units_per_tile;
    const int n_first = u_first / p.ru;
    StackTile cur = stack_tile(p, n_first, u_first - n_first * p.ru, c, KE);
    fetch_stack<IO, PW, NS>(p, lane, slide_src + cur.plane0 * p.plane, cur, staged);

    // The taps of the sliding pass, wavefront-uniform: scalar registers.  The fused 7x7 kernel has no room for 49 of
    // them beside its other scalars (the compiler then parks those in vector lanes and fetches them back around every
    // staging step, some 230 lane reads per tile), and filters from 9x9 up have more taps than there are scalar
    // registers: those keep the taps in the lanes of one to three vector registers and bring each filter row into
    // scalar registers when the window walk reaches it, K*K lane reads per tile and four rows live at a time.
    constexpr bool kRollTaps = (FUSED && K == 7) || K > 7;
    constexpr int kTapRegs = (KK + 63) / 64;
    float tap[kRollTaps ? 1 : KK];
    float tap_lanes[kRollTaps ? kTapRegs : 1];
    if constexpr (kRollTaps) {
#pragma unroll
        for (int i = 0; i < kTapRegs; ++i) {
            const int t = min(64 * i + (static_cast<int>(threadIdx.x) & 63), KK - 1);
            tap_lanes[i] = Io<IO>::in(static_cast<const IO *>(p.taps)[c * KK + ((FUSED || FLIP) ? KK - 1 - t : t)]);
        }
    } else {
#pragma unroll
        for (int t = 0; t < KK; ++t) {
            const float v = Io<IO>::in(static_cast<const IO *>(p.taps)[c * KK + ((FUSED || FLIP) ? KK - 1 - t : t)]);
            tap[t] = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v)));
        }
    }

    // this lane's place in every tile: unit ul of the tile, column block cb
    const int ul = div_magic(threadIdx.x, p.ncb_magic);
    const int cb = threadIdx.x - ul * p.ncb;
    const int ox = 4 * cb;

    float acc[FUSED ? KK : 1];
#pragma unroll
    for (int t = 0; t < (FUSED ? KK : 1); ++t) acc[t] = 0.f;

    // chunk k takes tiles k, k + chunks, ...: at any moment the grid works on a narrow window of images
    for (int tile = chunk; tile < p.tiles; tile += p.chunks) {
        const bool more = tile + p.chunks < p.tiles;
        // (forward: the windows of the previous tile are read until here; fused: the slide image was last read
        // before the previous tile's second barrier)
        if (!FUSED && tile != chunk) __syncthreads();
        commit_stack<IO, NS, ANY_WIDTH>(p, lane, lds_slide, cur, staged);
        __syncthreads();
        StackTile nxt_tile = cur;
        if (more) {
            const int r_raw = cur.r0 + p.step_r;
            const bool carry = r_raw >= p.ru;
            nxt_tile = stack_tile(p, cur.n0 + p.step_n + (carry ? 1 : 0), carry ? r_raw - p.ru : r_raw, c, KE);
        }
        if constexpr (FUSED) fetch_stack<IO, PW, NS>(p, lane, static_cast<const IO *>(p.x) + cur.plane0 * p.plane, cur, staged);
        else if (more) fetch_stack<IO, PW, NS>(p, lane, slide_src + nxt_tile.plane0 * p.plane, nxt_tile, staged);

        // this lane's unit: image n0 + nrel, row unit r
        const int q = cur.r0 + ul;
        const int nrel = div_magic(q, p.ru_magic);
        const int r = q - __mul24(nrel, p.ru);
        const bool has_item = ul < cur.units_here;
        const int base_off = (has_item ? __mul24(nrel, p.vh) + r * BH - cur.vrel0 : 0) * p.pitch + kSlack + ox;
        const float *sbase = lds_slide + base_off;

        float sums[BH][4];
        float g[FUSED ? BH : 1][4];
#pragma unroll
        for (int b = 0; b < BH; ++b)
#pragma unroll
            for (int o = 0; o < 4; ++o) sums[b][o] = 0.f;
        {
            float nxt[4 * NV];
            load_window_row<NV>(sbase, nxt);
            float trow[kRollTaps ? K : 1][K];
            if constexpr (kRollTaps) {  // (keeps the lane reads inside the tile loop)
#pragma unroll
                for (int i = 0; i < kTapRegs; ++i) asm volatile("" : "+v"(tap_lanes[i]));
            }
#pragma unroll
            for (int wr = 0; wr < WIN_ROWS; ++wr) {
                float win[4 * NV];
#pragma unroll
                for (int i = 0; i < 4 * NV; ++i) win[i] = nxt[i];
                if (wr + 1 < WIN_ROWS) load_window_row<NV>(sbase + (wr + 1) * p.pitch, nxt);
                if constexpr (kRollTaps) {
                    if (wr % D == 0 && wr / D < K) {
#pragma unroll
                        for (int tx = 0; tx < K; ++tx)
                            trow[wr / D < K ? wr / D : 0][tx] = __int_as_float(__builtin_amdgcn_readlane(
                                __float_as_int(tap_lanes[((wr / D) * K + tx) / 64]), ((wr / D) * K + tx) % 64));
                    }
                }
                if constexpr (FUSED) {
                    // the lane's own gy block sits K/2 rows and columns into its window
                    const int gb = wr - PW;
                    if (gb >= 0 && gb < BH) {
#pragma unroll
                        for (int o = 0; o < 4; ++o)
                            g[gb >= 0 && gb < BH ? gb : 0][o] = (has_item && r * BH + gb < p.h) ? win[o + PW] : 0.f;
                    }
                }
#pragma unroll
                for (int b = 0; b < BH; ++b) {
                    const int dy = wr - b;
                    if (dy < 0 || dy >= KE || dy % D != 0) continue;
                    const int ty = dy / D;
#pragma unroll
                    for (int tx = 0; tx < K; ++tx)
#pragma unroll
                        for (int o = 0; o < 4; ++o)
                            sums[b][o] = fmaf(win[o + tx * D], kRollTaps ? trow[kRollTaps ? ty : 0][tx] : tap[kRollTaps ? 0 : ty * K + tx], sums[b][o]);
                }
                pin_registers(sums);
            }
        }
        {
            // branch-free: rows past the end of the image (and lanes without a unit) store out of range
            const __amdgpu_buffer_rsrc_t view = buffer_view(static_cast<IO *>(p.out) + cur.plane0 * p.plane,
                                                            (static_cast<long>(cur.n_span - 1) * p.img_stride + p.plane) * ES);
            const unsigned o0 = (static_cast<unsigned>(nrel) * static_cast<unsigned>(p.img_stride) + ox) * ES;
#pragma unroll
            for (int b = 0; b < BH; ++b) {
                const int oy = r * BH + b;
                const bool ok = has_item && oy < p.h;
                if constexpr (ANY_WIDTH)
                    view_store_first<IO>(view, ok ? o0 + __mul24(oy, p.w) * ES : kOob, p.w - ox, p.w & 3, sums[b][0], sums[b][1],
                                         sums[b][2], sums[b][3]);
                else
                    view_store4<IO>(view, ok ? o0 + __mul24(oy, p.w) * ES : kOob, sums[b][0], sums[b][1], sums[b][2], sums[b][3]);
            }
        }

        if constexpr (FUSED) {
            commit_stack<IO, NS, ANY_WIDTH>(p, lane, lds_x, cur, staged);
            __syncthreads();
            if (more) fetch_stack<IO, PW, NS>(p, lane, slide_src + nxt_tile.plane0 * p.plane, nxt_tile, staged);
            const float *base = lds_x + base_off;
            float nxt[4 * NV];
            load_window_row<NV>(base, nxt);
#pragma unroll
            for (int wr = 0; wr < WIN_ROWS; ++wr) {
                float win[4 * NV];
#pragma unroll
                for (int i = 0; i < 4 * NV; ++i) win[i] = nxt[i];
                if (wr + 1 < WIN_ROWS) load_window_row<NV>(base + (wr + 1) * p.pitch, nxt);
#pragma unroll
                for (int b = 0; b < BH; ++b) {
                    const int dy = wr - b;
                    if (dy < 0 || dy >= KE || dy % D != 0) continue;
                    const int ty = dy / D;
#pragma unroll
                    for (int tx = 0; tx < K; ++tx)
#pragma unroll
                        for (int o = 0; o < 4; ++o) acc[ty * K + tx] = fmaf(g[b][o], win[o + tx * D], acc[ty * K + tx]);
                }
                pin_registers(acc);
            }
        }
        cur = nxt_tile;
    }

    if constexpr (FUSED) {
        __syncthreads();  // the tile images are dead; their LDS is reused for the reduction
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
            p.partial[(static_cast<long>(c) * p.chunks + chunk) * KK + threadIdx.x] = s;
        }
    }
}

// Geometry the stacked kernels take: stride 1, "same" padding D * (K/2), K x K taps at dilation D with (K, D) in
// {(5,1), (7,1), (3,2), (5,2)}, rows of whole groups of four elements, and a plane too large for two of them to share a
// workgroup (those shapes keep the several-planes mode of the general kernels).
// (3x3 at dilation 1 stays with the general kernels: they wait for HBM, not for the vector unit, and measured the same
// or faster: 112x112 C=32 fused backward 124-130 us here against 127, 56x56 C=144 152-158 against 132-144)
bool stack_shape(int K, int D)
{
    if (DWCONV_STACK_BIGK) return D == 1 && K == DWCONV_STACK_BIGK;
    return (D == 1 && (K == 5 || K == 7)) || (D == 2 && (K == 3 || K == 5));
}
// 16-bit elements, 3x3 at dilation 1, rows under 96 elements (from there on the kernels with 16-bit LDS images serve):
// the general kernels are bound by their vector instructions with such tensors (the fused 56x56 backward keeps the
// vector units 91 % busy with 196 of 256 lanes at work, 144 on a 48x48 map), and full lanes pay.  Measured by width
// with square bf16 maps, C = 144, batch 128, us stacked / general: fused backward 48: 78 / 95, 52: 90 / 97, 56: 97 / 98,
// 60: 114 / 139, 64: 120 / 142, 72: 155 / 174, 80: 187 / 191, 88: 209 / 260, 92: 285 / 269; forward 48: 48 / 50,
// 52: 60 / 52, 56: 64 / 56, 60: 70 / 76, 64: 62 / 69, 68: 103 / 97, 72: 94 / 100, 76: 117 / 104, 80: 129 / 107,
// 84: 143 / 130, 88: 138 / 140, 92: 173 / 152.  The forward pass takes the stacked kernel only at the widths where it
// won by more than the noise.
bool stack_shape_half(int K, int D, int w, bool fused)
{
    if (DWCONV_STACK_BIGK || K != 3 || D != 1 || !env_int("DWCONV_STACK_K3_16", 1)) return false;
    if (fused) return w <= 88;
    if (env_set("DWCONV_STACK_K3_16_FWD_W")) return w <= env_int("DWCONV_STACK_K3_16_FWD_W", 0);
    return w == 48 || w == 60 || w == 64 || w == 72;
}

bool make_plan(StackPlan &p, int K, int D, int batch, int channel, int h, int w, size_t esize, bool fused, int target_wgs,
               bool half_io = false)
{
    if (!stack_shape(K, D) && !(half_io && stack_shape_half(K, D, w, fused))) return false;
    // (filters from 9x9 up have no other tuned kernel: their small planes come here too, from two row units and two
    // column blocks on: the in-kernel divisions need divisors of at least 2)
    if (w < (K > 7 ? 8 : 16) || h < (K > 7 ? 5 : 8)) return false;
    const int ncb = ceil_div(w, 4);
    if (ncb > kThreads) return false;
    const int ru = ceil_div(h, kStackBH);
    if (K <= 7 && 2 * ru * ncb <= kThreads) return false;
    const long plane = static_cast<long>(h) * w;
    if (plane >= (1l << 23) || static_cast<long>(channel) * plane >= (1l << 28)) return false;
    const int ke = (K - 1) * D + 1, padw = D * (K / 2);
    p.batch = batch;
    p.channel = channel;
    p.h = h;
    p.w = w;
    p.plane = static_cast<int>(plane);
    p.img_stride = static_cast<int>(channel * plane);
    p.ru = ru;
    p.vh = h + padw;
    p.ncb = ncb;
    const int side = ceil_div(padw, 4);  // float4 slots of zeros on either side of a row
    p.pitch = round_up(w, 4) + 8 * side + 8;  // kSlack + 4 * side columns of zeros + w + as many zeros + kSlack
    p.spr = ncb + 2 * side;
    const long total_units = static_cast<long>(batch) * ru;
    if (total_units >= (1l << 30)) return false;
    p.total_units = static_cast<int>(total_units);
    // (two workgroups to a CU either way; with the 12 padding rows of a 13x13 filter between stacked 14-row images the
    // full 64 KiB hold a sixth more units: fused backward on 14x14 C=384, batch 64, 216 -> 185 us; 9x9 and 11x11 and
    // the 5x5 / 7x7 layers measured 1-2 % slower with it)
    const int budget = env_int("DWCONV_STACK_LDS", (K >= 13 ? 64 : 56) * 1024);
    int units = kThreads / ncb;
    auto rows_for = [&](int u) { return u * kStackBH + ke - 1 + padw * ((u - 1) / ru + 2); };
    // (and at most eight loads per lane and image: they wait in registers while the workgroup computes)
    p.rpp = kThreads / p.spr;
    while (units > 1 && (static_cast<long>(rows_for(units)) * p.pitch * 4 * (fused ? 2 : 1) > budget ||
                         rows_for(units) > 8 * p.rpp))
        --units;
    if (rows_for(units) > 8 * p.rpp) return false;
    if (static_cast<long>(rows_for(units)) * p.pitch * 4 * (fused ? 2 : 1) > budget) return false;
    p.units_per_tile = units;
    const int rows = rows_for(units);
    p.img_floats = rows * p.pitch;
    p.slots_per_lane = ceil_div(rows, p.rpp);
    // 16-bit reciprocals: stacked rows of a tile, units counted from the tile's first image
    if (rows + p.vh >= 65536 || ru + units >= 65536) return false;
    // a tile's images must lie within one buffer view
    const long span_images = (units - 1) / ru + 3;
    if ((span_images * p.img_stride + plane) * static_cast<long>(esize) >= static_cast<long>(kOob)) return false;
    p.tiles = ceil_div(p.total_units, units);
    int chunks = ceil_div(target_wgs, channel);
    if (chunks > p.tiles) chunks = p.tiles;
    if (chunks < 1) chunks = 1;
    if (static_cast<long>(channel) * chunks > 0x7fffffffL) return false;
    p.chunks = chunks;
    const long step = static_cast<long>(chunks) * units;
    p.step_n = static_cast<int>(step / ru);
    p.step_r = static_cast<int>(step % ru);
    p.ncb_magic = magic_u16(ncb);
    p.ru_magic = magic_u16(ru);
    p.vh_magic = magic_u16(p.vh);
    p.spr_magic = magic_u16(p.spr);
    return true;
}

size_t lds_bytes(const StackPlan &p, int K, bool fused)
{
    const size_t tile = static_cast<size_t>(p.img_floats) * 4 * (fused ? 2 : 1);
    const size_t red = static_cast<size_t>(kThreads / 64) * K * K * 4;
    return tile > red ? tile : red;
}

// Workgroups of the fused kernel: one resident round (three per compute unit by its registers and LDS) for 7x7
// filters (56x56 C=96 at batch 64: 768 workgroups 95 us, 1536 105, 2304 104); 5x5 filters do not care (256x256 C=64:
// 189-197 us from 768 to 6144).
// Larger filters like 7x7: 768 against 1536 on 56x56 9x9 126 against 136 us, 28x28 11x11 131 against 150, 14x14 13x13
// 220 against 277 (the K*K sums of a workgroup are reduced once per workgroup).
int bwd_target_wgs(int K) { return env_int("DWCONV_STACK_WGS", K >= 7 ? 768 : 1536); }

// fn.template operator()<K, D>() for the supported (K, D)
template <typename Fn>
void for_shape(int K, int D, Fn &&fn)
{
#if DWCONV_STACK_BIGK
    if (K == DWCONV_STACK_BIGK && D == 1) fn.template operator()<DWCONV_STACK_BIGK, 1>();
#else
    if (K == 3 && D == 1) fn.template operator()<3, 1>();
    if (K == 5 && D == 1) fn.template operator()<5, 1>();
    if (K == 7 && D == 1) fn.template operator()<7, 1>();
    if (K == 3 && D == 2) fn.template operator()<3, 2>();
    if (K == 5 && D == 2) fn.template operator()<5, 2>();
#endif
}

template <typename IO, bool FUSED>
struct StackLaunch {
    const StackPlan &p;
    bool rot;
    size_t shmem;
    hipStream_t stream;
    bool any_width = false;
    template <int K, int D>
    void operator()()
    {
        if constexpr (K == 3 && D == 1 && sizeof(IO) == 4) return;  // (16-bit elements only: stack_shape_half)
        const dim3 grid(static_cast<unsigned>(p.channel * p.chunks)), block(kThreads);
        const bool six = p.slots_per_lane <= 6;
        if (any_width) launch<K, D, true>(grid, block, six);
        else launch<K, D, false>(grid, block, six);
    }
    template <int K, int D, bool AW>
    void launch(dim3 grid, dim3 block, bool six)
    {
        if constexpr (FUSED) {
            if (six) hipLaunchKernelGGL((stack_kernel<IO, K, D, true, true, 6, AW>), grid, block, shmem, stream, p);
            else hipLaunchKernelGGL((stack_kernel<IO, K, D, true, true, 8, AW>), grid, block, shmem, stream, p);
        } else if (rot) {
            if (six) hipLaunchKernelGGL((stack_kernel<IO, K, D, false, true, 6, AW>), grid, block, shmem, stream, p);
            else hipLaunchKernelGGL((stack_kernel<IO, K, D, false, true, 8, AW>), grid, block, shmem, stream, p);
        } else {
            if (six) hipLaunchKernelGGL((stack_kernel<IO, K, D, false, false, 6, AW>), grid, block, shmem, stream, p);
            else hipLaunchKernelGGL((stack_kernel<IO, K, D, false, false, 8, AW>), grid, block, shmem, stream, p);
        }
    }
};

// Which instance serves tensors of rows `w` wide at these bases: 0 = the aligned one, 1 = ANY_WIDTH, -1 = neither
// (16-bit rows that do not all start on 32-bit boundaries: the general kernels take those).
template <typename IO>
int stack_width_mode(int w, std::initializer_list<const IO *> bases)
{
    bool aligned = w % 4 == 0, dword = sizeof(IO) == 4 || w % 2 == 0;
    for (const IO *b : bases) {
        aligned = aligned && aligned4(b);
        dword = dword && (reinterpret_cast<uintptr_t>(b) & 3) == 0;
    }
    if (aligned) return 0;
    return dword && env_int("DWCONV_RAGGED_VIEWS", 1) ? 1 : -1;
}

size_t stack_backward_workspace(int K, int D, int batch, int channel, int h, int w)
{
    if (!env_int("DWCONV_STACK", 1)) return 0;
#if !DWCONV_STACK_BIGK
    if (D == 1 && K == 9) return stack_bigk_workspace<9>(batch, channel, h, w);
    if (D == 1 && K == 11) return stack_bigk_workspace<11>(batch, channel, h, w);
    if (D == 1 && K == 13) return stack_bigk_workspace<13>(batch, channel, h, w);
#endif
    StackPlan p{};
    // (the plan does not depend on the element size except through the view-extent check: the larger one)
    // (and a 16-bit caller may take the 3x3 instance)
    if (!make_plan(p, K, D, batch, channel, h, w, 4, true, bwd_target_wgs(K), true)) return 0;
    return static_cast<size_t>(channel) * p.chunks * K * K * sizeof(float);
}

template <typename IO>
int launch_stack_backward(const IO *in, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes, int K, int D,
                          int batch, int channel, int h, int w, hipStream_t stream)
{
    if (!env_int("DWCONV_STACK", 1)) return -1;
#if !DWCONV_STACK_BIGK
    if (D == 1 && K == 9) return stack_bigk_backward<9, IO>(in, gy, taps, gx, gw, ws, ws_bytes, batch, channel, h, w, stream);
    if (D == 1 && K == 11) return stack_bigk_backward<11, IO>(in, gy, taps, gx, gw, ws, ws_bytes, batch, channel, h, w, stream);
    if (D == 1 && K == 13) return stack_bigk_backward<13, IO>(in, gy, taps, gx, gw, ws, ws_bytes, batch, channel, h, w, stream);
#endif
    const int width_mode = stack_width_mode<IO>(w, {in, gy, gx});
    if (width_mode < 0) return -1;
    StackPlan p{};
    if (!make_plan(p, K, D, batch, channel, h, w, 4, true, bwd_target_wgs(K), sizeof(IO) == 2)) return -1;
    const size_t need = static_cast<size_t>(channel) * p.chunks * K * K * sizeof(float);
    if (ws == nullptr || ws_bytes < need)
        return fail(DWCONV_ERR_WORKSPACE, "grad-weight needs a workspace of %zu bytes, got %zu", need, ws_bytes);
    p.x = in;
    p.gy = gy;
    p.taps = taps;
    p.out = gx;
    p.partial = static_cast<float *>(ws);
    for_shape(K, D, StackLaunch<IO, true>{p, true, lds_bytes(p, K, true), stream, width_mode == 1});
    const int rc = check_launch("stack_kernel");
    if (rc != DWCONV_OK) return rc;
    note_variant("bwd_stack%s<k%d,d%d,s1> units%d tiles%d chunks%d%s", sizeof(IO) == 2 ? "16" : "", K, D, p.units_per_tile,
                 p.tiles, p.chunks, width_mode == 1 ? " anywidth" : "");
    return launch_wgrad_final(static_cast<const float *>(ws), gw, channel, K * K, p.chunks, stream);
}

template <typename IO>
int launch_stack_forward(const IO *in, const IO *taps, IO *out, int K, int D, int batch, int channel, int h, int w, bool rot,
                         hipStream_t stream)
{
    if (!env_int("DWCONV_STACK", 1) || !env_int("DWCONV_STACK_FWD", 1)) return -1;
#if !DWCONV_STACK_BIGK
    if (D == 1 && K == 9) return stack_bigk_forward<9, IO>(in, taps, out, batch, channel, h, w, rot, stream);
    if (D == 1 && K == 11) return stack_bigk_forward<11, IO>(in, taps, out, batch, channel, h, w, rot, stream);
    if (D == 1 && K == 13) return stack_bigk_forward<13, IO>(in, taps, out, batch, channel, h, w, rot, stream);
#endif
    const int width_mode = stack_width_mode<IO>(w, {in, static_cast<const IO *>(out)});
    if (width_mode < 0) return -1;
    // fp32 at dilation 1: the general tiled kernel has overtaken this one on 5x5 filters (square maps 48-256 wide: 2-29 %
    // faster; the 256x256 C=64 layer 104 against 114 us) and on 7x7 filters on wide rows (128: 9 %, 256: 38 %); 7x7 on
    // rows up to 116 stays here (56x56 C=96: 43 against 48 us), whole groups of four only (57-75 wide: even or slower).
    if (D == 1 && K <= 7 && sizeof(IO) == 4 && !env_set("DWCONV_STACK_FWD") && (K == 5 || w > 116 || width_mode == 1)) return -1;
    StackPlan p{};
    // (short-lived workgroups of one tile each measured best: 56x56 C=96 7x7 43 us with 4800, 46-50 with 1280-4096)
    if (!make_plan(p, K, D, batch, channel, h, w, 4, false, env_int("DWCONV_STACK_FWD_WGS", 8192), sizeof(IO) == 2)) return -1;
    p.x = in;
    p.taps = taps;
    p.out = out;
    for_shape(K, D, StackLaunch<IO, false>{p, rot, lds_bytes(p, K, false), stream, width_mode == 1});
    note_variant("tile_stack%s<k%d,d%d,s1,%s> units%d tiles%d chunks%d%s", sizeof(IO) == 2 ? "16" : "", K, D, rot ? "rot" : "fwd",
                 p.units_per_tile, p.tiles, p.chunks, width_mode == 1 ? " anywidth" : "");
    return check_launch("stack_kernel");
}

bool covers_bwd(const WgradGeometry &g)
{
    const int K = g.kernel_h;
    if (g.kernel_w != K || g.down_h != 1 || g.down_w != 1 || g.pad_h != K / 2 || g.pad_w != K / 2) return false;
    if (g.out_h != g.in_h || g.out_w != g.in_w) return false;
    return true;
}

// dilated, multiplier 1, stride 1, "same" padding: the geometry the dilated instances take
bool covers_general(const GeneralGeometry &g)
{
    const int K = g.kernel_h, D = g.dil_h;
    if (g.multiplier != 1 || g.kernel_w != K || g.dil_w != D || D < 2) return false;
    if (g.stride_h != 1 || g.stride_w != 1 || g.pad_h != D * (K / 2) || g.pad_w != D * (K / 2)) return false;
    if (g.out_h != g.in_h || g.out_w != g.in_w) return false;
    return stack_shape(K, D);
}

}  // namespace

#if DWCONV_STACK_BIGK

template <>
size_t stack_bigk_workspace<DWCONV_STACK_BIGK>(int batch, int channel, int h, int w)
{
    return stack_backward_workspace(DWCONV_STACK_BIGK, 1, batch, channel, h, w);
}
template <int K, typename IO>
int stack_bigk_forward(const IO *in, const IO *taps, IO *out, int batch, int channel, int h, int w, bool rot, hipStream_t stream)
{
    return launch_stack_forward<IO>(in, taps, out, K, 1, batch, channel, h, w, rot, stream);
}
template <int K, typename IO>
int stack_bigk_backward(const IO *in, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes, int batch,
                        int channel, int h, int w, hipStream_t stream)
{
    return launch_stack_backward<IO>(in, gy, taps, gx, gw, ws, ws_bytes, K, 1, batch, channel, h, w, stream);
}
#define DWCONV_INSTANTIATE(IO)                                                                                                \
    template int stack_bigk_forward<DWCONV_STACK_BIGK, IO>(const IO *, const IO *, IO *, int, int, int, int, bool, hipStream_t); \
    template int stack_bigk_backward<DWCONV_STACK_BIGK, IO>(const IO *, const IO *, const IO *, IO *, IO *, void *, size_t, int,  \
                                                            int, int, int, hipStream_t);
DWCONV_INSTANTIATE(float)
DWCONV_INSTANTIATE(half_t)
DWCONV_INSTANTIATE(bf16_t)
#undef DWCONV_INSTANTIATE

#else

size_t bwd_stack_workspace(const WgradGeometry &g)
{
    if (!covers_bwd(g)) return 0;
    return stack_backward_workspace(g.kernel_h, 1, g.batch, g.channel, g.in_h, g.in_w);
}

template <typename IO>
int try_launch_bwd_stack(const IO *in, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes,
                         const WgradGeometry &g, hipStream_t stream)
{
    if (!covers_bwd(g)) return -1;
    return launch_stack_backward<IO>(in, gy, taps, gx, gw, ws, ws_bytes, g.kernel_h, 1, g.batch, g.channel, g.in_h, g.in_w, stream);
}

template <typename IO>
int try_launch_fir_stack(const IO *in, const IO *taps, IO *out, const Geometry &g, hipStream_t stream)
{
    const int K = g.kernel_h;
    if (g.kernel_w != K || g.up_h != 1 || g.up_w != 1 || g.down_h != 1 || g.down_w != 1) return -1;
    if (g.pad_h0 != K / 2 || g.pad_w0 != K / 2 || g.out_h != g.in_h || g.out_w != g.in_w) return -1;
    if (g.epi.enabled()) return -1;  // the fused epilogue stays with the general kernel
    return launch_stack_forward<IO>(in, taps, out, K, 1, g.batch, g.channel, g.in_h, g.in_w, !g.forward, stream);
}

size_t general_stack_workspace(const GeneralGeometry &g)
{
    if (!covers_general(g)) return 0;
    return stack_backward_workspace(g.kernel_h, g.dil_h, g.batch, g.channel, g.in_h, g.in_w);
}

template <typename IO>
int try_launch_general_stack_forward(const IO *in, const IO *taps, IO *out, const GeneralGeometry &g, hipStream_t stream)
{
    if (!covers_general(g)) return -1;
    return launch_stack_forward<IO>(in, taps, out, g.kernel_h, g.dil_h, g.batch, g.channel, g.in_h, g.in_w, false, stream);
}

template <typename IO>
int try_launch_general_stack_backward(const IO *in, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes,
                                      const GeneralGeometry &g, hipStream_t stream)
{
    if (!covers_general(g)) return -1;
    return launch_stack_backward<IO>(in, gy, taps, gx, gw, ws, ws_bytes, g.kernel_h, g.dil_h, g.batch, g.channel, g.in_h,
                                     g.in_w, stream);
}

#define DWCONV_INSTANTIATE(IO)                                                                                        \
    template int try_launch_bwd_stack<IO>(const IO *, const IO *, const IO *, IO *, IO *, void *, size_t,             \
                                          const WgradGeometry &, hipStream_t);                                        \
    template int try_launch_fir_stack<IO>(const IO *, const IO *, IO *, const Geometry &, hipStream_t);               \
    template int try_launch_general_stack_forward<IO>(const IO *, const IO *, IO *, const GeneralGeometry &,          \
                                                      hipStream_t);                                                   \
    template int try_launch_general_stack_backward<IO>(const IO *, const IO *, const IO *, IO *, IO *, void *,        \
                                                       size_t, const GeneralGeometry &, hipStream_t);
DWCONV_INSTANTIATE(float)
DWCONV_INSTANTIATE(half_t)
DWCONV_INSTANTIATE(bf16_t)
#undef DWCONV_INSTANTIATE

#endif  // DWCONV_STACK_BIGK

}  // namespace dwconv
