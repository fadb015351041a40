// LDS-tiled fp32 kernels for the forward and grad-input passes.
//
// Work decomposition (one workgroup of 256 lanes = 4 wavefronts per tile):
//   tile  = P consecutive (n,c) planes x a band of output rows x the full width.
//           Large maps use P = 1 and several row bands per plane; maps small
//           enough use whole planes and P > 1, so a wavefront carries several
//           channels.
//   load  = the input band (with its halo rows) is fetched with 128-bit loads
//           and scattered into an LDS image whose zero padding is materialised,
//           so the arithmetic below needs no bounds checks.
//   item  = a register block of BH x 4 outputs (8 wide for the stride-2
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
#include "dwconv_common.hpp"

#include <cstdlib>

namespace dwconv {

namespace {

constexpr int kThreads = 256;
constexpr int kSlack = 4;            // spare floats on both sides of every LDS row
constexpr int kLdsBudget = 48 * 1024;  // bytes of LDS one tile may take
constexpr int kXcds = 8;

struct TilePlan {
    const float *in;
    const float *taps;
    float *out;
    long planes;
    int channel;
    int in_h, in_w, out_h, out_w;
    int in_plane, out_plane;   // elements per plane
    int row_shift, col_shift;  // LDS row r / column c hold input row iy0 + r / column c - col_shift
    int rows_per_tile;         // output rows (down) or half-resolution rows (up) per tile
    int row_tiles;             // tiles per plane
    int planes_per_tile;
    int n_tiles;
    int lds_rows;              // rows of one plane image
    unsigned lds_rows_magic;
    int g_lo;                  // first (possibly negative) float4 column fetched per row
    int spr;                   // float4 slots per row
    unsigned spr_magic;
    int pitch;                 // floats per LDS row, slack included
    int plane_pitch;           // floats per plane image
    int ncb;                   // column blocks per row band
    unsigned ncb_magic;
    int items_per_plane;
    unsigned ipp_magic;
    int tap_base;              // float offset of the tap table in LDS
    int vec_in, vec_out;       // 128-bit global accesses are legal
};

// n / d through the reciprocal made by magic_u16(d); a zero reciprocal stands for d == 1.
__device__ __forceinline__ int fast_div(int n, unsigned magic)
{
    return magic ? static_cast<int>(__umulhi(static_cast<unsigned>(n), magic)) : n;
}

// Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.
// Give every XCD a contiguous run of tiles so that the row bands of one plane,
// which share halo rows, meet in the same L2.
__device__ __forceinline__ int xcd_contiguous_tile(int bid, int n_tiles)
{
    const int per = n_tiles / kXcds, rem = n_tiles - per * kXcds;
    const int xcd = bid % kXcds, k = bid / kXcds;
    return xcd * per + min(xcd, rem) + k;
}

// Copies the tap tables of the tile's planes into LDS, rotated by 180 degrees if FLIP.
template <int KK, bool FLIP>
__device__ __forceinline__ void stage_taps(const TilePlan &p, float *lds, long plane0, int nplanes)
{
    for (int i = threadIdx.x; i < nplanes * KK; i += kThreads) {
        const int pl = i / KK, t = i - pl * KK;
        const int c = static_cast<int>((plane0 + pl) % p.channel);
        lds[p.tap_base + i] = p.taps[c * KK + (FLIP ? KK - 1 - t : t)];
    }
}

// Fills the LDS image of the tile: every float4 slot of every row is written,
// with zeros where the row or the columns fall outside the plane.
__device__ __forceinline__ void stage_tile(const TilePlan &p, float *lds, long plane0, int nplanes, int iy0)
{
    const int total = nplanes * p.lds_rows * p.spr;
    for (int slot = threadIdx.x; slot < total; slot += kThreads) {
        const int rowidx = fast_div(slot, p.spr_magic);
        const int sc = slot - rowidx * p.spr;
        const int pl = fast_div(rowidx, p.lds_rows_magic);
        const int r = rowidx - pl * p.lds_rows;
        const int ix = 4 * (p.g_lo + sc);
        const int iy = iy0 + r;
        const bool row_ok = static_cast<unsigned>(iy) < static_cast<unsigned>(p.in_h);
        const float *src = p.in + (plane0 + pl) * p.in_plane + static_cast<long>(iy) * p.in_w + ix;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (p.vec_in) {
            if (row_ok && ix >= 0 && ix < p.in_w) v = *reinterpret_cast<const float4 *>(src);
        } else if (row_ok) {
            if (static_cast<unsigned>(ix + 0) < static_cast<unsigned>(p.in_w)) v.x = src[0];
            if (static_cast<unsigned>(ix + 1) < static_cast<unsigned>(p.in_w)) v.y = src[1];
            if (static_cast<unsigned>(ix + 2) < static_cast<unsigned>(p.in_w)) v.z = src[2];
            if (static_cast<unsigned>(ix + 3) < static_cast<unsigned>(p.in_w)) v.w = src[3];
        }
        float *dst = lds + pl * p.plane_pitch + r * p.pitch + kSlack + ix + p.col_shift;
        dst[0] = v.x;
        dst[1] = v.y;
        dst[2] = v.z;
        dst[3] = v.w;
    }
}

// up = 1, decimation S.  out[oy,ox] = sum_{ty,tx} in[oy*S - pad_h0 + ty, ox*S - pad_w0 + tx] * f[ty,tx].
template <int K, int S, bool FLIP, int BH>
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

    stage_taps<KK, FLIP>(p, lds, plane0, nplanes);
    stage_tile(p, lds, plane0, nplanes, oy0 * S - p.row_shift);
    __syncthreads();

    const int n_items = nplanes * p.items_per_plane;
    for (int item = threadIdx.x; item < n_items; item += kThreads) {
        const int pl = fast_div(item, p.ipp_magic);
        const int rem = item - pl * p.items_per_plane;
        const int rb = fast_div(rem, p.ncb_magic);
        const int cb = rem - rb * p.ncb;

        float tapv[KK];
#pragma unroll
        for (int t = 0; t < KK; ++t) tapv[t] = lds[p.tap_base + pl * KK + t];

        const float *base = lds + pl * p.plane_pitch + (rb * BH * S) * p.pitch + kSlack + 4 * cb * S;
        float acc[BH][4];
#pragma unroll
        for (int b = 0; b < BH; ++b)
#pragma unroll
            for (int o = 0; o < 4; ++o) acc[b][o] = 0.f;

#pragma unroll
        for (int wr = 0; wr < WIN_ROWS; ++wr) {
            float win[4 * NV];
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                const float4 q = *reinterpret_cast<const float4 *>(base + wr * p.pitch + 4 * v);
                win[4 * v + 0] = q.x;
                win[4 * v + 1] = q.y;
                win[4 * v + 2] = q.z;
                win[4 * v + 3] = q.w;
            }
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
        }

        const int ox = 4 * cb;
        float *dst = p.out + (plane0 + pl) * p.out_plane + ox;
#pragma unroll
        for (int b = 0; b < BH; ++b) {
            const int oy = oy0 + rb * BH + b;
            if (oy >= p.out_h) continue;
            float *row = dst + static_cast<long>(oy) * p.out_w;
            if (p.vec_out) {
                *reinterpret_cast<float4 *>(row) = make_float4(acc[b][0], acc[b][1], acc[b][2], acc[b][3]);
            } else {
#pragma unroll
                for (int o = 0; o < 4; ++o)
                    if (ox + o < p.out_w) row[o] = acc[b][o];
            }
        }
    }
}

// up = 2, no decimation, taps rotated.  With pad0 = 2m - E (E = pad0 & 1, m = (pad0+E)/2) and the
// rotated filter g shifted by E (g'[t] = g[t-E]):
//   out[2q + r] = sum_a in[q - m + r + a] * g'[r + 2a]      along each axis,
// i.e. a stride-1 correlation per output parity r with every other tap.
template <int K, int EY, int EX, int BQ>
__global__ __launch_bounds__(kThreads) void fir_up2_kernel(const TilePlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int KK = K * K;
    constexpr int KAY = (K + EY + 1) / 2, KAX = (K + EX + 1) / 2;
    constexpr int WIN_ROWS = BQ + KAY;
    static_assert(KAX + 3 < 8, "column window must fit two float4s");

    const int tile = xcd_contiguous_tile(blockIdx.x, p.n_tiles);
    const int pg = tile / p.row_tiles, rt = tile - pg * p.row_tiles;
    const long plane0 = static_cast<long>(pg) * p.planes_per_tile;
    const int nplanes = static_cast<int>(min(static_cast<long>(p.planes_per_tile), p.planes - plane0));
    const int qy0 = rt * p.rows_per_tile;

    stage_taps<KK, true>(p, lds, plane0, nplanes);
    stage_tile(p, lds, plane0, nplanes, qy0 - p.row_shift);
    __syncthreads();

    const int n_items = nplanes * p.items_per_plane;
    for (int item = threadIdx.x; item < n_items; item += kThreads) {
        const int pl = fast_div(item, p.ipp_magic);
        const int rem = item - pl * p.items_per_plane;
        const int rb = fast_div(rem, p.ncb_magic);
        const int cb = rem - rb * p.ncb;

        float tapv[KK];
#pragma unroll
        for (int t = 0; t < KK; ++t) tapv[t] = lds[p.tap_base + pl * KK + t];

        const float *base = lds + pl * p.plane_pitch + (rb * BQ) * p.pitch + kSlack + 4 * cb;
        float acc[2 * BQ][8];
#pragma unroll
        for (int b = 0; b < 2 * BQ; ++b)
#pragma unroll
            for (int o = 0; o < 8; ++o) acc[b][o] = 0.f;

#pragma unroll
        for (int wr = 0; wr < WIN_ROWS; ++wr) {
            float win[8];
            {
                const float4 q0 = *reinterpret_cast<const float4 *>(base + wr * p.pitch);
                const float4 q1 = *reinterpret_cast<const float4 *>(base + wr * p.pitch + 4);
                win[0] = q0.x; win[1] = q0.y; win[2] = q0.z; win[3] = q0.w;
                win[4] = q1.x; win[5] = q1.y; win[6] = q1.z; win[7] = q1.w;
            }
#pragma unroll
            for (int bq = 0; bq < BQ; ++bq)
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    const int a = wr - bq - r;
                    if (a < 0 || a >= KAY) continue;
                    const int fy = r + 2 * a - EY;
                    if (fy < 0 || fy >= K) continue;
#pragma unroll
                    for (int xq = 0; xq < 4; ++xq)
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
        }

        const int ox = 8 * cb;
        float *dst = p.out + (plane0 + pl) * p.out_plane + ox;
#pragma unroll
        for (int b = 0; b < 2 * BQ; ++b) {
            const int oy = 2 * (qy0 + rb * BQ) + b;
            if (oy >= p.out_h) continue;
            float *row = dst + static_cast<long>(oy) * p.out_w;
            if (p.vec_out) {
                if (ox < p.out_w)
                    *reinterpret_cast<float4 *>(row) = make_float4(acc[b][0], acc[b][1], acc[b][2], acc[b][3]);
                if (ox + 4 < p.out_w)
                    *reinterpret_cast<float4 *>(row + 4) = make_float4(acc[b][4], acc[b][5], acc[b][6], acc[b][7]);
            } else {
#pragma unroll
                for (int o = 0; o < 8; ++o)
                    if (ox + o < p.out_w) row[o] = acc[b][o];
            }
        }
    }
}

int floor_div(int a, int b)
{
    int q = a / b;
    if ((a % b != 0) && ((a < 0) != (b < 0))) --q;
    return q;
}

int env_int(const char *name, int dflt)
{
    const char *e = std::getenv(name);
    if (e == nullptr || e[0] == '\0') return dflt;
    return std::atoi(e);
}

// Fills in the tiling of `p` for a plane whose output is split into `row_units`
// units of rows (BH output rows or BQ half-resolution rows each) and `ncb` column
// blocks.  `rows_for(units)` gives the LDS rows a band of that many units needs.
// Returns false when even the smallest tile exceeds the LDS budget.
template <typename RowsFor>
bool plan_tiles(TilePlan &p, int row_units, int unit_rows, int used_cols, int taps_per_plane, RowsFor rows_for)
{
    const int target_items = env_int("DWCONV_TILE_ITEMS", 2 * kThreads);
    p.pitch = kSlack + round_up(used_cols, 4) + kSlack;
    p.g_lo = floor_div(-p.col_shift, 4);
    p.spr = ceil_div(used_cols - p.col_shift, 4) - p.g_lo;

    auto bytes = [&](int units, int planes) {
        return static_cast<long>(planes) * (static_cast<long>(rows_for(units)) * p.pitch + taps_per_plane) * 4;
    };

    const int ipp_full = row_units * p.ncb;
    int units_per_tile, planes_per_tile;
    if (ipp_full <= target_items / 2) {
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
    p.lds_rows = rows_for(units_per_tile);
    p.plane_pitch = p.lds_rows * p.pitch;
    p.items_per_plane = units_per_tile * p.ncb;
    p.tap_base = planes_per_tile * p.plane_pitch;
    const long groups = (p.planes + planes_per_tile - 1) / planes_per_tile;
    const long tiles = groups * p.row_tiles;
    if (tiles > 0x7fffffffL) return false;
    p.n_tiles = static_cast<int>(tiles);
    // the in-kernel divisions use a 16-bit reciprocal
    if (planes_per_tile * p.lds_rows * p.spr >= 65536 || planes_per_tile * p.items_per_plane >= 65536) return false;
    p.lds_rows_magic = magic_u16(p.lds_rows);
    p.spr_magic = magic_u16(p.spr);
    p.ncb_magic = magic_u16(p.ncb);
    p.ipp_magic = magic_u16(p.items_per_plane);
    return true;
}

size_t lds_bytes(const TilePlan &p, int taps_per_plane)
{
    return static_cast<size_t>(p.planes_per_tile) * (p.plane_pitch + taps_per_plane) * 4;
}

template <int K, int S, bool FLIP, int BH>
int launch_down(TilePlan &p, hipStream_t stream)
{
    constexpr int NV = (3 * S + K + 3) / 4;
    p.ncb = ceil_div(p.out_w, 4);
    const int used_cols = 4 * (p.ncb - 1) * S + 4 * NV;
    auto rows_for = [](int units) { return (units * BH - 1) * S + K; };
    if (!plan_tiles(p, ceil_div(p.out_h, BH), BH, used_cols, K * K, rows_for)) return -1;
    hipLaunchKernelGGL((fir_down_kernel<K, S, FLIP, BH>), dim3(p.n_tiles), dim3(kThreads), lds_bytes(p, K * K),
                       stream, p);
    note_variant("tile_down<k%d,s%d,%s,bh%d> P%d rows%d vin%d vout%d", K, S, FLIP ? "rot" : "fwd", BH,
                 p.planes_per_tile, p.rows_per_tile, p.vec_in, p.vec_out);
    return check_launch("fir_down_kernel");
}

template <int K, int S, bool FLIP>
int launch_down_bh(TilePlan &p, hipStream_t stream)
{
    const int forced = env_int("DWCONV_TILE_BH", 0);
    const bool seven = forced ? forced == 7 : (p.out_h % 7 == 0 || p.out_h > 64) && p.out_h % 4 != 0;
    return seven ? launch_down<K, S, FLIP, 7>(p, stream) : launch_down<K, S, FLIP, 4>(p, stream);
}

template <int K, int EY, int EX>
int launch_up2(TilePlan &p, hipStream_t stream)
{
    constexpr int BQ = 2;
    constexpr int KAY = (K + EY + 1) / 2;
    p.ncb = ceil_div(p.out_w, 8);
    const int used_cols = 4 * (p.ncb - 1) + 8;
    auto rows_for = [](int units) { return units * BQ + KAY; };
    if (!plan_tiles(p, ceil_div(ceil_div(p.out_h, 2), BQ), BQ, used_cols, K * K, rows_for)) return -1;
    hipLaunchKernelGGL((fir_up2_kernel<K, EY, EX, BQ>), dim3(p.n_tiles), dim3(kThreads), lds_bytes(p, K * K), stream,
                       p);
    note_variant("tile_up2<k%d,e%d%d,bq%d> P%d rows%d vin%d vout%d", K, EY, EX, BQ, p.planes_per_tile,
                 p.rows_per_tile, p.vec_in, p.vec_out);
    return check_launch("fir_up2_kernel");
}

template <int K>
int launch_up2_parity(TilePlan &p, int ey, int ex, hipStream_t stream)
{
    if (ey == 0 && ex == 0) return launch_up2<K, 0, 0>(p, stream);
    if (ey == 0 && ex == 1) return launch_up2<K, 0, 1>(p, stream);
    if (ey == 1 && ex == 0) return launch_up2<K, 1, 0>(p, stream);
    return launch_up2<K, 1, 1>(p, stream);
}

}  // namespace

int try_launch_fir_tiled(const float *in, const float *taps, float *out, const Geometry &g, hipStream_t stream)
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
    p.in_h = g.in_h;
    p.in_w = g.in_w;
    p.out_h = g.out_h;
    p.out_w = g.out_w;
    p.in_plane = g.in_h * g.in_w;
    p.out_plane = g.out_h * g.out_w;
    p.vec_in = (g.in_w % 4 == 0) && aligned16(in);
    p.vec_out = (g.out_w % 4 == 0) && aligned16(out);

    if (g.up_h == 1 && g.up_w == 1 && g.down_h == g.down_w && (g.down_h == 1 || g.down_h == 2)) {
        p.row_shift = g.pad_h0;
        p.col_shift = g.pad_w0;
        const bool rot = !g.forward;
        if (g.down_h == 1) {
            if (K == 3) return rot ? launch_down_bh<3, 1, true>(p, stream) : launch_down_bh<3, 1, false>(p, stream);
            if (K == 5) return rot ? launch_down_bh<5, 1, true>(p, stream) : launch_down_bh<5, 1, false>(p, stream);
            return rot ? launch_down_bh<7, 1, true>(p, stream) : launch_down_bh<7, 1, false>(p, stream);
        }
        if (rot) return -1;
        if (K == 3) return launch_down_bh<3, 2, false>(p, stream);
        if (K == 5) return launch_down_bh<5, 2, false>(p, stream);
        return launch_down_bh<7, 2, false>(p, stream);
    }
    if (g.up_h == 2 && g.up_w == 2 && g.down_h == 1 && g.down_w == 1 && !g.forward) {
        const int ey = g.pad_h0 & 1, ex = g.pad_w0 & 1;
        p.row_shift = (g.pad_h0 + ey) / 2;
        p.col_shift = (g.pad_w0 + ex) / 2;
        if (K == 3) return launch_up2_parity<3>(p, ey, ex, stream);
        if (K == 5) return launch_up2_parity<5>(p, ey, ex, stream);
        return launch_up2_parity<7>(p, ey, ex, stream);
    }
    return -1;
}

}  // namespace dwconv
