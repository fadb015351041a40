// Fused backward pass (grad-weight + grad-input) for stride-2 layers on large maps (fp32, fp16 or bf16 tensors).
//
// Workgroup (channel c, chunk k) walks tiles (image n, band of rows).  Per tile two images are staged
// in LDS: the band of x the grad-weight sums need, and the (four times smaller) band of gy.  A lane
// owns BQ x 2 elements of gy:
//   grad-input : out[2q + r] = sum_a gy[q - m + r + a] * rot'[r + 2a] along each axis (the zero-stuffed
//                gradient never exists); the lane's 2*BQ x 4 block of gx goes straight to memory
//                with 128-bit stores that are contiguous across lanes;
//   grad-weight: its gy elements (the centre of the window it just walked) against the x window
//                they touch, accumulated in K*K registers for the whole chunk, then reduced in a fixed
//                order exactly like the stride-1 kernel (DPP within a wavefront, LDS across
//                wavefronts) into partial[c][k][tap].
// gy is read from HBM once for both gradients; the reference reads it twice
// (torch_dwconv/dwconv.py:56-68) and x K*K times (torch_dwconv/dwconv_kernel.cu:260-306).
#include "dwconv_tile_common.hpp"

#include <type_traits>

namespace dwconv {

namespace {

constexpr int kFusedLdsBudget = 36 * 1024;    // both images of a tile

struct BwdS2Plan {
    StageLayout sx;   // x image: row r holds x row 2*q0 - pad + r, column c holds x column c - pad
    StageLayout sg;   // gy image: row r holds gy row q0 - m + r, column c holds gy column c - m
    const void *x;    // element type IO of the kernel template
    const void *gy;
    const void *taps;
    void *gx;
    float *partial;
    int channel;
    int pad;          // forward padding (both axes)
    int m;            // (K - 1 - pad + E) / 2
    int g_base;       // float offset of the gy image in LDS
    int rows_per_tile;  // half-resolution rows per tile
    int row_tiles;
    int tiles_per_group, chunks;
    int ncb;
    unsigned ncb_magic;
    int n_items;
    int bq;
    int vec_gx;
    bool prefetch;    // two-step staging, if the tensors turn out to be reachable through buffer views
};


// E = parity of the transposed problem's leading pad K - 1 - pad (the same on both axes).
// BQ: half-resolution rows per lane (4; 2 for planes too low to give every lane a block of 4).
// VIEWS: x, gy and gx all go through buffer views (sx.vec_in == sg.vec_in == vec_gx == 2), nothing else compiled in.
// PF (with VIEWS): the images travel in two steps (fetch_rows / commit_rows), each one's loads in flight during an
// arithmetic phase.  Order of a tile, two barriers as without PF: [gy of this tile is in registers] commit gy |
// barrier | issue the loads of x | grad-input from the gy windows | commit x | barrier | issue the loads of the next
// tile's gy | grad-weight sums over the x windows.
constexpr int kPrefetchSlots = 8;  // loads per lane and image at most (the planner checks rows_fit)

template <typename IO, int K, int E, int BQ, bool VIEWS, bool PF = false>
__global__ __launch_bounds__(kThreads) void bwd_s2_kernel(const BwdS2Plan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    const IO *const x = static_cast<const IO *>(p.x);
    const IO *const gy = static_cast<const IO *>(p.gy);
    constexpr int KK = K * K;
    constexpr int KA = (K + E + 1) / 2;
    constexpr int GW_ROWS = BQ + KA;                  // gy window rows
    constexpr int NWG = 2 * ((KA + 2 + 1) / 2);       // gy window columns, as float2s
    constexpr int XW_ROWS = (BQ - 1) * 2 + K;         // x window rows
    constexpr int NVX = (K + 2 + 3) / 4;              // x window columns, as float4s

    // every XCD (own L2) gets a contiguous run of workgroups: chunks k and k + 1 of a channel walk neighbouring
    // bands in step and share their halo rows (-2 % on the 112x112 layer)
    const int wg = xcd_contiguous_tile(blockIdx.x, gridDim.x);
    const int c = wg / p.chunks;
    const int chunk = wg - c * p.chunks;

    const bool has_item = static_cast<int>(threadIdx.x) < p.n_items;
    const int item = has_item ? threadIdx.x : 0;
    const int rb = fast_div(item, p.ncb_magic);
    const int cb = item - rb * p.ncb;
    const float *base_x = lds + (rb * BQ * 2) * p.sx.pitch + kSlack + 4 * cb;
    const float *base_g = lds + p.g_base + (rb * BQ) * p.sg.pitch + kSlack + 2 * cb;

    float rot[KK];
#pragma unroll
    for (int t = 0; t < KK; ++t) rot[t] = Io<IO>::in(static_cast<const IO *>(p.taps)[c * KK + KK - 1 - t]);
    float wacc[KK];
#pragma unroll
    for (int t = 0; t < KK; ++t) wacc[t] = 0.f;

    static_assert(!PF || VIEWS, "the two-step staging goes through buffer views");
    RowLane lane_x{}, lane_g{};
    typename Raw4<IO>::type staged[PF ? kPrefetchSlots : 1];
    if constexpr (PF) {
        lane_x = row_lane<IO>(p.sx);
        lane_g = row_lane<IO>(p.sg);
        if (chunk < p.tiles_per_group) {
            const int n = chunk / p.row_tiles, rt = chunk - n * p.row_tiles;
            fetch_rows<IO, kPrefetchSlots>(p.sg, lane_g, gy + (static_cast<long>(n) * p.channel + c) * p.sg.in_plane,
                                           rt * p.rows_per_tile - p.m, staged);
        }
    }

    for (int tile = chunk; tile < p.tiles_per_group; tile += p.chunks) {
        const int n = tile / p.row_tiles, rt = tile - n * p.row_tiles;
        const long plane0 = static_cast<long>(n) * p.channel + c;
        const int q0 = rt * p.rows_per_tile;

        if constexpr (PF) {
            // (every lane read its gy windows of the previous tile before that tile's second barrier)
            commit_rows<IO, kPrefetchSlots>(p.sg, lane_g, lds + p.g_base, staged);
            __syncthreads();
            fetch_rows<IO, kPrefetchSlots>(p.sx, lane_x, x + plane0 * p.sx.in_plane, 2 * q0 - p.pad, staged);
        } else {
            if (tile != chunk) __syncthreads();  // the previous tile's window reads are done
            // fp32: two 16-byte loads in flight per lane and image (not four): -3 % on the 112x112 layer, the two
            // images' loads overlap.  16-bit elements: four 8-byte loads, the same bytes in flight (112x112 C=96
            // 176 -> 166 us).
            constexpr int kInFlight = sizeof(IO) == 2 ? 4 : 2;
            stage_tile<IO, VIEWS, kInFlight>(p.sx, x, lds, plane0, 1, 2 * q0 - p.pad);
            stage_tile<IO, VIEWS, kInFlight>(p.sg, gy, lds + p.g_base, plane0, 1, q0 - p.m);
            __syncthreads();
        }

        // ---- gy window: grad-input block, and this lane's gy elements from the window's centre
        float g[BQ][2];
        float xacc[2 * BQ][4];
#pragma unroll
        for (int b = 0; b < 2 * BQ; ++b)
#pragma unroll
            for (int o = 0; o < 4; ++o) xacc[b][o] = 0.f;
        float nxg[NWG];
        load_window_row2<NWG / 2>(base_g, nxg);
#pragma unroll
        for (int wr = 0; wr < GW_ROWS; ++wr) {
            float win[NWG];
#pragma unroll
            for (int i = 0; i < NWG; ++i) win[i] = nxg[i];
            if (wr + 1 < GW_ROWS) load_window_row2<NWG / 2>(base_g + (wr + 1) * p.sg.pitch, nxg);
            if (wr >= p.m && wr - p.m < BQ) {
                // the centre row index depends on m (1 or 2 for the kernels served here): select at run time
#pragma unroll
                for (int bq = 0; bq < BQ; ++bq)
                    if (wr - p.m == bq) {
                        g[bq][0] = has_item ? (p.m == 1 ? win[1] : (p.m == 2 ? win[2] : win[0])) : 0.f;
                        g[bq][1] = has_item ? (p.m == 1 ? win[2] : (p.m == 2 ? win[3] : win[1])) : 0.f;
                    }
            }
#pragma unroll
            for (int bq = 0; bq < BQ; ++bq)
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    const int a = wr - bq - r;
                    if (a < 0 || a >= KA) continue;
                    const int fy = r + 2 * a - E;
                    if (fy < 0 || fy >= K) continue;
#pragma unroll
                    for (int xq = 0; xq < 2; ++xq)
#pragma unroll
                        for (int rx = 0; rx < 2; ++rx)
#pragma unroll
                            for (int ax = 0; ax < KA; ++ax) {
                                const int fx = rx + 2 * ax - E;
                                if (fx < 0 || fx >= K) continue;
                                xacc[2 * bq + r][2 * xq + rx] =
                                    fmaf(win[xq + rx + ax], rot[fy * K + fx], xacc[2 * bq + r][2 * xq + rx]);
                            }
                }
            pin_registers(xacc);
        }
        if (VIEWS || p.vec_gx >= 2) {
            // branch-free: rows and column blocks past the end of the plane store out of range
            const int ox = 4 * cb;
            const __amdgpu_buffer_rsrc_t view = buffer_view(static_cast<IO *>(p.gx) + plane0 * p.sx.in_plane, static_cast<long>(p.sx.in_plane) * sizeof(IO));  // this plane only
            const bool col_ok = has_item && ox < p.sx.in_w;
            bool done = false;
            if constexpr (!VIEWS) {
                if (p.vec_gx == 3) {  // rows of any width: the block that ends a row may be short
#pragma unroll
                    for (int b = 0; b < 2 * BQ; ++b) {
                        const int oy = 2 * (q0 + rb * BQ) + b;
                        const bool ok = col_ok && oy < p.sx.in_h;
                        view_store_first<IO>(view, ok ? (oy * p.sx.in_w + ox) * static_cast<unsigned>(sizeof(IO)) : kOob,
                                             p.sx.in_w - ox, p.sx.in_w & 3, xacc[b][0], xacc[b][1], xacc[b][2], xacc[b][3]);
                    }
                    done = true;
                }
            }
            if (!done) {
#pragma unroll
                for (int b = 0; b < 2 * BQ; ++b) {
                    const int oy = 2 * (q0 + rb * BQ) + b;
                    const bool ok = col_ok && oy < p.sx.in_h;
                    view_store4<IO>(view, ok ? (oy * p.sx.in_w + ox) * static_cast<unsigned>(sizeof(IO)) : kOob, xacc[b][0],
                                    xacc[b][1], xacc[b][2], xacc[b][3]);
                }
            }
        } else if (!VIEWS && has_item) {
            const int ox = 4 * cb;
            IO *dst = static_cast<IO *>(p.gx) + plane0 * p.sx.in_plane + ox;
#pragma unroll
            for (int b = 0; b < 2 * BQ; ++b) {
                const int oy = 2 * (q0 + rb * BQ) + b;
                if (oy >= p.sx.in_h) continue;
                IO *row = dst + static_cast<long>(oy) * p.sx.in_w;
                if (p.vec_gx) {
                    if (ox < p.sx.in_w) store4<IO>(row, xacc[b][0], xacc[b][1], xacc[b][2], xacc[b][3]);
                } else {
#pragma unroll
                    for (int o = 0; o < 4; ++o)
                        if (ox + o < p.sx.in_w) row[o] = Io<IO>::out(xacc[b][o]);
                }
            }
        }

        if constexpr (PF) {
            // (every lane read its x windows of the previous tile before this tile's first barrier)
            commit_rows<IO, kPrefetchSlots>(p.sx, lane_x, lds, staged);
            __syncthreads();
            const int next = tile + p.chunks;
            if (next < p.tiles_per_group) {
                const int nn = next / p.row_tiles, nrt = next - nn * p.row_tiles;
                fetch_rows<IO, kPrefetchSlots>(p.sg, lane_g, gy + (static_cast<long>(nn) * p.channel + c) * p.sg.in_plane,
                                               nrt * p.rows_per_tile - p.m, staged);
            }
        }

        // ---- x window: grad-weight sums
        float nxx[4 * NVX];
        load_window_row<NVX>(base_x, nxx);
#pragma unroll
        for (int wr = 0; wr < XW_ROWS; ++wr) {
            float win[4 * NVX];
#pragma unroll
            for (int i = 0; i < 4 * NVX; ++i) win[i] = nxx[i];
            if (wr + 1 < XW_ROWS) load_window_row<NVX>(base_x + (wr + 1) * p.sx.pitch, nxx);
#pragma unroll
            for (int bq = 0; bq < BQ; ++bq) {
                const int ty = wr - 2 * bq;
                if (ty < 0 || ty >= K) continue;
#pragma unroll
                for (int tx = 0; tx < K; ++tx)
#pragma unroll
                    for (int o = 0; o < 2; ++o) wacc[ty * K + tx] = fmaf(g[bq][o], win[2 * o + tx], wacc[ty * K + tx]);
            }
            pin_registers(wacc);
        }
    }

    __syncthreads();  // the images are dead; their LDS is reused for the reduction
#pragma unroll
    for (int t = 0; t < KK; ++t) {
        const float s = wave_sum_to_last_lane(wacc[t]);
        if ((threadIdx.x & 63) == 63) lds[(threadIdx.x >> 6) * KK + t] = s;
    }
    __syncthreads();
    if (threadIdx.x < KK) {
        float s = lds[threadIdx.x];
        for (int w = 1; w < static_cast<int>(blockDim.x) / 64; ++w) s += lds[w * KK + threadIdx.x];
        p.partial[(static_cast<long>(c) * p.chunks + chunk) * KK + threadIdx.x] = s;
    }
}

template <int K>
bool plan_bwd_s2(BwdS2Plan &p, const WgradGeometry &g, int kBq, size_t esize)
{
    const int pad0 = K - 1 - g.pad_h;  // leading pad of the transposed problem
    const int E = pad0 & 1;
    const int KA = (K + E + 1) / 2;
    const int NWG = 2 * ((KA + 2 + 1) / 2);
    const int NVX = (K + 2 + 3) / 4;
    p.channel = g.channel;
    p.bq = kBq;
    p.pad = g.pad_h;
    p.m = (pad0 + E) / 2;
    if (p.m > 2) return false;
    p.ncb = ceil_div(std::max((g.in_w + 1) / 2, g.out_w), 2);
    if (p.ncb > kThreads) return false;

    p.sx.in_h = g.in_h;
    p.sx.in_w = g.in_w;
    p.sx.in_plane = g.in_h * g.in_w;
    p.sx.col_shift = g.pad_w;
    layout_columns(p.sx, 4 * (p.ncb - 1) + 4 * NVX);
    p.sg.in_h = g.out_h;
    p.sg.in_w = g.out_w;
    p.sg.in_plane = g.out_h * g.out_w;
    p.sg.col_shift = p.m;
    layout_columns(p.sg, 2 * (p.ncb - 1) + NWG);

    const int qrows = std::max((g.in_h + 1) / 2, g.out_h);
    const int row_units = ceil_div(qrows, kBq);
    auto rows_x = [&](int units) { return (units * kBq - 1) * 2 + K; };
    auto rows_g = [&](int units) { return units * kBq + KA; };
    auto bytes = [&](int units) {
        return (static_cast<long>(rows_x(units)) * p.sx.pitch + static_cast<long>(rows_g(units)) * p.sg.pitch) * 4;
    };
    int units = kThreads / p.ncb;
    if (units < 1) units = 1;
    if (units > row_units) units = row_units;
    const int budget = env_int("DWCONV_FUSED_LDS", kFusedLdsBudget);
    while (units > 1 && bytes(units) > budget) --units;
    if (bytes(units) > 60 * 1024) return false;
    const int bands = ceil_div(row_units, units);
    units = ceil_div(row_units, bands);
    p.rows_per_tile = units * kBq;
    p.row_tiles = bands;
    if (!layout_rows(p.sx, rows_x(units), 1) || !layout_rows(p.sg, rows_g(units), 1)) return false;
    p.g_base = p.sx.plane_pitch;
    p.n_items = units * p.ncb;
    p.ncb_magic = magic_u16(p.ncb);
    const long tiles = static_cast<long>(g.batch) * bands;
    if (tiles > 0x7fffffffL) return false;
    p.tiles_per_group = static_cast<int>(tiles);
    // Workgroups in all.  The fp32 5x5 / 7x7 kernels gain from twice as many, shorter chunks; the 3x3 one does not, and with 16-bit elements, where the kernel is bound by
    // instruction issue, the per-workgroup prologue and reduction make more chunks 8-15 % slower.
    // Two-step staging (see the kernel) is for 16-bit elements, where the arithmetic is long against the bytes: 56x56
    // 5x5 bf16 88 -> 81 us, 112x112 3x3 bf16 162 -> 156.  It needs several tiles per workgroup, and its registers
    // leave room for four workgroups per CU (three with 7x7 filters), so the workgroups are counted to fill the chip
    // three times over, rounded down (with one chunk more per channel, a fourth, nearly empty round: +5 %).  With fp32
    // elements it gains on some layers and loses on others inside a training step (48x48 5x5 92 -> 85 us, 56x56 117 ->
    // 124, 64x64 137 -> 142; 3x3 112x112 274 -> 287): those kernels wait for memory with all their loads in flight
    // as they are, and stay as they were.  The choice is made from the geometry alone, so that the workspace query
    // and the launch agree; tensors that then turn out to be misaligned run the one-step kernel on the same chunks.
    const int pf_mode = env_int("DWCONV_S2_PREFETCH", 1);  // 0: never, 1: 16-bit elements, 2: wherever it fits
    p.prefetch = (pf_mode == 2 || (pf_mode == 1 && esize == 2)) && rows_fit(p.sx, kPrefetchSlots) &&
                 rows_fit(p.sg, kPrefetchSlots) && g.in_w % 4 == 0 && g.out_w % 4 == 0 &&
                 stage_vector_mode(p.sx, 1, esize) == 2 && stage_vector_mode(p.sg, 1, esize) == 2 &&
                 vector_mode(1, p.sx.in_plane, esize) == 2;
    int chunks;
    if (p.prefetch) {
        chunks = env_int("DWCONV_WGRAD_WGS", kCus * (K == 7 ? 3 : 4) * 3) / g.channel;
    } else {
        // (5x5 fp32: 6144 against 12288 measured 3-8 % faster on 48- to 64-wide maps, the same at 75 and 128 x 96;
        // 3x3 fp32: on maps 96 wide and more three workgroups per CU, all resident from the start, against 3072: 2-7 %
        // faster on 96-, 112- and 120-wide layers; 38 x 38 likes twice as many, 129 -> 121 us)
        const int wgs = K >= 5 && esize == 4 ? 6144 : (K == 3 && esize == 4 ? (g.in_w >= 96 ? 768 : (g.in_w < 48 ? 6144 : 3072)) : 3072);
        chunks = ceil_div(env_int(K == 3 ? "DWCONV_S2_WGS_K3" : "DWCONV_WGRAD_WGS", wgs), g.channel);
    }
    if (chunks > p.tiles_per_group) chunks = p.tiles_per_group;
    if (chunks < 1) chunks = 1;
    p.chunks = chunks;
    if (static_cast<long>(g.channel) * chunks > 0x7fffffffL) return false;
    return true;
}

template <typename IO, int K>
long bwd_s2_case(int mode, const IO *x, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws,
                 size_t ws_bytes, const WgradGeometry &g, hipStream_t stream)
{
    // blocks of 4 half-resolution rows, or of 2 when that is what it takes to give most lanes an item
    const int qrows = std::max((g.in_h + 1) / 2, g.out_h), pairs = ceil_div(std::max((g.in_w + 1) / 2, g.out_w), 2);
    const int bq = ceil_div(qrows, 4) * pairs * 2 <= kThreads ? 2 : 4;
    BwdS2Plan p{};
    if (!plan_bwd_s2<K>(p, g, bq, sizeof(IO))) return -1;
    const size_t need = static_cast<size_t>(g.channel) * p.chunks * K * K * sizeof(float);
    if (mode == 0) return static_cast<long>(need);
    if (ws == nullptr || ws_bytes < need)
        return fail(DWCONV_ERR_WORKSPACE, "backward needs a workspace of %zu bytes, got %zu", need, ws_bytes);
    p.x = x;
    p.gy = gy;
    p.taps = taps;
    p.gx = gx;
    p.partial = static_cast<float *>(ws);
    p.sx.vec_in = row_vector_mode(g.in_w, x);
    p.sg.vec_in = row_vector_mode(g.out_w, gy);
    p.vec_gx = row_vector_mode(g.in_w, gx, false);
    // (rows of any width, mode 3, need the view; the aligned modes choose between pointer and view)
    const int x_view = stage_vector_mode(p.sx, 1, sizeof(IO)), g_view = stage_vector_mode(p.sg, 1, sizeof(IO));
    const int gx_view = vector_mode(1, p.sx.in_plane, sizeof(IO));
    p.sx.vec_in = p.sx.vec_in == 1 ? x_view : (p.sx.vec_in == 3 && x_view == 2 ? 3 : 0);
    p.sg.vec_in = p.sg.vec_in == 1 ? g_view : (p.sg.vec_in == 3 && g_view == 2 ? 3 : 0);
    p.vec_gx = p.vec_gx == 1 ? gx_view : (p.vec_gx == 3 && gx_view == 2 ? 3 : 0);
    const size_t images = static_cast<size_t>(p.sx.plane_pitch + p.sg.plane_pitch) * 4;
    const size_t red = static_cast<size_t>(kThreads / 64) * K * K * 4;
    const size_t shmem = images > red ? images : red;
    const int E = (K - 1 - g.pad_h) & 1;
    const dim3 grid(g.channel * p.chunks), block(kThreads)  /* all 256 lanes stage the images even when the tile has fewer items */;
    const bool views = p.sx.vec_in == 2 && p.sg.vec_in == 2 && p.vec_gx == 2 && !env_int("DWCONV_NO_VIEW_ONLY", 0);
    const bool prefetch = views && p.prefetch;
    auto launch = [&](auto kernel) { hipLaunchKernelGGL(kernel, grid, block, shmem, stream, p); };
    auto pick = [&](auto e, auto b) {
        constexpr int kE = decltype(e)::value, kB = decltype(b)::value;
        if (prefetch) launch(bwd_s2_kernel<IO, K, kE, kB, true, true>);
        else if (views) launch(bwd_s2_kernel<IO, K, kE, kB, true>);
        else launch(bwd_s2_kernel<IO, K, kE, kB, false>);
    };
    using std::integral_constant;
    if (bq == 2) {
        if (E) pick(integral_constant<int, 1>{}, integral_constant<int, 2>{});
        else pick(integral_constant<int, 0>{}, integral_constant<int, 2>{});
    } else if (E) pick(integral_constant<int, 1>{}, integral_constant<int, 4>{});
    else pick(integral_constant<int, 0>{}, integral_constant<int, 4>{});
    const int rc = check_launch("bwd_s2_kernel");
    if (rc != DWCONV_OK) return rc;
    note_variant("bwd_tile_s2%s<k%d,e%d,bq%d> rows%d chunks%d vin%d vgy%d vgx%d%s", sizeof(IO) == 2 ? "16" : "", K, E, bq,
                 p.rows_per_tile, p.chunks, p.sx.vec_in, p.sg.vec_in, p.vec_gx, prefetch ? " pf" : "");
    return launch_wgrad_final(p.partial, gw, g.channel, K * K, p.chunks, stream);
}

template <typename IO>
long bwd_s2_any(int mode, const IO *x, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws,
                size_t ws_bytes, const WgradGeometry &g, hipStream_t stream)
{
    if (env_int("DWCONV_NO_FUSED_TILE", 0)) return -1;
    const int K = g.kernel_h;
    if (g.kernel_w != K || g.down_h != 2 || g.down_w != 2) return -1;
    if (g.pad_h != g.pad_w || g.pad_h < 0 || g.pad_h > K - 1) return -1;
    if (g.in_h < 1 || g.in_w < 1 || g.out_h < 1 || g.out_w < 1) return -1;
    if (static_cast<long>(g.in_h) * g.in_w >= (1l << 30)) return -1;
    if (K == 3) return bwd_s2_case<IO, 3>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
    if (K == 5) return bwd_s2_case<IO, 5>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
    if (K == 7) return bwd_s2_case<IO, 7>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
    return -1;
}

}  // namespace

size_t bwd_s2_workspace(const WgradGeometry &g)
{
    // partial sums are fp32 whatever the element type
    const long n = bwd_s2_any<float>(0, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, g, nullptr);
    return n > 0 ? static_cast<size_t>(n) : 0;
}

template <typename IO>
int try_launch_bwd_s2(const IO *in, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes,
                      const WgradGeometry &g, hipStream_t stream)
{
    return static_cast<int>(bwd_s2_any<IO>(1, in, gy, taps, gx, gw, ws, ws_bytes, g, stream));
}

template int try_launch_bwd_s2<float>(const float *, const float *, const float *, float *, float *, void *, size_t,
                                      const WgradGeometry &, hipStream_t);
template int try_launch_bwd_s2<half_t>(const half_t *, const half_t *, const half_t *, half_t *, half_t *, void *, size_t,
                                       const WgradGeometry &, hipStream_t);
template int try_launch_bwd_s2<bf16_t>(const bf16_t *, const bf16_t *, const bf16_t *, bf16_t *, bf16_t *, void *, size_t,
                                       const WgradGeometry &, hipStream_t);

}  // namespace dwconv
