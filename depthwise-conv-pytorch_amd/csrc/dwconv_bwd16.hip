// Fused backward pass of stride-1 "same" layers for 16-bit tensors (fp16, bf16) whose rows are whole groups of
// eight elements: grad-input and grad-weight from one pass over x and gy.
//
// Same decomposition as the fused kernel of dwconv_wgrad.hip (workgroup = channel group x chunk of tiles, one item
// per lane, per-lane tap sums reduced in a fixed order at the end, a second pass adds the chunks), with the LDS
// images kept in the tensors' own 16-bit format and two-element dot products (see dwconv_tile16.hip):
//   gx[oy,ox]   = sum gy[oy - pad + ty, ox - pad + tx] * f[K-1-ty, K-1-tx]   ceil(K/2) dot products per filter row
//   gw[ty,tx]  += sum_{o} gy[oy,ox+o] * x[oy - pad + ty, ox + o - pad + tx]  four dot products per tap, filter row
//                                                                             and row of the lane's 8-wide block
// Replaces, for these tensors, the two launches of torch_dwconv/dwconv.py:48-70 (dwconv_kernel.cu:69-181 with the
// rotated filter, and :260-306).
#include "dwconv_tile16_common.hpp"

namespace dwconv {

namespace {

struct Bwd16Plan {
    Image16 im;            // the x images; the gy images have the same layout
    const void *x;
    const void *gy;
    const void *taps;
    void *gx;
    float *partial;
    int batch, channel;
    int rows_per_tile, row_tiles;
    int planes_per_tile;   // channels a workgroup carries
    int groups;            // channel groups
    int chunks;            // chunks per channel group
    int tiles_per_group;   // batch * row_tiles
    int tiles_per_chunk;
    int strided;           // chunk k takes tiles k, k + chunks, ... instead of a contiguous range
    int ncb;
    unsigned ncb_magic;
    int items_per_plane;
    unsigned ipp_magic;
    int g_base;            // dword offset of the gy images in LDS
    int dump;              // slot index of a spare slot
    int lout;              // grad-input leaves through LDS as one linear stream per plane
};

template <typename IO, int K, int BH>
__global__ __launch_bounds__(kThreads) void bwd16_kernel(const Bwd16Plan p)
{
    extern __shared__ float4 lds_raw[];
    uint32_t *lds32 = reinterpret_cast<uint32_t *>(lds_raw);
    float *ldsf = reinterpret_cast<float *>(lds_raw);
    constexpr int KK = K * K;
    constexpr int PAD = K / 2;
    constexpr int PW1 = PAD & 1;
    constexpr int KP = (K + 1) / 2;
    constexpr int OWI = 8;
    constexpr int WIN_ROWS = BH - 1 + K;
    constexpr int NDW = (PW1 + OWI - 1 + K - 1) / 2 + 1;  // dwords of a window row
    const IO *const x = static_cast<const IO *>(p.x);
    const IO *const gy = static_cast<const IO *>(p.gy);

    const int group = blockIdx.x / p.chunks;
    const int chunk = blockIdx.x - group * p.chunks;
    const int c0 = group * p.planes_per_tile;
    const int nplanes = min(p.planes_per_tile, p.channel - c0);
    const int t_begin = p.strided ? chunk : chunk * p.tiles_per_chunk;
    const int t_end = p.strided ? p.tiles_per_group : min(p.tiles_per_group, t_begin + p.tiles_per_chunk);
    const int t_step = p.strided ? p.chunks : 1;
    const int n_items = nplanes * p.items_per_plane;

    // One item per lane (the planner guarantees n_items <= blockDim.x): its place in the tile is fixed.
    const bool has_item = static_cast<int>(threadIdx.x) < n_items;
    const bool wave_has_item = __builtin_amdgcn_readfirstlane(threadIdx.x) < n_items;
    const int item = has_item ? threadIdx.x : 0;
    const int pl = fast_div(item, p.ipp_magic);
    const int rem = item - __mul24(pl, p.items_per_plane);
    const int rb = fast_div(rem, p.ncb_magic);
    const int cb = rem - __mul24(rb, p.ncb);
    const int rpitch = p.im.rp;  // dwords per image row
    // The lane's window starts at logical dword 4 * cb + PH of image row rb * BH (its first element lies
    // (PAD + PW1) / 2 dwords left of the lane's block, which starts at dword 4 + 4 * cb); window dword i is LDS dword
    // xbase[swz(PH + i)].  The gy images lie g_base dwords on.
    constexpr int PH = 4 - (PAD + PW1) / 2;
    const uint32_t *xbase = lds32 + __mul24(pl, p.im.pp) + __mul24(rb * BH, p.im.rp) + 5 * cb;
    const uint32_t *gbase = xbase + p.g_base;
    // the lane's own block of gy, PAD rows into its window: logical dwords 4 * cb + 4 ...
    const uint32_t *gown = gbase + PAD * p.im.rp + 5;

    // rotated taps in pairs: [ty][0..KP-1] = (t[2j], t[2j+1]) (the last pair of an odd K is (t, 0)), [ty][KP] = (0, t)
    uint32_t tp[K][KP + 1];
    float t0_last;
    {
        const uint16_t *f = static_cast<const uint16_t *>(p.taps) + (c0 + pl) * KK;
        auto tap = [&](int ty, int tx) -> uint32_t { return tx < K ? f[(K - 1 - ty) * K + (K - 1 - tx)] : 0u; };
#pragma unroll
        for (int ty = 0; ty < K; ++ty) {
#pragma unroll
            for (int j = 0; j < KP; ++j) tp[ty][j] = tap(ty, 2 * j) | (tap(ty, 2 * j + 1) << 16);
            tp[ty][KP] = tap(ty, K - 1) << 16;
        }
        t0_last = Io<IO>::in(__builtin_bit_cast(IO, static_cast<uint16_t>(tap(0, K - 1))));
    }

    float acc[KK];
#pragma unroll
    for (int t = 0; t < KK; ++t) acc[t] = 0.f;

    const u32x4 *linear = reinterpret_cast<const u32x4 *>(lds_raw);
    for (int tile = t_begin; tile < t_end; tile += t_step) {
        const int n = tile / p.row_tiles, rt = tile - n * p.row_tiles;
        const long plane0 = static_cast<long>(n) * p.channel + c0;
        const int oy0 = rt * p.rows_per_tile;

        if (tile != t_begin) __syncthreads();  // the previous tile's window reads are done
        stage_image16(p.im, x + plane0 * p.im.in_plane, lds32, p.dump, nplanes, oy0 - PAD);
        stage_image16(p.im, gy + plane0 * p.im.in_plane, lds32 + p.g_base, p.dump - p.g_base / 5, nplanes, oy0 - PAD);
        __syncthreads();
        uint32_t packed[BH][OWI / 2];  // the lane's block of grad-input as 16-bit pairs
        // (uniform per wavefront: those without an item skip the arithmetic but meet every barrier)
        if (wave_has_item) {
        // ---- grad-input: the gy window against the rotated taps ----
        {
            float xacc[BH][OWI];
            uint32_t win[2][NDW];
#pragma unroll
            for (int i = 0; i < NDW; ++i) win[0][i] = gbase[swz(PH + i)];
#pragma unroll
            for (int wr = 0; wr < WIN_ROWS; ++wr) {
                const uint32_t(&d)[NDW] = win[wr & 1];
                if (wr + 1 < WIN_ROWS) {
#pragma unroll
                    for (int i = 0; i < NDW; ++i) win[(wr + 1) & 1][i] = gbase[(wr + 1) * rpitch + swz(PH + i)];
                }
                uint32_t q[NDW];  // pairs that start at an odd element
#pragma unroll
                for (int i = 0; i + 1 < NDW; ++i) q[i] = __builtin_amdgcn_alignbit(d[i + 1], d[i], 16);
                // the element under the last tap of each output: alone in its half for the dot product, and as fp32
                // for the output row this window row starts
                uint32_t last[OWI];
                float lastf[OWI];
#pragma unroll
                for (int o = 0; o < OWI; ++o) {
                    const int e = PW1 + o + K - 1;
                    last[o] = (e & 1) ? (d[e >> 1] & 0xffff0000u) : (d[e >> 1] & 0x0000ffffu);
                    const uint16_t h = static_cast<uint16_t>((e & 1) ? d[e >> 1] >> 16 : d[e >> 1] & 0xffffu);
                    lastf[o] = Io<IO>::in(__builtin_bit_cast(IO, h));
                }
#pragma unroll
                for (int b = 0; b < BH; ++b) {
                    const int ty = wr - b;
                    if (ty < 0 || ty >= K) continue;
#pragma unroll
                    for (int o = 0; o < OWI; ++o) {
                        const int el = PW1 + o + K - 1;
                        if (ty == 0) xacc[b][o] = lastf[o] * t0_last;
                        else xacc[b][o] = dot2<IO>(last[o], (el & 1) ? tp[ty][KP] : tp[ty][KP - 1], xacc[b][o]);
#pragma unroll
                        for (int j = 0; j < K / 2; ++j) {
                            const int e = PW1 + o + 2 * j;
                            xacc[b][o] = dot2<IO>((e & 1) ? q[e >> 1] : d[e >> 1], tp[ty][j], xacc[b][o]);
                        }
                    }
                }
#pragma unroll
                for (int b = 0; b < BH; ++b)
                    if (b <= wr) pin_registers(xacc[b]);  // the rows that have been started
            }
#pragma unroll
            for (int b = 0; b < BH; ++b)
#pragma unroll
                for (int m = 0; m < OWI / 2; ++m) {
                    if constexpr (std::is_same<IO, bf16_t>::value) packed[b][m] = bf16_pack2(xacc[b][2 * m], xacc[b][2 * m + 1]);
                    else packed[b][m] = f16_pack2(xacc[b][2 * m], xacc[b][2 * m + 1]);
                }
            if (!p.lout) {
                // branch-free: rows past the end of the plane (and lanes without an item) store out of range
                const __amdgpu_buffer_rsrc_t view =
                    buffer_view(static_cast<IO *>(p.gx) + plane0 * p.im.in_plane, static_cast<long>(nplanes) * p.im.in_plane * sizeof(IO));
                const unsigned o0 = (__mul24(pl, p.im.in_plane) + cb * OWI) * 2u;
#pragma unroll
                for (int b = 0; b < BH; ++b) {
                    const int oy = oy0 + rb * BH + b;
                    const bool ok = has_item && oy < p.im.in_h;
                    u32x4 t;
                    t.x = packed[b][0]; t.y = packed[b][1]; t.z = packed[b][2]; t.w = packed[b][3];
                    __builtin_amdgcn_raw_buffer_store_b128(t, view, ok ? o0 + __mul24(oy, p.im.in_w) * 2u : kOob, 0, kStoreStreaming);
                }
            }
        }

        // ---- grad-weight: the lane's block of gy against its x window ----
        if (has_item) {
            // gy rows past the end of the plane are zero in the image, so they add nothing
            uint32_t g[BH][OWI / 2];
#pragma unroll
            for (int b = 0; b < BH; ++b)
#pragma unroll
                for (int m = 0; m < OWI / 2; ++m) g[b][m] = gown[b * rpitch + m];
            uint32_t win[2][NDW];
#pragma unroll
            for (int i = 0; i < NDW; ++i) win[0][i] = xbase[swz(PH + i)];
#pragma unroll
            for (int wr = 0; wr < WIN_ROWS; ++wr) {
                const uint32_t(&d)[NDW] = win[wr & 1];
                if (wr + 1 < WIN_ROWS) {
#pragma unroll
                    for (int i = 0; i < NDW; ++i) win[(wr + 1) & 1][i] = xbase[(wr + 1) * rpitch + swz(PH + i)];
                }
                uint32_t q[NDW];
#pragma unroll
                for (int i = 0; i + 1 < NDW; ++i) q[i] = __builtin_amdgcn_alignbit(d[i + 1], d[i], 16);
#pragma unroll
                for (int b = 0; b < BH; ++b) {
                    const int ty = wr - b;
                    if (ty < 0 || ty >= K) continue;
#pragma unroll
                    for (int tx = 0; tx < K; ++tx)
#pragma unroll
                        for (int m = 0; m < OWI / 2; ++m) {
                            const int e = PW1 + 2 * m + tx;
                            acc[ty * K + tx] = dot2<IO>(g[b][m], (e & 1) ? q[e >> 1] : d[e >> 1], acc[ty * K + tx]);
                        }
                }
                pin_registers(acc);
            }
        }
        }  // wave_has_item

        if (p.lout) {
            // The packed rows go back into LDS in the layout the band has in memory, over the x images, and leave as
            // one linear stream per plane (16 bytes per lane, 1 KiB per wavefront and store): rows that are not whole
            // 128-byte lines (56 elements) would otherwise leave as partial lines.
            const int rows_here = min(p.rows_per_tile, p.im.in_h - oy0);
            const int run = rows_here * p.im.in_w;  // elements per plane, a multiple of eight
            __syncthreads();                        // every window has been read
            if (has_item) {
#pragma unroll
                for (int b = 0; b < BH; ++b) {
                    if (rb * BH + b < rows_here) {
                        // (16 bytes per lane at a multiple of 16 bytes: one conflict-free 128-bit write)
                        u32x4 t;
                        t.x = packed[b][0]; t.y = packed[b][1]; t.z = packed[b][2]; t.w = packed[b][3];
                        *reinterpret_cast<u32x4 *>(lds32 + ((__mul24(pl, run) + __mul24(rb * BH + b, p.im.in_w) + cb * OWI) >> 1)) = t;
                    }
                }
            }
            __syncthreads();
            const __amdgpu_buffer_rsrc_t view =
                buffer_view(static_cast<IO *>(p.gx) + plane0 * p.im.in_plane, static_cast<long>(nplanes) * p.im.in_plane * sizeof(IO));
            const int run8 = run >> 3;
            for (int q = 0; q < nplanes; ++q) {
                const unsigned o0 = (__mul24(q, p.im.in_plane) + __mul24(oy0, p.im.in_w)) * 2u;
                for (int i = threadIdx.x; i < run8; i += blockDim.x)
                    __builtin_amdgcn_raw_buffer_store_b128(linear[q * run8 + i], view, o0 + i * 16u, 0, kStoreStreaming);
            }
        }
    }

    __syncthreads();  // the images are dead; their LDS is reused for the reduction
    float *out = p.partial + (static_cast<long>(c0) * p.chunks + chunk) * KK;
    if (p.planes_per_tile == 1) {
        // every lane worked on the same channel: wavefront sums, then the four wavefronts in order
#pragma unroll
        for (int t = 0; t < KK; ++t) {
            const float s = wave_sum_to_last_lane(acc[t]);
            if ((threadIdx.x & 63) == 63) ldsf[(threadIdx.x >> 6) * KK + t] = s;
        }
        __syncthreads();
        if (threadIdx.x < KK) {
            float s = ldsf[threadIdx.x];
#pragma unroll
            for (int w = 1; w < kThreads / 64; ++w) s += ldsf[w * KK + threadIdx.x];
            out[threadIdx.x] = s;
        }
    } else {
        // lanes [pl*ipp, (pl+1)*ipp) hold channel c0+pl: transpose through LDS, then add each run front to back
#pragma unroll
        for (int t = 0; t < KK; ++t) ldsf[t * kRedPitch + threadIdx.x] = acc[t];
        __syncthreads();
        for (int e = threadIdx.x; e < nplanes * KK; e += blockDim.x) {
            const int q = e / KK, t = e - q * KK;
            const float *col = ldsf + t * kRedPitch + q * p.items_per_plane;
            float s = 0.f;
            for (int i = 0; i < p.items_per_plane; ++i) s += col[i];
            out[static_cast<long>(q) * p.chunks * KK + t] = s;
        }
    }
}

// The kernel covers: stride 1, pad K/2 on both axes, K in {3,5,7}, width a multiple of eight.
bool covers(const WgradGeometry &g)
{
    const int K = g.kernel_h;
    if (!env_int("DWCONV_BWD16", 1)) return false;
    if (g.kernel_w != K || (K != 3 && K != 5 && K != 7)) return false;
    if (g.down_h != 1 || g.down_w != 1 || g.pad_h != K / 2 || g.pad_w != K / 2) return false;
    if (g.out_h != g.in_h || g.out_w != g.in_w || g.in_h < 1) return false;
    // Rows of at least 96 elements: with 8-wide blocks a narrower plane has too few of them to occupy the lanes
    // (56 x 56: 98 blocks of 4 x 8), and the kernel of dwconv_wgrad.hip with its 4-wide blocks measured faster there
    // (96 against 102-112 us on the 56 x 56 3x3 layer of the stack).
    if (g.in_w % 8 != 0 || g.in_w < env_int("DWCONV_T16_MIN_W", 96)) return false;
    if (static_cast<long>(g.in_h) * g.in_w >= (1l << 30)) return false;
    return true;
}

template <int K, int BH>
bool make_plan(Bwd16Plan &p, const WgradGeometry &g)
{
    // workgroups in flight: a few tiles each, so that loading the taps and reducing the tap sums is paid once per
    // several tiles (112 x 112 3x3: 86 chunks of 3 tiles 73 us, 256 chunks of one 78 us)
    const int target_wgs = env_int("DWCONV_WGRAD_WGS", K == 7 ? 1536 : 3072);
    const int budget = env_int("DWCONV_BWD16_LDS", 40 * 1024);
    p.batch = g.batch;
    p.channel = g.channel;
    p.im.in_h = g.in_h;
    p.im.in_w = g.in_w;
    p.im.in_plane = g.in_h * g.in_w;
    p.ncb = g.in_w / 8;
    // windows reach input column (in_w - 1) + K/2, and its pair partner
    layout_image16(p.im, g.in_w - 1 + K / 2 + 1);
    auto rows_for = [](int units) { return units * BH - 1 + K; };
    auto tile_bytes = [&](int units, int planes) { return static_cast<long>(planes) * rows_for(units) * p.im.rp * 4 * 2 + 20; };
    const int row_units = ceil_div(g.in_h, BH);
    const int ipp_full = row_units * p.ncb;
    int units_per_tile, planes_per_tile;
    if (2 * ipp_full <= kThreads && g.channel > 1) {
        // whole planes, P channels side by side, one item per lane
        units_per_tile = row_units;
        planes_per_tile = std::min(kThreads / ipp_full, g.channel);
        while (planes_per_tile > 1 && tile_bytes(units_per_tile, planes_per_tile) > budget) --planes_per_tile;
        if (tile_bytes(units_per_tile, planes_per_tile) > budget) return false;
    } else {
        planes_per_tile = 1;
        units_per_tile = std::max(1, std::min(row_units, kThreads / p.ncb));
        while (units_per_tile > 1 && tile_bytes(units_per_tile, 1) > budget) --units_per_tile;
        if (tile_bytes(units_per_tile, 1) > budget) return false;
        units_per_tile = ceil_div(row_units, ceil_div(row_units, units_per_tile));
    }
    p.planes_per_tile = planes_per_tile;
    p.rows_per_tile = units_per_tile * BH;
    p.row_tiles = ceil_div(row_units, units_per_tile);
    if (!finish_image16(p.im, rows_for(units_per_tile), planes_per_tile)) return false;
    p.items_per_plane = units_per_tile * p.ncb;
    if (planes_per_tile * p.items_per_plane > kThreads) return false;  // one item per lane
    p.ncb_magic = magic_u16(p.ncb);
    p.ipp_magic = magic_u16(p.items_per_plane);
    p.g_base = planes_per_tile * p.im.pp;
    p.dump = 2 * planes_per_tile * p.im.lds_rows * (p.im.pitch / 8);
    p.groups = ceil_div(g.channel, planes_per_tile);
    const long tiles_per_group = static_cast<long>(g.batch) * p.row_tiles;
    if (tiles_per_group > 0x7fffffffL) return false;
    p.tiles_per_group = static_cast<int>(tiles_per_group);
    int chunks = std::max(1, std::min(p.tiles_per_group, ceil_div(target_wgs, p.groups)));
    p.tiles_per_chunk = ceil_div(p.tiles_per_group, chunks);
    p.chunks = ceil_div(p.tiles_per_group, p.tiles_per_chunk);
    if (static_cast<long>(p.groups) * p.chunks > 0x7fffffffL) return false;
    p.strided = env_int("DWCONV_WGRAD_STRIDED", 1);
    p.lout = env_int("DWCONV_BWD16_LOUT", 1);
    return true;
}

template <int K, int BH>
size_t lds_bytes(const Bwd16Plan &p)
{
    const size_t tile = static_cast<size_t>(p.dump + 1) * 20;
    const size_t red = p.planes_per_tile == 1 ? static_cast<size_t>(kThreads / 64) * K * K * 4
                                              : static_cast<size_t>(K) * K * kRedPitch * 4;
    return tile > red ? tile : red;
}

// fn.template operator()<K, BH>() for the instance that covers g
template <typename Fn>
void dispatch(const WgradGeometry &g, Fn &&fn)
{
    const int forced = env_int("DWCONV_TILE_BH", 0);
    const bool seven = forced ? forced == 7 : (g.out_h % 7 == 0 || g.out_h > 64) && g.out_h % 4 != 0;
    const int K = g.kernel_h;
    if (K == 3) { if (seven) fn.template operator()<3, 7>(); else fn.template operator()<3, 4>(); }
    if (K == 5) { if (seven) fn.template operator()<5, 7>(); else fn.template operator()<5, 4>(); }
    if (K == 7) { if (seven) fn.template operator()<7, 7>(); else fn.template operator()<7, 4>(); }
}

struct WorkspaceQuery {
    const WgradGeometry &g;
    size_t bytes = 0;
    template <int K, int BH>
    void operator()()
    {
        Bwd16Plan p{};
        if (make_plan<K, BH>(p, g)) bytes = static_cast<size_t>(p.groups) * p.planes_per_tile * p.chunks * K * K * sizeof(float);
    }
};

template <typename IO>
struct Launcher {
    const IO *x;
    const IO *gy;
    const IO *taps;
    IO *gx;
    IO *gw;
    void *ws;
    size_t ws_bytes;
    const WgradGeometry &g;
    hipStream_t stream;
    int rc = -1;
    template <int K, int BH>
    void operator()()
    {
        Bwd16Plan p{};
        if (!make_plan<K, BH>(p, g)) return;
        const size_t need = static_cast<size_t>(p.groups) * p.planes_per_tile * p.chunks * K * K * sizeof(float);
        if (ws == nullptr || ws_bytes < need) {
            rc = fail(DWCONV_ERR_WORKSPACE, "grad-weight needs a workspace of %zu bytes, got %zu", need, ws_bytes);
            return;
        }
        p.x = x;
        p.gy = gy;
        p.taps = taps;
        p.gx = gx;
        p.partial = static_cast<float *>(ws);
        const size_t shmem = lds_bytes<K, BH>(p);
        hipLaunchKernelGGL((bwd16_kernel<IO, K, BH>), dim3(p.groups * p.chunks), dim3(kThreads), shmem, stream, p);
        rc = check_launch("bwd16_kernel");
        if (rc != DWCONV_OK) return;
        note_variant("bwd_tile16_dot2<k%d,s1,bh%d> P%d rows%d chunks%d%s", K, BH, p.planes_per_tile, p.rows_per_tile, p.chunks,
                     p.lout ? " ldsout" : "");
        rc = launch_wgrad_final(static_cast<const float *>(ws), gw, g.channel, K * K, p.chunks, stream);
    }
};

}  // namespace

size_t bwd_tiled16_workspace(const WgradGeometry &g)
{
    if (!covers(g)) return 0;
    WorkspaceQuery q{g};
    dispatch(g, q);
    return q.bytes;
}

template <typename IO>
int try_launch_bwd_tiled16(const IO *in, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes,
                           const WgradGeometry &g, hipStream_t stream)
{
    static_assert(sizeof(IO) == 2, "16-bit element types");
    if (!covers(g)) return -1;
    if (reinterpret_cast<uintptr_t>(in) % 16 != 0 || reinterpret_cast<uintptr_t>(gy) % 16 != 0 || reinterpret_cast<uintptr_t>(gx) % 16 != 0)
        return -1;
    Launcher<IO> l{in, gy, taps, gx, gw, ws, ws_bytes, g, stream};
    dispatch(g, l);
    return l.rc;
}

template int try_launch_bwd_tiled16<half_t>(const half_t *, const half_t *, const half_t *, half_t *, half_t *, void *, size_t,
                                            const WgradGeometry &, hipStream_t);
template int try_launch_bwd_tiled16<bf16_t>(const bf16_t *, const bf16_t *, const bf16_t *, bf16_t *, bf16_t *, void *, size_t,
                                            const WgradGeometry &, hipStream_t);

}  // namespace dwconv
