// LDS-tiled forward / stride-1 grad-input kernel for 16-bit tensors (fp16, bf16) whose rows are whole groups of
// eight elements.
//
// The tiled kernels of dwconv_tile.hip widen every element to fp32 on its way into LDS.  With 16-bit tensors they
// are bound by the vector unit, not by memory: the same instructions move half the bytes.  This kernel keeps the
// elements as loaded, two per dword:
//   load  = eight elements (16 bytes) per lane and load, written to LDS as they are; a lane keeps its column and
//           walks down the rows, so a slot costs a handful of integer instructions.
//   taps  = packed in pairs (t[2j], t[2j+1]) as the tensor's own 16-bit values.
//   item  = BH x 8 outputs (stride 1) or BH x 4 outputs (stride 2) per lane.  A window row is read as dwords; the
//           pairs that start at an odd element are formed with one v_alignbit each, and every output takes
//           ceil(K/2) two-element dot products (v_dot2c_f32_f16 / v_dot2c_f32_bf16: exact products, fp32 sum) per
//           filter row instead of K multiply-adds.  The last tap of a row has no partner: its element is isolated
//           with a mask (a garbage partner times a zero tap would turn an Inf next to the window into a NaN).
// Same results as the fp32-image kernel up to the order of the fp32 additions.
// Replaces, for these tensors, what torch_dwconv/dwconv_kernel.cu:69-181 computes with `scalar_t` = half.
#include "dwconv_tile16_common.hpp"

namespace dwconv {

namespace {

struct Tile16Plan {
    const void *in;
    const void *taps;
    void *out;
    long planes;
    int channel;
    Image16 im;
    int out_h, out_w, out_plane;
    int pad_h, pad_w;
    int rows_per_tile;     // output rows per tile, a multiple of BH
    int row_tiles;         // tiles per plane
    int planes_per_tile;
    int n_tiles;
    int ncb;               // column blocks per row
    unsigned ncb_magic;
    int items_per_plane;
    unsigned ipp_magic;
    int tap_base;          // dword offset of the tap tables in LDS
    int dump;              // slot index of a spare slot
    int lout;              // results leave through LDS as one linear stream per plane (one item per lane)
    Epilogue epi;
};

// PW1: parity of the left padding (the first element of a lane's window is the high half of a dword when odd).
// EPI: the epilogue of the fused forward entry points is compiled in (its temporaries cost 12 registers, a wavefront
// of occupancy, also when it is switched off at run time).
template <typename IO, int K, int S, int PW1, bool FLIP, int BH, bool EPI>
__global__ __launch_bounds__(kThreads) void fir_down16_kernel(const Tile16Plan p)
{
    extern __shared__ float4 lds_raw[];
    uint32_t *lds32 = reinterpret_cast<uint32_t *>(lds_raw);
    constexpr int OWI = S == 1 ? 8 : 4;      // outputs per item and row
    constexpr int KP = (K + 1) / 2;          // tap pairs per filter row
    constexpr int TPP = K * (KP + 1);        // dwords of a plane's tap table: KP pairs and the last tap as (0, t)
    constexpr int WIN_ROWS = (BH - 1) * S + K;
    constexpr int NDW = (PW1 + (OWI - 1) * S + K - 1) / 2 + 1;  // dwords of a window row

    const int tile = xcd_contiguous_tile(blockIdx.x, p.n_tiles);
    const int pg = tile / p.row_tiles, rt = tile - pg * p.row_tiles;
    const long plane0 = static_cast<long>(pg) * p.planes_per_tile;
    const int nplanes = static_cast<int>(min(static_cast<long>(p.planes_per_tile), p.planes - plane0));
    const int oy0 = rt * p.rows_per_tile;
    const int iy0 = oy0 * S - p.pad_h;
    const int c0 = static_cast<int>(plane0 % p.channel);

    // tap tables
    for (int i = threadIdx.x; i < nplanes * TPP; i += blockDim.x) {
        const int pl = i / TPP, t = i - pl * TPP;
        const int ty = t / (KP + 1), j = t - ty * (KP + 1);
        const uint16_t *f = static_cast<const uint16_t *>(p.taps) + ((c0 + pl) % p.channel) * (K * K);
        auto tap = [&](int x) -> uint32_t {
            if (x >= K) return 0u;
            return FLIP ? f[(K - 1 - ty) * K + (K - 1 - x)] : f[ty * K + x];
        };
        lds32[p.tap_base + i] = j < KP ? (tap(2 * j) | (tap(2 * j + 1) << 16)) : (tap(K - 1) << 16);
    }

    stage_image16(p.im, static_cast<const IO *>(p.in) + plane0 * p.im.in_plane, lds32, p.dump, nplanes, iy0);
    __syncthreads();

    const int n_items = nplanes * p.items_per_plane;
    const __amdgpu_buffer_rsrc_t oview =
        buffer_view(static_cast<IO *>(p.out) + plane0 * p.out_plane, static_cast<long>(nplanes) * p.out_plane * sizeof(IO));
    // the BH x OWI sums of one item, after the epilogue
    auto convolve = [&](int pl, int rb, int cb, float(&acc)[BH][OWI]) {
        uint32_t tp[K][KP + 1];
#pragma unroll
        for (int ty = 0; ty < K; ++ty)
#pragma unroll
            for (int j = 0; j <= KP; ++j) tp[ty][j] = lds32[p.tap_base + pl * TPP + ty * (KP + 1) + j];

        // the first filter row's last tap as fp32: its product starts every sum (a plain multiply needs no zeroed
        // accumulator, which the accumulating dot product would)
        const float t0_last = Io<IO>::in(__builtin_bit_cast(IO, static_cast<uint16_t>(tp[0][KP] >> 16)));
        // The lane's window starts at logical dword 4 * cb + PH of image row rb * BH * S (pad_w = K / 2 puts its first
        // element (K/2 + PW1) / 2 dwords left of the lane's block, which starts at dword 4 + 4 * cb); window dword i is
        // LDS dword base[swz(PH + i)].
        constexpr int PH = 4 - (K / 2 + PW1) / 2;
        const uint32_t *base = lds32 + __mul24(pl, p.im.pp) + __mul24(rb * BH * S, p.im.rp) + 5 * cb;
        const int rpitch = p.im.rp;  // dwords per image row
        // (no zero fill: the first product of every sum starts from the constant, see below)
        // window rows are read one ahead of their use, into alternating registers, and the sums pinned after every
        // row (see pin_registers)
        uint32_t win[2][NDW];
#pragma unroll
        for (int i = 0; i < NDW; ++i) win[0][i] = base[swz(PH + i)];
#pragma unroll
        for (int wr = 0; wr < WIN_ROWS; ++wr) {
            const uint32_t(&d)[NDW] = win[wr & 1];
            if (wr + 1 < WIN_ROWS) {
#pragma unroll
                for (int i = 0; i < NDW; ++i) win[(wr + 1) & 1][i] = base[(wr + 1) * rpitch + swz(PH + i)];
            }
            // pairs that start at an odd element
            uint32_t q[NDW];
#pragma unroll
            for (int i = 0; i + 1 < NDW; ++i) q[i] = __builtin_amdgcn_alignbit(d[i + 1], d[i], 16);
            // the element under the last tap of each output: alone in its half for the dot product, and as fp32 for
            // the output row this window row starts
            uint32_t last[OWI];
            float lastf[OWI];
#pragma unroll
            for (int o = 0; o < OWI; ++o) {
                const int e = PW1 + o * S + K - 1;
                last[o] = (e & 1) ? (d[e >> 1] & 0xffff0000u) : (d[e >> 1] & 0x0000ffffu);
                const uint16_t h = static_cast<uint16_t>((e & 1) ? d[e >> 1] >> 16 : d[e >> 1] & 0xffffu);
                lastf[o] = Io<IO>::in(__builtin_bit_cast(IO, h));
            }
#pragma unroll
            for (int b = 0; b < BH; ++b) {
                const int ty = wr - b * S;
                if (ty < 0 || ty >= K) continue;
#pragma unroll
                for (int o = 0; o < OWI; ++o) {
                    const int el = PW1 + o * S + K - 1;
                    if (ty == 0) acc[b][o] = lastf[o] * t0_last;
                    else acc[b][o] = dot2<IO>(last[o], (el & 1) ? tp[ty][KP] : tp[ty][KP - 1], acc[b][o]);
#pragma unroll
                    for (int j = 0; j < K / 2; ++j) {
                        const int e = PW1 + o * S + 2 * j;
                        acc[b][o] = dot2<IO>((e & 1) ? q[e >> 1] : d[e >> 1], tp[ty][j], acc[b][o]);
                    }
                }
            }
#pragma unroll
            for (int b = 0; b < BH; ++b)
                if (b * S <= wr) pin_registers(acc[b]);  // the rows that have been started
        }

        if constexpr (EPI) epilogue_apply_block<1>(acc, p.epi, (c0 + pl) % p.channel);
    };
    // a row of sums as packed 16-bit elements
    auto pack_row = [](const float(&a)[OWI], uint32_t(&t)[OWI / 2]) {
#pragma unroll
        for (int i = 0; i < OWI / 2; ++i) {
            if constexpr (std::is_same<IO, bf16_t>::value) t[i] = bf16_pack2(a[2 * i], a[2 * i + 1]);
            else t[i] = f16_pack2(a[2 * i], a[2 * i + 1]);
        }
    };

    if (p.lout) {
        // One item per lane (the planner guarantees it).  The packed sums go back into LDS in the layout the band has
        // in memory, over the image, and leave as one linear stream per plane: 16 bytes per lane, 1 KiB of
        // consecutive bytes per wavefront and store.  Lane-owned blocks write a row segment at a time; where a row is
        // not a whole number of 128-byte lines (56 elements: 112 bytes) their streaming stores leave partial lines.
        const bool has_item = static_cast<int>(threadIdx.x) < n_items;
        const int item = has_item ? threadIdx.x : 0;
        const int pl = fast_div(item, p.ipp_magic);
        const int rem = item - __mul24(pl, p.items_per_plane);
        const int rb = fast_div(rem, p.ncb_magic);
        const int cb = rem - __mul24(rb, p.ncb);
        const int rows_here = min(p.rows_per_tile, p.out_h - oy0);
        const int run = rows_here * p.out_w;  // elements per plane, a multiple of eight
        // Wavefronts with no item at all skip the arithmetic; lanes without one in the others compute item 0 again.
        // The sums never leave the arm that makes them (merged with the arm that has none, every sum would be zeroed
        // first); what leaves it are the packed rows, and every wavefront meets the one barrier after the branch.
        uint32_t packed[BH][OWI / 2];
#pragma unroll
        for (int b = 0; b < BH; ++b)
#pragma unroll
            for (int i = 0; i < OWI / 2; ++i) packed[b][i] = 0u;
        if (__builtin_amdgcn_readfirstlane(threadIdx.x) < n_items) {
            float acc[BH][OWI];
            convolve(pl, rb, cb, acc);
#pragma unroll
            for (int b = 0; b < BH; ++b) pack_row(acc[b], packed[b]);
        }
        __syncthreads();  // every window has been read: the image can be overwritten
        if (has_item) {
#pragma unroll
            for (int b = 0; b < BH; ++b) {
                if (rb * BH + b < rows_here) {
                    // (one 128- or 64-bit write per lane at a multiple of its size: conflict-free)
                    uint32_t *d = lds32 + ((__mul24(pl, run) + __mul24(rb * BH + b, p.out_w) + cb * OWI) >> 1);
                    if constexpr (OWI == 8) {
                        u32x4 v;
                        v.x = packed[b][0]; v.y = packed[b][1]; v.z = packed[b][2]; v.w = packed[b][3];
                        *reinterpret_cast<u32x4 *>(d) = v;
                    } else {
                        u32x2 v;
                        v.x = packed[b][0]; v.y = packed[b][1];
                        *reinterpret_cast<u32x2 *>(d) = v;
                    }
                }
            }
        }
        __syncthreads();
        const u32x4 *image = reinterpret_cast<const u32x4 *>(lds_raw);
        const int run8 = run >> 3;
        for (int q = 0; q < nplanes; ++q) {
            const unsigned o0 = (__mul24(q, p.out_plane) + __mul24(oy0, p.out_w)) * 2u;
            for (int i = threadIdx.x; i < run8; i += blockDim.x)
                __builtin_amdgcn_raw_buffer_store_b128(image[q * run8 + i], oview, o0 + i * 16u, 0, kStoreStreaming);
        }
        return;
    }

    for (int item = threadIdx.x; item < n_items; item += blockDim.x) {
        const int pl = fast_div(item, p.ipp_magic);
        const int rem = item - __mul24(pl, p.items_per_plane);
        const int rb = fast_div(rem, p.ncb_magic);
        const int cb = rem - __mul24(rb, p.ncb);
        float acc[BH][OWI];
        convolve(pl, rb, cb, acc);
        // branch-free: rows past the end of the plane store out of range
        const unsigned o0 = (__mul24(pl, p.out_plane) + cb * OWI) * 2u;
#pragma unroll
        for (int b = 0; b < BH; ++b) {
            const int oy = oy0 + rb * BH + b;
            const unsigned off = oy < p.out_h ? o0 + __mul24(oy, p.out_w) * 2u : kOob;
            uint32_t t[OWI / 2];
            pack_row(acc[b], t);
            if constexpr (OWI == 8) {
                u32x4 v;
                v.x = t[0]; v.y = t[1]; v.z = t[2]; v.w = t[3];
                __builtin_amdgcn_raw_buffer_store_b128(v, oview, off, 0, kStoreStreaming);
            } else {
                u32x2 v;
                v.x = t[0]; v.y = t[1];
                __builtin_amdgcn_raw_buffer_store_b64(v, oview, off, 0, kStoreStreaming);
            }
        }
    }
}

template <typename IO, int K, int S, int PW1, bool FLIP, int BH>
int launch_down16(Tile16Plan &p, hipStream_t stream)
{
    constexpr int OWI = S == 1 ? 8 : 4;
    constexpr int KP = (K + 1) / 2;
    constexpr int TPP = K * (KP + 1);
    const int threads = kThreads;
    const int target_items = env_int("DWCONV_TILE16_ITEMS", threads);
    const int budget = env_int("DWCONV_TILE16_LDS", S == 2 ? 32 * 1024 : 24 * 1024);

    p.ncb = p.out_w / OWI;
    // elements of a row the windows touch: up to input column (out_w - 1) * S - pad_w + K - 1, and its pair partner
    const int last_col = (p.out_w - 1) * S - p.pad_w + K;
    layout_image16(p.im, last_col);
    auto rows_for = [](int units) { return (units * BH - 1) * S + K; };
    auto bytes = [&](int units, int planes) {
        return static_cast<long>(planes) * (static_cast<long>(rows_for(units)) * p.im.rp * 4 + TPP * 4) + 20;
    };

    const int row_units = ceil_div(p.out_h, BH);
    const int ipp_full = row_units * p.ncb;
    int units_per_tile = 0, planes_per_tile = 0;
    if (2 * ipp_full <= target_items) {
        units_per_tile = row_units;
        planes_per_tile = target_items / ipp_full;
        while (planes_per_tile > 1 && bytes(units_per_tile, planes_per_tile) > budget) --planes_per_tile;
        if (static_cast<long>(planes_per_tile) > p.planes) planes_per_tile = static_cast<int>(p.planes);
        if (bytes(units_per_tile, planes_per_tile) > budget) planes_per_tile = 0;
    }
    if (planes_per_tile == 0) {
        planes_per_tile = 1;
        units_per_tile = std::max(1, std::min(row_units, target_items / p.ncb));
        while (units_per_tile > 1 && bytes(units_per_tile, 1) > budget) --units_per_tile;
        if (bytes(units_per_tile, 1) > budget) return -1;
        units_per_tile = ceil_div(row_units, ceil_div(row_units, units_per_tile));  // even out the bands
    }
    p.planes_per_tile = planes_per_tile;
    p.rows_per_tile = units_per_tile * BH;
    p.row_tiles = ceil_div(row_units, units_per_tile);
    if (!finish_image16(p.im, rows_for(units_per_tile), planes_per_tile)) return -1;
    p.items_per_plane = units_per_tile * p.ncb;
    if (planes_per_tile * p.items_per_plane >= 65536) return -1;  // 16-bit reciprocals
    if (static_cast<long>(planes_per_tile) * p.out_plane * 2 >= static_cast<long>(kOob)) return -1;
    p.ncb_magic = magic_u16(p.ncb);
    p.ipp_magic = magic_u16(p.items_per_plane);
    p.dump = planes_per_tile * p.im.lds_rows * (p.im.pitch / 8);
    p.tap_base = 5 * (p.dump + 1);
    const long tiles = ceil_div(p.planes, static_cast<long>(planes_per_tile)) * p.row_tiles;
    if (tiles > 0x7fffffffL) return -1;
    p.n_tiles = static_cast<int>(tiles);
    p.lout = env_int("DWCONV_T16_LOUT", 1) && planes_per_tile * p.items_per_plane <= threads &&
             (p.rows_per_tile * p.out_w) % 8 == 0 && p.out_plane % 8 == 0;
    const size_t lds = static_cast<size_t>(p.tap_base) * 4 + static_cast<size_t>(planes_per_tile) * TPP * 4;

    if (!FLIP && p.epi.enabled())
        hipLaunchKernelGGL((fir_down16_kernel<IO, K, S, PW1, FLIP, BH, !FLIP>), dim3(p.n_tiles), dim3(threads), lds, stream, p);
    else
        hipLaunchKernelGGL((fir_down16_kernel<IO, K, S, PW1, FLIP, BH, false>), dim3(p.n_tiles), dim3(threads), lds, stream, p);
    note_variant("tile_down16_dot2<k%d,s%d,%s,bh%d> P%d rows%d%s", K, S, FLIP ? "rot" : "fwd", BH, p.planes_per_tile, p.rows_per_tile,
                 p.lout ? " ldsout" : "");
    return check_launch("fir_down16_kernel");
}

template <typename IO, int K, int S, bool FLIP>
int launch_down16_parity(Tile16Plan &p, hipStream_t stream)
{
    const int forced = env_int("DWCONV_TILE_BH", 0);
    const bool seven = forced ? forced == 7 : (p.out_h % 7 == 0 || p.out_h > 64) && p.out_h % 4 != 0;
    constexpr int PW1 = (K / 2) & 1;  // the left padding is K / 2
    return seven ? launch_down16<IO, K, S, PW1, FLIP, 7>(p, stream) : launch_down16<IO, K, S, PW1, FLIP, 4>(p, stream);
}

}  // namespace

// -1 when the kernel does not cover g (the caller goes on to the fp32-image kernel).
template <typename IO>
int try_launch_fir_tiled16(const IO *in, const IO *taps, IO *out, const Geometry &g, hipStream_t stream)
{
    static_assert(sizeof(IO) == 2, "16-bit element types");
    if (!env_int("DWCONV_TILE16", 1)) return -1;
    const int K = g.kernel_h, S = g.down_h;
    if (g.kernel_w != K || (K != 3 && K != 5 && K != 7)) return -1;
    if (g.up_h != 1 || g.up_w != 1 || g.down_w != S || (S != 1 && S != 2)) return -1;
    if (S == 2 && !g.forward) return -1;
    // (the window's place within its LDS slots is a compile-time constant: left padding K/2 only)
    if (g.pad_h0 < 0 || g.pad_h0 > 7 || g.pad_w0 != K / 2) return -1;
    if (g.in_w % 8 != 0 || g.out_w % (S == 1 ? 8 : 4) != 0 || g.in_h < 1) return -1;
    // Input rows of at least 48 elements at stride 2 and 72 at stride 1: measured against the fp32-image and stacked
    // kernels on 48 ... 88 wide maps (batch 64, C = 144, bf16 and fp16), stride 2 is 3-29 % faster here at every
    // width, stride 1 6-19 % from 72 on (88 x 88 5x5: equal) and mixed below (56 x 56 3x3 and 7x7: 8-12 % slower;
    // narrower planes have too few 8-wide blocks to occupy the lanes).
    if (g.in_w < env_int("DWCONV_T16_MIN_W", S == 2 ? 48 : 72)) return -1;
    if (reinterpret_cast<uintptr_t>(in) % 16 != 0 || reinterpret_cast<uintptr_t>(out) % 16 != 0) return -1;
    if (static_cast<long>(g.in_h) * g.in_w >= (1l << 30) || static_cast<long>(g.out_h) * g.out_w >= (1l << 30)) return -1;

    Tile16Plan p{};
    p.in = in;
    p.taps = taps;
    p.out = out;
    p.planes = g.planes();
    p.channel = g.channel;
    p.epi = g.epi;
    p.im.in_h = g.in_h;
    p.im.in_w = g.in_w;
    p.im.in_plane = g.in_h * g.in_w;
    p.out_h = g.out_h;
    p.out_w = g.out_w;
    p.out_plane = g.out_h * g.out_w;
    p.pad_h = g.pad_h0;
    p.pad_w = g.pad_w0;
    const bool rot = !g.forward;
    if (S == 1) {
        if (K == 3) return rot ? launch_down16_parity<IO, 3, 1, true>(p, stream) : launch_down16_parity<IO, 3, 1, false>(p, stream);
        if (K == 5) return rot ? launch_down16_parity<IO, 5, 1, true>(p, stream) : launch_down16_parity<IO, 5, 1, false>(p, stream);
        return rot ? launch_down16_parity<IO, 7, 1, true>(p, stream) : launch_down16_parity<IO, 7, 1, false>(p, stream);
    }
    if (K == 3) return launch_down16_parity<IO, 3, 2, false>(p, stream);
    if (K == 5) return launch_down16_parity<IO, 5, 2, false>(p, stream);
    return launch_down16_parity<IO, 7, 2, false>(p, stream);
}

template int try_launch_fir_tiled16<half_t>(const half_t *, const half_t *, half_t *, const Geometry &, hipStream_t);
template int try_launch_fir_tiled16<bf16_t>(const bf16_t *, const bf16_t *, bf16_t *, const Geometry &, hipStream_t);

}  // namespace dwconv
