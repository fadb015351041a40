// LDS-tiled kernels for double tensors: the raw operator (forward, and grad-input as the transposed problem with
// up-sampling) and grad-weight, for any filter extent, up/down factors and pads.
//
// The reference instantiates its tiled kernels for double as for float (torch_dwconv/dwconv_kernel.cu:749, :860, :960,
// :999 `AT_DISPATCH_FLOATING_TYPES_AND_HALF`).  Here fp64 is what gradcheck and reference computations use, so one
// kernel pair with everything taken at run time, rather than the instance families of the 32- and 16-bit types:
//   * a workgroup stages a band of input rows (several whole planes where they are small) into LDS as doubles, in
//     input coordinates, with the zero padding materialised, so that the tap loop carries no bounds checks;
//   * a lane owns one output column and four output rows; consecutive lanes read consecutive doubles from LDS and
//     store consecutive doubles, 512 bytes per wavefront and row;
//   * up-sampling (grad-input of strided layers) keeps the image in input coordinates, and a lane walks only the taps
//     that meet a real input: every up-th row and column from a first one that depends on the output's position;
//   * grad-weight keeps 32 sums per lane in registers, cuts larger filters into passes of 32 taps, and leaves
//     partial sums per (channel, chunk of images) that a second kernel adds front to back: no atomics, and the same
//     bits on every run.
// With 8-byte elements these are bound by HBM for the 3x3 and 5x5 filters and by the LDS read per multiply-add above.
//
// The operator kernel is a template over the element type and is instantiated for float, fp16 and bf16 as well (LDS
// image and sums in fp32): there it is the last LDS-tiled stop before the one-lane-per-element kernel, for what the
// kernels of those types leave out: up-sampling with filters other than 3x3 / 5x5 / 7x7 (grad-input of strip,
// even-sized and large filters above stride 1), up and down together, pads that crop.
#include <algorithm>
#include <cstdlib>

#include "dwconv_common.hpp"

namespace dwconv {

namespace {

constexpr int kThreads = 256;
constexpr int kRows = 4;            // output rows per lane
constexpr int kLdsBytes = 40 * 1024;
constexpr int kSums = 32;           // grad-weight sums per lane and pass

__host__ __device__ inline int floor_div(int a, int b) { return a >= 0 ? a / b : -((-a + b - 1) / b); }

template <typename T>
struct FirPlan {
    const T *in;
    const T *taps;
    T *out;
    long planes;
    int channel;
    int in_h, in_w, out_h, out_w;
    int kh, kw, up_h, up_w, down_h, down_w;
    int dil_h, dil_w;  // dilation of the taps (up = 1 only)
    int flip;
    Epilogue epi;
    int planes_per_tile, rows_per_tile, row_tiles;
    int lds_rows, pitch;   // LDS image of one plane: lds_rows x pitch doubles
    int ix_first;          // input column of LDS column 0 (may be negative: zero padding)
    int first_h, first_w;  // up-sampled coordinate of tap 0 of output 0 (-pad0)
    int items_per_plane;   // (rows_per_tile / kRows) * out_w
    int n_tiles;
};

// Stages rows [iy_first, iy_first + lds_rows) x columns [ix_first, ix_first + pitch) of `planes` planes from `src`
// (`plane_stride` elements apart) into lds, zero outside the planes.
template <typename T>
__device__ inline void stage_f64(typename Io<T>::acc_t *lds, const T *src, int planes, long plane_stride, int in_h, int in_w,
                                 int iy_first, int ix_first, int lds_rows, int pitch)
{
    const int per_plane = lds_rows * pitch;
    const int total = planes * per_plane;
    for (int idx = threadIdx.x; idx < total; idx += blockDim.x) {
        const int pl = idx / per_plane;
        const int rem = idx - pl * per_plane;
        const int r = rem / pitch;
        const int col = rem - r * pitch;
        const int iy = iy_first + r, ix = ix_first + col;
        typename Io<T>::acc_t v = 0;
        if (iy >= 0 && iy < in_h && ix >= 0 && ix < in_w)
            v = Io<T>::in(src[pl * plane_stride + static_cast<long>(iy) * in_w + ix]);
        lds[idx] = v;
    }
}

// UP: the up-sampling factor of both axes when it is 1 or 2, 0 = taken from the plan (any, per axis).
template <typename T, int UP>
__global__ __launch_bounds__(kThreads) void fir_f64_kernel(const FirPlan<T> p)
{
    using A = typename Io<T>::acc_t;
    extern __shared__ double lds_raw_f64[];
    A *const lds_f64 = reinterpret_cast<A *>(lds_raw_f64);
    const int KK = p.kh * p.kw;
    const int up_h = UP ? UP : p.up_h, up_w = UP ? UP : p.up_w;
    const int pg = blockIdx.x / p.row_tiles, rt = blockIdx.x - pg * p.row_tiles;
    const long plane0 = static_cast<long>(pg) * p.planes_per_tile;
    const int nplanes = static_cast<int>(min(static_cast<long>(p.planes_per_tile), p.planes - plane0));
    const int oy0 = rt * p.rows_per_tile;

    // up-sampled row of tap 0 of this band's first output row, and the input row the image starts at
    const int u0 = oy0 * p.down_h + p.first_h;
    const int iy_first = floor_div(u0, up_h);
    const int e_h = u0 - iy_first * up_h;               // 0 <= e_h < up_h
    const int e_w = p.first_w - p.ix_first * up_w;      // 0 <= e_w < up_w

    A *ltaps = lds_f64 + p.planes_per_tile * p.lds_rows * p.pitch;
    for (int i = threadIdx.x; i < nplanes * KK; i += blockDim.x) {
        const int pl = i / KK, t = i - pl * KK;
        const int c = static_cast<int>((plane0 + pl) % p.channel);
        ltaps[i] = Io<T>::in(p.taps[static_cast<long>(c) * KK + (p.flip ? KK - 1 - t : t)]);
    }
    const long in_plane = static_cast<long>(p.in_h) * p.in_w;
    stage_f64(lds_f64, p.in + plane0 * in_plane, nplanes, in_plane, p.in_h, p.in_w, iy_first, p.ix_first, p.lds_rows, p.pitch);
    __syncthreads();

    const int n_items = nplanes * p.items_per_plane;
    for (int item = threadIdx.x; item < n_items; item += blockDim.x) {
        const int pl = item / p.items_per_plane;
        const int rem = item - pl * p.items_per_plane;
        const int rb = rem / p.out_w;
        const int ox = rem - rb * p.out_w;
        const A *img = lds_f64 + pl * p.lds_rows * p.pitch;
        const A *tp = ltaps + pl * KK;
        // offsets, in up-sampled steps, of tap (0, 0) of this lane's first output from the image's origin
        const int dy0 = e_h + rb * kRows * p.down_h;
        const int dx0 = e_w + ox * p.down_w;
        A acc[kRows];
#pragma unroll
        for (int b = 0; b < kRows; ++b) acc[b] = 0;
        if constexpr (UP == 1) {
            for (int ty = 0; ty < p.kh; ++ty) {
                int row[kRows];
#pragma unroll
                for (int b = 0; b < kRows; ++b) row[b] = (dy0 + b * p.down_h + ty * p.dil_h) * p.pitch;
                for (int tx = 0; tx < p.kw; ++tx) {
                    const A t = tp[ty * p.kw + tx];
                    const int col = dx0 + tx * p.dil_w;
#pragma unroll
                    for (int b = 0; b < kRows; ++b) acc[b] = fma(img[row[b] + col], t, acc[b]);
                }
            }
        } else {
            // Up-sampling: of the taps of an output only every up-th row and column meets a real input, the others
            // a stuffed zero.  The lane walks the ones that count: from the first tap row and column whose
            // up-sampled coordinate is a multiple of up, in steps of up, which are steps of one in the image.
            const int tx0 = (up_w - dx0 % up_w) % up_w;
            const int col0 = (dx0 + tx0) / up_w;
#pragma unroll
            for (int b = 0; b < kRows; ++b) {
                const int dyb = dy0 + b * p.down_h;
                const int ty0 = (up_h - dyb % up_h) % up_h;
                const A *r = img + ((dyb + ty0) / up_h) * p.pitch + col0;
                for (int ty = ty0; ty < p.kh; ty += up_h, r += p.pitch) {
                    const A *t = tp + ty * p.kw;
                    int col = 0;
                    for (int tx = tx0; tx < p.kw; tx += up_w, ++col) acc[b] = fma(r[col], t[tx], acc[b]);
                }
            }
        }
        const int c = static_cast<int>((plane0 + pl) % p.channel);
        T *dst = p.out + (plane0 + pl) * p.out_h * p.out_w + ox;
#pragma unroll
        for (int b = 0; b < kRows; ++b) {
            const int oy = oy0 + rb * kRows + b;
            if (oy < p.out_h) {
                A v = acc[b];
                if (!p.flip && p.epi.enabled()) v = epilogue_apply(v, p.epi, c);
                dst[static_cast<long>(oy) * p.out_w] = Io<T>::out(v);
            }
        }
    }
}

struct WgradPlan64 {
    const double *x;
    const double *gy;
    double *partial;
    int batch, channel;
    int in_h, in_w, out_h, out_w;
    int kh, kw, down_h, down_w, pad_h, pad_w, dil_h, dil_w;
    int rows_per_tile, row_tiles;
    int lds_rows, pitch;
    int items;  // (rows_per_tile / kRows) * out_w
    int images_per_tile;  // images of the channel staged side by side (small planes)
    int chunks, images_per_chunk;
};

// Sum over the 64 lanes of a wavefront in a fixed butterfly order.
__device__ inline double wave_sum_f64(double v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Workgroup (c, chunk, pass): taps [pass * kSums, +kSums) of channel c summed over the images of the chunk.
// (The sum of torch_dwconv/dwconv_kernel.cu:269-297.)
__global__ __launch_bounds__(kThreads) void wgrad_f64_kernel(const WgradPlan64 p)
{
    extern __shared__ double lds_f64[];
    __shared__ double wave_part[kThreads / 64][kSums];
    const int KK = p.kh * p.kw;
    const int c = blockIdx.x, chunk = blockIdx.y;
    const int t_first = blockIdx.z * kSums;
    const int nt = min(kSums, KK - t_first);
    const int ty_first = t_first / p.kw, tx_first = t_first - ty_first * p.kw;
    const int n0 = chunk * p.images_per_chunk, n1 = min(p.batch, n0 + p.images_per_chunk);

    double acc[kSums];
#pragma unroll
    for (int t = 0; t < kSums; ++t) acc[t] = 0.0;

    const long in_plane = static_cast<long>(p.in_h) * p.in_w;
    for (int n = n0; n < n1; n += p.images_per_tile) {
        const int images = min(p.images_per_tile, n1 - n);
        const long plane0 = static_cast<long>(n) * p.channel + c;
        for (int rt = 0; rt < p.row_tiles; ++rt) {
            const int oy0 = rt * p.rows_per_tile;
            __syncthreads();  // the previous band's reads are done
            stage_f64<double>(lds_f64, p.x + plane0 * in_plane, images, p.channel * in_plane, p.in_h, p.in_w, oy0 * p.down_h - p.pad_h,
                      -p.pad_w, p.lds_rows, p.pitch);
            __syncthreads();
            for (int item = threadIdx.x; item < images * p.items; item += blockDim.x) {
                const int im = item / p.items;
                const int rem = item - im * p.items;
                const int rb = rem / p.out_w;
                const int ox = rem - rb * p.out_w;
                const long plane = plane0 + static_cast<long>(im) * p.channel;
                double g[kRows];
#pragma unroll
                for (int b = 0; b < kRows; ++b) {
                    const int oy = oy0 + rb * kRows + b;
                    g[b] = oy < p.out_h ? p.gy[(plane * p.out_h + oy) * p.out_w + ox] : 0.0;
                }
                const double *base = lds_f64 + (im * p.lds_rows + rb * kRows * p.down_h) * p.pitch + ox * p.down_w;
                const int row_step = p.down_h * p.pitch;
                int ty = ty_first, tx = tx_first;
#pragma unroll
                for (int t = 0; t < kSums; ++t) {
                    if (t < nt) {  // (uniform)
                        const double *r = base + ty * p.dil_h * p.pitch + tx * p.dil_w;
                        double sum = acc[t];
#pragma unroll
                        for (int b = 0; b < kRows; ++b) sum = fma(g[b], r[b * row_step], sum);
                        acc[t] = sum;
                        if (++tx == p.kw) {
                            tx = 0;
                            ++ty;
                        }
                    }
                }
            }
        }
    }

#pragma unroll
    for (int t = 0; t < kSums; ++t) {
        if (t < nt) {
            const double sum = wave_sum_f64(acc[t]);
            if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6][t] = sum;
        }
    }
    __syncthreads();
    if (static_cast<int>(threadIdx.x) < nt) {
        double sum = wave_part[0][threadIdx.x];
#pragma unroll
        for (int w = 1; w < kThreads / 64; ++w) sum += wave_part[w][threadIdx.x];
        p.partial[(static_cast<long>(c) * p.chunks + chunk) * KK + t_first + threadIdx.x] = sum;
    }
}

// Pass 2: one lane per (c, tap) adds the chunk partials front to back.
__global__ void wgrad_f64_final_kernel(const double *__restrict__ partial, double *__restrict__ gw, const int channel_taps,
                                       const int taps, const int chunks)
{
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= channel_taps) return;
    const int c = e / taps, tap = e - c * taps;
    const double *p = partial + static_cast<long>(c) * chunks * taps + tap;
    double s = 0.0;
    for (int k = 0; k < chunks; ++k) s += p[static_cast<long>(k) * taps];
    gw[e] = s;
}

int f64_chunks(const WgradGeometry &g)
{
    // enough workgroups to cover the 256 CUs a few times over
    int want = ceil_div(2048, g.channel);
    want = std::max(1, std::min(want, g.batch));
    const int per = ceil_div(g.batch, want);
    return ceil_div(g.batch, per);
}

bool make_wgrad_plan(WgradPlan64 &p, const WgradGeometry &g, int dil_h, int dil_w)
{
    if (g.mult != 1 || g.dil != 1 || dil_h < 1 || dil_w < 1) return false;
    const long span_h = static_cast<long>(g.kernel_h - 1) * dil_h, span_w = static_cast<long>(g.kernel_w - 1) * dil_w;
    if (span_h > 4096 || span_w > 4096) return false;
    if (g.kernel_h < 1 || g.kernel_w < 1 || g.down_h < 1 || g.down_w < 1 || g.pad_h < 0 || g.pad_w < 0) return false;
    if (g.batch < 1 || g.channel < 1 || g.in_h < 1 || g.in_w < 1 || g.out_h < 1 || g.out_w < 1) return false;
    if (g.channel > 65535 * 32 || static_cast<long>(g.kernel_h) * g.kernel_w > 4096) return false;
    if (g.down_h > 64 || g.down_w > 64 || g.pad_h > 4096 || g.pad_w > 4096 || g.kernel_h > 4096 || g.kernel_w > 4096) return false;
    if (g.out_w > (1 << 20) || g.out_h > (1 << 20) || g.in_w > (1 << 20) || g.in_h > (1 << 20)) return false;
    p.batch = g.batch;
    p.channel = g.channel;
    p.in_h = g.in_h;
    p.in_w = g.in_w;
    p.out_h = g.out_h;
    p.out_w = g.out_w;
    p.kh = g.kernel_h;
    p.kw = g.kernel_w;
    p.down_h = g.down_h;
    p.down_w = g.down_w;
    p.pad_h = g.pad_h;
    p.pad_w = g.pad_w;
    p.dil_h = dil_h;
    p.dil_w = dil_w;
    const long pitch = static_cast<long>(g.out_w - 1) * g.down_w + span_w + 1;
    auto rows_for = [&](long units) { return (units * kRows - 1) * g.down_h + span_h + 1; };
    const int row_units = ceil_div(g.out_h, kRows);
    long units = std::max(1, std::min(row_units, ceil_div(2 * kThreads, g.out_w)));
    while (units > 1 && rows_for(units) * pitch * 8 > kLdsBytes) --units;
    if (rows_for(units) * pitch * 8 > kLdsBytes) return false;
    units = ceil_div(row_units, ceil_div(row_units, static_cast<int>(units)));  // even out the bands
    p.rows_per_tile = static_cast<int>(units) * kRows;
    p.row_tiles = ceil_div(row_units, static_cast<int>(units));
    p.lds_rows = static_cast<int>(rows_for(units));
    p.pitch = static_cast<int>(pitch);
    p.items = static_cast<int>(units) * g.out_w;
    p.chunks = f64_chunks(g);
    p.images_per_chunk = ceil_div(g.batch, p.chunks);
    // small planes: several images of the channel in LDS at once, so that the lanes have an item each
    p.images_per_tile = 1;
    if (p.row_tiles == 1 && 2 * p.items <= kThreads) {
        long images = std::min(kThreads / p.items, p.images_per_chunk);
        while (images > 1 && images * p.lds_rows * pitch * 8 > kLdsBytes) --images;
        p.images_per_tile = static_cast<int>(images);
    }
    if (p.chunks > 65535) return false;
    return true;
}

}  // namespace

template <typename T>
int try_launch_fir_lds(const T *in, const T *taps, T *out, const Geometry &g, hipStream_t stream)
{
    constexpr int kElem = sizeof(typename Io<T>::acc_t);
    if (g.mult != 1 || g.dil_h < 1 || g.dil_w < 1) return -1;
    if ((g.dil_h != 1 || g.dil_w != 1) && (g.up_h != 1 || g.up_w != 1)) return -1;  // dilated taps: without up-sampling
    if (g.kernel_h < 1 || g.kernel_w < 1 || g.up_h < 1 || g.up_w < 1 || g.down_h < 1 || g.down_w < 1) return -1;
    if (g.in_h < 1 || g.in_w < 1 || g.out_h < 1 || g.out_w < 1 || g.planes() < 1) return -1;
    if (static_cast<long>(g.kernel_h) * g.kernel_w > 4096 || g.kernel_h > 4096 || g.kernel_w > 4096) return -1;
    if (g.up_h > 64 || g.up_w > 64 || g.down_h > 64 || g.down_w > 64) return -1;
    const long span_h = static_cast<long>(g.kernel_h - 1) * g.dil_h, span_w = static_cast<long>(g.kernel_w - 1) * g.dil_w;
    if (span_h > 4096 || span_w > 4096) return -1;
    if (std::abs(g.pad_h0) > 4096 || std::abs(g.pad_w0) > 4096) return -1;
    if (g.out_w > (1 << 20) || g.out_h > (1 << 20) || g.in_w > (1 << 20) || g.in_h > (1 << 20)) return -1;

    FirPlan<T> p{};
    p.in = in;
    p.taps = taps;
    p.out = out;
    p.planes = g.planes();
    p.channel = g.channel;
    p.in_h = g.in_h;
    p.in_w = g.in_w;
    p.out_h = g.out_h;
    p.out_w = g.out_w;
    p.kh = g.kernel_h;
    p.kw = g.kernel_w;
    p.up_h = g.up_h;
    p.up_w = g.up_w;
    p.down_h = g.down_h;
    p.down_w = g.down_w;
    p.dil_h = g.dil_h;
    p.dil_w = g.dil_w;
    p.flip = !g.forward;
    p.epi = g.epi;
    p.first_h = -g.pad_h0;
    p.first_w = -g.pad_w0;
    // columns: up-sampled coordinates -pad_w0 .. (out_w - 1) * down_w - pad_w0 + kw - 1
    p.ix_first = floor_div(-g.pad_w0, g.up_w);
    const long u_last_w = static_cast<long>(g.out_w - 1) * g.down_w - g.pad_w0 + span_w;
    const long pitch = floor_div(static_cast<int>(u_last_w), g.up_w) - p.ix_first + 1;
    // rows of a band of `units` * kRows output rows: the worst case over the band's alignment to the up-sampling grid
    auto rows_for = [&](long units) { return ((units * kRows - 1) * g.down_h + span_h + g.up_h - 1) / g.up_h + 1; };
    const long KK = static_cast<long>(g.kernel_h) * g.kernel_w;
    auto bytes = [&](long units, long planes) { return planes * (rows_for(units) * pitch + KK) * kElem; };
    const int row_units = ceil_div(g.out_h, kRows);
    const long ipp_full = static_cast<long>(row_units) * g.out_w;
    long units, planes_per_tile;
    if (2 * ipp_full <= kThreads) {
        // whole planes, several per tile
        units = row_units;
        planes_per_tile = std::min<long>(kThreads / ipp_full, g.planes());
        while (planes_per_tile > 1 && bytes(units, planes_per_tile) > kLdsBytes) --planes_per_tile;
        if (bytes(units, planes_per_tile) > kLdsBytes) return -1;
    } else {
        planes_per_tile = 1;
        units = std::max(1, std::min(row_units, ceil_div(2 * kThreads, g.out_w)));
        while (units > 1 && bytes(units, 1) > kLdsBytes) --units;
        if (bytes(units, 1) > kLdsBytes) return -1;
        units = ceil_div(row_units, ceil_div(row_units, static_cast<int>(units)));  // even out the bands
    }
    p.planes_per_tile = static_cast<int>(planes_per_tile);
    p.rows_per_tile = static_cast<int>(units) * kRows;
    p.row_tiles = ceil_div(row_units, static_cast<int>(units));
    p.lds_rows = static_cast<int>(rows_for(units));
    p.pitch = static_cast<int>(pitch);
    p.items_per_plane = static_cast<int>(units) * g.out_w;
    const long tiles = (g.planes() + planes_per_tile - 1) / planes_per_tile * p.row_tiles;
    if (tiles > 0x7fffffffL) return -1;
    p.n_tiles = static_cast<int>(tiles);
    const size_t shmem = static_cast<size_t>(bytes(units, planes_per_tile));
    const dim3 grid(static_cast<unsigned>(p.n_tiles)), block(kThreads);
    if (g.up_h == 1 && g.up_w == 1) hipLaunchKernelGGL((fir_f64_kernel<T, 1>), grid, block, shmem, stream, p);
    else if (g.up_h == 2 && g.up_w == 2) hipLaunchKernelGGL((fir_f64_kernel<T, 2>), grid, block, shmem, stream, p);
    else hipLaunchKernelGGL((fir_f64_kernel<T, 0>), grid, block, shmem, stream, p);
    char dil[24] = "";
    if (p.dil_h != 1 || p.dil_w != 1) std::snprintf(dil, sizeof(dil), " d%dx%d", p.dil_h, p.dil_w);
    note_variant("tile_%s<k%dx%d,u%dx%d,s%dx%d,%s> P%d rows%d%s", sizeof(T) == 8 ? "f64" : (sizeof(T) == 4 ? "gen" : "gen16"), p.kh, p.kw, p.up_h,
                 p.up_w, p.down_h, p.down_w, p.flip ? "rot" : "fwd", p.planes_per_tile, p.rows_per_tile, dil);
    return check_launch("fir_f64_kernel");
}

template int try_launch_fir_lds<double>(const double *, const double *, double *, const Geometry &, hipStream_t);
template int try_launch_fir_lds<float>(const float *, const float *, float *, const Geometry &, hipStream_t);
template int try_launch_fir_lds<half_t>(const half_t *, const half_t *, half_t *, const Geometry &, hipStream_t);
template int try_launch_fir_lds<bf16_t>(const bf16_t *, const bf16_t *, bf16_t *, const Geometry &, hipStream_t);

size_t wgrad_f64_workspace(const WgradGeometry &g, int dil_h, int dil_w)
{
    WgradPlan64 p{};
    if (!make_wgrad_plan(p, g, dil_h, dil_w)) return 0;
    return static_cast<size_t>(g.channel) * p.chunks * g.kernel_h * g.kernel_w * sizeof(double);
}

int try_launch_wgrad_f64(const double *in, const double *gy, double *gw, void *ws, size_t ws_bytes, const WgradGeometry &g,
                         hipStream_t stream, int dil_h, int dil_w)
{
    WgradPlan64 p{};
    if (!make_wgrad_plan(p, g, dil_h, dil_w)) return -1;
    const int KK = g.kernel_h * g.kernel_w;
    const size_t need = static_cast<size_t>(g.channel) * p.chunks * KK * sizeof(double);
    if (ws == nullptr || ws_bytes < need)
        return fail(DWCONV_ERR_WORKSPACE, "grad-weight needs a workspace of %zu bytes, got %zu", need, ws_bytes);
    p.x = in;
    p.gy = gy;
    p.partial = static_cast<double *>(ws);
    const int passes = ceil_div(KK, kSums);
    if (passes > 65535 || g.channel > 0x7fffffff / KK) return -1;
    const size_t shmem = static_cast<size_t>(p.images_per_tile) * p.lds_rows * p.pitch * 8;
    hipLaunchKernelGGL(wgrad_f64_kernel, dim3(static_cast<unsigned>(g.channel), static_cast<unsigned>(p.chunks), static_cast<unsigned>(passes)),
                       dim3(kThreads), shmem, stream, p);
    int rc = check_launch("wgrad_f64_kernel");
    if (rc != DWCONV_OK) return rc;
    const int total = g.channel * KK;
    hipLaunchKernelGGL(wgrad_f64_final_kernel, dim3(ceil_div(total, 256)), dim3(256), 0, stream, p.partial, gw, total, KK, p.chunks);
    char dil[24] = "";
    if (dil_h != 1 || dil_w != 1) std::snprintf(dil, sizeof(dil), " d%dx%d", dil_h, dil_w);
    note_variant("wgrad_f64<k%dx%d,s%dx%d> P%d rows%d chunks%d passes%d%s", p.kh, p.kw, p.down_h, p.down_w, p.images_per_tile,
                 p.rows_per_tile, p.chunks, passes, dil);
    return check_launch("wgrad_f64_final_kernel");
}

}  // namespace dwconv
