// Whole-plane kernels for small feature maps (width 7, 14 or 28, "same" padding); element type fp32, fp16 or
// bf16, LDS and arithmetic fp32.
//
// Planes of a small map are tiny (196 B to 3 KiB) and sit back to back in memory,
// so the only way to move them at HBM speed is to treat a run of P planes as one
// flat stream: 128-bit loads of the run into LDS (same layout as in memory, no
// index arithmetic), arithmetic out of LDS, results back into LDS in their
// memory layout, 128-bit stores of the run.  One wavefront (a 64-lane workgroup,
// so no cross-wave barrier exists) owns a run; a CU holds about ten such
// wavefronts, each with several loads in flight.
//
// A lane owns BH full-width output rows of one plane.  Because it holds whole
// rows, which taps fall off the left/right edge is known at compile time (they
// are simply not emitted); rows above/below the plane are replaced by zeros
// with a select.  The reference's counterpart (torch_dwconv/dwconv_kernel.cu:308-442,
// :444-588) keeps a zero-filled padded tile in shared memory and re-reads every
// tap for every output.
//
//   small_down_kernel : up = 1, decimation S; forward, and grad-input of stride-1 layers (FLIP)
//   small_up2_kernel  : up = 2, taps rotated; grad-input of stride-2 layers
// (grad-weight and the fused backward of these maps: dwconv_small_bwd.hip)
#include "dwconv_small_common.hpp"

namespace dwconv {

namespace {

struct SmallPlan {
    const void *in;    // element type IO of the kernel template
    const void *taps;
    void *out;
    long planes;
    int channel;
    int in_h, out_h;
    int pad_h;             // leading zero rows (down) or m = (pad0 + E) / 2 (up2)
    int planes_per_run;    // P
    int lanes_per_plane;   // LPP
    unsigned lpp_magic;
    Epilogue epi;          // forward kernels: applied to every sum before it is stored
};

// out[oy,ox] = sum_{ty,tx} in[oy*S - pad_h + ty, ox*S - K/2 + tx] * f[ty,tx], planes W wide.
template <typename IO, int W, int K, int S, bool FLIP, int BH>
__global__ __launch_bounds__(kWave) void small_down_kernel(const SmallPlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int OW = (W - 1) / S + 1;
    constexpr int PW = K / 2;
    constexpr int WIN_ROWS = (BH - 1) * S + K;

    const long plane0 = static_cast<long>(blockIdx.x) * p.planes_per_run;
    const int nplanes = static_cast<int>(min(static_cast<long>(p.planes_per_run), p.planes - plane0));
    const int in_plane = p.in_h * W, out_plane = p.out_h * OW;

    const int pl_raw = fast_div(threadIdx.x, p.lpp_magic);
    const int rb = threadIdx.x - pl_raw * p.lanes_per_plane;
    const bool active = pl_raw < nplanes;
    const int pl = active ? pl_raw : 0;

    float tapv[K * K];
    load_taps<K * K, FLIP>(static_cast<const IO *>(p.taps), static_cast<int>((plane0 + pl) % p.channel), tapv);
    run_to_lds(static_cast<const IO *>(p.in) + plane0 * in_plane, lds, nplanes * in_plane);
    __syncthreads();

    float acc[BH][OW];
#pragma unroll
    for (int b = 0; b < BH; ++b)
#pragma unroll
        for (int o = 0; o < OW; ++o) acc[b][o] = 0.f;

    const int oy0 = rb * BH;
    const float *plane = lds + pl * in_plane;
    // rows are read one ahead of their use and the sums pinned after every row (see pin_registers)
    float nxt[W];
    bool nxt_ok;
    {
        const int iy = oy0 * S - p.pad_h;
        nxt_ok = static_cast<unsigned>(iy) < static_cast<unsigned>(p.in_h);
        lds_load_row<W>(plane + (nxt_ok ? iy : 0) * W, nxt);
    }
#pragma unroll
    for (int wr = 0; wr < WIN_ROWS; ++wr) {
        float row[W];
#pragma unroll
        for (int i = 0; i < W; ++i) row[i] = nxt_ok ? nxt[i] : 0.f;
        if (wr + 1 < WIN_ROWS) {
            const int iy = oy0 * S - p.pad_h + wr + 1;
            nxt_ok = static_cast<unsigned>(iy) < static_cast<unsigned>(p.in_h);
            lds_load_row<W>(plane + (nxt_ok ? iy : 0) * W, nxt);
        }
#pragma unroll
        for (int b = 0; b < BH; ++b) {
            const int ty = wr - b * S;
            if (ty < 0 || ty >= K) continue;
#pragma unroll
            for (int tx = 0; tx < K; ++tx)
#pragma unroll
                for (int o = 0; o < OW; ++o) {
                    const int ix = o * S - PW + tx;
                    if (ix < 0 || ix >= W) continue;
                    acc[b][o] = fmaf(row[ix], tapv[ty * K + tx], acc[b][o]);
                }
        }
        pin_registers(acc);
    }
    if constexpr (!FLIP) {
        if (p.epi.enabled()) {
            epilogue_apply_block<1>(acc, p.epi, static_cast<int>((plane0 + pl) % p.channel));
        }
    }
    __syncthreads();  // every lane has read its input rows: the run can be overwritten in place

    if (active) {
        float *dst = lds + pl * out_plane;
#pragma unroll
        for (int b = 0; b < BH; ++b)
            if (oy0 + b < p.out_h) lds_store_row<OW>(dst + (oy0 + b) * OW, acc[b]);
    }
    __syncthreads();
    lds_to_run(static_cast<IO *>(p.out) + plane0 * out_plane, lds, nplanes * out_plane);
}

// up = 2, taps rotated, "same" padding of the forward conv (leading pad of the transposed problem = K/2):
//   out[2q + r] = sum_a in[q - m + r + a] * g'[r + 2a],  g'[t] = g[t - E],  E = (K/2) & 1,  m = (K/2 + E) / 2.
// Input planes are W wide, output planes 2W wide; a lane owns output rows 2q, 2q+1.
template <typename IO, int W, int K>
__global__ __launch_bounds__(kWave) void small_up2_kernel(const SmallPlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int OW = 2 * W;
    constexpr int E = (K / 2) & 1;
    constexpr int M = (K / 2 + E) / 2;
    constexpr int KA = (K + E + 1) / 2;
    constexpr int WIN_ROWS = KA + 1;

    const long plane0 = static_cast<long>(blockIdx.x) * p.planes_per_run;
    const int nplanes = static_cast<int>(min(static_cast<long>(p.planes_per_run), p.planes - plane0));
    const int in_plane = p.in_h * W, out_plane = p.out_h * OW;

    const int pl_raw = fast_div(threadIdx.x, p.lpp_magic);
    const int q = threadIdx.x - pl_raw * p.lanes_per_plane;
    const bool active = pl_raw < nplanes;
    const int pl = active ? pl_raw : 0;

    float tapv[K * K];
    load_taps<K * K, true>(static_cast<const IO *>(p.taps), static_cast<int>((plane0 + pl) % p.channel), tapv);
    run_to_lds(static_cast<const IO *>(p.in) + plane0 * in_plane, lds, nplanes * in_plane);
    __syncthreads();

    float acc[2][OW];
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int o = 0; o < OW; ++o) acc[r][o] = 0.f;

    const float *plane = lds + pl * in_plane;
    float nxt[W];
    bool nxt_ok;
    {
        const int iy = q - p.pad_h;
        nxt_ok = static_cast<unsigned>(iy) < static_cast<unsigned>(p.in_h);
        lds_load_row<W>(plane + (nxt_ok ? iy : 0) * W, nxt);
    }
#pragma unroll
    for (int wr = 0; wr < WIN_ROWS; ++wr) {
        float row[W];
#pragma unroll
        for (int i = 0; i < W; ++i) row[i] = nxt_ok ? nxt[i] : 0.f;
        if (wr + 1 < WIN_ROWS) {
            const int iy = q - p.pad_h + wr + 1;
            nxt_ok = static_cast<unsigned>(iy) < static_cast<unsigned>(p.in_h);
            lds_load_row<W>(plane + (nxt_ok ? iy : 0) * W, nxt);
        }
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int a = wr - r;
            if (a < 0 || a >= KA) continue;
            const int fy = r + 2 * a - E;
            if (fy < 0 || fy >= K) continue;
#pragma unroll
            for (int o = 0; o < OW; ++o) {
                const int xq = o / 2, rx = o % 2;
#pragma unroll
                for (int ax = 0; ax < KA; ++ax) {
                    const int fx = rx + 2 * ax - E;
                    const int ix = xq - M + rx + ax;
                    if (fx < 0 || fx >= K || ix < 0 || ix >= W) continue;
                    acc[r][o] = fmaf(row[ix], tapv[fy * K + fx], acc[r][o]);
                }
            }
        }
        pin_registers(acc);
    }
    __syncthreads();

    if (active) {
        float *dst = lds + pl * out_plane;
#pragma unroll
        for (int r = 0; r < 2; ++r)
            if (2 * q + r < p.out_h) lds_store_row<OW>(dst + (2 * q + r) * OW, acc[r]);
    }
    __syncthreads();
    lds_to_run(static_cast<IO *>(p.out) + plane0 * out_plane, lds, nplanes * out_plane);
}

size_t small_lds_bytes(int planes, int in_plane, int out_plane)
{
    return static_cast<size_t>(planes) * (in_plane > out_plane ? in_plane : out_plane) * 4;
}

// Planes per wavefront: as many as there are lane slots, a multiple of 4 when a plane is not a
// multiple of 4 elements (so that every run starts on a 4-element boundary), within the LDS budget.
int planes_per_run(int lanes_per_plane, int in_plane, int out_plane, long planes)
{
    int P = kWave / lanes_per_plane;
    while (P > 0 && small_lds_bytes(P, in_plane, out_plane) > 16 * 1024) --P;
    if (in_plane % 4 != 0 || out_plane % 4 != 0) P -= P % 4;
    if (static_cast<long>(P) > planes && in_plane % 4 == 0 && out_plane % 4 == 0) P = static_cast<int>(planes);
    return P;
}

template <typename IO, int W, int K, int S, bool FLIP, int BH>
int launch_small_down(SmallPlan &p, hipStream_t stream)
{
    constexpr int OW = (W - 1) / S + 1;
    p.lanes_per_plane = ceil_div(p.out_h, BH);
    if (p.lanes_per_plane > kWave) return -1;
    const int in_plane = p.in_h * W, out_plane = p.out_h * OW;
    p.planes_per_run = planes_per_run(p.lanes_per_plane, in_plane, out_plane, p.planes);
    if (p.planes_per_run < 1) return -1;
    p.lpp_magic = magic_u16(p.lanes_per_plane);
    const long runs = (p.planes + p.planes_per_run - 1) / p.planes_per_run;
    if (runs > 0x7fffffffL) return -1;
    const size_t shmem = small_lds_bytes(p.planes_per_run, in_plane, out_plane);
    hipLaunchKernelGGL((small_down_kernel<IO, W, K, S, FLIP, BH>), dim3(static_cast<unsigned>(runs)), dim3(kWave), shmem,
                       stream, p);
    note_variant("small_down%s<w%d,k%d,s%d,%s,bh%d> P%d", sizeof(IO) == 2 ? "16" : "", W, K, S, FLIP ? "rot" : "fwd", BH,
                 p.planes_per_run);
    return check_launch("small_down_kernel");
}

template <typename IO, int W, int K>
int launch_small_up2(SmallPlan &p, hipStream_t stream)
{
    p.lanes_per_plane = ceil_div(p.out_h, 2);
    if (p.lanes_per_plane > kWave) return -1;
    const int in_plane = p.in_h * W, out_plane = p.out_h * 2 * W;
    p.planes_per_run = planes_per_run(p.lanes_per_plane, in_plane, out_plane, p.planes);
    if (p.planes_per_run < 1) return -1;
    p.lpp_magic = magic_u16(p.lanes_per_plane);
    const long runs = (p.planes + p.planes_per_run - 1) / p.planes_per_run;
    if (runs > 0x7fffffffL) return -1;
    const size_t shmem = small_lds_bytes(p.planes_per_run, in_plane, out_plane);
    hipLaunchKernelGGL((small_up2_kernel<IO, W, K>), dim3(static_cast<unsigned>(runs)), dim3(kWave), shmem, stream, p);
    note_variant("small_up2%s<w%d,k%d> P%d", sizeof(IO) == 2 ? "16" : "", W, K, p.planes_per_run);
    return check_launch("small_up2_kernel");
}

template <typename IO, int W, int K>
int launch_small_down_any(SmallPlan &p, int S, bool rot, hipStream_t stream)
{
    constexpr int BH1 = W == 7 ? 7 : 2;
    if (S == 1) {
        if constexpr (W == 7) {
            // one lane per plane needs 64 planes per wavefront: with few planes that leaves most CUs idle,
            // so give a plane four lanes (two rows each) instead
            if (p.planes < 64l * 2048)
                return rot ? launch_small_down<IO, W, K, 1, true, 2>(p, stream) : launch_small_down<IO, W, K, 1, false, 2>(p, stream);
        }
        if constexpr (W != 7) {
            // One output row per lane (twice the lanes per plane, half the planes per wavefront, 80 instead of 140
            // registers) against two: 28x28 maps gain with every filter and element type (fp32 5x5 C=240 43.3 -> 39.0 us,
            // 7x7 C=192 27.8 -> 20.4, bf16 5x5 30.7 -> 28.4); 14x14 maps gain 1-2 us in fp32 with 3x3 and 5x5 filters
            // and lose 1-3 us with 7x7 filters or 16-bit elements.
            const bool one_row = W == 28 || (sizeof(IO) == 4 && K <= 5);
            if (env_int("DWCONV_SMALL_BH", one_row ? 1 : 2) == 1)
                return rot ? launch_small_down<IO, W, K, 1, true, 1>(p, stream) : launch_small_down<IO, W, K, 1, false, 1>(p, stream);
        }
        return rot ? launch_small_down<IO, W, K, 1, true, BH1>(p, stream) : launch_small_down<IO, W, K, 1, false, BH1>(p, stream);
    }
    if constexpr (W % 2 == 0) {
        if (S == 2 && !rot) return launch_small_down<IO, W, K, 2, false, 1>(p, stream);
    }
    return -1;
}

template <typename IO, int W>
int launch_small_down_k(SmallPlan &p, int K, int S, bool rot, hipStream_t stream)
{
    if (K == 3) return launch_small_down_any<IO, W, 3>(p, S, rot, stream);
    if (K == 5) return launch_small_down_any<IO, W, 5>(p, S, rot, stream);
    if (K == 7) return launch_small_down_any<IO, W, 7>(p, S, rot, stream);
    return -1;
}

template <typename IO, int W>
int launch_small_up2_k(SmallPlan &p, int K, hipStream_t stream)
{
    if (K == 3) return launch_small_up2<IO, W, 3>(p, stream);
    if (K == 5) return launch_small_up2<IO, W, 5>(p, stream);
    if (K == 7) return launch_small_up2<IO, W, 7>(p, stream);
    return -1;
}


}  // namespace

template <typename IO>
int try_launch_fir_small(const IO *in, const IO *taps, IO *out, const Geometry &g, hipStream_t stream)
{
    if (env_int("DWCONV_NO_SMALL", 0)) return -1;
    const int K = g.kernel_h;
    if (g.kernel_w != K || (K != 3 && K != 5 && K != 7)) return -1;
    if (!aligned4(in) || !aligned4(out)) return -1;
    if (g.in_h < 1 || g.in_h > 64 || g.out_h < 1 || g.out_h > 128) return -1;
    SmallPlan p{};
    p.in = in;
    p.taps = taps;
    p.out = out;
    p.planes = g.planes();
    p.channel = g.channel;
    p.epi = g.epi;
    p.in_h = g.in_h;
    p.out_h = g.out_h;
    const int W = g.in_w;
    if (g.up_h == 1 && g.up_w == 1 && g.down_h == g.down_w && (g.down_h == 1 || g.down_h == 2)) {
        const int S = g.down_h;
        // full-width rows with the column padding of a "same" convolution
        if (g.pad_w0 != K / 2 || g.out_w != (W - 1) / S + 1) return -1;
        if (g.pad_h0 < 0 || g.pad_h0 > 7) return -1;
        p.pad_h = g.pad_h0;
        if (W == 7) return launch_small_down_k<IO, 7>(p, K, S, !g.forward, stream);
        if (W == 14) return launch_small_down_k<IO, 14>(p, K, S, !g.forward, stream);
        if (W == 28) return launch_small_down_k<IO, 28>(p, K, S, !g.forward, stream);
        return -1;
    }
    if (g.up_h == 2 && g.up_w == 2 && g.down_h == 1 && g.down_w == 1 && !g.forward) {
        if (g.pad_w0 != K / 2 || g.pad_h0 != K / 2 || g.out_w != 2 * W) return -1;
        const int E = (K / 2) & 1;
        p.pad_h = (K / 2 + E) / 2;
        if (W == 7) return launch_small_up2_k<IO, 7>(p, K, stream);
        if (W == 14) return launch_small_up2_k<IO, 14>(p, K, stream);
        return -1;
    }
    return -1;
}

template int try_launch_fir_small<float>(const float *, const float *, float *, const Geometry &, hipStream_t);
template int try_launch_fir_small<half_t>(const half_t *, const half_t *, half_t *, const Geometry &, hipStream_t);
template int try_launch_fir_small<bf16_t>(const bf16_t *, const bf16_t *, bf16_t *, const Geometry &, hipStream_t);

}  // namespace dwconv
