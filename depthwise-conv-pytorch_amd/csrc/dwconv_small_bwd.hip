// Backward pass for small feature maps (7, 14 or 28 wide, "same" padding): grad-weight alone, or
// grad-weight and grad-input in one sweep.
//
// Wavefront (channel group g, chunk k): for every image of the chunk the x planes and the gy planes of
// the group's channels are streamed into LDS as two flat runs (128-bit loads).  While one image is
// being processed the runs of the next one are already in flight into registers.  A lane keeps one
// channel for the whole chunk:
//   grad-weight: the lane holds BH rows of gy and adds gy * x into K*K register sums; at the end the
//                lanes of a channel are added front to back through LDS -> partial[c][k][tap]
//                (the sum of torch_dwconv/dwconv_kernel.cu:269-297 and :535-586, without atomics);
//   grad-input : (fused variant) the same gy planes, still in LDS, are correlated with the rotated
//                taps; the rows replace the x run in LDS and leave with 128-bit stores.  gy is read from
//                HBM once for both gradients (the reference reads it twice, torch_dwconv/dwconv.py:56-68).
#include "dwconv_small_common.hpp"

namespace dwconv {

namespace {

constexpr int kRunRegs = 7;  // float4s per lane that hold one run of the next image
constexpr int kRunFloats = kRunRegs * kWave * 4;
constexpr int kSmallRedPitch = kWave + 1;

struct SmallBwdPlan {
    const void *x;    // element type IO of the kernel template
    const void *gy;
    const void *taps;
    void *gx;
    float *partial;
    int batch, channel;
    int in_h, out_h;
    int pad_h;
    int planes_per_run;  // channels per wavefront
    int lanes_per_plane;
    unsigned lpp_magic;
    int chunks, images_per_chunk;
};

// Issues the loads of a run of n elements (n >= 4, g aligned to four elements); slots past the end re-read the
// last group of four.
template <typename IO>
__device__ __forceinline__ void run_fetch(const IO *__restrict__ g, int n, typename Raw4<IO>::type (&v)[kRunRegs])
{
    const int n4 = n >> 2;
#pragma unroll
    for (int u = 0; u < kRunRegs; ++u) v[u] = load4_raw<IO>(g + 4 * min(static_cast<int>(threadIdx.x) + u * kWave, n4 - 1));
}

template <typename IO>
__device__ __forceinline__ void run_commit(const IO *__restrict__ g, float *lds, int n,
                                           const typename Raw4<IO>::type (&v)[kRunRegs])
{
    const int n4 = n >> 2;
#pragma unroll
    for (int u = 0; u < kRunRegs; ++u) {
        // slots past the end of the run hold its last group of four again (run_fetch) and rewrite it in place
        reinterpret_cast<float4 *>(lds)[min(static_cast<int>(threadIdx.x) + u * kWave, n4 - 1)] = widen4<IO>(v[u]);
    }
    const int tail = n4 * 4 + threadIdx.x;
    if (tail < n) lds[tail] = Io<IO>::in(g[tail]);
}

// PF: the runs of the next image are fetched into registers while the current image is processed
// (56 registers in fp32, 28 for 16-bit elements; dropped for the fp32 7x7 filter, whose sums and taps already take 98).
template <typename IO, int W, int K, int S, int BH, bool GX, bool PF = (K < 7 || sizeof(IO) == 2)>
__global__ __launch_bounds__(kWave) void small_bwd_kernel(const SmallBwdPlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int OW = (W - 1) / S + 1;
    constexpr int PW = K / 2;
    constexpr int KK = K * K;
    constexpr int WIN_ROWS = (BH - 1) * S + K;
    static_assert(S == 1 || BH == 1, "stride-2 lanes own one gy row");

    const int group = blockIdx.x / p.chunks;
    const int chunk = blockIdx.x - group * p.chunks;
    const int c0 = group * p.planes_per_run;
    const int nplanes = min(p.planes_per_run, p.channel - c0);
    const int n0 = chunk * p.images_per_chunk;
    const int n1 = min(p.batch, n0 + p.images_per_chunk);
    const int in_plane = p.in_h * W, out_plane = p.out_h * OW;
    const int nx = nplanes * in_plane, ng = nplanes * out_plane;
    float *lds_x = lds;
    float *lds_g = lds + p.planes_per_run * in_plane;

    const int pl_raw = fast_div(threadIdx.x, p.lpp_magic);
    const int rb = threadIdx.x - pl_raw * p.lanes_per_plane;
    const bool active = pl_raw < nplanes;
    const int pl = active ? pl_raw : 0;
    const int oy0 = rb * BH;

    float wacc[KK];
#pragma unroll
    for (int t = 0; t < KK; ++t) wacc[t] = 0.f;
    float tapv[GX ? KK : 1];
    if constexpr (GX) load_taps<KK, true>(static_cast<const IO *>(p.taps), c0 + pl, tapv);

    const IO *const x = static_cast<const IO *>(p.x);
    const IO *const gy = static_cast<const IO *>(p.gy);
    typename Raw4<IO>::type rx[kRunRegs], rg[kRunRegs];
    if constexpr (PF) {
        const long plane0 = static_cast<long>(n0) * p.channel + c0;
        run_fetch(x + plane0 * in_plane, nx, rx);
        run_fetch(gy + plane0 * out_plane, ng, rg);
    }

    for (int n = n0; n < n1; ++n) {
        const long plane0 = static_cast<long>(n) * p.channel + c0;
        if (n != n0) __syncthreads();  // the previous image is done with the LDS runs
        if constexpr (!PF) {
            run_fetch(x + plane0 * in_plane, nx, rx);
            run_fetch(gy + plane0 * out_plane, ng, rg);
        }
        run_commit(x + plane0 * in_plane, lds_x, nx, rx);
        run_commit(gy + plane0 * out_plane, lds_g, ng, rg);
        __syncthreads();
        if (PF && n + 1 < n1) {
            const long plane1 = plane0 + p.channel;
            run_fetch(x + plane1 * in_plane, nx, rx);
            run_fetch(gy + plane1 * out_plane, ng, rg);
        }

        // ---- grad-weight: this lane's gy rows against the x rows they touch
        {
            float g[BH][OW];
#pragma unroll
            for (int b = 0; b < BH; ++b) {
                const bool ok = active && oy0 + b < p.out_h;
                lds_load_row<OW>(lds_g + pl * out_plane + (ok ? oy0 + b : 0) * OW, g[b]);
#pragma unroll
                for (int o = 0; o < OW; ++o) g[b][o] = ok ? g[b][o] : 0.f;
            }
            const float *plane = lds_x + pl * in_plane;
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
                            wacc[ty * K + tx] = fmaf(g[b][o], row[ix], wacc[ty * K + tx]);
                        }
                }
                pin_registers(wacc);
            }
        }

        // ---- grad-input (fused variant): gy planes in LDS against the rotated taps
        if constexpr (GX) {
            constexpr int XR = S == 1 ? BH : 2;  // gx rows per lane
            float xacc[XR][W];
#pragma unroll
            for (int b = 0; b < XR; ++b)
#pragma unroll
                for (int o = 0; o < W; ++o) xacc[b][o] = 0.f;
            const float *gplane = lds_g + pl * out_plane;
            if constexpr (S == 1) {
                // gx[iy,ix] = sum_{ty,tx} gy[iy - PW + ty, ix - PW + tx] * rot[ty,tx]   (out extent == in extent)
                float nxt[OW];
                bool nxt_ok;
                {
                    const int gyr = oy0 - PW;
                    nxt_ok = static_cast<unsigned>(gyr) < static_cast<unsigned>(p.out_h);
                    lds_load_row<OW>(gplane + (nxt_ok ? gyr : 0) * OW, nxt);
                }
#pragma unroll
                for (int wr = 0; wr < BH - 1 + K; ++wr) {
                    float row[OW];
#pragma unroll
                    for (int i = 0; i < OW; ++i) row[i] = nxt_ok ? nxt[i] : 0.f;
                    if (wr + 1 < BH - 1 + K) {
                        const int gyr = oy0 - PW + wr + 1;
                        nxt_ok = static_cast<unsigned>(gyr) < static_cast<unsigned>(p.out_h);
                        lds_load_row<OW>(gplane + (nxt_ok ? gyr : 0) * OW, nxt);
                    }
#pragma unroll
                    for (int b = 0; b < BH; ++b) {
                        const int ty = wr - b;
                        if (ty < 0 || ty >= K) continue;
#pragma unroll
                        for (int tx = 0; tx < K; ++tx)
#pragma unroll
                            for (int o = 0; o < W; ++o) {
                                const int ix = o - PW + tx;
                                if (ix < 0 || ix >= OW) continue;
                                xacc[b][o] = fmaf(row[ix], tapv[ty * K + tx], xacc[b][o]);
                            }
                    }
                    pin_registers(xacc);
                }
            } else {
                // gx[2q + r] = sum_a gy[q - M + r + a] * rot'[r + 2a], rot'[t] = rot[t - E]  (see small_up2_kernel)
                constexpr int E = PW & 1;
                constexpr int M = (PW + E) / 2;
                constexpr int KA = (K + E + 1) / 2;
                float nxt[OW];
                bool nxt_ok;
                {
                    const int gyr = rb - M;
                    nxt_ok = static_cast<unsigned>(gyr) < static_cast<unsigned>(p.out_h);
                    lds_load_row<OW>(gplane + (nxt_ok ? gyr : 0) * OW, nxt);
                }
#pragma unroll
                for (int wr = 0; wr < KA + 1; ++wr) {
                    float row[OW];
#pragma unroll
                    for (int i = 0; i < OW; ++i) row[i] = nxt_ok ? nxt[i] : 0.f;
                    if (wr + 1 < KA + 1) {
                        const int gyr = rb - M + wr + 1;
                        nxt_ok = static_cast<unsigned>(gyr) < static_cast<unsigned>(p.out_h);
                        lds_load_row<OW>(gplane + (nxt_ok ? gyr : 0) * OW, nxt);
                    }
#pragma unroll
                    for (int r = 0; r < 2; ++r) {
                        const int a = wr - r;
                        if (a < 0 || a >= KA) continue;
                        const int fy = r + 2 * a - E;
                        if (fy < 0 || fy >= K) continue;
#pragma unroll
                        for (int o = 0; o < W; ++o) {
                            const int xq = o / 2, rxp = o % 2;
#pragma unroll
                            for (int ax = 0; ax < KA; ++ax) {
                                const int fx = rxp + 2 * ax - E;
                                const int ix = xq - M + rxp + ax;
                                if (fx < 0 || fx >= K || ix < 0 || ix >= OW) continue;
                                xacc[r][o] = fmaf(row[ix], tapv[fy * K + fx], xacc[r][o]);
                            }
                        }
                    }
                    pin_registers(xacc);
                }
            }
            __syncthreads();  // every lane is done with the x run: overwrite it with the gx run
            if (active) {
                float *dst = lds_x + pl * in_plane;
                const int row0 = S == 1 ? oy0 : 2 * rb;
#pragma unroll
                for (int b = 0; b < XR; ++b)
                    if (row0 + b < p.in_h) lds_store_row<W>(dst + (row0 + b) * W, xacc[b]);
            }
            __syncthreads();
            lds_to_run(static_cast<IO *>(p.gx) + plane0 * in_plane, lds_x, nx);
        }
    }

    __syncthreads();  // the runs are dead; reuse the LDS to bring the lanes of each channel together
#pragma unroll
    for (int t = 0; t < KK; ++t) lds[t * kSmallRedPitch + threadIdx.x] = wacc[t];
    __syncthreads();
    for (int e = threadIdx.x; e < nplanes * KK; e += kWave) {
        const int q = e / KK, t = e - q * KK;
        const float *col = lds + t * kSmallRedPitch + q * p.lanes_per_plane;
        float s = 0.f;
        for (int i = 0; i < p.lanes_per_plane; ++i) s += col[i];
        p.partial[(static_cast<long>(c0 + q) * p.chunks + chunk) * KK + t] = s;
    }
}

template <int W, int K, int S, int BH>
bool plan_small_bwd(SmallBwdPlan &p, const WgradGeometry &g)
{
    constexpr int OW = (W - 1) / S + 1;
    p.batch = g.batch;
    p.channel = g.channel;
    p.in_h = g.in_h;
    p.out_h = g.out_h;
    p.pad_h = g.pad_h;
    p.lanes_per_plane = ceil_div(g.out_h, BH);
    if (p.lanes_per_plane > kWave) return false;
    const int in_plane = g.in_h * W, out_plane = g.out_h * OW;
    const bool odd = in_plane % 4 != 0 || out_plane % 4 != 0;
    if (odd && g.channel % 4 != 0) return false;  // runs of every image must start on a 4-element boundary
    int P = kWave / p.lanes_per_plane;
    if (P > g.channel) P = g.channel;
    // a run must fit the registers that prefetch it
    while (P > 0 && (P * in_plane > kRunFloats || P * out_plane > kRunFloats)) --P;
    if (odd) P -= P % 4;
    if (P < 1) return false;
    p.planes_per_run = P;
    p.lpp_magic = magic_u16(p.lanes_per_plane);
    const int groups = ceil_div(g.channel, P);
    // At these register counts two wavefronts fit a SIMD, 2048 the device: the grid stays within that one resident
    // round (rounded down: 2112 wavefronts instead of 1536 cost the 28x28 7x7 backward 58 us instead of 47, the 64
    // stragglers run their whole chunk alone).
    int chunks = env_int("DWCONV_SMALL_WGRAD_WAVES", 2048) / groups;
    if (chunks > g.batch) chunks = g.batch;
    if (chunks < 1) chunks = 1;
    p.images_per_chunk = ceil_div(g.batch, chunks);
    p.chunks = ceil_div(g.batch, p.images_per_chunk);
    return true;
}

// mode 0: report the workspace bytes; mode 1: grad-weight; mode 2: grad-weight + grad-input.
// Returns -1 when this family does not cover g.
template <typename IO, int W, int K, int S, int BH>
long small_bwd_case(int mode, const IO *x, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws,
                    size_t ws_bytes, const WgradGeometry &g, hipStream_t stream)
{
    constexpr int OW = (W - 1) / S + 1;
    SmallBwdPlan p{};
    if (!plan_small_bwd<W, K, S, BH>(p, g)) return -1;
    const size_t need = static_cast<size_t>(g.channel) * p.chunks * K * K * sizeof(float);
    if (mode == 0) return static_cast<long>(need);
    if (ws == nullptr || ws_bytes < need)
        return fail(DWCONV_ERR_WORKSPACE, "grad-weight needs a workspace of %zu bytes, got %zu", need, ws_bytes);
    p.x = x;
    p.gy = gy;
    p.taps = taps;
    p.gx = gx;
    p.partial = static_cast<float *>(ws);
    const size_t runs = static_cast<size_t>(p.planes_per_run) * (g.in_h * W + g.out_h * OW) * 4;
    const size_t red = static_cast<size_t>(K) * K * kSmallRedPitch * 4;
    const size_t shmem = runs > red ? runs : red;
    const int groups = ceil_div(g.channel, p.planes_per_run);
    if (mode == 2)
        hipLaunchKernelGGL((small_bwd_kernel<IO, W, K, S, BH, true>), dim3(groups * p.chunks), dim3(kWave), shmem, stream, p);
    else
        hipLaunchKernelGGL((small_bwd_kernel<IO, W, K, S, BH, false>), dim3(groups * p.chunks), dim3(kWave), shmem, stream, p);
    const int rc = check_launch("small_bwd_kernel");
    if (rc != DWCONV_OK) return rc;
    note_variant("%s%s<w%d,k%d,s%d,bh%d> P%d chunks%d", mode == 2 ? "small_bwd" : "small_wgrad",
                 sizeof(IO) == 2 ? "16" : "", W, K, S, BH, p.planes_per_run, p.chunks);
    return launch_wgrad_final(p.partial, gw, g.channel, K * K, p.chunks, stream);
}

template <typename IO, int W, int K>
long small_bwd_s(int mode, const IO *x, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws,
                 size_t ws_bytes, const WgradGeometry &g, hipStream_t stream)
{
    constexpr int BH1 = W == 7 ? 4 : (W == 14 ? 2 : 1);
    if (g.down_h == 1) {
        if constexpr (W == 7 && sizeof(IO) == 4 && K >= 5) {
            // 7x7 maps, fp32, 5x5 and 7x7 filters: two rows per lane (four lanes per plane) instead of four (two lanes):
            // C=1152 5x5 30.9 -> 29.8 us, C=768 7x7 at batch 64 26.0 -> 23.1; 3x3 filters and 16-bit elements lose 1-2 us
            if (env_int("DWCONV_SMALL_BWD_BH", 2) == 2)
                return small_bwd_case<IO, W, K, 1, 2>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
        }
        return small_bwd_case<IO, W, K, 1, BH1>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
    }
    if constexpr (W % 2 == 0) {
        if (g.down_h == 2) return small_bwd_case<IO, W, K, 2, 1>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
    }
    return -1;
}

template <typename IO, int W>
long small_bwd_k(int mode, const IO *x, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws,
                 size_t ws_bytes, const WgradGeometry &g, hipStream_t stream)
{
    if (g.kernel_h == 3) return small_bwd_s<IO, W, 3>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
    if (g.kernel_h == 5) return small_bwd_s<IO, W, 5>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
    if (g.kernel_h == 7) return small_bwd_s<IO, W, 7>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
    return -1;
}

template <typename IO>
long small_bwd_any(int mode, const IO *x, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws,
                   size_t ws_bytes, const WgradGeometry &g, hipStream_t stream)
{
    if (env_int("DWCONV_NO_SMALL", 0)) return -1;
    const int K = g.kernel_h, S = g.down_h;
    if (g.kernel_w != K || g.down_w != S || (S != 1 && S != 2)) return -1;
    if (g.pad_w != K / 2 || g.pad_h < 0 || g.pad_h > 7) return -1;
    if (g.in_h < 1 || g.in_h > 64 || g.out_h < 1 || g.out_h > 64) return -1;
    if (g.out_w != (g.in_w - 1) / S + 1) return -1;
    if (mode == 2) {
        // the fused variant writes every gx row from the lane that owns the matching gy rows
        if (g.pad_h != K / 2) return -1;
        if (S == 1 && g.out_h != g.in_h) return -1;
        if (S == 2 && (g.in_h != 2 * g.out_h || g.in_w != 2 * g.out_w)) return -1;
        if (!aligned4(gx)) return -1;
    }
    if (mode != 0 && (!aligned4(x) || !aligned4(gy))) return -1;
    if (g.in_w == 7) return small_bwd_k<IO, 7>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
    if (g.in_w == 14) return small_bwd_k<IO, 14>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
    if (g.in_w == 28) return small_bwd_k<IO, 28>(mode, x, gy, taps, gx, gw, ws, ws_bytes, g, stream);
    return -1;
}

}  // namespace

size_t wgrad_small_workspace(const WgradGeometry &g)
{
    // partial sums are fp32 whatever the element type
    const long n = small_bwd_any<float>(0, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, g, nullptr);
    return n > 0 ? static_cast<size_t>(n) : 0;
}

template <typename IO>
int try_launch_wgrad_small(const IO *in, const IO *gy, IO *gw, void *ws, size_t ws_bytes, const WgradGeometry &g,
                           hipStream_t stream)
{
    return static_cast<int>(small_bwd_any<IO>(1, in, gy, nullptr, nullptr, gw, ws, ws_bytes, g, stream));
}

template <typename IO>
int try_launch_bwd_small(const IO *in, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes,
                         const WgradGeometry &g, hipStream_t stream)
{
    return static_cast<int>(small_bwd_any<IO>(2, in, gy, taps, gx, gw, ws, ws_bytes, g, stream));
}

#define DWCONV_INSTANTIATE(IO)                                                                                        \
    template int try_launch_wgrad_small<IO>(const IO *, const IO *, IO *, void *, size_t, const WgradGeometry &,      \
                                            hipStream_t);                                                             \
    template int try_launch_bwd_small<IO>(const IO *, const IO *, const IO *, IO *, IO *, void *, size_t,             \
                                          const WgradGeometry &, hipStream_t);
DWCONV_INSTANTIATE(float)
DWCONV_INSTANTIATE(half_t)
DWCONV_INSTANTIATE(bf16_t)
#undef DWCONV_INSTANTIATE

}  // namespace dwconv
