// Backward pass for small feature maps (up to 32 elements wide, "same" column padding): grad-weight alone, or
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
// Width instances (exact or ragged) as in dwconv_small_fir.hpp: W is the width of x, or its capacity class.
#pragma once

#include "dwconv_small_common.hpp"

namespace dwconv {

namespace {

// float4s per lane that hold one run (the planes of a wavefront's channels in one image): 1792 floats for the
// 7-, 14- and 28-wide instances (nine 14 x 14 planes, two 28 x 28 ones), 2048 for the others (eight 16 x 16 or
// 15 x 15 planes, two 32 x 32 ones)
constexpr int run_regs(int w) { return (w == 7 || w == 14 || w == 28) ? 7 : 8; }
constexpr int run_floats(int w) { return run_regs(w) * kWave * 4; }
constexpr int kSmallRedPitch = kWave + 1;

struct SmallBwdPlan {
    const void *x;    // element type IO of the kernel template
    const void *gy;
    const void *taps;
    void *gx;
    float *partial;
    int batch, channel;
    int in_h, out_h;
    int in_w, out_w;     // real widths (the kernels of an exact instance use their template constant)
    int pad_h;
    int planes_per_run;  // channels per wavefront
    int g_off;           // float offset of the gy run's span in LDS (a multiple of four)
    int zero_off;        // float offset of the row of zeros in LDS (a multiple of four)
    int lds_x_floats, lds_g_floats;  // LDS images of the two runs (host side only)
    int lds_x_off;       // float offset of the x run's span (0)
    int lp_in, lp_out;   // ragged instances: LDS row pitch of the x / gy rows (width | 1)
    unsigned magic_in, magic_out;  // ... and the reciprocals for padded_index (0: pitch == width, flat copies)
    int lanes_per_plane;
    unsigned lpp_magic;
    int chunks, images_per_chunk;
};

// Issues the loads of a run of n elements (n >= 4, g aligned to four elements); slots past the end re-read the
// last group of four.
template <typename IO, int RR>
__device__ __forceinline__ void run_fetch(const IO *__restrict__ g, int n, typename Raw4<IO>::type (&v)[RR])
{
    const int n4 = n >> 2;
#pragma unroll
    for (int u = 0; u < RR; ++u) v[u] = load4_raw<IO>(g + 4 * min(static_cast<int>(threadIdx.x) + u * kWave, n4 - 1));
}

template <typename IO, int RR, int GPR = 0>
__device__ __forceinline__ void run_commit(const IO *__restrict__ g, float *lds, int n,
                                           const typename Raw4<IO>::type (&v)[RR])
{
    const int n4 = n >> 2;
#pragma unroll
    for (int u = 0; u < RR; ++u) {
        // slots past the end of the run hold its last group of four again (run_fetch) and rewrite it in place
        reinterpret_cast<float4 *>(lds)[lds_group<GPR>(min(static_cast<int>(threadIdx.x) + u * kWave, n4 - 1))] = widen4<IO>(v[u]);
    }
    // (a run with padded rows is whole groups of four)
    const int tail = n4 * 4 + threadIdx.x;
    if (GPR == 0 && tail < n) lds[tail] = Io<IO>::in(g[tail]);
}

// PF: the runs of the next image are fetched into registers while the current image is processed
// (56-64 registers in fp32, half for 16-bit elements; dropped for the fp32 7x7 filter, whose sums and taps already
// take 98, and for fp32 rows beyond 28 elements, whose row registers do: with it the 32-wide 5x5 instance needs 280
// registers, one wavefront per SIMD).
// The same for rows at pitch width + 1 in LDS (ragged even widths; see run_to_lds_rows).
template <typename IO, int RR>
__device__ __forceinline__ void run_commit_rows(const IO *__restrict__ g, float *lds, int n, int head, unsigned magic, int dump,
                                                const typename Raw4<IO>::type (&v)[RR])
{
    const int n4 = n >> 2;
#pragma unroll
    for (int u = 0; u < RR; ++u) {
        const float4 w = widen4<IO>(v[u]);
        const int i = 4 * min(static_cast<int>(threadIdx.x) + u * kWave, n4 - 1) - head;
        lds[i >= 0 ? padded_index(i, magic) : dump] = w.x;
        lds[i + 1 >= 0 ? padded_index(i + 1, magic) : dump] = w.y;
        lds[i + 2 >= 0 ? padded_index(i + 2, magic) : dump] = w.z;
        lds[padded_index(i + 3, magic)] = w.w;
    }
    const int tail = n4 * 4 + threadIdx.x;
    if (tail < n && tail >= head) lds[padded_index(tail - head, magic)] = Io<IO>::in(g[tail]);
}

// PAD: LDS rows of 8, 16 or 32 floats get four spare floats (see lds_row_pitch)
// D: dilation of the taps (stride 1 only; the padding is then D * (K/2)).
template <typename IO, int W, bool RAG, int K, int S, int BH, bool GX, bool PAD, int D = 1,
          bool PF = (sizeof(IO) == 2 || (K < 7 && (RAG || W <= 28 || K == 3)))>
__global__ __launch_bounds__(kWave) void small_bwd_kernel(const SmallBwdPlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int OW = (W - 1) / S + 1;  // gy columns a lane handles (the real count when exact)
    constexpr int RR = run_regs(W);
    const int w_in = RAG ? p.in_w : W, w_out = RAG ? p.out_w : OW;
    constexpr int KE = (K - 1) * D + 1;  // rows and columns the dilated taps span
    constexpr int PW = D * (K / 2);
    static_assert(D == 1 || S == 1, "dilation comes with stride 1");
    constexpr int KK = K * K;
    constexpr int WIN_ROWS = (BH - 1) * S + KE;
    static_assert(S == 1 || BH == 1, "stride-2 lanes own one gy row");

    const int group = blockIdx.x / p.chunks;
    const int chunk = blockIdx.x - group * p.chunks;
    const int c0 = group * p.planes_per_run;
    const int nplanes = min(p.planes_per_run, p.channel - c0);
    const int n0 = chunk * p.images_per_chunk;
    const int n1 = min(p.batch, n0 + p.images_per_chunk);
    // row pitch in LDS (padded for rows of 8, 16 or 32 floats, see lds_row_pitch) and the plane pitch that follows
    constexpr int GI = PAD ? lds_row_groups(W, RAG) : 0, GO = PAD ? lds_row_groups(OW, RAG) : 0;
    // (ragged even widths: pitch width + 1, element-wise copies)
    const int lp_in = RAG ? p.lp_in : (GI ? lds_row_pitch(W, RAG) : W), lp_out = RAG ? p.lp_out : (GO ? lds_row_pitch(OW, RAG) : OW);
    const bool pad_in = RAG && p.magic_in != 0, pad_out = RAG && p.magic_out != 0;
    const int in_plane = p.in_h * w_in, out_plane = p.out_h * w_out;
    const int lin_plane = p.in_h * lp_in, lout_plane = p.out_h * lp_out;
    const int nx = nplanes * in_plane, ng = nplanes * out_plane;
    float *lds_x = lds;
    float *lds_g = lds + p.g_off;
    const float *zrow = lds + p.zero_off;  // stands in for the rows above and below a plane (cleared before the first barrier)
    clear_zero_row<W>(lds + p.zero_off);

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
    typename Raw4<IO>::type rx[RR], rg[RR];
    // A run that starts off a 4-element boundary is moved as the aligned span around it (see lds_to_run): hx / hg
    // elements of the neighbouring run come first in its LDS image.
    if constexpr (PF) {
        const long plane0 = static_cast<long>(n0) * p.channel + c0;
        const long x0 = plane0 * in_plane, g0 = plane0 * out_plane;
        run_fetch<IO, RR>(x + (x0 - (x0 & 3)), nx + static_cast<int>(x0 & 3), rx);
        run_fetch<IO, RR>(gy + (g0 - (g0 & 3)), ng + static_cast<int>(g0 & 3), rg);
    }

    for (int n = n0; n < n1; ++n) {
        const long plane0 = static_cast<long>(n) * p.channel + c0;
        const long x0 = plane0 * in_plane, g0 = plane0 * out_plane;
        const int hx = static_cast<int>(x0 & 3), hg = static_cast<int>(g0 & 3);
        if (n != n0) __syncthreads();  // the previous image is done with the LDS runs
        if constexpr (!PF) {
            run_fetch<IO, RR>(x + (x0 - hx), nx + hx, rx);
            run_fetch<IO, RR>(gy + (g0 - hg), ng + hg, rg);
        }
        if (pad_in) run_commit_rows<IO, RR>(x + (x0 - hx), lds_x, nx + hx, hx, p.magic_in, p.zero_off - 1 - p.lds_x_off, rx);
        else run_commit<IO, RR, GI>(x + (x0 - hx), lds_x, nx + hx, rx);
        if (pad_out) run_commit_rows<IO, RR>(gy + (g0 - hg), lds_g, ng + hg, hg, p.magic_out, p.zero_off - 1 - p.g_off, rg);
        else run_commit<IO, RR, GO>(gy + (g0 - hg), lds_g, ng + hg, rg);
        __syncthreads();
        if (PF && n + 1 < n1) {
            const long x1 = (plane0 + p.channel) * in_plane, g1 = (plane0 + p.channel) * out_plane;
            run_fetch<IO, RR>(x + (x1 - (x1 & 3)), nx + static_cast<int>(x1 & 3), rx);
            run_fetch<IO, RR>(gy + (g1 - (g1 & 3)), ng + static_cast<int>(g1 & 3), rg);
        }

        // ---- grad-weight: this lane's gy rows against the x rows they touch
        {
            float g[BH][OW];
#pragma unroll
            for (int b = 0; b < BH; ++b) {
                const bool ok = active && oy0 + b < p.out_h;
                lds_load_row_w<OW, RAG>(ok ? lds_g + (pad_out ? 0 : hg) + pl * lout_plane + (oy0 + b) * lp_out : zrow, g[b], w_out);
            }
            const float *plane = lds_x + (pad_in ? 0 : hx) + pl * lin_plane;
            // rows are read one ahead of their use and the sums pinned after every row (see pin_registers)
            auto row_at = [&](int iy) { return static_cast<unsigned>(iy) < static_cast<unsigned>(p.in_h) ? plane + iy * lp_in : zrow; };
            float nxt[W];
            lds_load_row_w<W, RAG>(row_at(oy0 * S - p.pad_h), nxt, w_in);
#pragma unroll
            for (int wr = 0; wr < WIN_ROWS; ++wr) {
                float row[W];
#pragma unroll
                for (int i = 0; i < W; ++i) row[i] = nxt[i];
                if (wr + 1 < WIN_ROWS) lds_load_row_w<W, RAG>(row_at(oy0 * S - p.pad_h + wr + 1), nxt, w_in);
#pragma unroll
                for (int b = 0; b < BH; ++b) {
                    const int dy = wr - b * S;
                    if (dy < 0 || dy >= KE || dy % D != 0) continue;
                    const int ty = dy / D;
#pragma unroll
                    for (int tx = 0; tx < K; ++tx)
#pragma unroll
                        for (int o = 0; o < OW; ++o) {
                            const int ix = o * S - PW + tx * D;
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
            const float *gplane = lds_g + (pad_out ? 0 : hg) + pl * lout_plane;
            auto grow_at = [&](int gyr) { return static_cast<unsigned>(gyr) < static_cast<unsigned>(p.out_h) ? gplane + gyr * lp_out : zrow; };
            if constexpr (S == 1) {
                // gx[iy,ix] = sum_{ty,tx} gy[iy - PW + ty, ix - PW + tx] * rot[ty,tx]   (out extent == in extent)
                float nxt[OW];
                lds_load_row_w<OW, RAG>(grow_at(oy0 - PW), nxt, w_out);
#pragma unroll
                for (int wr = 0; wr < BH - 1 + KE; ++wr) {
                    float row[OW];
#pragma unroll
                    for (int i = 0; i < OW; ++i) row[i] = nxt[i];
                    if (wr + 1 < BH - 1 + KE) lds_load_row_w<OW, RAG>(grow_at(oy0 - PW + wr + 1), nxt, w_out);
#pragma unroll
                    for (int b = 0; b < BH; ++b) {
                        const int dy = wr - b;
                        if (dy < 0 || dy >= KE || dy % D != 0) continue;
                        const int ty = dy / D;
#pragma unroll
                        for (int tx = 0; tx < K; ++tx)
#pragma unroll
                            for (int o = 0; o < W; ++o) {
                                const int ix = o - PW + tx * D;
                                if (ix < 0 || ix >= OW) continue;
                                xacc[b][o] = fmaf(row[ix], tapv[ty * K + tx], xacc[b][o]);
                            }
                    }
                    pin_registers(xacc);
                }
            } else {
                // gx[2q + r] = sum_a gy[q - M + r + a] * rot'[r + 2a], rot'[t] = rot[t - E]  (see small_up2_kernel)
                constexpr int E = (K / 2) & 1;
                constexpr int M = (K / 2 + E) / 2;
                constexpr int KA = (K + E + 1) / 2;
                float nxt[OW];
                lds_load_row_w<OW, RAG>(grow_at(rb - M), nxt, w_out);
#pragma unroll
                for (int wr = 0; wr < KA + 1; ++wr) {
                    float row[OW];
#pragma unroll
                    for (int i = 0; i < OW; ++i) row[i] = nxt[i];
                    if (wr + 1 < KA + 1) lds_load_row_w<OW, RAG>(grow_at(rb - M + wr + 1), nxt, w_out);
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
                float *dst = lds_x + (pad_in ? 0 : hx) + pl * lin_plane;
                const int row0 = S == 1 ? oy0 : 2 * rb;
#pragma unroll
                for (int b = 0; b < XR; ++b)
                    if (row0 + b < p.in_h) lds_store_row_w<W, RAG>(dst + (row0 + b) * lp_in, xacc[b], w_in);
            }
            __syncthreads();
            if (pad_in) lds_to_run_rows(static_cast<IO *>(p.gx) + (x0 - hx), lds_x, nx + hx, hx, p.magic_in);
            else lds_to_run<IO, GI>(static_cast<IO *>(p.gx) + (x0 - hx), lds_x, nx + hx, hx);
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

template <int W, bool RAG, int K, int S, int BH, bool PAD>
bool plan_small_bwd(SmallBwdPlan &p, const WgradGeometry &g)
{
    constexpr int OW = (W - 1) / S + 1;
    p.batch = g.batch;
    p.channel = g.channel;
    p.in_h = g.in_h;
    p.out_h = g.out_h;
    p.in_w = g.in_w;
    p.out_w = g.out_w;
    p.pad_h = g.pad_h;
    p.lanes_per_plane = ceil_div(g.out_h, BH);
    if (p.lanes_per_plane > kWave) return false;
    const int in_plane = g.in_h * g.in_w, out_plane = g.out_h * g.out_w;
    const bool odd = in_plane % 4 != 0 || out_plane % 4 != 0;
    int P = kWave / p.lanes_per_plane;
    if (P > g.channel) P = g.channel;
    // a run (with the up to three elements in front of one that starts off a 4-element boundary) must fit the
    // registers that prefetch it
    const int head = odd ? 3 : 0;
    while (P > 0 && (P * in_plane + head > run_floats(W) || P * out_plane + head > run_floats(W))) --P;
    // whole groups of four channels keep every run on a 4-element boundary (if the channel count allows it too)
    if (odd && P >= 4) P -= P % 4;
    if (P < 1) return false;
    if (in_plane < 4 || out_plane < 4) return false;
    p.planes_per_run = P;
    // LDS images: rows at their LDS pitch
    p.lp_in = RAG ? ragged_pitch(g.in_w) : g.in_w;
    p.lp_out = RAG ? ragged_pitch(g.out_w) : g.out_w;
    p.magic_in = RAG ? ragged_magic(g.in_w) : 0;
    p.magic_out = RAG ? ragged_magic(g.out_w) : 0;
    p.lds_x_off = 0;
    p.lds_x_floats = P * g.in_h * ((PAD && lds_row_groups(W, RAG)) ? lds_row_pitch(W, RAG) : p.lp_in);
    p.lds_g_floats = P * g.out_h * ((PAD && lds_row_groups(OW, RAG)) ? lds_row_pitch(OW, RAG) : p.lp_out);
    p.g_off = round_up(p.lds_x_floats + head, 4);
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

template <typename IO, int W, bool RAG, int K, int S, int BH, bool PAD, int D = 1>
long small_bwd_case(int mode, const SmallBwdArgs &a, const WgradGeometry &g, hipStream_t stream)
{
    SmallBwdPlan p{};
    if (!plan_small_bwd<W, RAG, K, S, BH, PAD>(p, g)) return -1;
    const size_t need = static_cast<size_t>(g.channel) * p.chunks * K * K * sizeof(float);
    if (mode == 0) return static_cast<long>(need);
    if (a.ws == nullptr || a.ws_bytes < need)
        return fail(DWCONV_ERR_WORKSPACE, "grad-weight needs a workspace of %zu bytes, got %zu", need, a.ws_bytes);
    p.x = a.x;
    p.gy = a.gy;
    p.taps = a.taps;
    p.gx = a.gx;
    p.partial = static_cast<float *>(a.ws);
    // (ragged rows are read up to W - 1 floats past their end: spare floats behind the gy run)
    p.zero_off = round_up(p.g_off + p.lds_g_floats + 4 + (RAG ? W : 0), 4);
    const size_t runs = static_cast<size_t>(p.zero_off + zero_row_floats(W)) * 4;
    const size_t red = static_cast<size_t>(K) * K * kSmallRedPitch * 4;
    const size_t shmem = runs > red ? runs : red;
    const int groups = ceil_div(g.channel, p.planes_per_run);
    if (mode == 2)
        hipLaunchKernelGGL((small_bwd_kernel<IO, W, RAG, K, S, BH, true, PAD, D>), dim3(groups * p.chunks), dim3(kWave), shmem, stream, p);
    else
        hipLaunchKernelGGL((small_bwd_kernel<IO, W, RAG, K, S, BH, false, PAD, D>), dim3(groups * p.chunks), dim3(kWave), shmem, stream, p);
    const int rc = check_launch("small_bwd_kernel");
    if (rc != DWCONV_OK) return rc;
    note_variant("%s%s<%s%d,k%d,s%d,bh%d%s%s> P%d chunks%d", mode == 2 ? "small_bwd" : "small_wgrad",
                 sizeof(IO) == 2 ? "16" : "", RAG ? "r" : "w", W, K, S, BH, PAD ? ",pad" : "", D == 2 ? ",d2" : "",
                 p.planes_per_run, p.chunks);
    return launch_wgrad_final(p.partial, static_cast<IO *>(a.gw), g.channel, K * K, p.chunks, stream);
}

// Rows of gy per lane, measured on the 7-, 14- and 28-wide maps and carried over to their neighbours: up to 8
// columns four rows (two lanes per 7x7 plane), but two with fp32 5x5 / 7x7 filters (C=1152 5x5 30.9 -> 29.8 us,
// C=768 7x7 at batch 64 26.0 -> 23.1; 3x3 filters and 16-bit elements lose 1-2 us); up to 16 columns two rows; wider
// maps and stride 2 one row.
template <typename IO, int W, bool RAG, int K>
long small_bwd_s(int mode, const SmallBwdArgs &a, const WgradGeometry &g, hipStream_t stream)
{
    constexpr int BH1 = W <= 8 ? ((sizeof(IO) == 4 && K >= 5) ? 2 : 4) : (W <= 16 ? 2 : 1);
    // LDS rows padded where the measurements say so: 32-wide maps (5x5 C=240 115 -> 80 us, 3x3 stride 2 80 -> 54) and
    // 16-wide ones at stride 2 (one row per lane: 47.5 -> 42.6 us); 16-wide stride 1 (two rows per lane) and 8-wide
    // maps did not change
    constexpr bool PAD1 = !RAG && W == 32, PAD2 = !RAG && (W == 32 || W == 16);
    if (g.dil != 1) {
        // dilation 2: stride 1, 3x3 and 5x5 taps, both gradients
        if constexpr (K <= 5) {
            if (g.dil == 2 && g.down_h == 1) return small_bwd_case<IO, W, RAG, K, 1, BH1, PAD1, 2>(mode, a, g, stream);
        }
        return -1;
    }
    if (g.down_h == 1) return small_bwd_case<IO, W, RAG, K, 1, BH1, PAD1>(mode, a, g, stream);
    if (g.down_h == 2) return small_bwd_case<IO, W, RAG, K, 2, 1, PAD2>(mode, a, g, stream);
    return -1;
}

}  // namespace

template <int W, bool RAG, typename IO>
long small_bwd_width(int mode, const SmallBwdArgs &a, const WgradGeometry &g, hipStream_t stream)
{
    if (g.kernel_h == 3) return small_bwd_s<IO, W, RAG, 3>(mode, a, g, stream);
    if (g.kernel_h == 5) return small_bwd_s<IO, W, RAG, 5>(mode, a, g, stream);
    if (g.kernel_h == 7) return small_bwd_s<IO, W, RAG, 7>(mode, a, g, stream);
    return -1;
}

}  // namespace dwconv
