// Whole-plane fp32 kernels for small feature maps (width 7, 14 or 28, "same" padding).
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
//   small_wgrad_kernel: grad-weight pass 1 (lane keeps its channel across the images of a chunk)
#include "dwconv_tile_common.hpp"

namespace dwconv {

namespace {

constexpr int kWave = 64;

struct SmallPlan {
    const float *in;
    const float *taps;
    float *out;
    long planes;
    int channel;
    int in_h, out_h;
    int pad_h;             // leading zero rows (down) or m = (pad0 + E) / 2 (up2)
    int planes_per_run;    // P
    int lanes_per_plane;   // LPP
    unsigned lpp_magic;
};

// ---- LDS rows -----------------------------------------------------------------------------
template <int N>
__device__ __forceinline__ void lds_load_row(const float *p, float (&r)[N])
{
    if constexpr (N % 4 == 0) {
#pragma unroll
        for (int i = 0; i < N / 4; ++i) {
            const float4 v = reinterpret_cast<const float4 *>(p)[i];
            r[4 * i] = v.x; r[4 * i + 1] = v.y; r[4 * i + 2] = v.z; r[4 * i + 3] = v.w;
        }
    } else if constexpr (N % 2 == 0) {
#pragma unroll
        for (int i = 0; i < N / 2; ++i) {
            const float2 v = reinterpret_cast<const float2 *>(p)[i];
            r[2 * i] = v.x; r[2 * i + 1] = v.y;
        }
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) r[i] = p[i];
    }
}

template <int N>
__device__ __forceinline__ void lds_store_row(float *p, const float *r)
{
    if constexpr (N % 4 == 0) {
#pragma unroll
        for (int i = 0; i < N / 4; ++i)
            reinterpret_cast<float4 *>(p)[i] = make_float4(r[4 * i], r[4 * i + 1], r[4 * i + 2], r[4 * i + 3]);
    } else if constexpr (N % 2 == 0) {
#pragma unroll
        for (int i = 0; i < N / 2; ++i) reinterpret_cast<float2 *>(p)[i] = make_float2(r[2 * i], r[2 * i + 1]);
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) p[i] = r[i];
    }
}

// ---- flat runs between global memory and LDS ---------------------------------------------------
// `g` is 16-byte aligned; n floats; the last partial float4 (only at the very end of a tensor) goes scalar.
// Loads are issued kRunBatch at a time before any of them is consumed, so their latencies overlap.
constexpr int kRunBatch = 8;

__device__ __forceinline__ void run_to_lds(const float *__restrict__ g, float *lds, int n)
{
    const int n4 = n >> 2;
    for (int base = threadIdx.x; base < n4; base += kWave * kRunBatch) {
        float4 v[kRunBatch];
        // out-of-range slots re-read the last float4 of the run (always a valid address) and are not stored
#pragma unroll
        for (int u = 0; u < kRunBatch; ++u)
            v[u] = reinterpret_cast<const float4 *>(g)[min(base + u * kWave, n4 - 1)];
#pragma unroll
        for (int u = 0; u < kRunBatch; ++u)
            if (base + u * kWave < n4) reinterpret_cast<float4 *>(lds)[base + u * kWave] = v[u];
    }
    const int tail = n4 * 4 + threadIdx.x;
    if (tail < n) lds[tail] = g[tail];
}

// Two runs at once (grad-weight: x and gy of the same planes): all loads of a batch of both runs fly together.
__device__ __forceinline__ void runs_to_lds(const float *__restrict__ ga, float *la, int na,
                                            const float *__restrict__ gb, float *lb, int nb)
{
    const int na4 = na >> 2, nb4 = nb >> 2;
    const int nmax = na4 > nb4 ? na4 : nb4;
    constexpr int U = kRunBatch / 2;
    for (int base = threadIdx.x; base < nmax; base += kWave * U) {
        float4 va[U], vb[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            va[u] = reinterpret_cast<const float4 *>(ga)[min(base + u * kWave, na4 - 1)];
            vb[u] = reinterpret_cast<const float4 *>(gb)[min(base + u * kWave, nb4 - 1)];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (base + u * kWave < na4) reinterpret_cast<float4 *>(la)[base + u * kWave] = va[u];
            if (base + u * kWave < nb4) reinterpret_cast<float4 *>(lb)[base + u * kWave] = vb[u];
        }
    }
    const int ta = na4 * 4 + threadIdx.x, tb = nb4 * 4 + threadIdx.x;
    if (ta < na) la[ta] = ga[ta];
    if (tb < nb) lb[tb] = gb[tb];
}

__device__ __forceinline__ void lds_to_run(float *__restrict__ g, const float *lds, int n)
{
    const int n4 = n >> 2;
    constexpr int U = 4;
    for (int base = threadIdx.x; base < n4; base += kWave * U) {
        float4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = reinterpret_cast<const float4 *>(lds)[min(base + u * kWave, n4 - 1)];
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (base + u * kWave < n4) reinterpret_cast<float4 *>(g)[base + u * kWave] = v[u];
    }
    const int tail = n4 * 4 + threadIdx.x;
    if (tail < n) g[tail] = lds[tail];
}

// This lane's K*K taps straight from global memory (the lanes of one plane read the same addresses).
template <int KK, bool FLIP>
__device__ __forceinline__ void load_taps(const float *__restrict__ taps, int c, float (&t)[KK])
{
#pragma unroll
    for (int i = 0; i < KK; ++i) t[i] = taps[c * KK + (FLIP ? KK - 1 - i : i)];
}

// out[oy,ox] = sum_{ty,tx} in[oy*S - pad_h + ty, ox*S - K/2 + tx] * f[ty,tx], planes W wide.
template <int W, int K, int S, bool FLIP, int BH>
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
    load_taps<K * K, FLIP>(p.taps, static_cast<int>((plane0 + pl) % p.channel), tapv);
    run_to_lds(p.in + plane0 * in_plane, lds, nplanes * in_plane);
    __syncthreads();

    float acc[BH][OW];
#pragma unroll
    for (int b = 0; b < BH; ++b)
#pragma unroll
        for (int o = 0; o < OW; ++o) acc[b][o] = 0.f;

    const int oy0 = rb * BH;
    const float *plane = lds + pl * in_plane;
#pragma unroll
    for (int wr = 0; wr < WIN_ROWS; ++wr) {
        const int iy = oy0 * S - p.pad_h + wr;
        const bool ok = static_cast<unsigned>(iy) < static_cast<unsigned>(p.in_h);
        float row[W];
        lds_load_row<W>(plane + (ok ? iy : 0) * W, row);
#pragma unroll
        for (int i = 0; i < W; ++i) row[i] = ok ? row[i] : 0.f;
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
    }
    __syncthreads();  // every lane has read its input rows: the run can be overwritten in place

    if (active) {
        float *dst = lds + pl * out_plane;
#pragma unroll
        for (int b = 0; b < BH; ++b)
            if (oy0 + b < p.out_h) lds_store_row<OW>(dst + (oy0 + b) * OW, acc[b]);
    }
    __syncthreads();
    lds_to_run(p.out + plane0 * out_plane, lds, nplanes * out_plane);
}

// up = 2, taps rotated, "same" padding of the forward conv (leading pad of the transposed problem = K/2):
//   out[2q + r] = sum_a in[q - m + r + a] * g'[r + 2a],  g'[t] = g[t - E],  E = (K/2) & 1,  m = (K/2 + E) / 2.
// Input planes are W wide, output planes 2W wide; a lane owns output rows 2q, 2q+1.
template <int W, int K>
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
    load_taps<K * K, true>(p.taps, static_cast<int>((plane0 + pl) % p.channel), tapv);
    run_to_lds(p.in + plane0 * in_plane, lds, nplanes * in_plane);
    __syncthreads();

    float acc[2][OW];
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int o = 0; o < OW; ++o) acc[r][o] = 0.f;

    const float *plane = lds + pl * in_plane;
#pragma unroll
    for (int wr = 0; wr < WIN_ROWS; ++wr) {
        const int iy = q - p.pad_h + wr;
        const bool ok = static_cast<unsigned>(iy) < static_cast<unsigned>(p.in_h);
        float row[W];
        lds_load_row<W>(plane + (ok ? iy : 0) * W, row);
#pragma unroll
        for (int i = 0; i < W; ++i) row[i] = ok ? row[i] : 0.f;
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
    }
    __syncthreads();

    if (active) {
        float *dst = lds + pl * out_plane;
#pragma unroll
        for (int r = 0; r < 2; ++r)
            if (2 * q + r < p.out_h) lds_store_row<OW>(dst + (2 * q + r) * OW, acc[r]);
    }
    __syncthreads();
    lds_to_run(p.out + plane0 * out_plane, lds, nplanes * out_plane);
}

size_t small_lds_bytes(int planes, int in_plane, int out_plane)
{
    return static_cast<size_t>(planes) * (in_plane > out_plane ? in_plane : out_plane) * 4;
}

// Planes per wavefront: as many as there are lane slots, a multiple of 4 when a plane is not a
// multiple of 4 floats (so that every run starts on a 16-byte boundary), within the LDS budget.
int planes_per_run(int lanes_per_plane, int in_plane, int out_plane, long planes)
{
    int P = kWave / lanes_per_plane;
    while (P > 0 && small_lds_bytes(P, in_plane, out_plane) > 16 * 1024) --P;
    if (in_plane % 4 != 0 || out_plane % 4 != 0) P -= P % 4;
    if (static_cast<long>(P) > planes && in_plane % 4 == 0 && out_plane % 4 == 0) P = static_cast<int>(planes);
    return P;
}

template <int W, int K, int S, bool FLIP, int BH>
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
    hipLaunchKernelGGL((small_down_kernel<W, K, S, FLIP, BH>), dim3(static_cast<unsigned>(runs)), dim3(kWave), shmem,
                       stream, p);
    note_variant("small_down<w%d,k%d,s%d,%s,bh%d> P%d", W, K, S, FLIP ? "rot" : "fwd", BH, p.planes_per_run);
    return check_launch("small_down_kernel");
}

template <int W, int K>
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
    hipLaunchKernelGGL((small_up2_kernel<W, K>), dim3(static_cast<unsigned>(runs)), dim3(kWave), shmem, stream, p);
    note_variant("small_up2<w%d,k%d> P%d", W, K, p.planes_per_run);
    return check_launch("small_up2_kernel");
}

template <int W, int K>
int launch_small_down_any(SmallPlan &p, int S, bool rot, hipStream_t stream)
{
    constexpr int BH1 = W == 7 ? 7 : 2;
    if (S == 1) return rot ? launch_small_down<W, K, 1, true, BH1>(p, stream) : launch_small_down<W, K, 1, false, BH1>(p, stream);
    if constexpr (W % 2 == 0) {
        if (S == 2 && !rot) return launch_small_down<W, K, 2, false, 1>(p, stream);
    }
    return -1;
}

template <int W>
int launch_small_down_k(SmallPlan &p, int K, int S, bool rot, hipStream_t stream)
{
    if (K == 3) return launch_small_down_any<W, 3>(p, S, rot, stream);
    if (K == 5) return launch_small_down_any<W, 5>(p, S, rot, stream);
    if (K == 7) return launch_small_down_any<W, 7>(p, S, rot, stream);
    return -1;
}

template <int W>
int launch_small_up2_k(SmallPlan &p, int K, hipStream_t stream)
{
    if (K == 3) return launch_small_up2<W, 3>(p, stream);
    if (K == 5) return launch_small_up2<W, 5>(p, stream);
    if (K == 7) return launch_small_up2<W, 7>(p, stream);
    return -1;
}


// ---- grad-weight ------------------------------------------------------------------------------------
struct SmallWgradPlan {
    const float *x;
    const float *gy;
    float *partial;
    int batch, channel;
    int in_h, out_h;
    int pad_h;
    int planes_per_run;   // channels per wavefront
    int lanes_per_plane;
    unsigned lpp_magic;
    int chunks, images_per_chunk;
};

constexpr int kSmallRedPitch = kWave + 1;

// Wavefront (channel group g, chunk k): for every image of the chunk, the x and gy planes of the
// group's channels are streamed into LDS as two flat runs; a lane holds BH rows of gy of one channel
// and adds gy * x into its K*K register sums.  The lanes of one channel are then summed front to
// back through LDS and stored as partial[c][k][tap]  (sum of torch_dwconv/dwconv_kernel.cu:269-297).
template <int W, int K, int S, int BH>
__global__ __launch_bounds__(kWave) void small_wgrad_kernel(const SmallWgradPlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int OW = (W - 1) / S + 1;
    constexpr int PW = K / 2;
    constexpr int KK = K * K;
    constexpr int WIN_ROWS = (BH - 1) * S + K;

    const int group = blockIdx.x / p.chunks;
    const int chunk = blockIdx.x - group * p.chunks;
    const int c0 = group * p.planes_per_run;
    const int nplanes = min(p.planes_per_run, p.channel - c0);
    const int n0 = chunk * p.images_per_chunk;
    const int n1 = min(p.batch, n0 + p.images_per_chunk);
    const int in_plane = p.in_h * W, out_plane = p.out_h * OW;
    float *lds_x = lds;
    float *lds_g = lds + p.planes_per_run * in_plane;

    const int pl_raw = fast_div(threadIdx.x, p.lpp_magic);
    const int rb = threadIdx.x - pl_raw * p.lanes_per_plane;
    const bool active = pl_raw < nplanes;
    const int pl = active ? pl_raw : 0;
    const int oy0 = rb * BH;

    float acc[KK];
#pragma unroll
    for (int t = 0; t < KK; ++t) acc[t] = 0.f;

    for (int n = n0; n < n1; ++n) {
        const long plane0 = static_cast<long>(n) * p.channel + c0;
        if (n != n0) __syncthreads();
        runs_to_lds(p.x + plane0 * in_plane, lds_x, nplanes * in_plane, p.gy + plane0 * out_plane, lds_g,
                    nplanes * out_plane);
        __syncthreads();

        float g[BH][OW];
#pragma unroll
        for (int b = 0; b < BH; ++b) {
            const bool ok = active && oy0 + b < p.out_h;
            lds_load_row<OW>(lds_g + pl * out_plane + (ok ? oy0 + b : 0) * OW, g[b]);
#pragma unroll
            for (int o = 0; o < OW; ++o) g[b][o] = ok ? g[b][o] : 0.f;
        }
        const float *plane = lds_x + pl * in_plane;
#pragma unroll
        for (int wr = 0; wr < WIN_ROWS; ++wr) {
            const int iy = oy0 * S - p.pad_h + wr;
            const bool ok = static_cast<unsigned>(iy) < static_cast<unsigned>(p.in_h);
            float row[W];
            lds_load_row<W>(plane + (ok ? iy : 0) * W, row);
#pragma unroll
            for (int i = 0; i < W; ++i) row[i] = ok ? row[i] : 0.f;
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
                        acc[ty * K + tx] = fmaf(g[b][o], row[ix], acc[ty * K + tx]);
                    }
            }
        }
    }

    __syncthreads();  // the runs are dead; reuse the LDS to bring the lanes of each channel together
#pragma unroll
    for (int t = 0; t < KK; ++t) lds[t * kSmallRedPitch + threadIdx.x] = acc[t];
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
bool plan_small_wgrad(SmallWgradPlan &p, const WgradGeometry &g)
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
    if (odd && g.channel % 4 != 0) return false;  // runs of every image must start on a 16-byte boundary
    int P = kWave / p.lanes_per_plane;
    if (P > g.channel) P = g.channel;
    while (P > 0 && static_cast<long>(P) * (in_plane + out_plane) * 4 > 32 * 1024) --P;
    if (odd) P -= P % 4;
    if (P < 1) return false;
    p.planes_per_run = P;
    p.lpp_magic = magic_u16(p.lanes_per_plane);
    const int groups = ceil_div(g.channel, P);
    int chunks = ceil_div(env_int("DWCONV_SMALL_WGRAD_WAVES", 4096), groups);
    if (chunks > g.batch) chunks = g.batch;
    if (chunks < 1) chunks = 1;
    p.images_per_chunk = ceil_div(g.batch, chunks);
    p.chunks = ceil_div(g.batch, p.images_per_chunk);
    return true;
}

template <int W, int K, int S, int BH>
size_t small_wgrad_lds(const SmallWgradPlan &p)
{
    constexpr int OW = (W - 1) / S + 1;
    const size_t runs = static_cast<size_t>(p.planes_per_run) * (p.in_h * W + p.out_h * OW) * 4;
    const size_t red = static_cast<size_t>(K) * K * kSmallRedPitch * 4;
    return runs > red ? runs : red;
}

// mode 0: report the workspace bytes; mode 1: launch.  Returns -1 when this family does not cover g.
template <int W, int K, int S, int BH>
long small_wgrad_case(int mode, const float *x, const float *gy, float *gw, void *ws, size_t ws_bytes,
                      const WgradGeometry &g, hipStream_t stream)
{
    SmallWgradPlan p{};
    if (!plan_small_wgrad<W, K, S, BH>(p, g)) return -1;
    const size_t need = static_cast<size_t>(g.channel) * p.chunks * K * K * sizeof(float);
    if (mode == 0) return static_cast<long>(need);
    if (ws == nullptr || ws_bytes < need)
        return fail(DWCONV_ERR_WORKSPACE, "grad-weight needs a workspace of %zu bytes, got %zu", need, ws_bytes);
    p.x = x;
    p.gy = gy;
    p.partial = static_cast<float *>(ws);
    const size_t shmem = small_wgrad_lds<W, K, S, BH>(p);
    const int groups = ceil_div(g.channel, p.planes_per_run);
    hipLaunchKernelGGL((small_wgrad_kernel<W, K, S, BH>), dim3(groups * p.chunks), dim3(kWave), shmem, stream, p);
    int rc = check_launch("small_wgrad_kernel");
    if (rc != DWCONV_OK) return rc;
    note_variant("small_wgrad<w%d,k%d,s%d,bh%d> P%d chunks%d", W, K, S, BH, p.planes_per_run, p.chunks);
    return launch_wgrad_final(p.partial, gw, g.channel, K * K, p.chunks, stream);
}

template <int W, int K>
long small_wgrad_s(int mode, const float *x, const float *gy, float *gw, void *ws, size_t ws_bytes,
                   const WgradGeometry &g, hipStream_t stream)
{
    constexpr int BH1 = W == 7 ? 4 : 2;
    if (g.down_h == 1) return small_wgrad_case<W, K, 1, BH1>(mode, x, gy, gw, ws, ws_bytes, g, stream);
    if constexpr (W % 2 == 0) {
        if (g.down_h == 2) return small_wgrad_case<W, K, 2, 1>(mode, x, gy, gw, ws, ws_bytes, g, stream);
    }
    return -1;
}

template <int W>
long small_wgrad_k(int mode, const float *x, const float *gy, float *gw, void *ws, size_t ws_bytes,
                   const WgradGeometry &g, hipStream_t stream)
{
    if (g.kernel_h == 3) return small_wgrad_s<W, 3>(mode, x, gy, gw, ws, ws_bytes, g, stream);
    if (g.kernel_h == 5) return small_wgrad_s<W, 5>(mode, x, gy, gw, ws, ws_bytes, g, stream);
    if (g.kernel_h == 7) return small_wgrad_s<W, 7>(mode, x, gy, gw, ws, ws_bytes, g, stream);
    return -1;
}

long small_wgrad_any(int mode, const float *x, const float *gy, float *gw, void *ws, size_t ws_bytes,
                     const WgradGeometry &g, hipStream_t stream)
{
    if (env_int("DWCONV_NO_SMALL", 0)) return -1;
    const int K = g.kernel_h, S = g.down_h;
    if (g.kernel_w != K || g.down_w != S || (S != 1 && S != 2)) return -1;
    if (g.pad_w != K / 2 || g.pad_h < 0 || g.pad_h > 7) return -1;
    if (g.in_h < 1 || g.in_h > 64 || g.out_h < 1 || g.out_h > 64) return -1;
    if (g.out_w != (g.in_w - 1) / S + 1) return -1;
    if (mode == 1 && (!aligned16(x) || !aligned16(gy))) return -1;
    if (g.in_w == 7) return small_wgrad_k<7>(mode, x, gy, gw, ws, ws_bytes, g, stream);
    if (g.in_w == 14) return small_wgrad_k<14>(mode, x, gy, gw, ws, ws_bytes, g, stream);
    if (g.in_w == 28) return small_wgrad_k<28>(mode, x, gy, gw, ws, ws_bytes, g, stream);
    return -1;
}

}  // namespace

int try_launch_fir_small(const float *in, const float *taps, float *out, const Geometry &g, hipStream_t stream)
{
    if (env_int("DWCONV_NO_SMALL", 0)) return -1;
    const int K = g.kernel_h;
    if (g.kernel_w != K || (K != 3 && K != 5 && K != 7)) return -1;
    if (!aligned16(in) || !aligned16(out)) return -1;
    if (g.in_h < 1 || g.in_h > 64 || g.out_h < 1 || g.out_h > 128) return -1;
    SmallPlan p{};
    p.in = in;
    p.taps = taps;
    p.out = out;
    p.planes = g.planes();
    p.channel = g.channel;
    p.in_h = g.in_h;
    p.out_h = g.out_h;
    const int W = g.in_w;
    if (g.up_h == 1 && g.up_w == 1 && g.down_h == g.down_w && (g.down_h == 1 || g.down_h == 2)) {
        const int S = g.down_h;
        // full-width rows with the column padding of a "same" convolution
        if (g.pad_w0 != K / 2 || g.out_w != (W - 1) / S + 1) return -1;
        if (g.pad_h0 < 0 || g.pad_h0 > 7) return -1;
        p.pad_h = g.pad_h0;
        if (W == 7) return launch_small_down_k<7>(p, K, S, !g.forward, stream);
        if (W == 14) return launch_small_down_k<14>(p, K, S, !g.forward, stream);
        if (W == 28) return launch_small_down_k<28>(p, K, S, !g.forward, stream);
        return -1;
    }
    if (g.up_h == 2 && g.up_w == 2 && g.down_h == 1 && g.down_w == 1 && !g.forward) {
        if (g.pad_w0 != K / 2 || g.pad_h0 != K / 2 || g.out_w != 2 * W) return -1;
        const int E = (K / 2) & 1;
        p.pad_h = (K / 2 + E) / 2;
        if (W == 7) return launch_small_up2_k<7>(p, K, stream);
        if (W == 14) return launch_small_up2_k<14>(p, K, stream);
        return -1;
    }
    return -1;
}

}  // namespace dwconv

namespace dwconv {

size_t wgrad_small_workspace(const WgradGeometry &g)
{
    const long n = small_wgrad_any(0, nullptr, nullptr, nullptr, nullptr, 0, g, nullptr);
    return n > 0 ? static_cast<size_t>(n) : 0;
}

int try_launch_wgrad_small(const float *in, const float *gy, float *gw, void *ws, size_t ws_bytes,
                           const WgradGeometry &g, hipStream_t stream)
{
    return static_cast<int>(small_wgrad_any(1, in, gy, gw, ws, ws_bytes, g, stream));
}

}  // namespace dwconv
