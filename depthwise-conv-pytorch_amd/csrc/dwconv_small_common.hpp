// Helpers shared by the whole-plane kernels for small feature maps: LDS rows of a
// compile-time width and flat runs of planes between global memory and LDS.
#pragma once

#include "dwconv_tile_common.hpp"

namespace dwconv {

constexpr int kWave = 64;

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
// `g` is aligned to four elements; n elements; the last partial group of four (only at the very end of a
// tensor) goes scalar.  LDS always holds fp32.
// Loads are issued kRunBatch at a time before any of them is consumed, so their latencies overlap.
constexpr int kRunBatch = 8;

template <typename IO>
__device__ __forceinline__ void run_to_lds(const IO *__restrict__ g, float *lds, int n)
{
    const int n4 = n >> 2;
    for (int base = threadIdx.x; base < n4; base += kWave * kRunBatch) {
        float4 v[kRunBatch];
        // slots past the end of the run re-read its last group of four and write it to the same place again:
        // no branch around either access
#pragma unroll
        for (int u = 0; u < kRunBatch; ++u)
            v[u] = load4<IO>(g + 4 * min(base + u * kWave, n4 - 1));
#pragma unroll
        for (int u = 0; u < kRunBatch; ++u) reinterpret_cast<float4 *>(lds)[min(base + u * kWave, n4 - 1)] = v[u];
    }
    const int tail = n4 * 4 + threadIdx.x;
    if (tail < n) lds[tail] = Io<IO>::in(g[tail]);
}

// Two runs at once (grad-weight: x and gy of the same planes): all loads of a batch of both runs fly together.
template <typename IO>
__device__ __forceinline__ void runs_to_lds(const IO *__restrict__ ga, float *la, int na,
                                            const IO *__restrict__ gb, float *lb, int nb)
{
    const int na4 = na >> 2, nb4 = nb >> 2;
    const int nmax = na4 > nb4 ? na4 : nb4;
    constexpr int U = kRunBatch / 2;
    for (int base = threadIdx.x; base < nmax; base += kWave * U) {
        float4 va[U], vb[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            va[u] = load4<IO>(ga + 4 * min(base + u * kWave, na4 - 1));
            vb[u] = load4<IO>(gb + 4 * min(base + u * kWave, nb4 - 1));
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            reinterpret_cast<float4 *>(la)[min(base + u * kWave, na4 - 1)] = va[u];
            reinterpret_cast<float4 *>(lb)[min(base + u * kWave, nb4 - 1)] = vb[u];
        }
    }
    const int ta = na4 * 4 + threadIdx.x, tb = nb4 * 4 + threadIdx.x;
    if (ta < na) la[ta] = Io<IO>::in(ga[ta]);
    if (tb < nb) lb[tb] = Io<IO>::in(gb[tb]);
}

template <typename IO>
__device__ __forceinline__ void lds_to_run(IO *__restrict__ g, const float *lds, int n)
{
    const int n4 = n >> 2;
    constexpr int U = 4;
    const __amdgpu_buffer_rsrc_t view = buffer_view(g, static_cast<long>(n) * sizeof(IO));  // g is uniform: one run per wavefront
    for (int base = threadIdx.x; base < n4; base += kWave * U) {
        float4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = reinterpret_cast<const float4 *>(lds)[min(base + u * kWave, n4 - 1)];
        // branch-free: groups past the end of the run store out of range of the view and are dropped
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = base + u * kWave;
            view_store4<IO>(view, i < n4 ? i * 4u * static_cast<unsigned>(sizeof(IO)) : kOob, v[u].x, v[u].y, v[u].z, v[u].w);
        }
    }
    const int tail = n4 * 4 + threadIdx.x;
    if (tail < n) g[tail] = Io<IO>::out(lds[tail]);
}

// This lane's K*K taps straight from global memory (the lanes of one plane read the same addresses).
template <int KK, bool FLIP, typename IO>
__device__ __forceinline__ void load_taps(const IO *__restrict__ taps, int c, float (&t)[KK])
{
#pragma unroll
    for (int i = 0; i < KK; ++i) t[i] = Io<IO>::in(taps[c * KK + (FLIP ? KK - 1 - i : i)]);
}

}  // namespace dwconv
