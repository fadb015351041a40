// Helpers shared by the whole-plane kernels for small feature maps: LDS rows of a
// compile-time width (or capacity) and flat runs of planes between global memory and LDS.
#pragma once

#include "dwconv_tile_common.hpp"

namespace dwconv {

constexpr int kWave = 64;

// ---- plans and per-width entry points ---------------------------------------------------------------------
// Width instances of the whole-plane kernels: exact widths, and ragged capacity classes for every other width.
// Each instance is its own translation unit (dwconv_small_width.hip); the dispatchers call them through the
// function templates declared below.
#define DWCONV_SMALL_EXACT_WIDTHS(X) X(6) X(7) X(8) X(9) X(10) X(12) X(14) X(15) X(16) X(18) X(20) X(24) X(28) X(30) X(32)
#define DWCONV_SMALL_RAGGED_WIDTHS(X) X(8) X(16) X(24) X(32)

inline bool small_width_is_exact(int w)
{
    switch (w) {
#define DWCONV_CASE(WV) case WV:
        DWCONV_SMALL_EXACT_WIDTHS(DWCONV_CASE)
#undef DWCONV_CASE
        return true;
    default:
        return false;
    }
}
// capacity class of a width that has no exact instance; 0 when it is too wide for this family
inline int small_ragged_class(int w) { return w < 1 || w > 32 ? 0 : (w + 7) / 8 * 8; }

struct SmallPlan {
    const void *in;    // element type IO of the kernel template
    const void *taps;
    void *out;
    long planes;
    int channel;
    int in_h, out_h;
    int in_w, out_w;       // real widths (the kernels of an exact instance use their template constant)
    int pad_h;             // leading zero rows (down) or m = (pad0 + E) / 2 (up2)
    int planes_per_run;    // P
    int lanes_per_plane;   // LPP
    unsigned lpp_magic;
    int zero_off;          // float offset of the row of zeros in LDS (a multiple of four)
    int lp_in, lp_out;     // ragged instances: LDS row pitch of the input / output rows (width | 1)
    unsigned magic_in, magic_out;  // ... and the reciprocals for padded_index (0: pitch == width, flat copies)
    Epilogue epi;          // forward kernels: applied to every sum before it is stored
};

// Launches the forward / grad-input kernel of width instance (W, RAG) for p: K in {3,5,7}; up2 = false: decimation
// S in {1,2}, taps rotated if `rot`, dilation D (2 only for 3x3 / 5x5 forward at stride 1); up2 = true: the
// transposed stride-2 problem.  -1 when the instance does not cover the case.
template <int W, bool RAG, typename IO>
int small_fir_width(SmallPlan &p, int K, int S, int D, bool rot, bool up2, hipStream_t stream);

struct SmallBwdArgs {
    const void *x;    // element type IO
    const void *gy;
    const void *taps;
    void *gx;
    void *gw;
    void *ws;
    size_t ws_bytes;
};

// mode 0: workspace bytes of the grad-weight partial sums; mode 1: grad-weight; mode 2: grad-weight + grad-input.
// Returns -1 when the instance does not cover g, a dwconv_status otherwise (mode 0: the byte count).
template <int W, bool RAG, typename IO>
long small_bwd_width(int mode, const SmallBwdArgs &a, const WgradGeometry &g, hipStream_t stream);

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

// Width-aware forms.  RAG = false: the row is exactly N elements.  RAG = true: N is a capacity and the real width
// (N - 7 .. N, uniform) comes at run time: a row starts anywhere, so it is read element by element, up to N - 1 floats
// past its end (the LDS allocation of a ragged kernel ends with N spare floats), and what was read past the real
// width is replaced by zero (a select under a wavefront-uniform condition, and only for the last seven columns:
// a capacity class spans eight widths).
//
// Rows above or below the plane are not masked element by element: every kernel keeps a row of zeros in LDS
// (zero_row_floats(W) floats, cleared by clear_zero_row) and points the read at it instead, one select on the address.
template <int N, bool RAG>
__device__ __forceinline__ void lds_load_row_w(const float *p, float (&r)[N], int w)
{
    if constexpr (RAG) {
#pragma unroll
        for (int i = 0; i < N; ++i) r[i] = p[i];
#pragma unroll
        for (int i = (N > 7 ? N - 7 : 0); i < N; ++i) r[i] = i < w ? r[i] : 0.f;
    } else {
        lds_load_row<N>(p, r);
    }
}

constexpr int zero_row_floats(int w) { return (w + 3) / 4 * 4 + 8; }

// LDS pitch of a row of n elements.  Lanes sit one or a few rows apart; rows of 8, 16 or 32 floats put them a power
// of two apart and onto two or four of the 64 banks (row reads of a 32 x 32 plane then take eight times their
// conflict-free time, and the LDS, not the vector unit, bounds the kernel), so exact instances give such rows four
// spare floats: lane strides of 12, 20 and 36 floats spread 128-bit reads over all banks.  The flat copies between
// memory and LDS then skip one group of four after every n / 4 (a shift: lds_group below).  Ragged rows of an
// even width (lanes a row apart would meet on 32 / gcd(width, 64) banks with their element reads: a 24-wide map ran
// at half the speed of a 28-wide one) are laid out at pitch width + 1: the copies between memory and LDS then go
// element by element (row = index * magic >> 18, see padded_index); odd widths keep the flat copy.
constexpr int lds_row_pitch(int n, bool rag) { return (!rag && (n == 8 || n == 16 || n == 32)) ? n + 4 : n; }
// groups of four per memory row when the LDS rows are padded, else 0
constexpr int lds_row_groups(int n, bool rag) { return lds_row_pitch(n, rag) != n ? n / 4 : 0; }

// LDS group index of group i of a flat run; GPR = groups of four per row where rows are padded (a power of two), else 0
template <int GPR>
__device__ __forceinline__ int lds_group(int i)
{
    if constexpr (GPR == 0) return i;
    else return i + i / GPR;
}

// LDS pitch of ragged rows of w elements, and the reciprocal that finds the row of a flat index (0: no padding)
// (from 10 columns on: on 6-wide maps the element-wise copies cost more than the conflicts, 14.1 -> 16.2 us forward
// and 25.4 -> 30.3 backward at C=1152; 12-wide maps gain 15-25 %, 24-wide ones 45 %)
inline bool ragged_padded(int w) { return (w & 1) == 0 && w >= 10; }
inline int ragged_pitch(int w) { return ragged_padded(w) ? w + 1 : w; }
inline unsigned ragged_magic(int w) { return ragged_padded(w) ? static_cast<unsigned>(((1u << 18) + w - 1) / w) : 0u; }
// LDS index of element i (0 <= i < 8192) of a flat run of rows laid out at pitch width + 1
__device__ __forceinline__ int padded_index(int i, unsigned magic) { return i + static_cast<int>(__umul24(i, magic) >> 18); }

template <int W>
__device__ __forceinline__ void clear_zero_row(float *zrow)
{
    static_assert(zero_row_floats(W) / 4 <= kWave, "one float4 per lane");
    if (threadIdx.x < zero_row_floats(W) / 4) reinterpret_cast<float4 *>(zrow)[threadIdx.x] = make_float4(0.f, 0.f, 0.f, 0.f);
}

template <int N, bool RAG>
__device__ __forceinline__ void lds_store_row_w(float *p, const float *r, int w)
{
    if constexpr (RAG) {
#pragma unroll
        for (int i = 0; i < N; ++i)
            if (i < w) p[i] = r[i];
    } else {
        lds_store_row<N>(p, r);
    }
}

// ---- flat runs between global memory and LDS ---------------------------------------------------
// `g` is aligned to four elements; n elements; the last partial group of four (only at the very end of a
// tensor) goes scalar.  LDS always holds fp32.
// Loads are issued kRunBatch at a time before any of them is consumed, so their latencies overlap.
constexpr int kRunBatch = 8;

template <typename IO, int GPR = 0>
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
        for (int u = 0; u < kRunBatch; ++u) reinterpret_cast<float4 *>(lds)[lds_group<GPR>(min(base + u * kWave, n4 - 1))] = v[u];
    }
    // (a run with padded rows is whole groups of four)
    const int tail = n4 * 4 + threadIdx.x;
    if (GPR == 0 && tail < n) lds[tail] = Io<IO>::in(g[tail]);
}

// The same for rows at pitch width + 1 in LDS (ragged even widths): element i of the run proper (the span minus its
// `head` elements of the neighbouring run, which go to the spare float at `dump`) lands at padded_index(i).
template <typename IO>
__device__ __forceinline__ void run_to_lds_rows(const IO *__restrict__ g, float *lds, int n, int head, unsigned magic, int dump)
{
    const int n4 = n >> 2;
    for (int base = threadIdx.x; base < n4; base += kWave * kRunBatch) {
        float4 v[kRunBatch];
#pragma unroll
        for (int u = 0; u < kRunBatch; ++u)
            v[u] = load4<IO>(g + 4 * min(base + u * kWave, n4 - 1));
#pragma unroll
        for (int u = 0; u < kRunBatch; ++u) {
            const int i = 4 * min(base + u * kWave, n4 - 1) - head;
            lds[i >= 0 ? padded_index(i, magic) : dump] = v[u].x;
            lds[i + 1 >= 0 ? padded_index(i + 1, magic) : dump] = v[u].y;
            lds[i + 2 >= 0 ? padded_index(i + 2, magic) : dump] = v[u].z;
            lds[padded_index(i + 3, magic)] = v[u].w;
        }
    }
    const int tail = n4 * 4 + threadIdx.x;
    if (tail < n && tail >= head) lds[padded_index(tail - head, magic)] = Io<IO>::in(g[tail]);
}

template <typename IO>
__device__ __forceinline__ void lds_to_run_rows(IO *__restrict__ g, const float *lds, int n, int head, unsigned magic)
{
    const int n4 = n >> 2;
    constexpr int U = 4;
    const __amdgpu_buffer_rsrc_t view = buffer_view(g, static_cast<long>(n) * sizeof(IO));
    for (int base = threadIdx.x; base < n4; base += kWave * U) {
        float4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = 4 * min(base + u * kWave, n4 - 1) - head;
            v[u].x = lds[padded_index(max(i, 0), magic)];
            v[u].y = lds[padded_index(max(i + 1, 0), magic)];
            v[u].z = lds[padded_index(max(i + 2, 0), magic)];
            v[u].w = lds[padded_index(i + 3, magic)];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = base + u * kWave;
            const bool whole = i < n4 && (i > 0 || head == 0);
            view_store4<IO>(view, whole ? i * 4u * static_cast<unsigned>(sizeof(IO)) : kOob, v[u].x, v[u].y, v[u].z, v[u].w);
        }
    }
    const int t = threadIdx.x;
    if (head != 0 && n4 > 0 && t >= head && t < 4) g[t] = Io<IO>::out(lds[padded_index(t - head, magic)]);
    const int tail = n4 * 4 + t;
    if (tail < n && tail >= head) g[tail] = Io<IO>::out(lds[padded_index(tail - head, magic)]);
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

// A run that starts `head` elements (1..3) past a 4-element boundary is moved as the aligned span that contains it:
// `g` points at that boundary, `n` counts the head too, and the run's first element sits at lds[head].  Loading such a
// span reads up to three elements of the neighbouring run (harmless); storing it must not write them: the first
// group of four goes out element by element, from `head` on.
template <typename IO, int GPR = 0>
__device__ __forceinline__ void lds_to_run(IO *__restrict__ g, const float *lds, int n, int head = 0)
{
    const int n4 = n >> 2;
    constexpr int U = 4;
    const __amdgpu_buffer_rsrc_t view = buffer_view(g, static_cast<long>(n) * sizeof(IO));  // g is uniform: one run per wavefront
    for (int base = threadIdx.x; base < n4; base += kWave * U) {
        float4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = reinterpret_cast<const float4 *>(lds)[lds_group<GPR>(min(base + u * kWave, n4 - 1))];
        // branch-free: groups past the end of the run store out of range of the view and are dropped
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = base + u * kWave;
            const bool whole = i < n4 && (i > 0 || head == 0);
            view_store4<IO>(view, whole ? i * 4u * static_cast<unsigned>(sizeof(IO)) : kOob, v[u].x, v[u].y, v[u].z, v[u].w);
        }
    }
    if constexpr (GPR == 0) {
        const int t = threadIdx.x;
        if (head != 0 && n4 > 0 && t >= head && t < 4) g[t] = Io<IO>::out(lds[t]);
        const int tail = n4 * 4 + t;
        if (tail < n && tail >= head) g[tail] = Io<IO>::out(lds[tail]);
    }
}

// This lane's K*K taps straight from global memory (the lanes of one plane read the same addresses).
template <int KK, bool FLIP, typename IO>
__device__ __forceinline__ void load_taps(const IO *__restrict__ taps, int c, float (&t)[KK])
{
#pragma unroll
    for (int i = 0; i < KK; ++i) t[i] = Io<IO>::in(taps[c * KK + (FLIP ? KK - 1 - i : i)]);
}

}  // namespace dwconv
