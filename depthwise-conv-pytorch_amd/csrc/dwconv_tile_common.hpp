// Device and host helpers shared by the LDS-tiled kernels (forward/grad-input
// and grad-weight): the LDS image of a band of input rows and how it is filled.
#pragma once

#include "dwconv_common.hpp"

#include <cstdlib>
#include <type_traits>

namespace dwconv {

constexpr int kThreads = 256;           // lanes per workgroup (4 wavefronts)
constexpr int kSlack = 4;               // spare floats on both sides of every LDS row
constexpr int kLdsBudget = 48 * 1024;   // bytes of LDS one tile may take
constexpr int kXcds = 8;
constexpr int kCus = 256;                 // compute units of an MI355X

// The LDS image of a tile: `planes` images of `lds_rows` rows of `pitch` floats.
// Row r, column c (after the slack) of an image holds input row iy0 + r, column c - col_shift,
// or zero where that falls outside the plane.
struct StageLayout {
    int in_h, in_w, in_plane;
    int col_shift;
    int lds_rows;
    unsigned lds_rows_magic;
    int g_lo;   // first (possibly negative) float4 column fetched per row
    int spr;    // float4 slots per row
    unsigned spr_magic;
    int pitch;        // floats per LDS row, slack included
    int plane_pitch;  // floats per plane image
    int vec_in;       // 0: element loads; 1: four elements per load (in_w % 4 == 0, base aligned to four elements);
                      // 2: the same through a buffer view (the tile's planes span less than kOob bytes);
                      // 3: through a view with rows of any width at any element alignment: a slot's load starts
                      //    on an element boundary only, and what it reads past the end of its row is zeroed
};

// Four consecutive elements (aligned to four elements) as fp32, and back.
template <typename IO>
__device__ __forceinline__ float4 load4(const IO *p);
template <>
__device__ __forceinline__ float4 load4<float>(const float *p)
{
    return *reinterpret_cast<const float4 *>(p);
}
template <>
__device__ __forceinline__ float4 load4<half_t>(const half_t *p)
{
    const uint2 raw = *reinterpret_cast<const uint2 *>(p);
    union { uint32_t u; half_t h[2]; } a, b;
    a.u = raw.x;
    b.u = raw.y;
    return make_float4(static_cast<float>(a.h[0]), static_cast<float>(a.h[1]), static_cast<float>(b.h[0]),
                       static_cast<float>(b.h[1]));
}
template <>
__device__ __forceinline__ float4 load4<bf16_t>(const bf16_t *p)
{
    const uint2 raw = *reinterpret_cast<const uint2 *>(p);
    return make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u), __uint_as_float(raw.y << 16),
                       __uint_as_float(raw.y & 0xffff0000u));
}

template <typename IO>
__device__ __forceinline__ void store4(IO *p, float a, float b, float c, float d);
template <>
__device__ __forceinline__ void store4<float>(float *p, float a, float b, float c, float d)
{
    *reinterpret_cast<float4 *>(p) = make_float4(a, b, c, d);
}
template <>
__device__ __forceinline__ void store4<half_t>(half_t *p, float a, float b, float c, float d)
{
    *reinterpret_cast<uint2 *>(p) = make_uint2(f16_pack2(a, b), f16_pack2(c, d));
}
template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t *p, float a, float b, float c, float d)
{
    *reinterpret_cast<uint2 *>(p) = make_uint2(bf16_pack2(a, b), bf16_pack2(c, d));
}

// The same four elements as loaded, not yet widened: half the registers for the 16-bit types.
template <typename IO>
struct Raw4 {
    using type = float4;
};
template <>
struct Raw4<half_t> {
    using type = uint2;
};
template <>
struct Raw4<bf16_t> {
    using type = uint2;
};
template <typename IO>
__device__ __forceinline__ typename Raw4<IO>::type load4_raw(const IO *p)
{
    return *reinterpret_cast<const typename Raw4<IO>::type *>(p);
}
template <typename IO>
__device__ __forceinline__ float4 widen4(const typename Raw4<IO>::type &raw);
template <>
__device__ __forceinline__ float4 widen4<float>(const float4 &raw)
{
    return raw;
}
template <>
__device__ __forceinline__ float4 widen4<half_t>(const uint2 &raw)
{
    union { uint32_t u; half_t h[2]; } a, b;
    a.u = raw.x;
    b.u = raw.y;
    return make_float4(static_cast<float>(a.h[0]), static_cast<float>(a.h[1]), static_cast<float>(b.h[0]),
                       static_cast<float>(b.h[1]));
}
template <>
__device__ __forceinline__ float4 widen4<bf16_t>(const uint2 &raw)
{
    return make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u), __uint_as_float(raw.y << 16),
                       __uint_as_float(raw.y & 0xffff0000u));
}

// ---- loads through a buffer view ------------------------------------------------------------------------------
// A raw buffer view of `bytes` bytes from `base` (both uniform): what the workgroup may really touch there.  A load
// whose byte offset is at or beyond the extent returns zeros and a store there is dropped, so an element outside the
// image needs no branch and no select: its offset is replaced by kOob, which is beyond every extent (extents are
// clamped to kOob; the planners keep every real offset below it).  Because the extent is the real span and not a
// blanket 2 GiB, an index slip in a kernel reads zeros or writes nothing instead of touching a neighbouring allocation.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
constexpr unsigned kOob = 0x80000000u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_view(const void *base, long bytes)
{
    const unsigned extent = bytes < static_cast<long>(kOob) ? static_cast<unsigned>(bytes) : kOob;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, extent, 0x00020000);
}

// CV consecutive elements at byte offset `off` of the view, widened to fp32.
template <typename IO, int CV>
__device__ __forceinline__ void view_load(__amdgpu_buffer_rsrc_t view, unsigned off, float (&v)[CV])
{
    if constexpr (CV * sizeof(IO) == 16) {
        const u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(view, off, 0, 0);
        v[0] = __uint_as_float(t.x); v[1] = __uint_as_float(t.y); v[2] = __uint_as_float(t.z); v[3] = __uint_as_float(t.w);
    } else if constexpr (CV * sizeof(IO) == 8) {
        const u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(view, off, 0, 0);
        if constexpr (sizeof(IO) == 4) {
            v[0] = __uint_as_float(t.x); v[1] = __uint_as_float(t.y);
        } else {
            const float4 w = widen4<IO>(make_uint2(t.x, t.y));
            v[0] = w.x; v[1] = w.y; v[2] = w.z; v[3] = w.w;
        }
    } else if constexpr (CV == 1) {
        static_assert(sizeof(IO) == 4, "a single element per lane is an fp32 one");
        v[0] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(view, off, 0, 0));
    } else {
        static_assert(CV == 2 && sizeof(IO) == 2, "two 16-bit elements");
        const unsigned t = __builtin_amdgcn_raw_buffer_load_b32(view, off, 0, 0);
        const float4 w = widen4<IO>(make_uint2(t, 0u));
        v[0] = w.x; v[1] = w.y;
    }
}
template <typename IO>
__device__ __forceinline__ float4 view_load4(__amdgpu_buffer_rsrc_t view, unsigned off)
{
    float v[4];
    view_load<IO, 4>(view, off, v);
    return make_float4(v[0], v[1], v[2], v[3]);
}

// Cache policy of result stores: non-temporal (the `nt` bit).  Results are written once and not read again by
// the kernel that makes them; as ordinary stores they sit dirty in the L2 / Infinity Cache until the reads of a
// later kernel push them out.  Streaming them took 2-8 % off every workload measured (both layouts, all element
// types); `sc0` alone changed nothing and `sc1 nt` was slower.
constexpr int kStoreTemporal = 0, kStoreStreaming = 2;

// Four results as elements at byte offset `off` of the view; dropped when `off` is at or beyond kOob.
template <typename IO, int POLICY = kStoreStreaming>
__device__ __forceinline__ void view_store4(__amdgpu_buffer_rsrc_t view, unsigned off, float a, float b, float c, float d)
{
    if constexpr (sizeof(IO) == 4) {
        u32x4 t;
        t.x = __float_as_uint(a); t.y = __float_as_uint(b); t.z = __float_as_uint(c); t.w = __float_as_uint(d);
        __builtin_amdgcn_raw_buffer_store_b128(t, view, off, 0, POLICY);
    } else {
        u32x2 t;
        if constexpr (std::is_same<IO, bf16_t>::value) {
            t.x = bf16_pack2(a, b); t.y = bf16_pack2(c, d);
        } else {
            t.x = f16_pack2(a, b); t.y = f16_pack2(c, d);
        }
        __builtin_amdgcn_raw_buffer_store_b64(t, view, off, 0, POLICY);
    }
}

// Two results as elements at byte offset `off` of the view; dropped when `off` is at or beyond kOob.
template <typename IO, int POLICY = kStoreStreaming>
__device__ __forceinline__ void view_store2(__amdgpu_buffer_rsrc_t view, unsigned off, float a, float b)
{
    if constexpr (sizeof(IO) == 4) {
        u32x2 t;
        t.x = __float_as_uint(a); t.y = __float_as_uint(b);
        __builtin_amdgcn_raw_buffer_store_b64(t, view, off, 0, POLICY);
    } else {
        unsigned t;
        if constexpr (std::is_same<IO, bf16_t>::value) t = bf16_pack2(a, b);
        else t = f16_pack2(a, b);
        __builtin_amdgcn_raw_buffer_store_b32(t, view, off, 0, POLICY);
    }
}

// One fp32 result at byte offset `off` of the view; dropped when `off` is at or beyond the extent.
template <typename IO, int POLICY = kStoreStreaming>
__device__ __forceinline__ void view_store1(__amdgpu_buffer_rsrc_t view, unsigned off, float a)
{
    static_assert(sizeof(IO) == 4, "a single element per lane is an fp32 one");
    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(a), view, off, 0, POLICY);
}

// A block of four results at byte offset `off`, which need only be a multiple of 4 bytes, of a row whose width leaves
// `rem` = width % 4 elements (uniform) to its last block: `n` is what is left of the row from the block's first column
// on, so n >= 4 for a whole block (one 128-bit store; 64 bits for 16-bit elements) and n == rem for the last one (a
// 64-bit and / or a 32-bit store; 16-bit elements, whose rows are even here: a 32-bit store).  Branch-free per lane: the
// stores that do not apply to a lane go out of range; the ones no lane needs are skipped under the uniform `rem`.
// Dropped when `off` is at or beyond kOob.  (16-bit tensors with rows that start 2 bytes past a 32-bit boundary do not
// come here: stored as 16 + 32 + 16 bits they measured slower than element by element.)
template <typename IO, int POLICY = kStoreStreaming>
__device__ __forceinline__ void view_store_first(__amdgpu_buffer_rsrc_t view, unsigned off, int n, int rem, float a, float b, float c,
                                                 float d)
{
    const bool tail = off < kOob && n < 4;
    view_store4<IO, POLICY>(view, n >= 4 ? off : kOob, a, b, c, d);
    if (rem & 2) view_store2<IO, POLICY>(view, tail ? off : kOob, a, b);
    if constexpr (sizeof(IO) == 4) {
        if (rem & 1) view_store1<IO, POLICY>(view, tail ? off + (rem == 3 ? 8u : 0u) : kOob, rem == 3 ? c : a);
    }
}

// Whether some row of a 16-bit tensor `width` elements wide that starts at `base` begins 2 bytes past a 32-bit boundary.
template <typename IO>
__device__ __forceinline__ bool mixed_row_starts(const IO *base, int width)
{
    return sizeof(IO) == 2 && ((width & 1) != 0 || (reinterpret_cast<uintptr_t>(base) & 2) != 0);
}

// Zeroes what a four-element load read past the `n` elements that were left of its row.
__device__ __forceinline__ void keep_first(float4 &v, int n)
{
    v.y = n > 1 ? v.y : 0.f;
    v.z = n > 2 ? v.z : 0.f;
    v.w = n > 3 ? v.w : 0.f;
}

// Views for rows of any width (vec_in == 3).  fp32: the plain view.  16 bits: every load must start on a 32-bit boundary,
// so the view starts at the boundary at or before `base` and ends at the one at or after the last byte (at most two
// bytes of the neighbouring planes, or of the allocation's own padding, on either side); `bias` is what a byte offset
// relative to `base` is increased by.
struct AnyWidthView {
    __amdgpu_buffer_rsrc_t view;
    unsigned bias;
};
template <typename IO>
__device__ __forceinline__ AnyWidthView any_width_view(const IO *base, long bytes)
{
    AnyWidthView v;
    if constexpr (sizeof(IO) == 4) {
        v.bias = 0;
        v.view = buffer_view(base, bytes);
    } else {
        v.bias = static_cast<unsigned>(reinterpret_cast<uintptr_t>(base) & 2);
        v.view = buffer_view(reinterpret_cast<const char *>(base) - v.bias, (bytes + v.bias + 3) & ~3l);
    }
    return v;
}
// Four consecutive elements at byte offset `off` (relative to the view's tensor; kOob: zeros) as fp32.  16 bits: three
// aligned dwords and two funnel shifts when the elements start in the middle of a dword.
template <typename IO>
__device__ __forceinline__ float4 any_width_load4(const AnyWidthView &v, unsigned off)
{
    if constexpr (sizeof(IO) == 4) {
        return view_load4<IO>(v.view, off);
    } else {
        typedef unsigned int u32x3 __attribute__((ext_vector_type(3)));
        const unsigned at = off < kOob ? off + v.bias : kOob;
        const u32x3 d = __builtin_amdgcn_raw_buffer_load_b96(v.view, at & ~3u, 0, 0);
        const unsigned sh = (at & 2u) << 3;
        return widen4<IO>(make_uint2(__builtin_amdgcn_alignbit(d.y, d.x, sh), __builtin_amdgcn_alignbit(d.z, d.y, sh)));
    }
}

// True when groups of four elements starting at `p` may be moved with one vector access.
template <typename IO>
inline bool aligned4(const IO *p)
{
    return (reinterpret_cast<uintptr_t>(p) & (4 * sizeof(IO) - 1)) == 0;
}

// n / d through the reciprocal made by magic_u16(d); a zero reciprocal stands for d == 1.
__device__ __forceinline__ int fast_div(int n, unsigned magic)
{
    return magic ? static_cast<int>(__umulhi(static_cast<unsigned>(n), magic)) : n;
}

// Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.
// Give every XCD a contiguous run of tiles so that the row bands of one plane,
// which share halo rows, meet in the same L2.
__device__ __forceinline__ int xcd_contiguous_tile(int bid, int n_tiles)
{
    const int per = n_tiles / kXcds, rem = n_tiles - per * kXcds;
    const int xcd = bid % kXcds, k = bid / kXcds;
    return xcd * per + min(xcd, rem) + k;
}

// Fills the LDS image of the tile: every float4 slot of every row is written,
// with zeros where the row or the columns fall outside the plane.  A lane issues
// the global loads of kStageBatch slots before it consumes any of them, so that
// their latencies overlap instead of adding up.
constexpr int kStageBatch = 4;

// VIEW_ONLY: the caller guarantees s.vec_in == 2, and the other two ways of loading are not compiled in.  The
// kernels keep an instance of each kind: with every alternative in one body, the values the unused ones need
// stay live and push the scalar registers past what the hardware has.
// BATCH: loads a lane has in flight at a time (kStageBatch unless a kernel measured better with another number).
// BY_ROWS: the view path walks rows per lane instead of linear slots (see there).  It needs fewer vector instructions
// and more registers: the forward kernels, which stage once, gain a few per cent from it (up to 10 % with 7x7
// filters); the backward kernels, which stage two images per chunk, lose a wavefront of occupancy and 2-8 %.
// ANY_WIDTH: vec_in == 3 (rows of any width) is looked for at run time; kernels that keep an instance of their own for
// such rows switch it off in the other one, which then carries none of it.
template <typename IO, bool VIEW_ONLY = false, int BATCH = kStageBatch, bool BY_ROWS = false, bool ANY_WIDTH = true>
__device__ __forceinline__ void stage_tile(const StageLayout &s, const IO *__restrict__ in, float *lds,
                                           long plane0, int nplanes, int iy0)
{
    constexpr int kStageBatch = BATCH;  // shadows the default within this function
    const int total = nplanes * s.lds_rows * s.spr;
    if (VIEW_ONLY || s.vec_in == 2 || (ANY_WIDTH && s.vec_in == 3)) {
        // (rows of any width, vec_in == 3: see StageLayout)
        const bool ragged = ANY_WIDTH && !VIEW_ONLY && s.vec_in == 3;
        // groups of four elements through a view of the tile's planes: slots outside the image read zeros
        const __amdgpu_buffer_rsrc_t view = buffer_view(in + plane0 * s.in_plane, static_cast<long>(nplanes) * s.in_plane * sizeof(IO));
        // (16-bit rows that do not all start on 32-bit boundaries are loaded from such boundaries: see any_width_view)
        AnyWidthView wide{view, 0};
        bool split = false;
        if constexpr (sizeof(IO) == 2 && ANY_WIDTH && !VIEW_ONLY) {
            split = ragged && mixed_row_starts(in + plane0 * s.in_plane, s.in_w);
            if (split) wide = any_width_view(in + plane0 * s.in_plane, static_cast<long>(nplanes) * s.in_plane * sizeof(IO));
        }
        auto load_slot = [&](unsigned off) -> float4 {
            if constexpr (sizeof(IO) == 2 && ANY_WIDTH && !VIEW_ONLY) {
                if (split) return any_width_load4<IO>(wide, off);
            }
            return view_load4<IO>(view, off);
        };
        if constexpr (BY_ROWS) {
            // A lane owns one float4 column and every rpp-th row: column, column check and the LDS column are
            // computed once, and per slot only the row moves (two additions, a range check, a select), where the
            // linear slot order below pays two divisions and four multiplies per slot.  Lanes beyond rpp whole
            // rows idle (none when the slots per row divide the workgroup).
            constexpr unsigned ES = sizeof(IO);
            const int nthreads = blockDim.x;
            const int rpp_raw = s.spr > 1 ? fast_div(nthreads, s.spr_magic) : nthreads;
            const int rpp = max(rpp_raw, 1);
            const int col_step = rpp_raw ? s.spr : nthreads;   // one trip unless a row has more slots than lanes
            const int rl = fast_div(threadIdx.x, s.spr_magic);
            const int total_rows = nplanes * s.lds_rows;
            if (rl >= rpp) return;
            for (int sc = threadIdx.x - __mul24(rl, s.spr); sc < s.spr; sc += col_step) {
                const int ix = 4 * (s.g_lo + sc);
                const bool col_ok = static_cast<unsigned>(ix) < static_cast<unsigned>(s.in_w);
                const int dcol = kSlack + ix + s.col_shift;
                const int left = s.in_w - ix;  // elements of the row from this column on
                if (nplanes == 1) {
                    // rows of the image that exist in the plane: [lo, lo + span)
                    const int lo = max(iy0, 0);
                    const unsigned span = static_cast<unsigned>(max(min(s.in_h, iy0 + s.lds_rows) - lo, 0));
                    const unsigned off_step = __mul24(rpp, s.in_w) * ES;
                    const int dst_step = __mul24(rpp, s.pitch);
                    int iy = iy0 + rl;
                    unsigned off = (__mul24(iy, s.in_w) + ix) * ES;
                    int dst = __mul24(rl, s.pitch) + dcol;
                    // whole batches first (the bound is uniform, so every store is unconditional), then one batch whose
                    // rows past the image go to the dump slot.  A store under a per-lane condition would drag its load
                    // into the conditional block, behind the other loads' wait.
                    const int dump = s.plane_pitch - 4;
                    int rb = 0;
                    for (; rb + rpp * kStageBatch <= s.lds_rows; rb += rpp * kStageBatch) {
                        float4 v[kStageBatch];
#pragma unroll
                        for (int u = 0; u < kStageBatch; ++u) {
                            const bool ok = col_ok && static_cast<unsigned>(iy + u * rpp - lo) < span;
                            v[u] = load_slot(ok ? off + u * off_step : kOob);
                        }
                        if (ragged) {
#pragma unroll
                            for (int u = 0; u < kStageBatch; ++u) keep_first(v[u], left);
                        }
#pragma unroll
                        for (int u = 0; u < kStageBatch; ++u) {
                            float *d = lds + dst + u * dst_step;  // (col_shift need not be a multiple of four)
                            d[0] = v[u].x;
                            d[1] = v[u].y;
                            d[2] = v[u].z;
                            d[3] = v[u].w;
                        }
                        iy += rpp * kStageBatch;
                        off += off_step * kStageBatch;
                        dst += dst_step * kStageBatch;
                    }
                    if (rb < s.lds_rows) {
                        float4 v[kStageBatch];
#pragma unroll
                        for (int u = 0; u < kStageBatch; ++u) {
                            const bool ok = col_ok && static_cast<unsigned>(iy + u * rpp - lo) < span;
                            v[u] = load_slot(ok ? off + u * off_step : kOob);
                        }
                        if (ragged) {
#pragma unroll
                            for (int u = 0; u < kStageBatch; ++u) keep_first(v[u], left);
                        }
#pragma unroll
                        for (int u = 0; u < kStageBatch; ++u) {
                            float *d = lds + (rb + rl + u * rpp < s.lds_rows ? dst + u * dst_step : dump);
                            d[0] = v[u].x;
                            d[1] = v[u].y;
                            d[2] = v[u].z;
                            d[3] = v[u].w;
                        }
                    }
                } else {
                    const int dump = nplanes * s.plane_pitch - 4;
                    for (int ra = rl; ra < total_rows; ra += rpp * kStageBatch) {
                        float4 v[kStageBatch];
                        int dst[kStageBatch];
#pragma unroll
                        for (int u = 0; u < kStageBatch; ++u) {
                            const bool live = ra + u * rpp < total_rows;
                            const int rc = min(ra + u * rpp, total_rows - 1);
                            const int pl = fast_div(rc, s.lds_rows_magic);
                            const int r = rc - __mul24(pl, s.lds_rows);
                            const int iy = iy0 + r;
                            const bool ok = live && col_ok && static_cast<unsigned>(iy) < static_cast<unsigned>(s.in_h);
                            const unsigned off = (__mul24(pl, s.in_plane) + __mul24(iy, s.in_w) + ix) * ES;
                            v[u] = load_slot(ok ? off : kOob);
                            dst[u] = live ? __mul24(pl, s.plane_pitch) + __mul24(r, s.pitch) + dcol : dump;
                        }
                        if (ragged) {
#pragma unroll
                            for (int u = 0; u < kStageBatch; ++u) keep_first(v[u], left);
                        }
#pragma unroll
                        for (int u = 0; u < kStageBatch; ++u) {
                            float *d = lds + dst[u];
                            d[0] = v[u].x;
                            d[1] = v[u].y;
                            d[2] = v[u].z;
                            d[3] = v[u].w;
                        }
                    }
                }
            }
            return;
        }
        for (int base = threadIdx.x; base < total; base += blockDim.x * kStageBatch) {
            float4 v[kStageBatch];
            int dst[kStageBatch];
#pragma unroll
            for (int u = 0; u < kStageBatch; ++u) {
                const bool live = base + u * static_cast<int>(blockDim.x) < total;
                const int slot = min(base + u * static_cast<int>(blockDim.x), total - 1);
                // 24-bit multiplies run at full rate, 32-bit ones at a quarter of it; vector_mode() guarantees
                // that the operands fit
                const int rowidx = fast_div(slot, s.spr_magic);
                const int sc = slot - __mul24(rowidx, s.spr);
                const int pl = nplanes == 1 ? 0 : fast_div(rowidx, s.lds_rows_magic);
                const int r = rowidx - __mul24(pl, s.lds_rows);
                const int ix = 4 * (s.g_lo + sc);
                const int iy = iy0 + r;
                const bool ok = live && static_cast<unsigned>(iy) < static_cast<unsigned>(s.in_h) &&
                                static_cast<unsigned>(ix) < static_cast<unsigned>(s.in_w);
                const unsigned off = (__mul24(pl, s.in_plane) + __mul24(iy, s.in_w) + ix) * static_cast<unsigned>(sizeof(IO));
                v[u] = load_slot(ok ? off : kOob);
                if (ragged) keep_first(v[u], s.in_w - ix);
                // slots past the end of the image (they hold zeros) go to the spare floats that end the image:
                // the right-hand slack of its last row, which no stored output depends on
                dst[u] = live ? __mul24(pl, s.plane_pitch) + __mul24(r, s.pitch) + kSlack + ix + s.col_shift
                              : nplanes * s.plane_pitch - 4;
            }
#pragma unroll
            for (int u = 0; u < kStageBatch; ++u) {
                float *d = lds + dst[u];
                d[0] = v[u].x;
                d[1] = v[u].y;
                d[2] = v[u].z;
                d[3] = v[u].w;
            }
        }
        return;
    }
    if constexpr (VIEW_ONLY) return;
    for (int base = threadIdx.x; base < total; base += blockDim.x * kStageBatch) {
        float4 v[kStageBatch];
        int dst[kStageBatch];
#pragma unroll
        for (int u = 0; u < kStageBatch; ++u) {
            const int slot = base + u * blockDim.x;
            v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            dst[u] = -1;
            if (slot < total) {
                const int rowidx = fast_div(slot, s.spr_magic);
                const int sc = slot - rowidx * s.spr;
                const int pl = fast_div(rowidx, s.lds_rows_magic);
                const int r = rowidx - pl * s.lds_rows;
                const int ix = 4 * (s.g_lo + sc);
                const int iy = iy0 + r;
                const bool row_ok = static_cast<unsigned>(iy) < static_cast<unsigned>(s.in_h);
                const IO *src = in + (plane0 + pl) * s.in_plane + static_cast<long>(iy) * s.in_w + ix;
                if (s.vec_in) {
                    if (row_ok && ix >= 0 && ix < s.in_w) v[u] = load4<IO>(src);
                } else if (row_ok) {
                    if (static_cast<unsigned>(ix + 0) < static_cast<unsigned>(s.in_w)) v[u].x = Io<IO>::in(src[0]);
                    if (static_cast<unsigned>(ix + 1) < static_cast<unsigned>(s.in_w)) v[u].y = Io<IO>::in(src[1]);
                    if (static_cast<unsigned>(ix + 2) < static_cast<unsigned>(s.in_w)) v[u].z = Io<IO>::in(src[2]);
                    if (static_cast<unsigned>(ix + 3) < static_cast<unsigned>(s.in_w)) v[u].w = Io<IO>::in(src[3]);
                }
                dst[u] = pl * s.plane_pitch + r * s.pitch + kSlack + ix + s.col_shift;
            }
        }
#pragma unroll
        for (int u = 0; u < kStageBatch; ++u) {
            if (dst[u] >= 0) {
                float *d = lds + dst[u];
                d[0] = v[u].x;
                d[1] = v[u].y;
                d[2] = v[u].z;
                d[3] = v[u].w;
            }
        }
    }
}

// Pins an accumulator array at this point of a fully unrolled loop nest.  The empty asm makes every
// element an input and an output, so all FMAs feeding it must be issued before, and its memory clobber
// keeps later LDS reads after it.  Without such pins the compiler sinks every FMA of a window below
// the LDS reads of all its rows and keeps the whole window in registers (several hundred VGPRs).
// It emits no instruction.
template <int N>
__device__ __forceinline__ void pin_registers(float (&a)[N])
{
#pragma unroll
    for (int i = 0; i < N; ++i) asm volatile("" : "+v"(a[i]) : : "memory");
}

template <int R, int C>
__device__ __forceinline__ void pin_registers(float (&a)[R][C])
{
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int c = 0; c < C; ++c) asm volatile("" : "+v"(a[r][c]) : : "memory");
}

// NV aligned float4s of an LDS row into registers.
template <int NV>
__device__ __forceinline__ void load_window_row(const float *row, float (&w)[4 * NV])
{
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const float4 q = reinterpret_cast<const float4 *>(row)[v];
        w[4 * v + 0] = q.x;
        w[4 * v + 1] = q.y;
        w[4 * v + 2] = q.z;
        w[4 * v + 3] = q.w;
    }
}

// NV2 aligned float2s of an LDS row into registers.
template <int NV2>
__device__ __forceinline__ void load_window_row2(const float *row, float (&w)[2 * NV2])
{
#pragma unroll
    for (int v = 0; v < NV2; ++v) {
        const float2 q = reinterpret_cast<const float2 *>(row)[v];
        w[2 * v + 0] = q.x;
        w[2 * v + 1] = q.y;
    }
}

// ---- fixed-order reductions of per-lane sums ----------------------------------------------------------------
template <int CTRL, int ROW_MASK, int BANK_MASK>
__device__ __forceinline__ float dpp_add(float v)
{
    const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, BANK_MASK, true);
    return v + __int_as_float(moved);
}

// Sum of the 64 lanes, delivered in lane 63; fixed association order.
__device__ __forceinline__ float wave_sum_to_last_lane(float v)
{
    v = dpp_add<0x111, 0xf, 0xf>(v);  // row_shr:1
    v = dpp_add<0x112, 0xf, 0xf>(v);  // row_shr:2
    v = dpp_add<0x114, 0xf, 0xf>(v);  // row_shr:4
    v = dpp_add<0x118, 0xf, 0xf>(v);  // row_shr:8  -> lane 15 of each row of 16 holds the row sum
    v = dpp_add<0x142, 0xa, 0xf>(v);  // row_bcast:15 into rows 1 and 3
    v = dpp_add<0x143, 0xc, 0xf>(v);  // row_bcast:31 into rows 2 and 3
    return v;
}

constexpr int kRedPitch = kThreads + 1;  // odd pitch: lanes of one wave reading one column spread over the banks

inline int floor_div(int a, int b)
{
    int q = a / b;
    if ((a % b != 0) && ((a < 0) != (b < 0))) --q;
    return q;
}

// Tuning overrides.  The planners' choices (rows per lane, workgroups, LDS budgets, which kernel family) can be
// overridden through DWCONV_* environment variables for measurements.  They are honoured only while DWCONV_TUNING=1 is
// set as well, so that a stray variable in a user's environment changes nothing; values that are not plain
// non-negative numbers up to 2^24 are ignored.
inline bool tuning_enabled()
{
    const char *t = std::getenv("DWCONV_TUNING");
    return t != nullptr && t[0] == '1' && t[1] == '\0';
}

inline int env_int(const char *name, int dflt)
{
    if (!tuning_enabled()) return dflt;
    const char *e = std::getenv(name);
    if (e == nullptr || e[0] == '\0') return dflt;
    char *end = nullptr;
    const long v = std::strtol(e, &end, 10);
    if (end == e || *end != '\0' || v < 0 || v > (1l << 24)) return dflt;
    return static_cast<int>(v);
}

// True when the override `name` is set (and overrides are enabled at all).
inline bool env_set(const char *name)
{
    if (!tuning_enabled()) return false;
    const char *e = std::getenv(name);
    return e != nullptr && e[0] != '\0';
}

// vec_in for a tile of `planes` planes of `in_plane` elements of `esize` bytes whose rows allow vector loads.
inline int vector_mode(long planes, long in_plane, size_t esize)
{
    const bool fits = planes * in_plane * static_cast<long>(esize) < static_cast<long>(kOob);
    return fits && env_int("DWCONV_STAGE_VIEW", 1) ? 2 : 1;
}

// How a tensor whose rows are `width` elements wide and which starts at `base` is moved, before the view conditions are
// known: 1 = groups of four aligned elements (stage_vector_mode / vector_mode then decide between 1 and 2), 3 = groups
// of four at any element alignment through a view (the caller drops to 0 where the view does not fit), 0 =
// element by element.
// `mixed_ok`: whether mode 3 is wanted also where rows of a 16-bit tensor start 2 bytes past a 32-bit boundary (odd
// widths, or a base there).  64- and 32-bit accesses from such addresses returned wrong data; loads are then made from
// the boundary before (any_width_load4: 150x150 -> 75x75 5x5 stride-2 forward in bf16 209 -> 130 us), stores stay
// element by element (`mixed_ok` false for results: in aligned pieces of 16 + 32 + 16 bits they were 3-10 % slower).
template <typename IO>
inline int unaligned_vector_mode(int width, const IO *base, bool mixed_ok)
{
    const bool mixed = sizeof(IO) == 2 && ((width & 1) != 0 || (reinterpret_cast<uintptr_t>(base) & 2) != 0);
    if (mixed && !mixed_ok) return 0;
    return env_int("DWCONV_RAGGED_VIEWS", 1) ? 3 : 0;
}
template <typename IO>
inline int row_vector_mode(int width, const IO *base, bool mixed_ok = true)
{
    return width % 4 == 0 && aligned4(base) ? 1 : unaligned_vector_mode<IO>(width, base, mixed_ok);
}

// ---- a one-plane image staged in two steps --------------------------------------------------------------
// fetch_rows issues a lane's loads into registers (elements as loaded), commit_rows writes them into the LDS image
// later: between the two the workgroup computes on the images already in LDS, with the next image's loads in
// flight.  A lane owns one float4 column and every rpp-th row (rpp = whole rows per sweep of the workgroup); trips
// that lie past the image for every lane are skipped under a uniform bound.  The planner checks rows_fit().
struct RowLane {
    int rl;         // first row (lanes beyond rpp whole rows stage nothing: rl is then past every image)
    int rpp;        // rows per sweep
    unsigned coff;  // byte offset of the column within a row of the tensor
    bool col_ok;    // the column lies inside the plane (else it reads as zeros)
    int dcol;       // float offset of the column within an LDS row
};

template <typename IO>
__device__ __forceinline__ RowLane row_lane(const StageLayout &s)
{
    RowLane l;
    l.rpp = fast_div(kThreads, s.spr_magic);
    const int rl = fast_div(threadIdx.x, s.spr_magic);
    const int ix = 4 * (s.g_lo + static_cast<int>(threadIdx.x) - __mul24(rl, s.spr));
    l.rl = rl < l.rpp ? rl : (1 << 20);
    l.coff = static_cast<unsigned>(ix) * static_cast<unsigned>(sizeof(IO));
    l.col_ok = static_cast<unsigned>(ix) < static_cast<unsigned>(s.in_w);
    l.dcol = kSlack + ix + s.col_shift;
    return l;
}

// `plane`: the tensor plane the image is cut from; LDS row r holds its row iy0 + r (zeros outside the plane).
template <typename IO, int NS>
__device__ __forceinline__ void fetch_rows(const StageLayout &s, const RowLane &l, const IO *__restrict__ plane, int iy0,
                                           typename Raw4<IO>::type (&v)[NS])
{
    constexpr unsigned ES = sizeof(IO);
    const __amdgpu_buffer_rsrc_t view = buffer_view(plane, static_cast<long>(s.in_plane) * ES);
    // (the lane's row is made opaque here and in commit_rows: what derives from it is then worked out where it is
    // used, an add and a select per slot, instead of being kept in registers from one tile to the next)
    int rl = l.rl;
    asm volatile("" : "+v"(rl));
#pragma unroll
    for (int u = 0; u < NS; ++u) {
        if (u * l.rpp >= s.lds_rows) break;  // uniform
        const int r = rl + u * l.rpp;
        const int iy = iy0 + r;
        const bool ok = r < s.lds_rows && l.col_ok && static_cast<unsigned>(iy) < static_cast<unsigned>(s.in_h);
        const unsigned off = __mul24(iy, s.in_w) * ES + l.coff;
        if constexpr (sizeof(IO) == 4) {
            const u32x4 q = __builtin_amdgcn_raw_buffer_load_b128(view, ok ? off : kOob, 0, 0);
            v[u] = make_float4(__uint_as_float(q.x), __uint_as_float(q.y), __uint_as_float(q.z), __uint_as_float(q.w));
        } else {
            const u32x2 q = __builtin_amdgcn_raw_buffer_load_b64(view, ok ? off : kOob, 0, 0);
            v[u] = make_uint2(q.x, q.y);
        }
    }
}

template <typename IO, int NS>
__device__ __forceinline__ void commit_rows(const StageLayout &s, const RowLane &l, float *lds,
                                            const typename Raw4<IO>::type (&v)[NS])
{
    const int dump = s.plane_pitch - 4;  // right-hand slack of the last row
    int rl = l.rl;
    asm volatile("" : "+v"(rl));
#pragma unroll
    for (int u = 0; u < NS; ++u) {
        if (u * l.rpp >= s.lds_rows) break;  // uniform
        const int r = rl + u * l.rpp;
        float *d = lds + (r < s.lds_rows ? __mul24(r, s.pitch) + l.dcol : dump);
        const float4 w = widen4<IO>(v[u]);
        d[0] = w.x;
        d[1] = w.y;
        d[2] = w.z;
        d[3] = w.w;
    }
}

// Whether an image can be staged that way with at most `ns` loads per lane.
inline bool rows_fit(const StageLayout &s, int ns)
{
    if (s.spr < 1 || s.spr > kThreads) return false;
    return s.lds_rows <= ns * (kThreads / s.spr);
}

// vec_in of a staged image: the view path also needs operands that fit its 24-bit multiplies.
inline int stage_vector_mode(const StageLayout &s, long planes, size_t esize)
{
    const bool dims = s.in_h < (1 << 23) && s.in_w < (1 << 23) && (planes == 1 || s.in_plane < (1 << 23));
    return dims ? vector_mode(planes, s.in_plane, esize) : 1;
}

// Row pitch and float4 slots of an image `used_cols` floats wide (col_shift must be set).
inline void layout_columns(StageLayout &s, int used_cols)
{
    s.pitch = kSlack + round_up(used_cols, 4) + kSlack;
    s.g_lo = floor_div(-s.col_shift, 4);
    s.spr = ceil_div(used_cols - s.col_shift, 4) - s.g_lo;
}

// Finishes the layout once the rows per image are known.  False if the 16-bit
// reciprocals the kernels divide with would not be exact.
inline bool layout_rows(StageLayout &s, int lds_rows, int planes_per_tile)
{
    s.lds_rows = lds_rows;
    s.plane_pitch = lds_rows * s.pitch;
    if (static_cast<long>(planes_per_tile) * lds_rows * s.spr >= 65536) return false;
    s.lds_rows_magic = magic_u16(lds_rows);
    s.spr_magic = magic_u16(s.spr);
    return true;
}

}  // namespace dwconv
