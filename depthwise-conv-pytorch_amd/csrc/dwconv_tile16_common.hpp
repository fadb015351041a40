// Shared by the kernels for 16-bit tensors that keep their LDS images in the tensors' own format (two elements
// per dword): the image layout, how it is filled, and the two-element dot product.
#pragma once

#include "dwconv_tile_common.hpp"

namespace dwconv {

constexpr int kPadL = 8;  // element j of an image row holds input column j - kPadL

// `planes` images of `lds_rows` rows of `pitch` 16-bit elements; a row is written in slots of eight elements
// (four dwords), `spr` of them, the first of which lies wholly left of the plane.
// In LDS a slot takes FIVE dwords, the fifth unused: lanes that own consecutive 8-element blocks then sit five
// dwords apart, an odd stride, and their two-dword reads fall on distinct banks.  With the slots packed (stride
// four) the same reads use half the banks twice over: the counters showed the LDS busy 60 % of the time, two thirds
// of it in bank conflicts.
struct Image16 {
    int in_h, in_w, in_plane;   // in_w is a multiple of eight
    int lds_rows;
    unsigned lds_rows_magic;
    int spr;
    unsigned spr_magic;
    int pitch;                  // elements per image row, a multiple of eight
    int rp;                     // dwords per image row in LDS: five per slot
    int pp;                     // dwords per plane image in LDS
};

// Row pitch and slots for windows that reach input column `last_col` at most.
inline void layout_image16(Image16 &im, int last_col)
{
    im.spr = ceil_div(kPadL + std::max(last_col + 1, im.in_w), 8);
    // eight spare elements per row keep the rows of consecutive row blocks off the same banks
    im.pitch = 8 * im.spr + 8;
    im.rp = 5 * (im.pitch / 8);
}

// False if the 16-bit reciprocals or the 24-bit multiplies of stage_image16 would not be exact.
inline bool finish_image16(Image16 &im, int lds_rows, int planes_per_tile)
{
    im.lds_rows = lds_rows;
    im.pp = lds_rows * im.rp;
    if (static_cast<long>(planes_per_tile) * lds_rows * im.spr >= 65536) return false;
    if (im.in_h >= (1 << 23) || im.in_w >= (1 << 23) || (planes_per_tile > 1 && im.in_plane >= (1 << 23))) return false;
    if (static_cast<long>(planes_per_tile) * im.in_plane * 2 >= static_cast<long>(kOob)) return false;
    im.spr_magic = magic_u16(im.spr);
    im.lds_rows_magic = magic_u16(lds_rows);
    return true;
}

// LDS dword of logical dword j of an image row (four data dwords per five).
__host__ __device__ constexpr int swz(int j) { return j + (j >> 2); }

template <typename IO>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c)
{
    if constexpr (std::is_same<IO, bf16_t>::value) {
        typedef __bf16 v2 __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2, a), __builtin_bit_cast(v2, b), c, false);
    } else {
        typedef _Float16 v2 __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(v2, a), __builtin_bit_cast(v2, b), c, false);
    }
}

// Fills the images of `nplanes` planes starting at `src` (plane stride im.in_plane) with input rows iy0 ...: every
// slot of every row is written, with zeros (loads beyond the view) outside the plane.  `image` is the first dword,
// `dump` the index of a spare slot.  A lane keeps its column and walks down the rows: per slot two additions, a range check and a
// select.  kBatch loads are in flight per lane.
template <typename IO, int kBatch = 4>
__device__ __forceinline__ void stage_image16(const Image16 &im, const IO *src, uint32_t *image, int dump, int nplanes, int iy0)
{
    const __amdgpu_buffer_rsrc_t view = buffer_view(src, static_cast<long>(nplanes) * im.in_plane * sizeof(IO));
    const int nthreads = blockDim.x;
    const int rpp_raw = fast_div(nthreads, im.spr_magic);
    const int rpp = max(rpp_raw, 1);                     // rows per pass of the workgroup
    const int col_step = rpp_raw ? im.spr : nthreads;    // one trip unless a row has more slots than lanes
    const int rl = fast_div(threadIdx.x, im.spr_magic);
    const int spitch = im.pitch >> 3;                    // in slots
    auto put = [&](int slot, const u32x4 &v) {
        uint32_t *d = image + slot * 5;
        d[0] = v.x;
        d[1] = v.y;
        d[2] = v.z;
        d[3] = v.w;
    };
    if (rl >= rpp) return;
    for (int sc = threadIdx.x - __mul24(rl, im.spr); sc < im.spr; sc += col_step) {
        const int ix = 8 * sc - kPadL;
        const bool col_ok = static_cast<unsigned>(ix) < static_cast<unsigned>(im.in_w);
        if (nplanes == 1) {
            const int lo = max(iy0, 0);
            const unsigned span = static_cast<unsigned>(max(min(im.in_h, iy0 + im.lds_rows) - lo, 0));
            const unsigned off_step = __mul24(rpp, im.in_w) * 2u;
            const int dst_step = __mul24(rpp, spitch);
            int iy = iy0 + rl;
            unsigned off = (__mul24(iy, im.in_w) + ix) * 2u;
            int dst = __mul24(rl, spitch) + sc;
            int rb = 0;
            // whole batches (uniform bound, unconditional stores), then one batch whose rows past the image go to
            // the spare slot.  A store under a per-lane condition would drag its load into the conditional block,
            // behind the other loads' wait.
            for (; rb + rpp * kBatch <= im.lds_rows; rb += rpp * kBatch) {
                u32x4 v[kBatch];
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    const bool ok = col_ok && static_cast<unsigned>(iy + u * rpp - lo) < span;
                    v[u] = __builtin_amdgcn_raw_buffer_load_b128(view, ok ? off + u * off_step : kOob, 0, 0);
                }
#pragma unroll
                for (int u = 0; u < kBatch; ++u) put(dst + u * dst_step, v[u]);
                iy += rpp * kBatch;
                off += off_step * kBatch;
                dst += dst_step * kBatch;
            }
            if (rb < im.lds_rows) {
                u32x4 v[kBatch];
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    const bool ok = col_ok && static_cast<unsigned>(iy + u * rpp - lo) < span;
                    v[u] = __builtin_amdgcn_raw_buffer_load_b128(view, ok ? off + u * off_step : kOob, 0, 0);
                }
#pragma unroll
                for (int u = 0; u < kBatch; ++u) put(rb + rl + u * rpp < im.lds_rows ? dst + u * dst_step : dump, v[u]);
            }
        } else {
            const int total_rows = nplanes * im.lds_rows;
            const int pslots = im.lds_rows * spitch;
            for (int ra = rl; ra < total_rows; ra += rpp * kBatch) {
                u32x4 v[kBatch];
                int dst[kBatch];
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    const bool live = ra + u * rpp < total_rows;
                    const int rc = min(ra + u * rpp, total_rows - 1);
                    const int pl = fast_div(rc, im.lds_rows_magic);
                    const int r = rc - __mul24(pl, im.lds_rows);
                    const int iy = iy0 + r;
                    const bool ok = live && col_ok && static_cast<unsigned>(iy) < static_cast<unsigned>(im.in_h);
                    const unsigned off = (__mul24(pl, im.in_plane) + __mul24(iy, im.in_w) + ix) * 2u;
                    v[u] = __builtin_amdgcn_raw_buffer_load_b128(view, ok ? off : kOob, 0, 0);
                    dst[u] = live ? __mul24(pl, pslots) + __mul24(r, spitch) + sc : dump;
                }
#pragma unroll
                for (int u = 0; u < kBatch; ++u) put(dst[u], v[u]);
            }
        }
    }
}

}  // namespace dwconv
