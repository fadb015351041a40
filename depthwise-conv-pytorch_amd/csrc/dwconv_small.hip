// Dispatch of the whole-plane forward / grad-input kernels for small feature maps (any plane up to 32 elements
// wide and 64 rows with "same" column padding; kernels and their description: dwconv_small_fir.hpp).  Picks the
// width instance: an exact one for widths 7, 8, 14, 16, 28, 32, else the ragged class that holds the width.
#include "dwconv_small_common.hpp"

namespace dwconv {

namespace {

template <typename IO>
int small_fir_any_width(SmallPlan &p, int width, bool exact_ok, int K, int S, int D, bool rot, bool up2, hipStream_t stream)
{
    if (exact_ok && small_width_is_exact(width)) {
#define DWCONV_CASE(WV) \
        if (width == WV) return small_fir_width<WV, false, IO>(p, K, S, D, rot, up2, stream);
        DWCONV_SMALL_EXACT_WIDTHS(DWCONV_CASE)
#undef DWCONV_CASE
    }
    const int cls = small_ragged_class(width);
#define DWCONV_CASE(WV) \
    if (cls == WV) return small_fir_width<WV, true, IO>(p, K, S, D, rot, up2, stream);
    DWCONV_SMALL_RAGGED_WIDTHS(DWCONV_CASE)
#undef DWCONV_CASE
    return -1;
}

}  // namespace

template <typename IO>
int try_launch_fir_small(const IO *in, const IO *taps, IO *out, const Geometry &g, hipStream_t stream, int dil)
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
    p.in_w = g.in_w;
    p.out_w = g.out_w;
    const int W = g.in_w;
    if (g.up_h == 1 && g.up_w == 1 && g.down_h == g.down_w && (g.down_h == 1 || g.down_h == 2)) {
        const int S = g.down_h;
        // full-width rows with the column padding of a "same" convolution
        if (g.pad_w0 != dil * (K / 2) || g.out_w != (W - 1) / S + 1) return -1;
        if (g.pad_h0 < 0 || g.pad_h0 > 7) return -1;
        p.pad_h = g.pad_h0;
        return small_fir_any_width<IO>(p, W, true, K, S, dil, !g.forward, false, stream);
    }
    if (dil == 1 && g.up_h == 2 && g.up_w == 2 && g.down_h == 1 && g.down_w == 1 && !g.forward) {
        // the transposed stride-2 problem: the output is 2W wide, or 2W - 1 when the forward input was odd
        if (g.pad_w0 != K / 2 || g.pad_h0 != K / 2 || (g.out_w != 2 * W && g.out_w != 2 * W - 1)) return -1;
        const int E = (K / 2) & 1;
        p.pad_h = (K / 2 + E) / 2;
        return small_fir_any_width<IO>(p, W, g.out_w == 2 * W, K, 1, 1, true, true, stream);
    }
    return -1;
}

template int try_launch_fir_small<float>(const float *, const float *, float *, const Geometry &, hipStream_t, int);
template int try_launch_fir_small<half_t>(const half_t *, const half_t *, half_t *, const Geometry &, hipStream_t, int);
template int try_launch_fir_small<bf16_t>(const bf16_t *, const bf16_t *, bf16_t *, const Geometry &, hipStream_t, int);

}  // namespace dwconv
