// Dispatch of the whole-plane grad-weight / fused backward kernels for small feature maps (any plane up to 32
// elements wide and 64 rows with "same" column padding; kernels and their description: dwconv_small_bwd.hpp).
#include "dwconv_small_common.hpp"

namespace dwconv {

namespace {

template <typename IO>
long small_bwd_any(int mode, const IO *x, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws,
                   size_t ws_bytes, const WgradGeometry &g, hipStream_t stream)
{
    if (env_int("DWCONV_NO_SMALL", 0)) return -1;
    const int K = g.kernel_h, S = g.down_h;
    if (g.kernel_w != K || g.down_w != S || (S != 1 && S != 2)) return -1;
    if (g.dil != 1 && (g.dil != 2 || S != 1 || K > 5)) return -1;
    if (g.pad_w != g.dil * (K / 2) || g.pad_h < 0 || g.pad_h > 7) return -1;
    if (g.in_h < 1 || g.in_h > 64 || g.out_h < 1 || g.out_h > 64) return -1;
    if (g.in_w < 1 || g.out_w != (g.in_w - 1) / S + 1) return -1;
    if (mode == 2) {
        // the fused variant writes every gx row from the lane that owns the matching gy rows
        if (g.pad_h != g.dil * (K / 2)) return -1;
        if (S == 1 && g.out_h != g.in_h) return -1;
        if (S == 2 && g.out_h != (g.in_h - 1) / 2 + 1) return -1;
        if (!aligned4(gx)) return -1;
    }
    if (mode != 0 && (!aligned4(x) || !aligned4(gy))) return -1;
    const SmallBwdArgs a{x, gy, taps, gx, gw, ws, ws_bytes};
    const int width = g.in_w;
    if (small_width_is_exact(width)) {
#define DWCONV_CASE(WV) \
        if (width == WV) return small_bwd_width<WV, false, IO>(mode, a, g, stream);
        DWCONV_SMALL_EXACT_WIDTHS(DWCONV_CASE)
#undef DWCONV_CASE
    }
    const int cls = small_ragged_class(width);
#define DWCONV_CASE(WV) \
    if (cls == WV) return small_bwd_width<WV, true, IO>(mode, a, g, stream);
    DWCONV_SMALL_RAGGED_WIDTHS(DWCONV_CASE)
#undef DWCONV_CASE
    return -1;
}

}  // namespace

size_t wgrad_small_workspace(const WgradGeometry &g)
{
    // partial sums are fp32 whatever the element type, but the rows per lane, and with them the chunk count, follow
    // the element size: the larger of the two plans
    const long n4 = small_bwd_any<float>(0, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, g, nullptr);
    const long n2 = small_bwd_any<half_t>(0, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, g, nullptr);
    const long n = n4 > n2 ? n4 : n2;
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
