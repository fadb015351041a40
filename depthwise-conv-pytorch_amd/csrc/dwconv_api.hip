// extern "C" surface of libdwconv_hip (declared in include/dwconv_hip.h):
// argument checks, kernel-family selection, error strings.
#include "dwconv_common.hpp"

#include <algorithm>
#include <mutex>
#include <type_traits>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace dwconv {

namespace {
thread_local char g_error[512] = "";
thread_local char g_variant[256] = "";

// DWCONV_FORCE_GENERIC=1 routes every call to the generic kernels (used by the
// tests to cover that path at fp32 as well).
bool force_generic()
{
    const char *e = std::getenv("DWCONV_FORCE_GENERIC");
    return e != nullptr && e[0] != '\0' && e[0] != '0';
}
}  // namespace

int fail(dwconv_status code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

void note_variant(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(g_variant, sizeof(g_variant), fmt, ap);
    va_end(ap);
}

int check_launch(const char *what)
{
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return fail(DWCONV_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return DWCONV_OK;
}

namespace {

int make_geometry(Geometry &g, const void *in, const void *taps, const void *out, int batch,
                  int channel, int in_h, int in_w, int kernel_h, int kernel_w, int up_h, int up_w,
                  int down_h, int down_w, int pad_h0, int pad_h1, int pad_w0, int pad_w1, int forward)
{
    if (batch < 0 || channel < 0 || in_h < 0 || in_w < 0)
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "negative tensor extent (%d,%d,%d,%d)", batch, channel,
                    in_h, in_w);
    if (kernel_h < 1 || kernel_w < 1)
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "kernel extent must be >= 1, got %dx%d", kernel_h,
                    kernel_w);
    if (up_h < 1 || up_w < 1 || down_h < 1 || down_w < 1)
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "up/down factors must be >= 1, got up %dx%d down %dx%d",
                    up_h, up_w, down_h, down_w);
    g = Geometry{batch, channel, in_h, in_w, kernel_h, kernel_w, up_h, up_w, down_h, down_w,
                 pad_h0, pad_h1, pad_w0, pad_w1, 0, 0, forward ? 1 : 0};
    g.out_h = dwconv_out_size(in_h, up_h, down_h, pad_h0, pad_h1, kernel_h);
    g.out_w = dwconv_out_size(in_w, up_w, down_w, pad_w0, pad_w1, kernel_w);
    if (g.out_h < 0) g.out_h = 0;
    if (g.out_w < 0) g.out_w = 0;
    const long long in_elems = 1ll * batch * channel * in_h * in_w;
    const long long out_elems = 1ll * batch * channel * g.out_h * g.out_w;
    if (in_elems >= (1ll << 40) || out_elems >= (1ll << 40))
        return fail(DWCONV_ERR_UNSUPPORTED, "tensor too large");
    if (out_elems > 0 && (taps == nullptr || out == nullptr || (in_elems > 0 && in == nullptr)))
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "null device pointer");
    return DWCONV_OK;
}

template <typename T>
int run_fir(const T *in, const T *taps, T *out, const Geometry &g, hipStream_t stream)
{
    if (g.planes() * g.out_h * g.out_w == 0) {
        note_variant("empty");
        return DWCONV_OK;
    }
    if constexpr (!std::is_same<T, double>::value) {
        if (!force_generic()) {
            int rc = try_launch_fir_small<T>(in, taps, out, g, stream);
            if (rc >= 0) return rc;
            if constexpr (sizeof(T) == 2) {
                rc = try_launch_fir_tiled16<T>(in, taps, out, g, stream);
                if (rc >= 0) return rc;
            }
            rc = try_launch_fir_stack<T>(in, taps, out, g, stream);
            if (rc >= 0) return rc;
            rc = try_launch_fir_tiled<T>(in, taps, out, g, stream);
            if (rc >= 0) return rc;
            rc = try_launch_fir_any<T>(in, taps, out, g, stream);
            if (rc >= 0) return rc;
        }
    }
    if (!force_generic()) {
        const int rc = try_launch_fir_lds<T>(in, taps, out, g, stream);
        if (rc >= 0) return rc;
    }
    return launch_fir_direct<T>(in, taps, out, g, stream);
}

int check_activation(int act)
{
    if (act < DWCONV_ACT_NONE || act > DWCONV_ACT_SILU)
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "unknown activation %d", act);
    return DWCONV_OK;
}

template <typename T>
int dwconv2d_any(const T *in, const T *taps, T *out, int batch, int channel, int in_h, int in_w,
                 int kernel_h, int kernel_w, int up_h, int up_w, int down_h, int down_w, int pad_h0,
                 int pad_h1, int pad_w0, int pad_w1, int forward, void *stream, const Epilogue &epi = Epilogue{})
{
    Geometry g;
    const int rc = make_geometry(g, in, taps, out, batch, channel, in_h, in_w, kernel_h, kernel_w,
                                 up_h, up_w, down_h, down_w, pad_h0, pad_h1, pad_w0, pad_w1, forward);
    if (rc != DWCONV_OK) return rc;
    g.epi = epi;
    return run_fir<T>(in, taps, out, g, static_cast<hipStream_t>(stream));
}

template <typename T>
int dwconv2d_small_any(const T *in, const T *taps, T *out, int batch, int channel, int in_h,
                       int in_w, int kernel_h, int kernel_w, int up_h, int up_w, int down_h,
                       int down_w, int pad_h, int pad_w, int forward, void *stream)
{
    if (up_h != 1 || up_w != 1 || down_h != 1 || down_w != 1)
        return fail(DWCONV_ERR_UNSUPPORTED,
                    "dwconv2d_small handles stride-1 same-size convolutions only (up %dx%d, down %dx%d)",
                    up_h, up_w, down_h, down_w);
    if (in_h > 32 || in_w > 32)
        return fail(DWCONV_ERR_UNSUPPORTED, "dwconv2d_small handles planes up to 32x32, got %dx%d",
                    in_h, in_w);
    if (kernel_h < 1 || kernel_w < 1)
        return fail(DWCONV_ERR_UNSUPPORTED, "dwconv2d_small needs a kernel of at least 1x1, got %dx%d", kernel_h, kernel_w);
    if (pad_h < 0 || pad_h >= kernel_h || pad_w < 0 || pad_w >= kernel_w)
        return fail(DWCONV_ERR_UNSUPPORTED, "dwconv2d_small needs 0 <= pad < kernel, got pad %dx%d kernel %dx%d",
                    pad_h, pad_w, kernel_h, kernel_w);
    // Same-size output: trailing pad = kernel - 1 - leading pad.
    return dwconv2d_any<T>(in, taps, out, batch, channel, in_h, in_w, kernel_h, kernel_w, 1, 1, 1, 1,
                           pad_h, kernel_h - 1 - pad_h, pad_w, kernel_w - 1 - pad_w, forward, stream);
}

int make_wgrad_geometry(WgradGeometry &g, const void *in, const void *gy, const void *gw, int batch,
                        int channel, int in_h, int in_w, int out_h, int out_w, int kernel_h,
                        int kernel_w, int up_h, int up_w, int down_h, int down_w, int pad_h, int pad_w)
{
    if (batch < 0 || channel < 0 || in_h < 0 || in_w < 0 || out_h < 0 || out_w < 0)
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "negative tensor extent");
    if (kernel_h < 1 || kernel_w < 1)
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "kernel extent must be >= 1, got %dx%d", kernel_h,
                    kernel_w);
    if (up_h != 1 || up_w != 1)
        return fail(DWCONV_ERR_UNSUPPORTED, "grad-weight is defined for up == 1 only, got %dx%d", up_h,
                    up_w);
    if (down_h < 1 || down_w < 1)
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "down factors must be >= 1");
    if (1ll * batch * channel * in_h * in_w >= (1ll << 40) ||
        1ll * batch * channel * out_h * out_w >= (1ll << 40))
        return fail(DWCONV_ERR_UNSUPPORTED, "tensor too large");
    if (channel > 0 && gw == nullptr)
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "null kernel_grad pointer");
    const bool has_work = 1ll * batch * channel * out_h * out_w > 0 && in_h > 0 && in_w > 0;
    if (has_work && (in == nullptr || gy == nullptr))
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "null device pointer");
    g = WgradGeometry{batch, channel, in_h, in_w, out_h, out_w, kernel_h, kernel_w, down_h, down_w,
                      pad_h, pad_w};
    return DWCONV_OK;
}

template <typename T>
size_t wgrad_workspace(const WgradGeometry &g)
{
    size_t need = wgrad_direct_workspace<T>(g);
    if constexpr (!std::is_same<T, double>::value) {
        const size_t t = wgrad_tiled_workspace(g);
        if (t > need) need = t;
        const size_t sm = wgrad_small_workspace(g);
        if (sm > need) need = sm;
        const size_t s2 = bwd_s2_workspace(g);
        if (s2 > need) need = s2;
        const size_t st = bwd_stack_workspace(g);
        if (st > need) need = st;
        const size_t any = wgrad_any_workspace(g, 1, 1);
        if (any > need) need = any;
        if constexpr (sizeof(T) == 2) {
            const size_t t16 = bwd_tiled16_workspace(g);
            if (t16 > need) need = t16;
        }
    } else {
        const size_t f64 = wgrad_f64_workspace(g);
        if (f64 > need) need = f64;
    }
    return need;
}

template <typename T>
int wgrad_any(const T *in, const T *gy, T *gw, void *ws, size_t ws_bytes, int batch, int channel,
              int in_h, int in_w, int out_h, int out_w, int kernel_h, int kernel_w, int up_h, int up_w,
              int down_h, int down_w, int pad_h, int pad_w, void *stream_)
{
    WgradGeometry g;
    const int rc = make_wgrad_geometry(g, in, gy, gw, batch, channel, in_h, in_w, out_h, out_w, kernel_h,
                                       kernel_w, up_h, up_w, down_h, down_w, pad_h, pad_w);
    if (rc != DWCONV_OK) return rc;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const long taps = static_cast<long>(channel) * kernel_h * kernel_w;
    if (taps == 0) {
        note_variant("empty");
        return DWCONV_OK;
    }
    if (1ll * batch * out_h * out_w == 0 || in_h == 0 || in_w == 0) {
        // nothing to sum: the gradient is zero (a fill kernel, not a memset node,
        // so that the call may be captured into a graph)
        note_variant("zero");
        return launch_fill_zero(gw, static_cast<size_t>(taps) * sizeof(T), stream);
    }
    if constexpr (!std::is_same<T, double>::value) {
        if (!force_generic()) {
            if (wgrad_small_workspace(g) > 0) {
                const int r = try_launch_wgrad_small<T>(in, gy, gw, ws, ws_bytes, g, stream);
                if (r >= 0) return r;
            }
            if (wgrad_tiled_workspace(g) > 0) {
                const int r = try_launch_wgrad_tiled<T>(in, gy, gw, ws, ws_bytes, g, stream);
                if (r >= 0) return r;
            }
            const int r = try_launch_wgrad_any<T>(in, gy, gw, ws, ws_bytes, g, 1, 1, stream);
            if (r >= 0) return r;
        }
    } else if (!force_generic()) {
        const int r = try_launch_wgrad_f64(in, gy, gw, ws, ws_bytes, g, stream);
        if (r >= 0) return r;
    }
    return launch_wgrad_direct<T>(in, gy, gw, ws, ws_bytes, g, stream);
}

// Both gradients of one layer.  Fused kernels where they exist; otherwise the two separate passes.
template <typename T>  // float, half_t or bf16_t
int backward_any(const T *in, const T *gy, const T *taps, T *gx, T *gw, void *ws, size_t ws_bytes, int batch,
                 int channel, int in_h, int in_w, int out_h, int out_w, int kernel_h, int kernel_w, int stride_h,
                 int stride_w, int pad_h, int pad_w, void *stream_)
{
    WgradGeometry g;
    int rc = make_wgrad_geometry(g, in, gy, gw, batch, channel, in_h, in_w, out_h, out_w, kernel_h, kernel_w, 1, 1,
                                 stride_h, stride_w, pad_h, pad_w);
    if (rc != DWCONV_OK) return rc;
    if (dwconv_out_size(in_h, 1, stride_h, pad_h, pad_h, kernel_h) != out_h ||
        dwconv_out_size(in_w, 1, stride_w, pad_w, pad_w, kernel_w) != out_w)
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "out_grad extent %dx%d does not match the convolution geometry",
                    out_h, out_w);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const bool has_work = 1ll * batch * channel * out_h * out_w > 0 && in_h > 0 && in_w > 0;
    if (has_work && !force_generic()) {
        if (taps == nullptr || gx == nullptr) return fail(DWCONV_ERR_INVALID_ARGUMENT, "null device pointer");
        rc = try_launch_bwd_small<T>(in, gy, taps, gx, gw, ws, ws_bytes, g, stream);
        if (rc >= 0) return rc;
        if constexpr (sizeof(T) == 2) {
            rc = try_launch_bwd_tiled16<T>(in, gy, taps, gx, gw, ws, ws_bytes, g, stream);
            if (rc >= 0) return rc;
        }
        rc = try_launch_bwd_stack<T>(in, gy, taps, gx, gw, ws, ws_bytes, g, stream);
        if (rc >= 0) return rc;
        rc = try_launch_bwd_tiled<T>(in, gy, taps, gx, gw, ws, ws_bytes, g, stream);
        if (rc >= 0) return rc;
        rc = try_launch_bwd_s2<T>(in, gy, taps, gx, gw, ws, ws_bytes, g, stream);
        if (rc >= 0) return rc;
    }
    // grad-input as the transposed problem (torch_dwconv/dwconv.py:39-44, :61-64), then grad-weight
    rc = dwconv2d_any<T>(gy, taps, gx, batch, channel, out_h, out_w, kernel_h, kernel_w, stride_h, stride_w, 1, 1,
                             kernel_h - pad_h - 1, in_h - out_h * stride_h + pad_h, kernel_w - pad_w - 1,
                             in_w - out_w * stride_w + pad_w, 0, stream_);
    if (rc != DWCONV_OK) return rc;
    char first[sizeof(g_variant)];
    std::snprintf(first, sizeof(first), "%s", g_variant);
    rc = wgrad_any<T>(in, gy, gw, ws, ws_bytes, batch, channel, in_h, in_w, out_h, out_w, kernel_h, kernel_w, 1, 1,
                          stride_h, stride_w, pad_h, pad_w, stream_);
    if (rc == DWCONV_OK) {
        char second[sizeof(g_variant)];
        std::snprintf(second, sizeof(second), "%s", g_variant);
        note_variant("%.120s + %.120s", first, second);
    }
    return rc;
}

// ---- channels-last entry points ----
int make_nhwc_geometry(NhwcGeometry &g, int batch, int channel, int in_h, int in_w, int kernel_h, int kernel_w,
                       int stride_h, int stride_w, int pad_h, int pad_w)
{
    if (batch < 0 || channel < 0 || in_h < 0 || in_w < 0)
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "negative tensor extent (batch %d, channel %d, input %dx%d)", batch,
                    channel, in_h, in_w);
    if (kernel_h < 1 || kernel_w < 1)
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "kernel extent must be >= 1, got %dx%d", kernel_h, kernel_w);
    if (stride_h < 1 || stride_w < 1)
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "stride must be >= 1, got %dx%d", stride_h, stride_w);
    if (pad_h < 0 || pad_w < 0) return fail(DWCONV_ERR_INVALID_ARGUMENT, "padding must be >= 0, got %dx%d", pad_h, pad_w);
    g = NhwcGeometry{batch, channel, in_h, in_w, 0, 0, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w};
    g.out_h = std::max(0, dwconv_out_size(in_h, 1, stride_h, pad_h, pad_h, kernel_h));
    g.out_w = std::max(0, dwconv_out_size(in_w, 1, stride_w, pad_w, pad_w, kernel_w));
    if (1ll * batch * channel * in_h * in_w >= (1ll << 40) || 1ll * batch * channel * g.out_h * g.out_w >= (1ll << 40))
        return fail(DWCONV_ERR_UNSUPPORTED, "tensor too large");
    return DWCONV_OK;
}

template <typename T>
int nhwc_forward_any(const T *in, const T *taps, T *out, int batch, int channel, int in_h, int in_w, int kernel_h,
                     int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w, void *stream,
                     const Epilogue &epi = Epilogue{})
{
    NhwcGeometry g;
    const int rc = make_nhwc_geometry(g, batch, channel, in_h, in_w, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w);
    if (rc != DWCONV_OK) return rc;
    g.epi = epi;
    const long long out_elems = 1ll * batch * channel * g.out_h * g.out_w;
    if (out_elems > 0 && (in == nullptr || taps == nullptr || out == nullptr))
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "null device pointer");
    return nhwc_forward<T>(in, taps, out, g, static_cast<hipStream_t>(stream));
}

template <typename T>
int nhwc_backward_any(const T *in, const T *gy, const T *taps, T *gx, T *gw, void *ws, size_t ws_bytes, int batch,
                      int channel, int in_h, int in_w, int out_h, int out_w, int kernel_h, int kernel_w, int stride_h,
                      int stride_w, int pad_h, int pad_w, void *stream_)
{
    NhwcGeometry g;
    int rc = make_nhwc_geometry(g, batch, channel, in_h, in_w, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w);
    if (rc != DWCONV_OK) return rc;
    if (g.out_h != std::max(0, out_h) || g.out_w != std::max(0, out_w))
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "out_grad extent %dx%d does not match the convolution geometry", out_h,
                    out_w);
    if (gx == nullptr && gw == nullptr) return fail(DWCONV_ERR_INVALID_ARGUMENT, "neither in_grad nor kernel_grad given");
    const bool has_out = 1ll * batch * channel * g.out_h * g.out_w > 0;
    if (has_out && gy == nullptr) return fail(DWCONV_ERR_INVALID_ARGUMENT, "null device pointer");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    char first[sizeof(g_variant)] = "";
    if (gx != nullptr && gw != nullptr && has_out && in != nullptr && taps != nullptr) {
        rc = nhwc_backward_fused<T>(in, gy, taps, gx, gw, ws, ws_bytes, g, stream);
        if (rc >= 0) return rc;
    }
    if (gx != nullptr) {
        if (has_out && taps == nullptr) return fail(DWCONV_ERR_INVALID_ARGUMENT, "null device pointer");
        rc = nhwc_grad_input<T>(gy, taps, gx, g, stream);
        if (rc != DWCONV_OK) return rc;
        std::snprintf(first, sizeof(first), "%s", g_variant);
    }
    if (gw != nullptr) {
        if (has_out && in_h > 0 && in_w > 0 && in == nullptr) return fail(DWCONV_ERR_INVALID_ARGUMENT, "null device pointer");
        rc = nhwc_grad_weight<T>(in, gy, gw, ws, ws_bytes, g, stream);
        if (rc != DWCONV_OK) return rc;
        if (gx != nullptr) {
            char second[sizeof(g_variant)];
            std::snprintf(second, sizeof(second), "%s", g_variant);
            note_variant("%.120s + %.120s", first, second);
        }
    }
    return DWCONV_OK;
}

// ---- dilation and depth multiplier ----
int make_general_geometry(GeneralGeometry &g, int batch, int channel, int in_h, int in_w, int multiplier, int kernel_h,
                          int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w)
{
    if (batch < 0 || channel < 0 || in_h < 0 || in_w < 0)
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "negative tensor extent (batch %d, channel %d, input %dx%d)", batch,
                    channel, in_h, in_w);
    if (multiplier < 1) return fail(DWCONV_ERR_INVALID_ARGUMENT, "depth multiplier must be >= 1, got %d", multiplier);
    if (kernel_h < 1 || kernel_w < 1)
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "kernel extent must be >= 1, got %dx%d", kernel_h, kernel_w);
    if (stride_h < 1 || stride_w < 1 || dil_h < 1 || dil_w < 1)
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "stride and dilation must be >= 1, got stride %dx%d dilation %dx%d",
                    stride_h, stride_w, dil_h, dil_w);
    if (pad_h < 0 || pad_w < 0) return fail(DWCONV_ERR_INVALID_ARGUMENT, "padding must be >= 0, got %dx%d", pad_h, pad_w);
    g = GeneralGeometry{batch, channel, multiplier, in_h, in_w, 0, 0, kernel_h, kernel_w, stride_h, stride_w,
                        pad_h, pad_w, dil_h, dil_w};
    const long span_h = 1l * dil_h * (kernel_h - 1) + 1, span_w = 1l * dil_w * (kernel_w - 1) + 1;
    const long oh = in_h + 2l * pad_h - span_h, ow = in_w + 2l * pad_w - span_w;
    g.out_h = oh < 0 ? 0 : static_cast<int>(oh / stride_h + 1);
    g.out_w = ow < 0 ? 0 : static_cast<int>(ow / stride_w + 1);
    if (1ll * batch * channel * in_h * in_w >= (1ll << 40) ||
        1ll * batch * channel * multiplier * g.out_h * g.out_w >= (1ll << 40) ||
        1ll * channel * multiplier * kernel_h * kernel_w >= (1ll << 31))
        return fail(DWCONV_ERR_UNSUPPORTED, "tensor too large");
    return DWCONV_OK;
}

inline bool is_plain(const GeneralGeometry &g) { return g.multiplier == 1 && g.dil_h == 1 && g.dil_w == 1; }
// multiplier 1, stride 1, the same dilation above 1 on both axes: what the whole-plane kernels may take
inline bool dilated_small(const GeneralGeometry &g)
{
    return g.multiplier == 1 && g.dil_h == g.dil_w && g.dil_h > 1 && g.stride_h == 1 && g.stride_w == 1 &&
           g.kernel_h == g.kernel_w && g.in_w <= 32;
}
inline WgradGeometry dilated_wgrad_geometry(const GeneralGeometry &g)
{
    WgradGeometry w{g.batch, g.channel, g.in_h, g.in_w, g.out_h, g.out_w, g.kernel_h, g.kernel_w, 1, 1, g.pad_h, g.pad_w};
    w.dil = g.dil_h;
    return w;
}

// Depth multiplier above 1 with the taps at dilation 1, square filters and one stride of 1 or 2: what the tiled
// kernels may take on maps large enough for one plane per tile (Geometry::mult, WgradGeometry::mult).
inline bool multiplied_tiled(const GeneralGeometry &g)
{
    return g.multiplier > 1 && g.dil_h == 1 && g.dil_w == 1 && g.kernel_h == g.kernel_w && g.stride_h == g.stride_w &&
           (g.stride_h == 1 || g.stride_h == 2);
}
inline WgradGeometry multiplied_wgrad_geometry(const GeneralGeometry &g)
{
    WgradGeometry w{g.batch, g.channel * g.multiplier, g.in_h, g.in_w, g.out_h, g.out_w, g.kernel_h, g.kernel_w,
                    g.stride_h, g.stride_w, g.pad_h, g.pad_w};
    w.mult = g.multiplier;
    return w;
}

template <typename T>
int general_forward_any(const T *in, const T *taps, T *out, int batch, int channel, int in_h, int in_w, int multiplier,
                        int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w, int dil_h,
                        int dil_w, void *stream)
{
    GeneralGeometry g;
    const int rc = make_general_geometry(g, batch, channel, in_h, in_w, multiplier, kernel_h, kernel_w, stride_h,
                                         stride_w, pad_h, pad_w, dil_h, dil_w);
    if (rc != DWCONV_OK) return rc;
    if (is_plain(g))  // the tuned kernels
        return dwconv2d_any<T>(in, taps, out, batch, channel, in_h, in_w, kernel_h, kernel_w, 1, 1, stride_h, stride_w,
                               pad_h, pad_h, pad_w, pad_w, 1, stream);
    const long long out_elems = 1ll * batch * channel * multiplier * g.out_h * g.out_w;
    if (out_elems > 0 && (in == nullptr || taps == nullptr || out == nullptr))
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "null device pointer");
    if constexpr (!std::is_same<T, double>::value) {
        if (!force_generic() && out_elems > 0) {
            int r = try_launch_general_stack_forward<T>(in, taps, out, g, static_cast<hipStream_t>(stream));
            if (r >= 0) return r;
            if (dilated_small(g)) {
                const Geometry gg{batch, channel, in_h, in_w, kernel_h, kernel_w, 1, 1, 1, 1, pad_h, pad_h, pad_w, pad_w,
                                  g.out_h, g.out_w, 1};
                r = try_launch_fir_small<T>(in, taps, out, gg, static_cast<hipStream_t>(stream), g.dil_h);
                if (r >= 0) return r;
            }
            if (multiplied_tiled(g)) {
                Geometry gg{batch, channel * multiplier, in_h, in_w, kernel_h, kernel_w, 1, 1, stride_h, stride_w,
                            pad_h, pad_h, pad_w, pad_w, g.out_h, g.out_w, 1};
                gg.mult = multiplier;
                r = try_launch_fir_tiled<T>(in, taps, out, gg, static_cast<hipStream_t>(stream));
                if (r >= 0) return r;
            }
            if (multiplier == 1) {  // any other dilation, stride or filter extent: the any-geometry tiled kernel
                Geometry gg{batch, channel, in_h, in_w, kernel_h, kernel_w, 1, 1, stride_h, stride_w,
                            pad_h, pad_h, pad_w, pad_w, g.out_h, g.out_w, 1};
                gg.dil_h = dil_h;
                gg.dil_w = dil_w;
                r = try_launch_fir_any<T>(in, taps, out, gg, static_cast<hipStream_t>(stream));
                if (r >= 0) return r;
            }
        }
    }
    if (!force_generic() && out_elems > 0 && multiplier == 1) {
        // the one-column-per-lane tiled kernel: double tensors, and what the kernels above left of the other types
        Geometry gg{batch, channel, in_h, in_w, kernel_h, kernel_w, 1, 1, stride_h, stride_w,
                    pad_h, pad_h, pad_w, pad_w, g.out_h, g.out_w, 1};
        gg.dil_h = dil_h;
        gg.dil_w = dil_w;
        const int r = try_launch_fir_lds<T>(in, taps, out, gg, static_cast<hipStream_t>(stream));
        if (r >= 0) return r;
    }
    return general_forward<T>(in, taps, out, g, static_cast<hipStream_t>(stream));
}

template <typename T>
size_t general_workspace_any(const GeneralGeometry &g)
{
    if (is_plain(g)) {
        const WgradGeometry w{g.batch, g.channel, g.in_h, g.in_w, g.out_h, g.out_w, g.kernel_h, g.kernel_w,
                              g.stride_h, g.stride_w, g.pad_h, g.pad_w};
        return wgrad_workspace<T>(w);
    }
    size_t need = general_grad_weight_workspace<T>(g);
    if constexpr (!std::is_same<T, double>::value) {
        const size_t st = general_stack_workspace(g);
        if (st > need) need = st;
        if (dilated_small(g)) {
            const size_t sm = wgrad_small_workspace(dilated_wgrad_geometry(g));
            if (sm > need) need = sm;
        }
        if (g.multiplier == 1) {
            const WgradGeometry wg{g.batch, g.channel, g.in_h, g.in_w, g.out_h, g.out_w, g.kernel_h, g.kernel_w,
                                   g.stride_h, g.stride_w, g.pad_h, g.pad_w};
            const size_t any = wgrad_any_workspace(wg, g.dil_h, g.dil_w);
            if (any > need) need = any;
        }
        if (multiplied_tiled(g)) {
            const size_t mt = wgrad_tiled_workspace(multiplied_wgrad_geometry(g));
            if (mt > need) need = mt;
        }
    } else if (g.multiplier == 1) {
        const WgradGeometry wg{g.batch, g.channel, g.in_h, g.in_w, g.out_h, g.out_w, g.kernel_h, g.kernel_w,
                               g.stride_h, g.stride_w, g.pad_h, g.pad_w};
        const size_t f64 = wgrad_f64_workspace(wg, g.dil_h, g.dil_w);
        if (f64 > need) need = f64;
    }
    return need;
}

template <typename T>
int general_backward_any(const T *in, const T *gy, const T *taps, T *gx, T *gw, void *ws, size_t ws_bytes, int batch,
                         int channel, int in_h, int in_w, int out_h, int out_w, int multiplier, int kernel_h,
                         int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w,
                         void *stream_)
{
    GeneralGeometry g;
    int rc = make_general_geometry(g, batch, channel, in_h, in_w, multiplier, kernel_h, kernel_w, stride_h, stride_w,
                                   pad_h, pad_w, dil_h, dil_w);
    if (rc != DWCONV_OK) return rc;
    if (g.out_h != std::max(0, out_h) || g.out_w != std::max(0, out_w))
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "out_grad extent %dx%d does not match the convolution geometry", out_h,
                    out_w);
    if (gx == nullptr || gw == nullptr) return fail(DWCONV_ERR_INVALID_ARGUMENT, "null gradient pointer");
    if (is_plain(g)) {
        if constexpr (std::is_same<T, double>::value) {
            // fp64 has no combined kernel: the two passes of the reference's backward (torch_dwconv/dwconv.py:56-68)
            rc = dwconv2d_any<T>(gy, taps, gx, batch, channel, out_h, out_w, kernel_h, kernel_w, stride_h, stride_w, 1,
                                 1, kernel_h - pad_h - 1, in_h - out_h * stride_h + pad_h, kernel_w - pad_w - 1,
                                 in_w - out_w * stride_w + pad_w, 0, stream_);
            if (rc != DWCONV_OK) return rc;
            return wgrad_any<T>(in, gy, gw, ws, ws_bytes, batch, channel, in_h, in_w, out_h, out_w, kernel_h, kernel_w,
                                1, 1, stride_h, stride_w, pad_h, pad_w, stream_);
        } else {
            return backward_any<T>(in, gy, taps, gx, gw, ws, ws_bytes, batch, channel, in_h, in_w, out_h, out_w,
                                   kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w, stream_);
        }
    }
    const bool has_out = 1ll * batch * channel * multiplier * g.out_h * g.out_w > 0;
    if (has_out && (gy == nullptr || taps == nullptr || (in_h > 0 && in_w > 0 && in == nullptr)))
        return fail(DWCONV_ERR_INVALID_ARGUMENT, "null device pointer");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if constexpr (!std::is_same<T, double>::value) {
        if (has_out && !force_generic()) {
            rc = try_launch_general_stack_backward<T>(in, gy, taps, gx, gw, ws, ws_bytes, g, stream);
            if (rc >= 0) return rc;
            if (dilated_small(g)) {
                rc = try_launch_bwd_small<T>(in, gy, taps, gx, gw, ws, ws_bytes, dilated_wgrad_geometry(g), stream);
                if (rc >= 0) return rc;
            }
            if (multiplied_tiled(g)) {
                // the two passes on their own; either falls back to the per-element kernels where the tiled one
                // does not take the shape
                const int s = g.stride_h;
                Geometry gi{batch, channel, g.out_h, g.out_w, kernel_h, kernel_w, s, s, 1, 1, kernel_h - pad_h - 1,
                            in_h - g.out_h * s + pad_h, kernel_w - pad_w - 1, in_w - g.out_w * s + pad_w, in_h, in_w, 0};
                gi.mult = multiplier;
                rc = gi.pad_h1 >= 0 && gi.pad_w1 >= 0 ? try_launch_fir_tiled<T>(gy, taps, gx, gi, stream) : -1;
                if (rc < 0) rc = general_grad_input<T>(gy, taps, gx, g, stream);
                if (rc != DWCONV_OK) return rc;
                char first[sizeof(g_variant)];
                std::snprintf(first, sizeof(first), "%s", g_variant);
                rc = try_launch_wgrad_tiled<T>(in, gy, gw, ws, ws_bytes, multiplied_wgrad_geometry(g), stream);
                if (rc < 0) rc = general_grad_weight<T>(in, gy, gw, ws, ws_bytes, g, stream);
                if (rc != DWCONV_OK) return rc;
                char second[sizeof(g_variant)];
                std::snprintf(second, sizeof(second), "%s", g_variant);
                note_variant("%.120s + %.120s", first, second);
                return DWCONV_OK;
            }
            if (multiplier == 1 && in_h > 0 && in_w > 0) {
                // any other dilation, stride or filter extent: the two passes through the any-geometry tiled kernels
                // (grad-input of a stride-1 layer is the correlation with the rotated taps; above stride 1 it stays
                // with the gather kernel); either falls back to the per-element kernels
                rc = -1;
                if (stride_h == 1 && stride_w == 1) {
                    Geometry gi{batch, channel, g.out_h, g.out_w, kernel_h, kernel_w, 1, 1, 1, 1,
                                dil_h * (kernel_h - 1) - pad_h, in_h - g.out_h + pad_h, dil_w * (kernel_w - 1) - pad_w,
                                in_w - g.out_w + pad_w, in_h, in_w, 0};
                    gi.dil_h = dil_h;
                    gi.dil_w = dil_w;
                    if (gi.pad_h0 >= 0 && gi.pad_w0 >= 0) rc = try_launch_fir_any<T>(gy, taps, gx, gi, stream);
                }
                if (rc < 0) rc = general_grad_input<T>(gy, taps, gx, g, stream);
                if (rc != DWCONV_OK) return rc;
                char first[sizeof(g_variant)];
                std::snprintf(first, sizeof(first), "%s", g_variant);
                const WgradGeometry wg{batch, channel, in_h, in_w, g.out_h, g.out_w, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w};
                rc = try_launch_wgrad_any<T>(in, gy, gw, ws, ws_bytes, wg, dil_h, dil_w, stream);
                if (rc < 0) rc = general_grad_weight<T>(in, gy, gw, ws, ws_bytes, g, stream);
                if (rc != DWCONV_OK) return rc;
                char second[sizeof(g_variant)];
                std::snprintf(second, sizeof(second), "%s", g_variant);
                note_variant("%.120s + %.120s", first, second);
                return DWCONV_OK;
            }
        }
    }
    if constexpr (std::is_same<T, double>::value) {
        if (has_out && !force_generic() && multiplier == 1 && in_h > 0 && in_w > 0) {
            // double tensors: grad-input of a stride-1 layer as the correlation with the rotated, dilated taps, and
            // grad-weight, through the fp64 tiled kernels; either falls back to the per-element kernels
            rc = -1;
            if (stride_h == 1 && stride_w == 1) {
                Geometry gi{batch, channel, g.out_h, g.out_w, kernel_h, kernel_w, 1, 1, 1, 1,
                            dil_h * (kernel_h - 1) - pad_h, in_h - g.out_h + pad_h, dil_w * (kernel_w - 1) - pad_w,
                            in_w - g.out_w + pad_w, in_h, in_w, 0};
                gi.dil_h = dil_h;
                gi.dil_w = dil_w;
                rc = try_launch_fir_lds<T>(gy, taps, gx, gi, stream);
            }
            if (rc < 0) rc = general_grad_input<T>(gy, taps, gx, g, stream);
            if (rc != DWCONV_OK) return rc;
            char first[sizeof(g_variant)];
            std::snprintf(first, sizeof(first), "%s", g_variant);
            const WgradGeometry wg{batch, channel, in_h, in_w, g.out_h, g.out_w, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w};
            rc = try_launch_wgrad_f64(in, gy, gw, ws, ws_bytes, wg, stream, dil_h, dil_w);
            if (rc < 0) rc = general_grad_weight<T>(in, gy, gw, ws, ws_bytes, g, stream);
            if (rc != DWCONV_OK) return rc;
            char second[sizeof(g_variant)];
            std::snprintf(second, sizeof(second), "%s", g_variant);
            note_variant("%.120s + %.120s", first, second);
            return DWCONV_OK;
        }
    }
    rc = general_grad_input<T>(gy, taps, gx, g, stream);
    if (rc != DWCONV_OK) return rc;
    return general_grad_weight<T>(in, gy, gw, ws, ws_bytes, g, stream);
}

}  // namespace
}  // namespace dwconv

// ---- scratch memory of the entry point that allocates nothing -------------------------------------------
// Partial grad-weight sums of dwconv2d_backward_noalloc_f32 live in this array instead of a caller's
// workspace.  Every device the library runs on holds its own copy, at its own address, until the process
// ends.  In host code the name is only a handle for hipGetSymbolAddress: kernels and copies get the
// per-device address that call returns, never the name itself.
static __device__ __align__(256) unsigned char scratch[DWCONV_NOALLOC_SCRATCH_BYTES];

namespace dwconv {
namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

// Address of `scratch` on the current device (looked up once per device).  The lookup is not a call to make
// while `stream` records a graph: a first call that arrives under capture is refused instead.
int scratch_of_current_device(void **ptr, hipStream_t stream)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(DWCONV_ERR_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(DWCONV_ERR_UNSUPPORTED, "device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        e = hipStreamIsCapturing(stream, &capture);
        if (e != hipSuccess) return fail(DWCONV_ERR_LAUNCH, "hipStreamIsCapturing: %s", hipGetErrorString(e));
        if (capture != hipStreamCaptureStatusNone)
            return fail(DWCONV_ERR_UNSUPPORTED,
                        "dwconv2d_backward_noalloc_f32: the first call on device %d looks up the scratch buffer's "
                        "address and must be made outside stream capture",
                        dev);
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr)
            return fail(DWCONV_ERR_LAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return DWCONV_OK;
}

}  // namespace
}  // namespace dwconv

using namespace dwconv;

extern "C" {

const char *dwconv_last_error(void) { return g_error; }
const char *dwconv_last_variant(void) { return g_variant; }
const char *dwconv_version(void) { return "dwconv_hip 0.1 gfx950"; }

int dwconv_out_size(int in, int up, int down, int pad0, int pad1, int k)
{
    if (down < 1) return 0;
    return (in * up + pad0 + pad1 - k + down) / down;
}

int dwconv_use_dwconv2d_small(int in_h, int in_w, int kernel_h, int kernel_w, int up_h, int up_w,
                              int down_h, int down_w, int pad_h, int pad_w)
{
    if (down_h != 1 || down_w != 1) return 0;
    if (in_h > 32 || in_w > 32) return 0;
    if (pad_h < 0 || pad_h >= kernel_h || pad_w < 0 || pad_w >= kernel_w) return 0;
    const int out_h = dwconv_out_size(in_h, up_h, 1, pad_h, pad_h, kernel_h);
    const int out_w = dwconv_out_size(in_w, up_w, 1, pad_w, pad_w, kernel_w);
    if (out_h != in_h || out_w != in_w) return 0;
    // the reference's lane budget: one lane per two rows must cover the taps
    return kernel_h * kernel_w <= (in_h + 1) / 2 * in_w ? 1 : 0;
}

int dwconv2d_f32(const float *input, const float *kernel, float *out, int batch, int channel,
                 int in_h, int in_w, int kernel_h, int kernel_w, int up_h, int up_w, int down_h,
                 int down_w, int pad_h0, int pad_h1, int pad_w0, int pad_w1, int forward, void *stream)
{
    return dwconv2d_any<float>(input, kernel, out, batch, channel, in_h, in_w, kernel_h, kernel_w, up_h,
                               up_w, down_h, down_w, pad_h0, pad_h1, pad_w0, pad_w1, forward, stream);
}

int dwconv2d_f64(const double *input, const double *kernel, double *out, int batch, int channel,
                 int in_h, int in_w, int kernel_h, int kernel_w, int up_h, int up_w, int down_h,
                 int down_w, int pad_h0, int pad_h1, int pad_w0, int pad_w1, int forward, void *stream)
{
    return dwconv2d_any<double>(input, kernel, out, batch, channel, in_h, in_w, kernel_h, kernel_w, up_h,
                                up_w, down_h, down_w, pad_h0, pad_h1, pad_w0, pad_w1, forward, stream);
}

int dwconv2d_small_f32(const float *input, const float *kernel, float *out, int batch, int channel,
                       int in_h, int in_w, int kernel_h, int kernel_w, int up_h, int up_w, int down_h,
                       int down_w, int pad_h, int pad_w, int forward, void *stream)
{
    return dwconv2d_small_any<float>(input, kernel, out, batch, channel, in_h, in_w, kernel_h, kernel_w,
                                     up_h, up_w, down_h, down_w, pad_h, pad_w, forward, stream);
}

int dwconv2d_small_f64(const double *input, const double *kernel, double *out, int batch, int channel,
                       int in_h, int in_w, int kernel_h, int kernel_w, int up_h, int up_w, int down_h,
                       int down_w, int pad_h, int pad_w, int forward, void *stream)
{
    return dwconv2d_small_any<double>(input, kernel, out, batch, channel, in_h, in_w, kernel_h, kernel_w,
                                      up_h, up_w, down_h, down_w, pad_h, pad_w, forward, stream);
}

size_t dwconv2d_backward_kernel_workspace_bytes(int batch, int channel, int in_h, int in_w, int out_h,
                                                int out_w, int kernel_h, int kernel_w, int down_h,
                                                int down_w, int pad_h, int pad_w, int elem_size)
{
    if (batch <= 0 || channel <= 0 || kernel_h < 1 || kernel_w < 1 || down_h < 1 || down_w < 1) return 0;
    const WgradGeometry g{batch, channel, in_h, in_w, out_h, out_w, kernel_h, kernel_w,
                          down_h, down_w, pad_h, pad_w};
    if (elem_size == 8) return wgrad_workspace<double>(g);
    if (elem_size == 2) return wgrad_workspace<half_t>(g);
    return wgrad_workspace<float>(g);
}

int dwconv2d_backward_kernel_f32(const float *input, const float *out_grad, float *kernel_grad,
                                 void *workspace, size_t workspace_bytes, int batch, int channel,
                                 int in_h, int in_w, int out_h, int out_w, int kernel_h, int kernel_w,
                                 int up_h, int up_w, int down_h, int down_w, int pad_h, int pad_w,
                                 void *stream)
{
    return wgrad_any<float>(input, out_grad, kernel_grad, workspace, workspace_bytes, batch, channel,
                            in_h, in_w, out_h, out_w, kernel_h, kernel_w, up_h, up_w, down_h, down_w,
                            pad_h, pad_w, stream);
}

int dwconv2d_backward_kernel_f64(const double *input, const double *out_grad, double *kernel_grad,
                                 void *workspace, size_t workspace_bytes, int batch, int channel,
                                 int in_h, int in_w, int out_h, int out_w, int kernel_h, int kernel_w,
                                 int up_h, int up_w, int down_h, int down_w, int pad_h, int pad_w,
                                 void *stream)
{
    return wgrad_any<double>(input, out_grad, kernel_grad, workspace, workspace_bytes, batch, channel,
                             in_h, in_w, out_h, out_w, kernel_h, kernel_w, up_h, up_w, down_h, down_w,
                             pad_h, pad_w, stream);
}

// ---- 16-bit element types (storage passed as unsigned short) ----
#define DWCONV_16BIT_ENTRY_POINTS(SUFFIX, TYPE)                                                                       \
    int dwconv2d_##SUFFIX(const unsigned short *input, const unsigned short *kernel, unsigned short *out, int batch,   \
                          int channel, int in_h, int in_w, int kernel_h, int kernel_w, int up_h, int up_w, int down_h, \
                          int down_w, int pad_h0, int pad_h1, int pad_w0, int pad_w1, int forward, void *stream)       \
    {                                                                                                                  \
        return dwconv2d_any<TYPE>(reinterpret_cast<const TYPE *>(input), reinterpret_cast<const TYPE *>(kernel),       \
                                  reinterpret_cast<TYPE *>(out), batch, channel, in_h, in_w, kernel_h, kernel_w, up_h, \
                                  up_w, down_h, down_w, pad_h0, pad_h1, pad_w0, pad_w1, forward, stream);              \
    }                                                                                                                  \
    int dwconv2d_small_##SUFFIX(const unsigned short *input, const unsigned short *kernel, unsigned short *out,        \
                                int batch, int channel, int in_h, int in_w, int kernel_h, int kernel_w, int up_h,      \
                                int up_w, int down_h, int down_w, int pad_h, int pad_w, int forward, void *stream)     \
    {                                                                                                                  \
        return dwconv2d_small_any<TYPE>(reinterpret_cast<const TYPE *>(input), reinterpret_cast<const TYPE *>(kernel), \
                                        reinterpret_cast<TYPE *>(out), batch, channel, in_h, in_w, kernel_h, kernel_w, \
                                        up_h, up_w, down_h, down_w, pad_h, pad_w, forward, stream);                    \
    }                                                                                                                  \
    int dwconv2d_backward_kernel_##SUFFIX(const unsigned short *input, const unsigned short *out_grad,                 \
                                          unsigned short *kernel_grad, void *workspace, size_t workspace_bytes,        \
                                          int batch, int channel, int in_h, int in_w, int out_h, int out_w,            \
                                          int kernel_h, int kernel_w, int up_h, int up_w, int down_h, int down_w,      \
                                          int pad_h, int pad_w, void *stream)                                          \
    {                                                                                                                  \
        return wgrad_any<TYPE>(reinterpret_cast<const TYPE *>(input), reinterpret_cast<const TYPE *>(out_grad),        \
                               reinterpret_cast<TYPE *>(kernel_grad), workspace, workspace_bytes, batch, channel,      \
                               in_h, in_w, out_h, out_w, kernel_h, kernel_w, up_h, up_w, down_h, down_w, pad_h, pad_w, \
                               stream);                                                                                \
    }                                                                                                                  \
    int dwconv2d_backward_##SUFFIX(const unsigned short *input, const unsigned short *out_grad,                        \
                                   const unsigned short *kernel, unsigned short *in_grad,                              \
                                   unsigned short *kernel_grad, void *workspace, size_t workspace_bytes, int batch,    \
                                   int channel, int in_h, int in_w, int out_h, int out_w, int kernel_h, int kernel_w,  \
                                   int stride_h, int stride_w, int pad_h, int pad_w, void *stream)                     \
    {                                                                                                                  \
        return backward_any<TYPE>(reinterpret_cast<const TYPE *>(input), reinterpret_cast<const TYPE *>(out_grad),     \
                                  reinterpret_cast<const TYPE *>(kernel), reinterpret_cast<TYPE *>(in_grad),           \
                                  reinterpret_cast<TYPE *>(kernel_grad), workspace, workspace_bytes, batch, channel,   \
                                  in_h, in_w, out_h, out_w, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w,      \
                                  stream);                                                                             \
    }
DWCONV_16BIT_ENTRY_POINTS(f16, half_t)
DWCONV_16BIT_ENTRY_POINTS(bf16, bf16_t)
#undef DWCONV_16BIT_ENTRY_POINTS

int dwconv2d_backward_f32(const float *input, const float *out_grad, const float *kernel, float *in_grad,
                          float *kernel_grad, void *workspace, size_t workspace_bytes, int batch, int channel,
                          int in_h, int in_w, int out_h, int out_w, int kernel_h, int kernel_w, int stride_h,
                          int stride_w, int pad_h, int pad_w, void *stream)
{
    return backward_any<float>(input, out_grad, kernel, in_grad, kernel_grad, workspace, workspace_bytes, batch,
                               channel, in_h, in_w, out_h, out_w, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w,
                               stream);
}

int dwconv2d_backward_noalloc_f32(const float *input, const float *out_grad, const float *kernel, float *in_grad,
                                  float *kernel_grad, int batch, int channel, int in_h, int in_w, int out_h,
                                  int out_w, int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h,
                                  int pad_w, void *stream)
{
    WgradGeometry g;
    const int rc = make_wgrad_geometry(g, input, out_grad, kernel_grad, batch, channel, in_h, in_w, out_h, out_w,
                                       kernel_h, kernel_w, 1, 1, stride_h, stride_w, pad_h, pad_w);
    if (rc != DWCONV_OK) return rc;
    const size_t need = (batch > 0 && channel > 0) ? wgrad_workspace<float>(g) : 0;
    if (need > sizeof(scratch))
        return fail(DWCONV_ERR_WORKSPACE,
                    "dwconv2d_backward_noalloc_f32: this geometry needs %zu bytes of scratch memory, the built-in "
                    "buffer holds %zu; call dwconv2d_backward_f32 with a workspace of your own",
                    need, sizeof(scratch));
    void *ws = nullptr;
    const int rs = scratch_of_current_device(&ws, static_cast<hipStream_t>(stream));
    if (rs != DWCONV_OK) return rs;
    return backward_any<float>(input, out_grad, kernel, in_grad, kernel_grad, ws, sizeof(scratch), batch, channel, in_h,
                               in_w, out_h, out_w, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w, stream);
}

// ---- channels-last tensors ----
size_t dwconv2d_backward_nhwc_workspace_bytes(int batch, int channel, int in_h, int in_w, int kernel_h, int kernel_w,
                                              int stride_h, int stride_w, int pad_h, int pad_w, int elem_size)
{
    NhwcGeometry g;
    if (make_nhwc_geometry(g, batch, channel, in_h, in_w, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w) != DWCONV_OK)
        return 0;
    if (batch == 0 || channel == 0) return 0;
    if (elem_size == 8) return nhwc_grad_weight_workspace<double>(g);
    if (elem_size == 2) return nhwc_grad_weight_workspace<half_t>(g);
    return nhwc_grad_weight_workspace<float>(g);
}

#define DWCONV_NHWC_ENTRY_POINTS(SUFFIX, CTYPE, TYPE)                                                                  \
    int dwconv2d_nhwc_##SUFFIX(const CTYPE *input, const CTYPE *kernel, CTYPE *out, int batch, int channel, int in_h,  \
                               int in_w, int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w, \
                               void *stream)                                                                           \
    {                                                                                                                  \
        return nhwc_forward_any<TYPE>(reinterpret_cast<const TYPE *>(input), reinterpret_cast<const TYPE *>(kernel),   \
                                      reinterpret_cast<TYPE *>(out), batch, channel, in_h, in_w, kernel_h, kernel_w,   \
                                      stride_h, stride_w, pad_h, pad_w, stream);                                       \
    }                                                                                                                  \
    int dwconv2d_backward_nhwc_##SUFFIX(const CTYPE *input, const CTYPE *out_grad, const CTYPE *kernel, CTYPE *in_grad, \
                                        CTYPE *kernel_grad, void *workspace, size_t workspace_bytes, int batch,        \
                                        int channel, int in_h, int in_w, int out_h, int out_w, int kernel_h,           \
                                        int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w, void *stream)  \
    {                                                                                                                  \
        return nhwc_backward_any<TYPE>(reinterpret_cast<const TYPE *>(input), reinterpret_cast<const TYPE *>(out_grad), \
                                       reinterpret_cast<const TYPE *>(kernel), reinterpret_cast<TYPE *>(in_grad),      \
                                       reinterpret_cast<TYPE *>(kernel_grad), workspace, workspace_bytes, batch,       \
                                       channel, in_h, in_w, out_h, out_w, kernel_h, kernel_w, stride_h, stride_w,      \
                                       pad_h, pad_w, stream);                                                          \
    }
DWCONV_NHWC_ENTRY_POINTS(f32, float, float)
DWCONV_NHWC_ENTRY_POINTS(f64, double, double)
DWCONV_NHWC_ENTRY_POINTS(f16, unsigned short, half_t)
DWCONV_NHWC_ENTRY_POINTS(bf16, unsigned short, bf16_t)
#undef DWCONV_NHWC_ENTRY_POINTS

// ---- forward with a fused per-channel scale / shift and activation ----
#define DWCONV_FUSED_ENTRY_POINTS(SUFFIX, CTYPE, TYPE, PTYPE)                                                          \
    int dwconv2d_fused_##SUFFIX(const CTYPE *input, const CTYPE *kernel, const PTYPE *scale, const PTYPE *shift,       \
                                CTYPE *out, int batch, int channel, int in_h, int in_w, int kernel_h, int kernel_w,    \
                                int stride_h, int stride_w, int pad_h, int pad_w, int activation, void *stream)        \
    {                                                                                                                  \
        if (check_activation(activation) != DWCONV_OK) return DWCONV_ERR_INVALID_ARGUMENT;                             \
        Epilogue epi;                                                                                                  \
        epi.scale = scale;                                                                                             \
        epi.shift = shift;                                                                                             \
        epi.act = activation;                                                                                          \
        return dwconv2d_any<TYPE>(reinterpret_cast<const TYPE *>(input), reinterpret_cast<const TYPE *>(kernel),       \
                                  reinterpret_cast<TYPE *>(out), batch, channel, in_h, in_w, kernel_h, kernel_w, 1, 1, \
                                  stride_h, stride_w, pad_h, pad_h, pad_w, pad_w, 1, stream, epi);                     \
    }                                                                                                                  \
    int dwconv2d_fused_nhwc_##SUFFIX(const CTYPE *input, const CTYPE *kernel, const PTYPE *scale, const PTYPE *shift,  \
                                     CTYPE *out, int batch, int channel, int in_h, int in_w, int kernel_h,             \
                                     int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w, int activation,   \
                                     void *stream)                                                                     \
    {                                                                                                                  \
        if (check_activation(activation) != DWCONV_OK) return DWCONV_ERR_INVALID_ARGUMENT;                             \
        Epilogue epi;                                                                                                  \
        epi.scale = scale;                                                                                             \
        epi.shift = shift;                                                                                             \
        epi.act = activation;                                                                                          \
        return nhwc_forward_any<TYPE>(reinterpret_cast<const TYPE *>(input), reinterpret_cast<const TYPE *>(kernel),   \
                                      reinterpret_cast<TYPE *>(out), batch, channel, in_h, in_w, kernel_h, kernel_w,   \
                                      stride_h, stride_w, pad_h, pad_w, stream, epi);                                  \
    }
DWCONV_FUSED_ENTRY_POINTS(f32, float, float, float)
DWCONV_FUSED_ENTRY_POINTS(f64, double, double, double)
DWCONV_FUSED_ENTRY_POINTS(f16, unsigned short, half_t, float)
DWCONV_FUSED_ENTRY_POINTS(bf16, unsigned short, bf16_t, float)
#undef DWCONV_FUSED_ENTRY_POINTS

// ---- backward of the fused epilogue ----
size_t dwconv2d_epilogue_backward_workspace_bytes(int batch, int channel, int out_h, int out_w, int channels_last)
{
    return epilogue_backward_workspace(batch, channel, out_h, out_w, channels_last != 0);
}

#define DWCONV_EPILOGUE_BACKWARD(SUFFIX, CTYPE, TYPE)                                                                  \
    int dwconv2d_epilogue_backward_##SUFFIX(const CTYPE *conv_out, const CTYPE *out_grad, const float *scale,           \
                                            const float *shift, CTYPE *conv_out_grad, float *scale_shift_grad,          \
                                            void *workspace, size_t workspace_bytes, int batch, int channel, int out_h, \
                                            int out_w, int activation, int channels_last, void *stream)                 \
    {                                                                                                                  \
        if (check_activation(activation) != DWCONV_OK) return DWCONV_ERR_INVALID_ARGUMENT;                             \
        if (batch < 0 || channel < 0 || out_h < 0 || out_w < 0)                                                        \
            return fail(DWCONV_ERR_INVALID_ARGUMENT, "negative tensor extent");                                        \
        if (channel > 0 && scale_shift_grad == nullptr) return fail(DWCONV_ERR_INVALID_ARGUMENT, "null gradient pointer"); \
        if (1ll * batch * channel * out_h * out_w == 0) {                                                              \
            note_variant("zero");                                                                                      \
            return launch_fill_zero(scale_shift_grad, static_cast<size_t>(channel) * 2 * sizeof(float),                \
                                    static_cast<hipStream_t>(stream));                                                 \
        }                                                                                                              \
        if (conv_out == nullptr || out_grad == nullptr || conv_out_grad == nullptr)                                    \
            return fail(DWCONV_ERR_INVALID_ARGUMENT, "null device pointer");                                           \
        return epilogue_backward<TYPE>(reinterpret_cast<const TYPE *>(conv_out), reinterpret_cast<const TYPE *>(out_grad), \
                                       scale, shift, reinterpret_cast<TYPE *>(conv_out_grad), scale_shift_grad, workspace, \
                                       workspace_bytes, batch, channel, out_h, out_w, activation, channels_last != 0,  \
                                       static_cast<hipStream_t>(stream));                                              \
    }
DWCONV_EPILOGUE_BACKWARD(f32, float, float)
DWCONV_EPILOGUE_BACKWARD(f16, unsigned short, half_t)
DWCONV_EPILOGUE_BACKWARD(bf16, unsigned short, bf16_t)
#undef DWCONV_EPILOGUE_BACKWARD

// ---- dilation and depth multiplier ----
size_t dwconv2d_general_backward_workspace_bytes(int batch, int channel, int in_h, int in_w, int multiplier,
                                                 int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h,
                                                 int pad_w, int dil_h, int dil_w, int elem_size)
{
    GeneralGeometry g;
    if (make_general_geometry(g, batch, channel, in_h, in_w, multiplier, kernel_h, kernel_w, stride_h, stride_w, pad_h,
                              pad_w, dil_h, dil_w) != DWCONV_OK)
        return 0;
    if (batch == 0 || channel == 0) return 0;
    if (elem_size == 8) return general_workspace_any<double>(g);
    if (elem_size == 2) return general_workspace_any<half_t>(g);
    return general_workspace_any<float>(g);
}

#define DWCONV_GENERAL_ENTRY_POINTS(SUFFIX, CTYPE, TYPE)                                                               \
    int dwconv2d_general_##SUFFIX(const CTYPE *input, const CTYPE *kernel, CTYPE *out, int batch, int channel,         \
                                  int in_h, int in_w, int multiplier, int kernel_h, int kernel_w, int stride_h,        \
                                  int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void *stream)              \
    {                                                                                                                  \
        return general_forward_any<TYPE>(reinterpret_cast<const TYPE *>(input), reinterpret_cast<const TYPE *>(kernel), \
                                         reinterpret_cast<TYPE *>(out), batch, channel, in_h, in_w, multiplier,        \
                                         kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, stream);  \
    }                                                                                                                  \
    int dwconv2d_general_backward_##SUFFIX(const CTYPE *input, const CTYPE *out_grad, const CTYPE *kernel,             \
                                           CTYPE *in_grad, CTYPE *kernel_grad, void *workspace,                        \
                                           size_t workspace_bytes, int batch, int channel, int in_h, int in_w,         \
                                           int out_h, int out_w, int multiplier, int kernel_h, int kernel_w,           \
                                           int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w,     \
                                           void *stream)                                                               \
    {                                                                                                                  \
        return general_backward_any<TYPE>(                                                                             \
            reinterpret_cast<const TYPE *>(input), reinterpret_cast<const TYPE *>(out_grad),                           \
            reinterpret_cast<const TYPE *>(kernel), reinterpret_cast<TYPE *>(in_grad),                                 \
            reinterpret_cast<TYPE *>(kernel_grad), workspace, workspace_bytes, batch, channel, in_h, in_w, out_h,      \
            out_w, multiplier, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, stream);            \
    }
DWCONV_GENERAL_ENTRY_POINTS(f32, float, float)
DWCONV_GENERAL_ENTRY_POINTS(f64, double, double)
DWCONV_GENERAL_ENTRY_POINTS(f16, unsigned short, half_t)
DWCONV_GENERAL_ENTRY_POINTS(bf16, unsigned short, bf16_t)
#undef DWCONV_GENERAL_ENTRY_POINTS

}  // extern "C"
