// Depthwise convolution with a dilation and a depth multiplier: the two options the reference's
// check_options turns away (torch_dwconv/dwconv.py:99-106: "dilations > 1", "in_channels != out_channels").
//
//   out[n, c*M + j, oy, ox] = sum_{ty,tx} in[n, c, oy*s - p + ty*d, ox*s - p + tx*d] * w[c*M + j, ty, tx]
//
// (what F.conv2d(groups=C, dilation=d) computes for a weight of shape (C*M, 1, KH, KW)), with its two gradients.
// One lane per result element, bounds-checked global reads, 64-bit indexing: correct for every geometry and element
// type, not tuned.  Calls with d == 1 and M == 1 never get here: the entry points hand those to the tuned kernels.
// Grad-weight is two-pass and bit-identical from run to run: partial[chunk][oc][tap] over chunks of the
// (image, row) range, then a fixed-order sum in fp64.
#include "dwconv_common.hpp"

#include <algorithm>

namespace dwconv {

namespace {

constexpr int kGeneralThreads = 256;

template <typename T>
__global__ __launch_bounds__(kGeneralThreads) void general_fwd_kernel(const T *__restrict__ in, const T *__restrict__ taps,
                                                                      T *__restrict__ out, const GeneralGeometry g,
                                                                      const long total)
{
    using acc_t = typename Io<T>::acc_t;
    const long e = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (e >= total) return;
    const int ox = static_cast<int>(e % g.out_w);
    long r = e / g.out_w;
    const int oy = static_cast<int>(r % g.out_h);
    r /= g.out_h;
    const int oc = static_cast<int>(r % (g.channel * g.multiplier));
    const long n = r / (g.channel * g.multiplier);
    const int c = oc / g.multiplier;
    const T *src = in + (n * g.channel + c) * g.in_h * g.in_w;
    const T *f = taps + static_cast<long>(oc) * g.kernel_h * g.kernel_w;
    acc_t s = 0;
    for (int ty = 0; ty < g.kernel_h; ++ty) {
        const int iy = oy * g.stride_h - g.pad_h + ty * g.dil_h;
        if (iy < 0 || iy >= g.in_h) continue;
        for (int tx = 0; tx < g.kernel_w; ++tx) {
            const int ix = ox * g.stride_w - g.pad_w + tx * g.dil_w;
            if (ix < 0 || ix >= g.in_w) continue;
            s += static_cast<acc_t>(Io<T>::in(src[static_cast<long>(iy) * g.in_w + ix])) *
                 static_cast<acc_t>(Io<T>::in(f[ty * g.kernel_w + tx]));
        }
    }
    out[e] = Io<T>::out(s);
}

// gx[n,c,iy,ix] = sum_{j<M} sum_{ty,tx} gy[n, c*M+j, oy, ox] * w[c*M+j, ty, tx]  with  oy*s = iy + p - ty*d  (same for x)
template <typename T>
__global__ __launch_bounds__(kGeneralThreads) void general_gx_kernel(const T *__restrict__ gy, const T *__restrict__ taps,
                                                                     T *__restrict__ gx, const GeneralGeometry g,
                                                                     const long total)
{
    using acc_t = typename Io<T>::acc_t;
    const long e = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (e >= total) return;
    const int ix = static_cast<int>(e % g.in_w);
    long r = e / g.in_w;
    const int iy = static_cast<int>(r % g.in_h);
    r /= g.in_h;
    const int c = static_cast<int>(r % g.channel);
    const long n = r / g.channel;
    acc_t s = 0;
    for (int j = 0; j < g.multiplier; ++j) {
        const int oc = c * g.multiplier + j;
        const T *src = gy + (n * g.channel * g.multiplier + oc) * g.out_h * g.out_w;
        const T *f = taps + static_cast<long>(oc) * g.kernel_h * g.kernel_w;
        for (int ty = 0; ty < g.kernel_h; ++ty) {
            const int ny = iy + g.pad_h - ty * g.dil_h;
            if (ny < 0 || ny % g.stride_h != 0) continue;
            const int oy = ny / g.stride_h;
            if (oy >= g.out_h) continue;
            for (int tx = 0; tx < g.kernel_w; ++tx) {
                const int nx = ix + g.pad_w - tx * g.dil_w;
                if (nx < 0 || nx % g.stride_w != 0) continue;
                const int ox = nx / g.stride_w;
                if (ox >= g.out_w) continue;
                s += static_cast<acc_t>(Io<T>::in(src[static_cast<long>(oy) * g.out_w + ox])) *
                     static_cast<acc_t>(Io<T>::in(f[ty * g.kernel_w + tx]));
            }
        }
    }
    gx[e] = Io<T>::out(s);
}

// Pass 1: lane = (oc, tap), block row = chunk of the (image, output row) pairs; partial[chunk][oc][tap].
template <typename T>
__global__ __launch_bounds__(kGeneralThreads) void general_gw_kernel(const T *__restrict__ x, const T *__restrict__ gy,
                                                                     void *__restrict__ partial_raw, const GeneralGeometry g,
                                                                     const long rows, const int chunks)
{
    using acc_t = typename Io<T>::acc_t;
    acc_t *partial = static_cast<acc_t *>(partial_raw);
    const int taps = g.kernel_h * g.kernel_w;
    const int oc_total = g.channel * g.multiplier;
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= oc_total * taps) return;
    const int oc = e / taps, t = e - oc * taps;
    const int ty = t / g.kernel_w, tx = t - ty * g.kernel_w;
    const int c = oc / g.multiplier;
    const long per = (rows + chunks - 1) / chunks;
    const long r0 = blockIdx.y * per, r1 = min(rows, r0 + per);
    acc_t s = 0;
    for (long r = r0; r < r1; ++r) {
        const long n = r / g.out_h;
        const int oy = static_cast<int>(r - n * g.out_h);
        const int iy = oy * g.stride_h - g.pad_h + ty * g.dil_h;
        if (iy < 0 || iy >= g.in_h) continue;
        const T *grow = gy + ((n * oc_total + oc) * g.out_h + oy) * g.out_w;
        const T *xrow = x + ((n * g.channel + c) * g.in_h + iy) * g.in_w;
        for (int ox = 0; ox < g.out_w; ++ox) {
            const int ix = ox * g.stride_w - g.pad_w + tx * g.dil_w;
            if (ix < 0 || ix >= g.in_w) continue;
            s += static_cast<acc_t>(Io<T>::in(grow[ox])) * static_cast<acc_t>(Io<T>::in(xrow[ix]));
        }
    }
    partial[static_cast<long>(blockIdx.y) * oc_total * taps + e] = s;
}

template <typename T>
__global__ __launch_bounds__(kGeneralThreads) void general_gw_final_kernel(const void *__restrict__ partial_raw,
                                                                           T *__restrict__ gw, const int total,
                                                                           const int chunks)
{
    using acc_t = typename Io<T>::acc_t;
    const acc_t *partial = static_cast<const acc_t *>(partial_raw);
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= total) return;
    double s = 0.0;
    for (int k = 0; k < chunks; ++k) s += static_cast<double>(partial[static_cast<long>(k) * total + e]);
    gw[e] = Io<T>::out(static_cast<acc_t>(s));
}

int general_chunks(const GeneralGeometry &g)
{
    const long rows = static_cast<long>(g.batch) * g.out_h;
    return static_cast<int>(std::max(1l, std::min(512l, rows / 4)));
}

}  // namespace

template <typename T>
int general_forward(const T *in, const T *taps, T *out, const GeneralGeometry &g, hipStream_t stream)
{
    const long total = static_cast<long>(g.batch) * g.channel * g.multiplier * g.out_h * g.out_w;
    if (total == 0) {
        note_variant("empty");
        return DWCONV_OK;
    }
    if ((total + kGeneralThreads - 1) / kGeneralThreads > 0x7fffffffL) return fail(DWCONV_ERR_UNSUPPORTED, "tensor too large");
    hipLaunchKernelGGL(general_fwd_kernel<T>, dim3(static_cast<unsigned>((total + kGeneralThreads - 1) / kGeneralThreads)),
                       dim3(kGeneralThreads), 0, stream, in, taps, out, g, total);
    note_variant("general_fwd<d%dx%d,m%d>", g.dil_h, g.dil_w, g.multiplier);
    return check_launch("general_fwd_kernel");
}

template <typename T>
int general_grad_input(const T *gy, const T *taps, T *gx, const GeneralGeometry &g, hipStream_t stream)
{
    const long total = static_cast<long>(g.batch) * g.channel * g.in_h * g.in_w;
    if (total == 0) {
        note_variant("empty");
        return DWCONV_OK;
    }
    if (static_cast<long>(g.out_h) * g.out_w * g.multiplier == 0) {
        note_variant("zero");
        return launch_fill_zero(gx, static_cast<size_t>(total) * sizeof(T), stream);
    }
    if ((total + kGeneralThreads - 1) / kGeneralThreads > 0x7fffffffL) return fail(DWCONV_ERR_UNSUPPORTED, "tensor too large");
    hipLaunchKernelGGL(general_gx_kernel<T>, dim3(static_cast<unsigned>((total + kGeneralThreads - 1) / kGeneralThreads)),
                       dim3(kGeneralThreads), 0, stream, gy, taps, gx, g, total);
    note_variant("general_gx<d%dx%d,m%d>", g.dil_h, g.dil_w, g.multiplier);
    return check_launch("general_gx_kernel");
}

template <typename T>
size_t general_grad_weight_workspace(const GeneralGeometry &g)
{
    return static_cast<size_t>(general_chunks(g)) * g.channel * g.multiplier * g.kernel_h * g.kernel_w *
           sizeof(typename Io<T>::acc_t);
}

template <typename T>
int general_grad_weight(const T *x, const T *gy, T *gw, void *ws, size_t ws_bytes, const GeneralGeometry &g,
                        hipStream_t stream)
{
    const int total = g.channel * g.multiplier * g.kernel_h * g.kernel_w;
    if (total == 0) {
        note_variant("empty");
        return DWCONV_OK;
    }
    const long rows = static_cast<long>(g.batch) * g.out_h;
    if (rows * g.out_w == 0 || g.in_h == 0 || g.in_w == 0) {
        note_variant("zero");
        return launch_fill_zero(gw, static_cast<size_t>(total) * sizeof(T), stream);
    }
    const size_t need = general_grad_weight_workspace<T>(g);
    if (ws == nullptr || ws_bytes < need)
        return fail(DWCONV_ERR_WORKSPACE, "grad-weight needs a workspace of %zu bytes, got %zu", need, ws_bytes);
    const int chunks = general_chunks(g);
    hipLaunchKernelGGL(general_gw_kernel<T>, dim3(ceil_div(total, kGeneralThreads), chunks), dim3(kGeneralThreads), 0,
                       stream, x, gy, ws, g, rows, chunks);
    int rc = check_launch("general_gw_kernel");
    if (rc != DWCONV_OK) return rc;
    hipLaunchKernelGGL(general_gw_final_kernel<T>, dim3(ceil_div(total, kGeneralThreads)), dim3(kGeneralThreads), 0, stream,
                       static_cast<const void *>(ws), gw, total, chunks);
    note_variant("general_gw<d%dx%d,m%d> chunks%d", g.dil_h, g.dil_w, g.multiplier, chunks);
    return check_launch("general_gw_final_kernel");
}

#define DWCONV_INSTANTIATE(T)                                                                                          \
    template int general_forward<T>(const T *, const T *, T *, const GeneralGeometry &, hipStream_t);                  \
    template int general_grad_input<T>(const T *, const T *, T *, const GeneralGeometry &, hipStream_t);               \
    template size_t general_grad_weight_workspace<T>(const GeneralGeometry &);                                         \
    template int general_grad_weight<T>(const T *, const T *, T *, void *, size_t, const GeneralGeometry &, hipStream_t);
DWCONV_INSTANTIATE(float)
DWCONV_INSTANTIATE(double)
DWCONV_INSTANTIATE(half_t)
DWCONV_INSTANTIATE(bf16_t)
#undef DWCONV_INSTANTIATE

}  // namespace dwconv
