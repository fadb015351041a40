// Generic kernels: any up/down/kernel/pad combination, float or double.
//
// These are the catch-all behind the tuned fp32 kernels (they also serve every
// fp64 call).  One lane produces one output element straight from global memory.
// The reference has no such catch-all: geometries outside its nine template
// instances run off the end of a non-void function
// (torch_dwconv/dwconv_kernel.cu:808-845).
#include "dwconv_common.hpp"

namespace dwconv {

namespace {

constexpr int kDirectThreads = 256;

// out[n,c,oy,ox] = sum_{ty,tx} U[oy*down_h - pad_h0 + ty, ox*down_w - pad_w0 + tx] * f[c,ty,tx]
// (the operator of torch_dwconv/dwconv_kernel.cu:69-181).
template <typename T>
__global__ __launch_bounds__(kDirectThreads) void fir_direct_kernel(
    const T *__restrict__ in, const T *__restrict__ taps, T *__restrict__ out, const Geometry g,
    const long total)
{
    const long step = static_cast<long>(gridDim.x) * blockDim.x;
    for (long idx = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x; idx < total;
         idx += step) {
        const int ox = static_cast<int>(idx % g.out_w);
        const long t1 = idx / g.out_w;
        const int oy = static_cast<int>(t1 % g.out_h);
        const long plane = t1 / g.out_h;
        const int c = static_cast<int>(plane % g.channel);
        const T *src = in + plane * g.in_h * g.in_w;
        const T *f = taps + static_cast<long>(c) * g.kernel_h * g.kernel_w;
        typename Io<T>::acc_t acc = 0;
        for (int ty = 0; ty < g.kernel_h; ++ty) {
            const int uy = oy * g.down_h - g.pad_h0 + ty;
            if (uy < 0 || uy % g.up_h != 0) continue;
            const int iy = uy / g.up_h;
            if (iy >= g.in_h) continue;
            for (int tx = 0; tx < g.kernel_w; ++tx) {
                const int ux = ox * g.down_w - g.pad_w0 + tx;
                if (ux < 0 || ux % g.up_w != 0) continue;
                const int ix = ux / g.up_w;
                if (ix >= g.in_w) continue;
                const T fv = g.forward ? f[ty * g.kernel_w + tx]
                                       : f[(g.kernel_h - 1 - ty) * g.kernel_w + (g.kernel_w - 1 - tx)];
                acc += Io<T>::in(fv) * Io<T>::in(src[static_cast<long>(iy) * g.in_w + ix]);
            }
        }
        if (g.epi.enabled()) acc = epilogue_apply(acc, g.epi, c);
        out[idx] = Io<T>::out(acc);
    }
}

// Sum over the 64 lanes of a wavefront in a fixed butterfly order.
template <typename T>
__device__ inline T wave_sum(T v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Pass 1 of the generic grad-weight: workgroup (c, chunk) sums
//   gy[n,c,oy,ox] * x[n,c, oy*down_h - pad_h + i, ox*down_w - pad_w + j]
// over the images of its chunk, one tap (i,j) after the other, and stores
// K*K partial sums.  (Sum of torch_dwconv/dwconv_kernel.cu:269-297.)
template <typename T>
__global__ __launch_bounds__(kDirectThreads) void wgrad_direct_partial_kernel(
    const T *__restrict__ in, const T *__restrict__ gy, typename Io<T>::acc_t *__restrict__ partial,
    const WgradGeometry g, const int chunks, const int images_per_chunk)
{
    using A = typename Io<T>::acc_t;
    __shared__ A wave_part[kDirectThreads / 64];
    const int c = blockIdx.x;
    const int chunk = blockIdx.y;
    const int n0 = chunk * images_per_chunk;
    const int n1 = min(g.batch, n0 + images_per_chunk);
    const int out_px = g.out_h * g.out_w;
    const int taps = g.kernel_h * g.kernel_w;
    for (int tap = 0; tap < taps; ++tap) {
        const int i = tap / g.kernel_w, j = tap - i * g.kernel_w;
        A acc = 0;
        for (int n = n0; n < n1; ++n) {
            const long plane = static_cast<long>(n) * g.channel + c;
            const T *x = in + plane * g.in_h * g.in_w;
            const T *d = gy + plane * out_px;
            for (int p = threadIdx.x; p < out_px; p += kDirectThreads) {
                const int oy = p / g.out_w, ox = p - oy * g.out_w;
                const int iy = oy * g.down_h - g.pad_h + i;
                const int ix = ox * g.down_w - g.pad_w + j;
                if (iy >= 0 && iy < g.in_h && ix >= 0 && ix < g.in_w)
                    acc += Io<T>::in(d[p]) * Io<T>::in(x[static_cast<long>(iy) * g.in_w + ix]);
            }
        }
        acc = wave_sum(acc);
        if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = acc;
        __syncthreads();
        if (threadIdx.x == 0) {
            A s = wave_part[0];
            for (int w = 1; w < kDirectThreads / 64; ++w) s += wave_part[w];
            partial[(static_cast<long>(c) * chunks + chunk) * taps + tap] = s;
        }
        __syncthreads();
    }
}

// Pass 2: one lane per (c, tap) adds the chunk partials front to back.
template <typename T>
__global__ void wgrad_direct_final_kernel(const typename Io<T>::acc_t *__restrict__ partial, T *__restrict__ gw,
                                          const int channel_taps, const int taps, const int chunks)
{
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= channel_taps) return;
    const int c = e / taps, tap = e - c * taps;
    const typename Io<T>::acc_t *p = partial + static_cast<long>(c) * chunks * taps + tap;
    typename Io<T>::acc_t s = 0;
    for (int k = 0; k < chunks; ++k) s += p[static_cast<long>(k) * taps];
    gw[e] = Io<T>::out(s);
}

__global__ void fill_zero_kernel(uint32_t *p, const size_t words)
{
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < words) p[i] = 0u;
}

int direct_chunks(const WgradGeometry &g)
{
    // enough workgroups to cover the 256 CUs a few times over
    int want = ceil_div(2048, g.channel);
    if (want < 1) want = 1;
    if (want > g.batch) want = g.batch;
    const int per = ceil_div(g.batch, want);
    return ceil_div(g.batch, per);
}

}  // namespace

int launch_fill_zero(void *p, size_t bytes, hipStream_t stream)
{
    const size_t words = bytes / 4;
    if (words == 0) return DWCONV_OK;
    hipLaunchKernelGGL(fill_zero_kernel, dim3(static_cast<unsigned>((words + 255) / 256)), dim3(256), 0,
                       stream, static_cast<uint32_t *>(p), words);
    return check_launch("fill_zero_kernel");
}

template <typename T>
int launch_fir_direct(const T *in, const T *taps, T *out, const Geometry &g, hipStream_t stream)
{
    const long total = g.planes() * g.out_h * g.out_w;
    if (total <= 0) return DWCONV_OK;
    long blocks = (total + kDirectThreads - 1) / kDirectThreads;
    if (blocks > 1 << 20) blocks = 1 << 20;
    hipLaunchKernelGGL(fir_direct_kernel<T>, dim3(static_cast<unsigned>(blocks)),
                       dim3(kDirectThreads), 0, stream, in, taps, out, g, total);
    note_variant("direct_%s", sizeof(T) == 4 ? "f32" : (sizeof(T) == 8 ? "f64" : "16"));
    return check_launch("fir_direct_kernel");
}

template <typename T>
size_t wgrad_direct_workspace(const WgradGeometry &g)
{
    return static_cast<size_t>(g.channel) * direct_chunks(g) * g.kernel_h * g.kernel_w * sizeof(typename Io<T>::acc_t);
}

template <typename T>
int launch_wgrad_direct(const T *in, const T *gy, T *gw, void *ws, size_t ws_bytes,
                        const WgradGeometry &g, hipStream_t stream)
{
    const size_t need = wgrad_direct_workspace<T>(g);
    if (ws == nullptr || ws_bytes < need)
        return fail(DWCONV_ERR_WORKSPACE, "grad-weight needs a workspace of %zu bytes, got %zu", need,
                    ws_bytes);
    const int chunks = direct_chunks(g);
    const int per = ceil_div(g.batch, chunks);
    const int taps = g.kernel_h * g.kernel_w;
    auto *partial = static_cast<typename Io<T>::acc_t *>(ws);
    hipLaunchKernelGGL(wgrad_direct_partial_kernel<T>, dim3(g.channel, chunks), dim3(kDirectThreads),
                       0, stream, in, gy, partial, g, chunks, per);
    int rc = check_launch("wgrad_direct_partial_kernel");
    if (rc != DWCONV_OK) return rc;
    const int total = g.channel * taps;
    hipLaunchKernelGGL(wgrad_direct_final_kernel<T>, dim3(ceil_div(total, 256)), dim3(256), 0, stream,
                       partial, gw, total, taps, chunks);
    note_variant("wgrad_direct_%s", sizeof(T) == 4 ? "f32" : (sizeof(T) == 8 ? "f64" : "16"));
    return check_launch("wgrad_direct_final_kernel");
}

template int launch_fir_direct<float>(const float *, const float *, float *, const Geometry &,
                                      hipStream_t);
template int launch_fir_direct<half_t>(const half_t *, const half_t *, half_t *, const Geometry &, hipStream_t);
template int launch_fir_direct<bf16_t>(const bf16_t *, const bf16_t *, bf16_t *, const Geometry &, hipStream_t);
template size_t wgrad_direct_workspace<half_t>(const WgradGeometry &);
template size_t wgrad_direct_workspace<bf16_t>(const WgradGeometry &);
template int launch_wgrad_direct<half_t>(const half_t *, const half_t *, half_t *, void *, size_t,
                                         const WgradGeometry &, hipStream_t);
template int launch_wgrad_direct<bf16_t>(const bf16_t *, const bf16_t *, bf16_t *, void *, size_t,
                                         const WgradGeometry &, hipStream_t);
template int launch_fir_direct<double>(const double *, const double *, double *, const Geometry &,
                                       hipStream_t);
template size_t wgrad_direct_workspace<float>(const WgradGeometry &);
template size_t wgrad_direct_workspace<double>(const WgradGeometry &);
template int launch_wgrad_direct<float>(const float *, const float *, float *, void *, size_t,
                                        const WgradGeometry &, hipStream_t);
template int launch_wgrad_direct<double>(const double *, const double *, double *, void *, size_t,
                                         const WgradGeometry &, hipStream_t);

}  // namespace dwconv
