// Backward of the fused forward epilogue  out = act(conv * scale[c] + shift[c])  (dwconv2d_fused_*).
//
// Given the convolution result `conv` (recomputed by the caller with the plain forward kernel; the fused
// forward keeps nothing but its inputs) and the gradient of `out`, one sweep produces
//   conv_grad  = out_grad * act'(z) * scale[c],          z = conv * scale[c] + shift[c]
//   scale_grad[c] = sum_{n,y,x} out_grad * act'(z) * conv
//   shift_grad[c] = sum_{n,y,x} out_grad * act'(z)
// conv_grad then goes through the ordinary backward kernels as out_grad.  Three tensor sweeps (two reads, one
// write) stand for the four elementwise backward passes autograd would run for mul, add and the activation.
// The per-channel sums are two-pass and bit-identical from run to run: partial[c][chunk][2] per workgroup
// (fixed-order tree in LDS), then the fixed-order fp64 sum shared with grad-weight.
// No counterpart in the reference, which has no epilogue (it rejects a bias, torch_dwconv/dwconv.py:108-109).
#include "dwconv_tile_common.hpp"

#include <algorithm>

namespace dwconv {

namespace {

constexpr int kEpiThreads = 256;

struct EpiBwdPlan {
    const void *conv;
    const void *out_grad;
    void *conv_grad;
    const float *scale;
    const float *shift;
    float *partial;
    int act;
    int channel;
    int outer;            // NCHW: images; channels-last: pixels of all images
    int inner;            // NCHW: elements per plane; channels-last: 1
    int chunks;
    int outer_per_chunk;
    int vec;              // groups of four elements may be moved with one access
};

// out_grad * d act(z) / dz.  Boundaries as PyTorch's own backward formulas: ReLU passes z > 0, ReLU6 passes 0 < z < 6.
__device__ __forceinline__ float act_backward(float z, float g, int act)
{
    if (act == DWCONV_ACT_RELU) return z > 0.f ? g : 0.f;
    if (act == DWCONV_ACT_RELU6) return (z > 0.f && z < 6.f) ? g : 0.f;
    if (act == DWCONV_ACT_SILU) {
        const float s = 1.f / (1.f + __expf(-z));
        return g * s * (1.f + z * (1.f - s));
    }
    return g;
}

// One element: returns conv_grad and adds to the two channel sums.
__device__ __forceinline__ float epi_element(float y, float g, float sc, float sh, int act, float &s_scale, float &s_shift)
{
    const float ga = act_backward(fmaf(y, sc, sh), g, act);
    s_scale = fmaf(ga, y, s_scale);
    s_shift += ga;
    return ga * sc;
}

// Sum of v over the workgroup, in a fixed order, valid in lane 0.
__device__ __forceinline__ float block_sum(float v, float *red)
{
    red[threadIdx.x] = v;
    __syncthreads();
#pragma unroll
    for (int half = kEpiThreads / 2; half > 0; half >>= 1) {
        if (static_cast<int>(threadIdx.x) < half) red[threadIdx.x] += red[threadIdx.x + half];
        __syncthreads();
    }
    const float s = red[0];
    __syncthreads();
    return s;
}

// NCHW: workgroup (channel c, chunk of images); lanes run along the plane.
template <typename IO>
__global__ __launch_bounds__(kEpiThreads) void epilogue_bwd_nchw_kernel(const EpiBwdPlan p)
{
    __shared__ float red[kEpiThreads];
    const int c = blockIdx.x, chunk = blockIdx.y;
    const int n0 = chunk * p.outer_per_chunk, n1 = min(p.outer, n0 + p.outer_per_chunk);
    const float sc = p.scale != nullptr ? p.scale[c] : 1.f, sh = p.shift != nullptr ? p.shift[c] : 0.f;
    const IO *const conv = static_cast<const IO *>(p.conv);
    const IO *const gy = static_cast<const IO *>(p.out_grad);
    IO *const g0 = static_cast<IO *>(p.conv_grad);
    float s_scale = 0.f, s_shift = 0.f;
    if (p.vec) {
        const int inner4 = p.inner >> 2;
        const int total = (n1 - n0) * inner4;
        for (int e = threadIdx.x; e < total; e += kEpiThreads) {
            const int n = e / inner4, i = e - n * inner4;
            const long off = (static_cast<long>(n0 + n) * p.channel + c) * p.inner + 4 * i;
            const float4 y = load4<IO>(conv + off), g = load4<IO>(gy + off);
            store4<IO>(g0 + off, epi_element(y.x, g.x, sc, sh, p.act, s_scale, s_shift),
                       epi_element(y.y, g.y, sc, sh, p.act, s_scale, s_shift),
                       epi_element(y.z, g.z, sc, sh, p.act, s_scale, s_shift),
                       epi_element(y.w, g.w, sc, sh, p.act, s_scale, s_shift));
        }
    } else {
        const int total = (n1 - n0) * p.inner;
        for (int e = threadIdx.x; e < total; e += kEpiThreads) {
            const int n = e / p.inner, i = e - n * p.inner;
            const long off = (static_cast<long>(n0 + n) * p.channel + c) * p.inner + i;
            g0[off] = Io<IO>::out(epi_element(Io<IO>::in(conv[off]), Io<IO>::in(gy[off]), sc, sh, p.act, s_scale, s_shift));
        }
    }
    const float t_scale = block_sum(s_scale, red), t_shift = block_sum(s_shift, red);
    if (threadIdx.x == 0) {
        float *dst = p.partial + (static_cast<long>(c) * p.chunks + chunk) * 2;
        dst[0] = t_scale;
        dst[1] = t_shift;
    }
}

// Channels-last: workgroup (64 channel lanes of CV channels each, chunk of pixels); the four wavefronts take
// every fourth pixel and are added in order at the end.
template <typename IO, int CV>
__global__ __launch_bounds__(kEpiThreads) void epilogue_bwd_nhwc_kernel(const EpiBwdPlan p)
{
    __shared__ float red[kEpiThreads / 64][64][2 * CV];
    const int cl = threadIdx.x & 63, pl = threadIdx.x >> 6;
    const int c0 = (blockIdx.x * 64 + cl) * CV;
    const int chunk = blockIdx.y;
    const int o0 = chunk * p.outer_per_chunk, o1 = min(p.outer, o0 + p.outer_per_chunk);
    const bool live = c0 < p.channel;
    const IO *const conv = static_cast<const IO *>(p.conv);
    const IO *const gy = static_cast<const IO *>(p.out_grad);
    IO *const g0 = static_cast<IO *>(p.conv_grad);
    float sc[CV], sh[CV], s_scale[CV], s_shift[CV];
#pragma unroll
    for (int v = 0; v < CV; ++v) {
        sc[v] = live && p.scale != nullptr ? p.scale[c0 + v] : 1.f;
        sh[v] = live && p.shift != nullptr ? p.shift[c0 + v] : 0.f;
        s_scale[v] = s_shift[v] = 0.f;
    }
    if (live) {
        for (int o = o0 + pl; o < o1; o += kEpiThreads / 64) {
            const long off = static_cast<long>(o) * p.channel + c0;
            if constexpr (CV == 4) {
                const float4 y = load4<IO>(conv + off), g = load4<IO>(gy + off);
                store4<IO>(g0 + off, epi_element(y.x, g.x, sc[0], sh[0], p.act, s_scale[0], s_shift[0]),
                           epi_element(y.y, g.y, sc[1], sh[1], p.act, s_scale[1], s_shift[1]),
                           epi_element(y.z, g.z, sc[2], sh[2], p.act, s_scale[2], s_shift[2]),
                           epi_element(y.w, g.w, sc[3], sh[3], p.act, s_scale[3], s_shift[3]));
            } else {
                g0[off] = Io<IO>::out(
                    epi_element(Io<IO>::in(conv[off]), Io<IO>::in(gy[off]), sc[0], sh[0], p.act, s_scale[0], s_shift[0]));
            }
        }
    }
#pragma unroll
    for (int v = 0; v < CV; ++v) {
        red[pl][cl][2 * v] = s_scale[v];
        red[pl][cl][2 * v + 1] = s_shift[v];
    }
    __syncthreads();
    if (pl == 0 && live) {
#pragma unroll
        for (int v = 0; v < CV; ++v) {
            float a = red[0][cl][2 * v], b = red[0][cl][2 * v + 1];
#pragma unroll
            for (int w = 1; w < kEpiThreads / 64; ++w) {
                a += red[w][cl][2 * v];
                b += red[w][cl][2 * v + 1];
            }
            float *dst = p.partial + (static_cast<long>(c0 + v) * p.chunks + chunk) * 2;
            dst[0] = a;
            dst[1] = b;
        }
    }
}

bool make_plan(EpiBwdPlan &p, int batch, int channel, int out_h, int out_w, bool channels_last)
{
    const long plane = static_cast<long>(out_h) * out_w;
    p.channel = channel;
    if (channels_last) {
        if (batch * plane >= (1l << 31)) return false;
        p.outer = static_cast<int>(batch * plane);
        p.inner = 1;
        const int groups = ceil_div(channel, 64 * (channel % 4 == 0 ? 4 : 1));
        int chunks = ceil_div(2048, groups);
        chunks = std::max(1, std::min(chunks, std::min(ceil_div(p.outer, 16), 65535)));
        p.outer_per_chunk = ceil_div(p.outer, chunks);
    } else {
        if (plane >= (1l << 30)) return false;
        p.outer = batch;
        p.inner = static_cast<int>(plane);
        int chunks = ceil_div(4096, std::max(channel, 1));
        chunks = std::max(1, std::min(chunks, std::min(batch, 65535)));
        p.outer_per_chunk = ceil_div(batch, chunks);
        // a chunk's elements of one channel are indexed with 32 bits
        while (static_cast<long>(p.outer_per_chunk) * plane >= (1l << 31)) p.outer_per_chunk = ceil_div(p.outer_per_chunk, 2);
        if (ceil_div(batch, p.outer_per_chunk) > 65535) return false;
    }
    p.chunks = ceil_div(p.outer, p.outer_per_chunk);
    return true;
}

}  // namespace

size_t epilogue_backward_workspace(int batch, int channel, int out_h, int out_w, bool channels_last)
{
    EpiBwdPlan p{};
    if (batch <= 0 || channel <= 0 || out_h <= 0 || out_w <= 0) return 0;
    if (!make_plan(p, batch, channel, out_h, out_w, channels_last)) return 0;
    return static_cast<size_t>(channel) * p.chunks * 2 * sizeof(float);
}

template <typename IO>
int epilogue_backward(const IO *conv, const IO *out_grad, const float *scale, const float *shift, IO *conv_grad,
                      float *param_grad, void *ws, size_t ws_bytes, int batch, int channel, int out_h, int out_w, int act,
                      bool channels_last, hipStream_t stream)
{
    EpiBwdPlan p{};
    if (!make_plan(p, batch, channel, out_h, out_w, channels_last)) return fail(DWCONV_ERR_UNSUPPORTED, "tensor too large");
    const size_t need = static_cast<size_t>(channel) * p.chunks * 2 * sizeof(float);
    if (ws == nullptr || ws_bytes < need)
        return fail(DWCONV_ERR_WORKSPACE, "the epilogue backward needs a workspace of %zu bytes, got %zu", need, ws_bytes);
    p.conv = conv;
    p.out_grad = out_grad;
    p.conv_grad = conv_grad;
    p.scale = scale;
    p.shift = shift;
    p.partial = static_cast<float *>(ws);
    p.act = act;
    const bool aligned = aligned4(conv) && aligned4(out_grad) && aligned4(conv_grad);
    if (channels_last) {
        p.vec = aligned && channel % 4 == 0;
        if (p.vec)
            hipLaunchKernelGGL((epilogue_bwd_nhwc_kernel<IO, 4>), dim3(ceil_div(channel, 256), p.chunks), dim3(kEpiThreads), 0,
                               stream, p);
        else
            hipLaunchKernelGGL((epilogue_bwd_nhwc_kernel<IO, 1>), dim3(ceil_div(channel, 64), p.chunks), dim3(kEpiThreads), 0,
                               stream, p);
    } else {
        p.vec = aligned && p.inner % 4 == 0;
        hipLaunchKernelGGL(epilogue_bwd_nchw_kernel<IO>, dim3(channel, p.chunks), dim3(kEpiThreads), 0, stream, p);
    }
    const int rc = check_launch("epilogue_bwd_kernel");
    if (rc != DWCONV_OK) return rc;
    note_variant("epilogue_bwd%s<%s,v%d> chunks%d", sizeof(IO) == 2 ? "16" : "", channels_last ? "nhwc" : "nchw", p.vec ? 4 : 1,
                 p.chunks);
    // param_grad[c][0] = scale_grad, [c][1] = shift_grad: the fixed-order fp64 sum over the chunks
    return launch_wgrad_final<float>(p.partial, param_grad, channel, 2, p.chunks, stream);
}

#define DWCONV_INSTANTIATE(IO)                                                                                          \
    template int epilogue_backward<IO>(const IO *, const IO *, const float *, const float *, IO *, float *, void *, size_t, \
                                       int, int, int, int, int, bool, hipStream_t);
DWCONV_INSTANTIATE(float)
DWCONV_INSTANTIATE(half_t)
DWCONV_INSTANTIATE(bf16_t)
#undef DWCONV_INSTANTIATE

}  // namespace dwconv
