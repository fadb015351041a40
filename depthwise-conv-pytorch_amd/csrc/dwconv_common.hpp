// Shared declarations of libdwconv_hip: geometry, error reporting and the
// launch functions each translation unit provides.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "dwconv_hip.h"

namespace dwconv {

// ---- element types at the boundary --------------------------------------------------------------------
// fp16 and bf16 tensors are read and written as such; all arithmetic and every partial sum is fp32
// (the reference accumulates halves in half, torch_dwconv/dwconv_kernel.cu:749 `AT_DISPATCH_..._AND_HALF`
// with `scalar_t v`; fp32 accumulation is strictly more accurate).
using half_t = _Float16;
struct bf16_t {
    uint16_t bits;
};

template <typename T>
struct Io {
    using acc_t = float;
    __host__ __device__ static float in(T v) { return static_cast<float>(v); }
    __host__ __device__ static T out(float v) { return static_cast<T>(v); }
};
template <>
struct Io<double> {
    using acc_t = double;
    __host__ __device__ static double in(double v) { return v; }
    __host__ __device__ static double out(double v) { return v; }
};
template <>
struct Io<bf16_t> {
    using acc_t = float;
    __host__ __device__ static float in(bf16_t v)
    {
        union { uint32_t u; float f; } c;
        c.u = static_cast<uint32_t>(v.bits) << 16;
        return c.f;
    }
    // Round to nearest even.  Device code uses the hardware conversion of gfx950 (v_cvt_pk_bf16_f32); the host
    // version computes the same bits for every finite value and keeps a NaN a NaN.
    __host__ __device__ static bf16_t out(float v)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        return bf16_t{__builtin_bit_cast(uint16_t, static_cast<__bf16>(v))};
#else
        union { uint32_t u; float f; } c;
        c.f = v;
        if ((c.u & 0x7fffffffu) > 0x7f800000u) return bf16_t{static_cast<uint16_t>((c.u >> 16) | 0x40u)};
        c.u += 0x7fffu + ((c.u >> 16) & 1u);
        return bf16_t{static_cast<uint16_t>(c.u >> 16)};
#endif
    }
};

// Two sums as a pair of fp16 / bf16 in one register: a single conversion instruction each on gfx950.
__device__ __forceinline__ uint32_t f16_pack2(float lo, float hi)
{
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}
__device__ __forceinline__ uint32_t bf16_pack2(float lo, float hi)
{
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

// What a forward kernel applies to each sum before storing it: v * scale[c] + shift[c], then an activation.
// scale / shift are per-channel arrays of the accumulation type (float; double for fp64 tensors) or null.
struct Epilogue {
    const void *scale = nullptr;
    const void *shift = nullptr;
    int act = DWCONV_ACT_NONE;  // dwconv_activation
    __host__ __device__ bool enabled() const { return scale != nullptr || shift != nullptr || act != DWCONV_ACT_NONE; }
};

// v * sigmoid(v).  fp32: hardware exp2 and reciprocal (1 ulp each), two quarter-rate instructions instead of
// the dozen of an IEEE division.
__device__ __forceinline__ float epilogue_silu(float v) { return v * __builtin_amdgcn_rcpf(1.f + __expf(-v)); }
__device__ __forceinline__ double epilogue_silu(double v) { return v / (1.0 + exp(-v)); }

template <typename A>
__device__ __forceinline__ A epilogue_apply(A v, const Epilogue &e, int c)
{
    if (e.scale != nullptr) v *= static_cast<const A *>(e.scale)[c];
    if (e.shift != nullptr) v += static_cast<const A *>(e.shift)[c];
    // comparisons written so that NaN passes through, as it does in torch
    if (e.act == DWCONV_ACT_RELU) v = v < A(0) ? A(0) : v;
    else if (e.act == DWCONV_ACT_RELU6) v = v < A(0) ? A(0) : (v > A(6) ? A(6) : v);
    else if (e.act == DWCONV_ACT_SILU) v = epilogue_silu(v);
    return v;
}

// The same for a lane's whole register block: the tests on the (uniform) options are made once, outside the
// element loops, so that the independent exp/rcp chains of the elements can overlap.  Element [r][j] belongs
// to channel c0 + (j % CPL) (CPL = 1: one channel for the whole block).
template <int CPL, int R, int C>
__device__ __forceinline__ void epilogue_apply_block(float (&acc)[R][C], const Epilogue &e, int c0)
{
    if (e.scale != nullptr || e.shift != nullptr) {
        float sc[CPL], sh[CPL];
#pragma unroll
        for (int v = 0; v < CPL; ++v) {
            sc[v] = e.scale != nullptr ? static_cast<const float *>(e.scale)[c0 + v] : 1.f;
            sh[v] = e.shift != nullptr ? static_cast<const float *>(e.shift)[c0 + v] : 0.f;
        }
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < C; ++j) acc[r][j] = fmaf(acc[r][j], sc[j % CPL], sh[j % CPL]);
    }
    if (e.act == DWCONV_ACT_RELU) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < C; ++j) acc[r][j] = acc[r][j] < 0.f ? 0.f : acc[r][j];
    } else if (e.act == DWCONV_ACT_RELU6) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < C; ++j) acc[r][j] = acc[r][j] < 0.f ? 0.f : (acc[r][j] > 6.f ? 6.f : acc[r][j]);
    } else if (e.act == DWCONV_ACT_SILU) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < C; ++j) acc[r][j] = epilogue_silu(acc[r][j]);
    }
}

// Geometry of one up/FIR/down call on dense NCHW planes.  The same fields as the
// reference's DWConv2dKernelParams (torch_dwconv/dwconv_kernel.cu:42-67), with the
// batch and channel extents folded into `planes` where a kernel does not need them.
struct Geometry {
    int batch, channel;
    int in_h, in_w;
    int kernel_h, kernel_w;
    int up_h, up_w;
    int down_h, down_w;
    int pad_h0, pad_h1, pad_w0, pad_w1;
    int out_h, out_w;
    int forward;
    Epilogue epi;  // forward convolutions only
    // Depth multiplier M (tiled kernels on larger maps only).  `channel` and planes() count the result's channels.
    // Forward: result plane (n, c) reads input plane (n, c / M) of an input with channel / M channels.  Backward:
    // result plane (n, c) adds up the planes (n, c * M + m) of an operand with channel * M channels, each with the
    // taps of its own channel.
    int mult = 1;
    // Dilation of the taps (the any-geometry tiled kernel only; every other kernel is handed 1).
    int dil_h = 1, dil_w = 1;
    long planes() const { return static_cast<long>(batch) * channel; }
};

// Geometry of a grad-weight call.
struct WgradGeometry {
    int batch, channel;
    int in_h, in_w;
    int out_h, out_w;
    int kernel_h, kernel_w;
    int down_h, down_w;
    int pad_h, pad_w;
    int dil = 1;  // dilation of the taps, both axes (the whole-plane kernels take 2 for 3x3 / 5x5 at stride 1)
    int mult = 1; // depth multiplier M (tiled grad-weight kernel only): `channel` counts the channels of out_grad and of
                  // the taps, the input has channel / M of them and plane (n, c) of out_grad meets input plane (n, c / M)
};

// Geometry of a channels-last call: input (N,H,W,C), output (N,OH,OW,C), taps (C,1,KH,KW).
struct NhwcGeometry {
    int batch, channel;
    int in_h, in_w;
    int out_h, out_w;
    int kernel_h, kernel_w;
    int stride_h, stride_w;
    int pad_h, pad_w;
    Epilogue epi;  // nhwc_forward only
};

// Geometry of a call with dilation and depth multiplier (NCHW): input (N,C,H,W), taps (C*M,1,KH,KW),
// output (N,C*M,OH,OW), OH = (H + 2*pad - dil*(KH-1) - 1) / stride + 1.
struct GeneralGeometry {
    int batch, channel, multiplier;
    int in_h, in_w;
    int out_h, out_w;
    int kernel_h, kernel_w;
    int stride_h, stride_w;
    int pad_h, pad_w;
    int dil_h, dil_w;
};

// Thread-local error/variant strings behind dwconv_last_error()/dwconv_last_variant().
int fail(dwconv_status code, const char *fmt, ...);
void note_variant(const char *fmt, ...);
int check_launch(const char *what);

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline int round_up(int a, int b) { return ceil_div(a, b) * b; }

// Reciprocal m with n / d == (n * m) >> 32 for 0 <= n < 65536 and 2 <= d < 65536;
// d == 1 is encoded as m == 0 (the kernels test for it).
inline unsigned magic_u16(unsigned d) { return d <= 1 ? 0u : static_cast<unsigned>((0x100000000ull + d - 1) / d); }

// ---- generic kernels (any geometry, float or double): dwconv_generic.hip ----
template <typename T>
int launch_fir_direct(const T *in, const T *taps, T *out, const Geometry &g, hipStream_t stream);
// Zero-fills `bytes` (a multiple of 4) with a kernel rather than a memset node.
int launch_fill_zero(void *p, size_t bytes, hipStream_t stream);
template <typename T>
size_t wgrad_direct_workspace(const WgradGeometry &g);
template <typename T>
int launch_wgrad_direct(const T *in, const T *gy, T *gw, void *ws, size_t ws_bytes,
                        const WgradGeometry &g, hipStream_t stream);

// ---- LDS-tiled fp64 kernels: dwconv_f64.hip (-1 when the geometry is not covered; workspace 0 likewise) ----
// The operator kernel takes any up/down factors, filter extent and pads, and every element type (fp32 image and sums for
// the 32- and 16-bit ones: their last tiled stop before the per-element kernel).
template <typename T>
int try_launch_fir_lds(const T *in, const T *taps, T *out, const Geometry &g, hipStream_t stream);
size_t wgrad_f64_workspace(const WgradGeometry &g, int dil_h = 1, int dil_w = 1);
int try_launch_wgrad_f64(const double *in, const double *gy, double *gw, void *ws, size_t ws_bytes, const WgradGeometry &g,
                         hipStream_t stream, int dil_h = 1, int dil_w = 1);

// ---- LDS-tiled fp32 kernels: dwconv_tile.hip ----
// Return DWCONV_OK after launching, a negative value (-1) when the geometry is
// outside what the tiled kernels cover (the caller then uses the generic kernel),
// or a positive dwconv_status on a launch error.
template <typename IO>  // float, half_t or bf16_t
int try_launch_fir_tiled(const IO *in, const IO *taps, IO *out, const Geometry &g, hipStream_t stream);
// The same for any filter extent, stride and dilation (up = 1): taps looped over at run time (dwconv_tile.hip).
template <typename IO>
int try_launch_fir_any(const IO *in, const IO *taps, IO *out, const Geometry &g, hipStream_t stream);
// The same for 16-bit tensors whose rows are whole groups of eight elements: raw 16-bit LDS image and two-element
// dot products (dwconv_tile16.hip).  -1 when it does not cover g.
template <typename IO>
int try_launch_fir_tiled16(const IO *in, const IO *taps, IO *out, const Geometry &g, hipStream_t stream);

// ---- whole-plane kernels for maps up to 32 wide: dwconv_small.hip (same return convention) ----
// dil: dilation of the taps (1, or 2 for 3x3 / 5x5 forward at stride 1 with padding 2 * (K/2))
template <typename IO>  // float, half_t or bf16_t
int try_launch_fir_small(const IO *in, const IO *taps, IO *out, const Geometry &g, hipStream_t stream, int dil = 1);

size_t wgrad_small_workspace(const WgradGeometry &g);  // 0 when the whole-plane kernel does not cover g
template <typename IO>
int try_launch_wgrad_small(const IO *in, const IO *gy, IO *gw, void *ws, size_t ws_bytes, const WgradGeometry &g,
                           hipStream_t stream);
// Fused grad-weight + grad-input for the same maps (gy read once); same return convention.
template <typename IO>
int try_launch_bwd_small(const IO *in, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes,
                         const WgradGeometry &g, hipStream_t stream);
// Pass 2 shared by the tiled and whole-plane grad-weight kernels:
// gw[c][tap] = sum over chunks of partial[c][chunk][tap] (fp32 partial sums, added in fp64 in a fixed order).
// The stacked-image kernels (dwconv_stack.hip) of one large filter size each, K = 9, 11, 13: translation units of their
// own.  -1 when the geometry is not covered.
template <int K>
size_t stack_bigk_workspace(int batch, int channel, int h, int w);
template <int K, typename IO>
int stack_bigk_forward(const IO *in, const IO *taps, IO *out, int batch, int channel, int h, int w, bool rot, hipStream_t stream);
template <int K, typename IO>
int stack_bigk_backward(const IO *in, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes, int batch,
                        int channel, int h, int w, hipStream_t stream);

// Grad-weight for any filter extent, stride and dilation (dwconv_wgrad.hip); workspace bytes (0: not covered) and launch.
size_t wgrad_any_workspace(const WgradGeometry &g, int dil_h, int dil_w);
template <typename IO>
int try_launch_wgrad_any(const IO *in, const IO *gy, IO *gw, void *ws, size_t ws_bytes, const WgradGeometry &g, int dil_h,
                         int dil_w, hipStream_t stream);

template <typename IO>
int launch_wgrad_final(const float *partial, IO *gw, int channel, int taps, int chunks, hipStream_t stream);

// ---- grad-weight with LDS tiles and a fixed-order two-pass reduction: dwconv_wgrad.hip ----
size_t wgrad_tiled_workspace(const WgradGeometry &g);  // 0 when the tiled kernel does not cover g
template <typename IO>
int try_launch_wgrad_tiled(const IO *in, const IO *gy, IO *gw, void *ws, size_t ws_bytes, const WgradGeometry &g,
                           hipStream_t stream);

// Fused grad-weight + grad-input with LDS tiles (stride 1, "same" padding); same return convention.
template <typename IO>
int try_launch_bwd_tiled(const IO *in, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes,
                         const WgradGeometry &g, hipStream_t stream);
// The same for 16-bit tensors whose rows are whole groups of eight elements: raw 16-bit LDS images and two-element
// dot products (dwconv_bwd16.hip).  bwd_tiled16_workspace is 0 where the kernel does not cover g.
size_t bwd_tiled16_workspace(const WgradGeometry &g);
template <typename IO>
int try_launch_bwd_tiled16(const IO *in, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes,
                           const WgradGeometry &g, hipStream_t stream);

// Stride-1 "same" layers with 5x5 / 7x7 filters on maps too wide for several planes per workgroup: one channel per
// workgroup over a stack of its images, taps in scalar registers (dwconv_stack.hip).  Same return convention.
size_t bwd_stack_workspace(const WgradGeometry &g);  // 0 when that kernel does not cover g
template <typename IO>
int try_launch_bwd_stack(const IO *in, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes,
                         const WgradGeometry &g, hipStream_t stream);
template <typename IO>
int try_launch_fir_stack(const IO *in, const IO *taps, IO *out, const Geometry &g, hipStream_t stream);
// The same kernels at dilation 2 (3x3 and 5x5 taps, multiplier 1, stride 1, padding 2 * (K/2)).
size_t general_stack_workspace(const GeneralGeometry &g);  // 0 when they do not cover g
template <typename IO>
int try_launch_general_stack_forward(const IO *in, const IO *taps, IO *out, const GeneralGeometry &g, hipStream_t stream);
template <typename IO>
int try_launch_general_stack_backward(const IO *in, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws,
                                      size_t ws_bytes, const GeneralGeometry &g, hipStream_t stream);

// The same for stride-2 layers: dwconv_bwd_s2.hip.
size_t bwd_s2_workspace(const WgradGeometry &g);  // 0 when that kernel does not cover g
template <typename IO>
int try_launch_bwd_s2(const IO *in, const IO *gy, const IO *taps, IO *gx, IO *gw, void *ws, size_t ws_bytes,
                      const WgradGeometry &g, hipStream_t stream);

// ---- channels-last kernels: dwconv_nhwc.hip (T = float, double, half_t or bf16_t) ----
template <typename T>
int nhwc_forward(const T *in, const T *taps, T *out, const NhwcGeometry &g, hipStream_t stream);
template <typename T>
int nhwc_grad_input(const T *gy, const T *taps, T *gx, const NhwcGeometry &g, hipStream_t stream);
template <typename T>
int nhwc_backward_fused(const T *x, const T *gy, const T *taps, T *gx, T *gw, void *ws, size_t ws_bytes,
                        const NhwcGeometry &g, hipStream_t stream);
template <typename T>
size_t nhwc_grad_weight_workspace(const NhwcGeometry &g);
template <typename T>
int nhwc_grad_weight(const T *x, const T *gy, T *gw, void *ws, size_t ws_bytes, const NhwcGeometry &g,
                     hipStream_t stream);

// ---- backward of the fused forward epilogue: dwconv_epilogue_bwd.hip (IO = float, half_t or bf16_t) ----
size_t epilogue_backward_workspace(int batch, int channel, int out_h, int out_w, bool channels_last);
template <typename IO>
int epilogue_backward(const IO *conv, const IO *out_grad, const float *scale, const float *shift, IO *conv_grad,
                      float *param_grad, void *ws, size_t ws_bytes, int batch, int channel, int out_h, int out_w, int act,
                      bool channels_last, hipStream_t stream);

// ---- dilation and depth multiplier: dwconv_general.hip (T = float, double, half_t or bf16_t) ----
template <typename T>
int general_forward(const T *in, const T *taps, T *out, const GeneralGeometry &g, hipStream_t stream);
template <typename T>
int general_grad_input(const T *gy, const T *taps, T *gx, const GeneralGeometry &g, hipStream_t stream);
template <typename T>
size_t general_grad_weight_workspace(const GeneralGeometry &g);
template <typename T>
int general_grad_weight(const T *x, const T *gy, T *gw, void *ws, size_t ws_bytes, const GeneralGeometry &g,
                        hipStream_t stream);

}  // namespace dwconv
