/*
 * libdwconv_hip -- depthwise conv2d (forward, grad-input, grad-weight) for
 * AMD MI355X (gfx950), plain C ABI.
 *
 * These entry points are what a binding of the reference's extension module
 * `torch_dwconv._C` (torch_dwconv/dwconv.cpp:60-67) needs: one C function per
 * bound function, taking raw device pointers and integer geometry instead of
 * torch::Tensor.  Tensors are dense NCHW, `kernel` is (C,1,KH,KW).  All
 * pointers are device pointers valid on the device that is current when the
 * call is made; `stream` is a hipStream_t (NULL = the null stream).  Calls
 * only enqueue work and return; nothing is synchronised and nothing is kept
 * after the call returns.  The library allocates no device memory.
 *
 * Return value: DWCONV_OK (0) or a dwconv_status error code.  After an error
 * dwconv_last_error() returns a message for the calling thread.
 *
 * Geometry common to all entry points (the reference's DWConv2dKernelParams,
 * torch_dwconv/dwconv_kernel.cu:42-67):
 *   up_*   zero-stuffing factor applied to the input before filtering
 *   down_* decimation applied after filtering (the conv stride)
 *   pad_*  zeros added before (pad_*0) and after (pad_*1) the stuffed input
 *   forward != 0: taps used as stored (cross-correlation);
 *   forward == 0: taps rotated by 180 degrees (the grad-input direction).
 */
#ifndef DWCONV_HIP_H
#define DWCONV_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum dwconv_status {
    DWCONV_OK = 0,
    DWCONV_ERR_INVALID_ARGUMENT = 1, /* null pointer, non-positive extent, ... */
    DWCONV_ERR_UNSUPPORTED = 2,      /* geometry outside what the entry point accepts */
    DWCONV_ERR_WORKSPACE = 3,        /* workspace missing or too small */
    DWCONV_ERR_LAUNCH = 4            /* HIP reported an error at launch */
} dwconv_status;

/* Activation of the fused forward entry points (dwconv2d_fused_*). */
typedef enum dwconv_activation {
    DWCONV_ACT_NONE = 0,
    DWCONV_ACT_RELU = 1,  /* max(v, 0) */
    DWCONV_ACT_RELU6 = 2, /* min(max(v, 0), 6) */
    DWCONV_ACT_SILU = 3   /* v * sigmoid(v) */
} dwconv_activation;

/* Message describing the last error returned to this thread ("" if none). */
const char *dwconv_last_error(void);

/* Library version string, e.g. "dwconv_hip 0.1 gfx950". */
const char *dwconv_version(void);

/* Output extent along one axis: (in*up + pad0 + pad1 - k + down) / down.
 * Replaces the arithmetic of make_conv2d_params,
 * torch_dwconv/dwconv_kernel.cu:612-615. */
int dwconv_out_size(int in, int up, int down, int pad0, int pad1, int k);

/* Replaces `_C.use_dwconv2d_small` (torch_dwconv/dwconv.cpp:60,
 * torch_dwconv/dwconv_kernel.cu:652-662): 1 when the geometry is a stride-1,
 * same-size convolution of a plane no larger than 32x32 that the whole-plane
 * entry point dwconv2d_small_* accepts, else 0. */
int dwconv_use_dwconv2d_small(int in_h, int in_w, int kernel_h, int kernel_w,
                              int up_h, int up_w, int down_h, int down_w,
                              int pad_h, int pad_w);

/* Replaces `_C.dwconv2d` (torch_dwconv/dwconv.cpp:27-35 ->
 * dwconv2d_op, torch_dwconv/dwconv_kernel.cu:847-869).
 *   out[n,c,oy,ox] = sum_{ty,tx} U[oy*down_h - pad_h0 + ty, ox*down_w - pad_w0 + tx] * f[c,ty,tx]
 * U = input with up-1 zeros stuffed after every sample, zero outside.
 * `out` holds batch*channel*out_h*out_w elements, out_* = dwconv_out_size(...).
 * Accepts every up>=1, down>=1, kernel extent >=1 and pad >= -(extent) (the
 * reference supports nine hard-coded combinations and is undefined elsewhere,
 * dwconv_kernel.cu:808-845).  Forward convolution: up=1, down=stride,
 * pad0=pad1=padding.  Grad-input: input=grad_output, up=stride, down=1,
 * pads = g_pad of torch_dwconv/dwconv.py:39-44, forward=0. */
int dwconv2d_f32(const float *input, const float *kernel, float *out,
                 int batch, int channel, int in_h, int in_w,
                 int kernel_h, int kernel_w, int up_h, int up_w,
                 int down_h, int down_w, int pad_h0, int pad_h1,
                 int pad_w0, int pad_w1, int forward, void *stream);
int dwconv2d_f64(const double *input, const double *kernel, double *out,
                 int batch, int channel, int in_h, int in_w,
                 int kernel_h, int kernel_w, int up_h, int up_w,
                 int down_h, int down_w, int pad_h0, int pad_h1,
                 int pad_w0, int pad_w1, int forward, void *stream);

/* Replaces `_C.dwconv2d_small` (torch_dwconv/dwconv.cpp:37-46 ->
 * dwconv2d_small_op, torch_dwconv/dwconv_kernel.cu:734-771): stride-1
 * convolution whose output has the input's extent; `pad_h`,`pad_w` zeros lead
 * each axis and kernel-1-pad trail it.  up_* and down_* must be 1 and the plane
 * at most 32x32 (DWCONV_ERR_UNSUPPORTED otherwise); the kernel may be any
 * size. */
int dwconv2d_small_f32(const float *input, const float *kernel, float *out,
                       int batch, int channel, int in_h, int in_w,
                       int kernel_h, int kernel_w, int up_h, int up_w,
                       int down_h, int down_w, int pad_h, int pad_w,
                       int forward, void *stream);
int dwconv2d_small_f64(const double *input, const double *kernel, double *out,
                       int batch, int channel, int in_h, int in_w,
                       int kernel_h, int kernel_w, int up_h, int up_w,
                       int down_h, int down_w, int pad_h, int pad_w,
                       int forward, void *stream);

/* Bytes of device scratch that dwconv2d_backward_kernel_* needs for this
 * geometry (0 is possible).  The reference allocates its own zero-filled
 * result and accumulates into it with atomics (dwconv_kernel.cu:1026, :304,
 * :583); here the caller lends a workspace for per-workgroup partial sums that
 * a second kernel adds up in a fixed order.  `elem_size` is 2 (fp16/bf16), 4 or 8. */
size_t dwconv2d_backward_kernel_workspace_bytes(int batch, int channel,
                                                int in_h, int in_w,
                                                int out_h, int out_w,
                                                int kernel_h, int kernel_w,
                                                int down_h, int down_w,
                                                int pad_h, int pad_w,
                                                int elem_size);

/* Replaces `_C.dwconv2d_backward_kernel` (torch_dwconv/dwconv.cpp:48-58 ->
 * dwconv2d_backward_kernel_op, torch_dwconv/dwconv_kernel.cu:1015-1036).
 *   kernel_grad[c,i,j] = sum_{n,oy,ox} out_grad[n,c,oy,ox] *
 *                        input[n,c, oy*down_h - pad_h + i, ox*down_w - pad_w + j]
 * (taps falling outside `input` contribute nothing).  kernel_grad (C*KH*KW
 * elements) is overwritten; it need not be zeroed.  The result is bit-identical
 * from run to run.  up_* must be 1 (the reference ignores it). */
int dwconv2d_backward_kernel_f32(const float *input, const float *out_grad,
                                 float *kernel_grad, void *workspace,
                                 size_t workspace_bytes, int batch, int channel,
                                 int in_h, int in_w, int out_h, int out_w,
                                 int kernel_h, int kernel_w, int up_h, int up_w,
                                 int down_h, int down_w, int pad_h, int pad_w,
                                 void *stream);
int dwconv2d_backward_kernel_f64(const double *input, const double *out_grad,
                                 double *kernel_grad, void *workspace,
                                 size_t workspace_bytes, int batch, int channel,
                                 int in_h, int in_w, int out_h, int out_w,
                                 int kernel_h, int kernel_w, int up_h, int up_w,
                                 int down_h, int down_w, int pad_h, int pad_w,
                                 void *stream);

/* fp16 (`_f16`) and bfloat16 (`_bf16`) twins of the three operations above: tensors hold 16-bit elements
 * (passed as `unsigned short` storage), every product and partial sum is fp32, results are rounded to
 * nearest-even once when stored.  The reference dispatches half for `_C.dwconv2d`, `_C.dwconv2d_small` and
 * the general grad-weight kernel (torch_dwconv/dwconv_kernel.cu:749, :860, :999) and accumulates in half.
 * Workspace for grad-weight: dwconv2d_backward_kernel_workspace_bytes(..., elem_size = 2). */
int dwconv2d_f16(const unsigned short *input, const unsigned short *kernel, unsigned short *out,
                 int batch, int channel, int in_h, int in_w, int kernel_h, int kernel_w,
                 int up_h, int up_w, int down_h, int down_w, int pad_h0, int pad_h1,
                 int pad_w0, int pad_w1, int forward, void *stream);
int dwconv2d_bf16(const unsigned short *input, const unsigned short *kernel, unsigned short *out,
                  int batch, int channel, int in_h, int in_w, int kernel_h, int kernel_w,
                  int up_h, int up_w, int down_h, int down_w, int pad_h0, int pad_h1,
                  int pad_w0, int pad_w1, int forward, void *stream);
int dwconv2d_small_f16(const unsigned short *input, const unsigned short *kernel,
                       unsigned short *out, int batch, int channel, int in_h, int in_w,
                       int kernel_h, int kernel_w, int up_h, int up_w, int down_h, int down_w,
                       int pad_h, int pad_w, int forward, void *stream);
int dwconv2d_small_bf16(const unsigned short *input, const unsigned short *kernel,
                        unsigned short *out, int batch, int channel, int in_h, int in_w,
                        int kernel_h, int kernel_w, int up_h, int up_w, int down_h, int down_w,
                        int pad_h, int pad_w, int forward, void *stream);
int dwconv2d_backward_kernel_f16(const unsigned short *input, const unsigned short *out_grad,
                                 unsigned short *kernel_grad, void *workspace,
                                 size_t workspace_bytes, int batch, int channel, int in_h, int in_w,
                                 int out_h, int out_w, int kernel_h, int kernel_w, int up_h, int up_w,
                                 int down_h, int down_w, int pad_h, int pad_w, void *stream);
int dwconv2d_backward_kernel_bf16(const unsigned short *input, const unsigned short *out_grad,
                                  unsigned short *kernel_grad, void *workspace,
                                  size_t workspace_bytes, int batch, int channel, int in_h, int in_w,
                                  int out_h, int out_w, int kernel_h, int kernel_w, int up_h, int up_w,
                                  int down_h, int down_w, int pad_h, int pad_w, void *stream);

/* Both gradients of one layer in one call: in_grad (batch*channel*in_h*in_w) and kernel_grad
 * (channel*kernel_h*kernel_w), from the forward input, the output gradient and the taps.
 * Stands for the two calls the reference's autograd Function makes in a row in its backward
 * (torch_dwconv/dwconv.py:56-68: `_C.dwconv2d` in the backward direction with g_pad, then
 * `_C.dwconv2d_backward_kernel`); the reference has no single function for it.  Results are
 * the same as those two calls give; where a fused kernel covers the geometry out_grad is read
 * from memory once instead of twice.  out_h/out_w must be the forward output extent for
 * (stride, pad).  Workspace as for dwconv2d_backward_kernel_f32. */
int dwconv2d_backward_f32(const float *input, const float *out_grad, const float *kernel,
                          float *in_grad, float *kernel_grad, void *workspace,
                          size_t workspace_bytes, int batch, int channel, int in_h, int in_w,
                          int out_h, int out_w, int kernel_h, int kernel_w, int stride_h,
                          int stride_w, int pad_h, int pad_w, void *stream);

/* fp16 / bfloat16 twins (fp32 products and sums, one rounding on store). */
int dwconv2d_backward_f16(const unsigned short *input, const unsigned short *out_grad,
                          const unsigned short *kernel, unsigned short *in_grad,
                          unsigned short *kernel_grad, void *workspace, size_t workspace_bytes,
                          int batch, int channel, int in_h, int in_w, int out_h, int out_w,
                          int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
                          void *stream);
int dwconv2d_backward_bf16(const unsigned short *input, const unsigned short *out_grad,
                           const unsigned short *kernel, unsigned short *in_grad,
                           unsigned short *kernel_grad, void *workspace, size_t workspace_bytes,
                           int batch, int channel, int in_h, int in_w, int out_h, int out_w,
                           int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
                           void *stream);

/* dwconv2d_backward_f32 for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): the same kernels and the same results, bit for
 * bit, but the partial grad-weight sums go to a buffer of DWCONV_NOALLOC_SCRATCH_BYTES that is part of
 * the library's device image, so there is no workspace argument and the call allocates nothing.  It has no
 * counterpart in the reference (whose backward allocates its results, torch_dwconv/dwconv_kernel.cu:782,
 * :1026).  A geometry whose dwconv2d_backward_kernel_workspace_bytes(..., elem_size = 4) exceeds
 * DWCONV_NOALLOC_SCRATCH_BYTES is refused with DWCONV_ERR_WORKSPACE before anything is launched.  Every
 * device holds one such buffer, shared by all calls on it: the kernels overwrite what they read from it,
 * so nothing needs clearing between calls, but two calls that overlap in time on one device (different
 * streams or threads) race on it -- run them on one stream or order them yourself.  The buffer's address
 * is looked up on the first call on each device; make that call outside stream capture (a first call on
 * a capturing stream returns DWCONV_ERR_UNSUPPORTED and launches nothing). */
#define DWCONV_NOALLOC_SCRATCH_BYTES (32u << 20)
int dwconv2d_backward_noalloc_f32(const float *input, const float *out_grad, const float *kernel,
                                  float *in_grad, float *kernel_grad, int batch, int channel,
                                  int in_h, int in_w, int out_h, int out_w, int kernel_h, int kernel_w,
                                  int stride_h, int stride_w, int pad_h, int pad_w, void *stream);

/* ---- channels-last (NHWC) tensors -------------------------------------------------------------
 * No counterpart in the reference, which makes every tensor NCHW-contiguous before its kernels run
 * (torch_dwconv/dwconv_kernel.cu:741, :855, :1023): these entry points serve callers whose activations are
 * channels-last, so that no layout conversion is needed either side of the op.  input is (N,H,W,C), out and
 * out_grad are (N,OH,OW,C) with OH = dwconv_out_size(H, 1, stride_h, pad_h, pad_h, kernel_h); kernel and
 * kernel_grad are (C,1,KH,KW) as everywhere else.  Same arithmetic as dwconv2d_* with up = 1,
 * down = stride, pad0 = pad1 = pad (forward) and as the reference's backward pair (dwconv.py:56-68). */
int dwconv2d_nhwc_f32(const float *input, const float *kernel, float *out, int batch, int channel,
                      int in_h, int in_w, int kernel_h, int kernel_w, int stride_h, int stride_w,
                      int pad_h, int pad_w, void *stream);
int dwconv2d_nhwc_f64(const double *input, const double *kernel, double *out, int batch, int channel,
                      int in_h, int in_w, int kernel_h, int kernel_w, int stride_h, int stride_w,
                      int pad_h, int pad_w, void *stream);
int dwconv2d_nhwc_f16(const unsigned short *input, const unsigned short *kernel, unsigned short *out,
                      int batch, int channel, int in_h, int in_w, int kernel_h, int kernel_w,
                      int stride_h, int stride_w, int pad_h, int pad_w, void *stream);
int dwconv2d_nhwc_bf16(const unsigned short *input, const unsigned short *kernel, unsigned short *out,
                       int batch, int channel, int in_h, int in_w, int kernel_h, int kernel_w,
                       int stride_h, int stride_w, int pad_h, int pad_w, void *stream);

/* Workspace (bytes) for dwconv2d_backward_nhwc_*; elem_size 2, 4 or 8. */
size_t dwconv2d_backward_nhwc_workspace_bytes(int batch, int channel, int in_h, int in_w,
                                              int kernel_h, int kernel_w, int stride_h, int stride_w,
                                              int pad_h, int pad_w, int elem_size);

/* Both gradients (either of in_grad, kernel_grad may be NULL to skip it).  kernel_grad is overwritten
 * and bit-identical from run to run.  With both asked for, layers with a 3x3 filter and pad 1 or a 5x5
 * filter and pad 2 are served by one kernel that reads out_grad once: stride 1 (3x3: any element type,
 * 5x5: fp32) and stride 2 on even extents (fp32); the workspace is needed even then. */
int dwconv2d_backward_nhwc_f32(const float *input, const float *out_grad, const float *kernel,
                               float *in_grad, float *kernel_grad, void *workspace,
                               size_t workspace_bytes, int batch, int channel, int in_h, int in_w,
                               int out_h, int out_w, int kernel_h, int kernel_w, int stride_h,
                               int stride_w, int pad_h, int pad_w, void *stream);
int dwconv2d_backward_nhwc_f64(const double *input, const double *out_grad, const double *kernel,
                               double *in_grad, double *kernel_grad, void *workspace,
                               size_t workspace_bytes, int batch, int channel, int in_h, int in_w,
                               int out_h, int out_w, int kernel_h, int kernel_w, int stride_h,
                               int stride_w, int pad_h, int pad_w, void *stream);
int dwconv2d_backward_nhwc_f16(const unsigned short *input, const unsigned short *out_grad,
                               const unsigned short *kernel, unsigned short *in_grad,
                               unsigned short *kernel_grad, void *workspace, size_t workspace_bytes,
                               int batch, int channel, int in_h, int in_w, int out_h, int out_w,
                               int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h,
                               int pad_w, void *stream);
int dwconv2d_backward_nhwc_bf16(const unsigned short *input, const unsigned short *out_grad,
                                const unsigned short *kernel, unsigned short *in_grad,
                                unsigned short *kernel_grad, void *workspace, size_t workspace_bytes,
                                int batch, int channel, int in_h, int in_w, int out_h, int out_w,
                                int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h,
                                int pad_w, void *stream);

/* ---- forward convolution with a fused epilogue ---------------------------------------------------
 *   out = act(conv(input, kernel) * scale[c] + shift[c])
 * for the step that follows a depthwise convolution in EfficientNet / MobileNet / ConvNeXt blocks: bias
 * (which the reference rejects, torch_dwconv/dwconv.py:108-109), a folded batch-norm (scale and shift) and
 * ReLU / ReLU6 / SiLU.  No counterpart in the reference.  scale and shift are device arrays of `channel`
 * entries in the accumulation type (float for f32/f16/bf16 tensors, double for f64); either may be NULL
 * (factor 1 / offset 0).  Saves the separate elementwise pass over `out` (one read and one write of it).
 * conv = dwconv2d_* with up = 1, down = stride, pad0 = pad1 = pad, forward = 1; `_nhwc`: channels-last tensors. */
int dwconv2d_fused_f32(const float *input, const float *kernel, const float *scale,
    const float *shift, float *out, int batch, int channel, int in_h, int in_w,
    int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
    int activation, void *stream);
int dwconv2d_fused_nhwc_f32(const float *input, const float *kernel, const float *scale,
    const float *shift, float *out, int batch, int channel, int in_h, int in_w,
    int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
    int activation, void *stream);
int dwconv2d_fused_f64(const double *input, const double *kernel, const double *scale,
    const double *shift, double *out, int batch, int channel, int in_h, int in_w,
    int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
    int activation, void *stream);
int dwconv2d_fused_nhwc_f64(const double *input, const double *kernel, const double *scale,
    const double *shift, double *out, int batch, int channel, int in_h, int in_w,
    int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
    int activation, void *stream);
int dwconv2d_fused_f16(const unsigned short *input, const unsigned short *kernel, const float *scale,
    const float *shift, unsigned short *out, int batch, int channel, int in_h, int in_w,
    int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
    int activation, void *stream);
int dwconv2d_fused_nhwc_f16(const unsigned short *input, const unsigned short *kernel, const float *scale,
    const float *shift, unsigned short *out, int batch, int channel, int in_h, int in_w,
    int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
    int activation, void *stream);
int dwconv2d_fused_bf16(const unsigned short *input, const unsigned short *kernel, const float *scale,
    const float *shift, unsigned short *out, int batch, int channel, int in_h, int in_w,
    int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
    int activation, void *stream);
int dwconv2d_fused_nhwc_bf16(const unsigned short *input, const unsigned short *kernel, const float *scale,
    const float *shift, unsigned short *out, int batch, int channel, int in_h, int in_w,
    int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
    int activation, void *stream);

/* Backward of that epilogue, for training through the fused forward (no counterpart in the reference).  The fused
 * forward keeps nothing but its inputs; in the backward pass the caller recomputes conv_out = conv(input, kernel)
 * with dwconv2d_* / dwconv2d_nhwc_* and calls this entry point, which makes in one sweep
 *   conv_out_grad       = out_grad * act'(z) * scale[c],   z = conv_out * scale[c] + shift[c]
 *   scale_shift_grad[c][0] = sum over (n,y,x) of out_grad * act'(z) * conv_out      (gradient of scale)
 *   scale_shift_grad[c][1] = sum over (n,y,x) of out_grad * act'(z)                 (gradient of shift)
 * conv_out_grad (it may alias conv_out) is then the out_grad of dwconv2d_backward_*.  Tensors are
 * (N,C,OH,OW) or, with channels_last != 0, (N,OH,OW,C); scale / shift may be NULL as in the forward;
 * scale_shift_grad holds 2 * channel floats and is bit-identical from run to run.  fp32 arithmetic. */
size_t dwconv2d_epilogue_backward_workspace_bytes(int batch, int channel, int out_h, int out_w, int channels_last);
int dwconv2d_epilogue_backward_f32(const float *conv_out, const float *out_grad, const float *scale, const float *shift,
    float *conv_out_grad, float *scale_shift_grad, void *workspace, size_t workspace_bytes, int batch, int channel,
    int out_h, int out_w, int activation, int channels_last, void *stream);
int dwconv2d_epilogue_backward_f16(const unsigned short *conv_out, const unsigned short *out_grad, const float *scale,
    const float *shift, unsigned short *conv_out_grad, float *scale_shift_grad, void *workspace, size_t workspace_bytes,
    int batch, int channel, int out_h, int out_w, int activation, int channels_last, void *stream);
int dwconv2d_epilogue_backward_bf16(const unsigned short *conv_out, const unsigned short *out_grad, const float *scale,
    const float *shift, unsigned short *conv_out_grad, float *scale_shift_grad, void *workspace, size_t workspace_bytes,
    int batch, int channel, int out_h, int out_w, int activation, int channels_last, void *stream);

/* ---- dilation and depth multiplier ------------------------------------------------------------------
 * The two options the reference's check_options refuses (torch_dwconv/dwconv.py:99-106): a dilation
 * above 1 and out_channels = multiplier * in_channels.  input (N,C,H,W); kernel and kernel_grad
 * (C*multiplier,1,KH,KW); out and out_grad (N,C*multiplier,OH,OW) with
 * OH = (H + 2*pad_h - dil_h*(KH-1) - 1) / stride_h + 1:
 *   out[n, c*M+j, oy, ox] = sum_{ty,tx} input[n, c, oy*stride - pad + ty*dil, ox*stride - pad + tx*dil] * kernel[c*M+j, ty, tx]
 * i.e. F.conv2d(groups=C, dilation=dil).  With multiplier 1 and dilation 1 the call is served by the tuned
 * kernels behind dwconv2d_* / dwconv2d_backward_*; otherwise by per-element kernels (correct, not tuned).
 * kernel_grad is bit-identical from run to run. */
size_t dwconv2d_general_backward_workspace_bytes(int batch, int channel, int in_h, int in_w,
                                                 int multiplier, int kernel_h, int kernel_w,
                                                 int stride_h, int stride_w, int pad_h, int pad_w,
                                                 int dil_h, int dil_w, int elem_size);
int dwconv2d_general_f32(const float *input, const float *kernel, float *out,
    int batch, int channel, int in_h, int in_w, int multiplier, int kernel_h, int kernel_w,
    int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void *stream);
int dwconv2d_general_backward_f32(const float *input, const float *out_grad, const float *kernel,
    float *in_grad, float *kernel_grad, void *workspace, size_t workspace_bytes,
    int batch, int channel, int in_h, int in_w, int out_h, int out_w, int multiplier,
    int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
    int dil_h, int dil_w, void *stream);
int dwconv2d_general_f64(const double *input, const double *kernel, double *out,
    int batch, int channel, int in_h, int in_w, int multiplier, int kernel_h, int kernel_w,
    int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void *stream);
int dwconv2d_general_backward_f64(const double *input, const double *out_grad, const double *kernel,
    double *in_grad, double *kernel_grad, void *workspace, size_t workspace_bytes,
    int batch, int channel, int in_h, int in_w, int out_h, int out_w, int multiplier,
    int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
    int dil_h, int dil_w, void *stream);
int dwconv2d_general_f16(const unsigned short *input, const unsigned short *kernel, unsigned short *out,
    int batch, int channel, int in_h, int in_w, int multiplier, int kernel_h, int kernel_w,
    int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void *stream);
int dwconv2d_general_backward_f16(const unsigned short *input, const unsigned short *out_grad, const unsigned short *kernel,
    unsigned short *in_grad, unsigned short *kernel_grad, void *workspace, size_t workspace_bytes,
    int batch, int channel, int in_h, int in_w, int out_h, int out_w, int multiplier,
    int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
    int dil_h, int dil_w, void *stream);
int dwconv2d_general_bf16(const unsigned short *input, const unsigned short *kernel, unsigned short *out,
    int batch, int channel, int in_h, int in_w, int multiplier, int kernel_h, int kernel_w,
    int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void *stream);
int dwconv2d_general_backward_bf16(const unsigned short *input, const unsigned short *out_grad, const unsigned short *kernel,
    unsigned short *in_grad, unsigned short *kernel_grad, void *workspace, size_t workspace_bytes,
    int batch, int channel, int in_h, int in_w, int out_h, int out_w, int multiplier,
    int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
    int dil_h, int dil_w, void *stream);

/* Tuning/diagnostic hook: name of the kernel variant the last successful call
 * on this thread launched (e.g. "tile_f32<k3,s1,v4>"), for benchmarks and tests. */
const char *dwconv_last_variant(void);

#ifdef __cplusplus
}
#endif

#endif /* DWCONV_HIP_H */
