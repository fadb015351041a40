/*
 * CPU oracle for the depthwise conv2d path of torch_dwconv.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is a plain-C, double-precision
 * restatement of what the reference's kernels compute.  It exists so that the
 * HIP kernels can be checked against something that does not share any code
 * with them.  Nothing in the shipped package may link, load or call it; only
 * the test-suite, the smoke check and the CPU-baseline leg of the benchmark do.
 *
 * Every function names the reference lines it restates (paths relative to the
 * reference checkout, torch_dwconv/...).
 *
 * How each function is pinned (see tests/test_oracle.py):
 *   oracle_out_size            - equals floor((H+2p-k)/s)+1 on a sweep, and the
 *                                g_pad identity of dwconv.py:39-44.
 *   oracle_use_dwconv2d_small  - hand-evaluated truth table.
 *   oracle_dwconv2d_f64        - torch F.conv2d fp64 (the oracle the reference's
 *                                own tests use, test/test_forward.py:14),
 *                                F.conv_transpose2d fp64 for the backward
 *                                direction, a 7-loop pure-Python brute force,
 *                                delta / box-filter / 1x1 closed forms, the
 *                                adjoint identity, committed golden vectors.
 *   oracle_dwconv2d_small_f64  - same, through its equivalence with the large op.
 *   oracle_backward_kernel_f64 - torch autograd fp64, brute force, adjoint
 *                                identity <w, gw> == <y, gy>, golden vectors.
 *
 * Build: gcc -O2 -fPIC -shared -fopenmp (see oracle/Makefile).
 */
#include <stddef.h>
#include <stdint.h>

/* dwconv_kernel.cu:612-615 (make_conv2d_params): output extent of the
 * up-sample / FIR / down-sample operator along one axis. */
int oracle_out_size(int in, int up, int down, int pad0, int pad1, int k)
{
    return (in * up + pad0 + pad1 - k + down) / down;
}

/* dwconv_kernel.cu:652-662 (use_dwconv2d_small): may the whole-plane
 * "small" kernel take this geometry? */
int oracle_use_dwconv2d_small(int in_h, int in_w, int kernel_h, int kernel_w,
                              int up_h, int up_w, int down_h, int down_w,
                              int pad_h, int pad_w)
{
    int out_h = oracle_out_size(in_h, up_h, down_h, pad_h, pad_h, kernel_h);
    int out_w = oracle_out_size(in_w, up_w, down_w, pad_w, pad_w, kernel_w);
    return down_h == 1 && down_w == 1 && in_h <= 32 && in_w <= 32 &&
           in_h == out_h && in_w == out_w && pad_h >= 0 && pad_h < kernel_h &&
           pad_w >= 0 && pad_w < kernel_w &&
           kernel_h * kernel_w <= (in_h + 1) / 2 * in_w;
}

/* Value of the zero-stuffed ("up-sampled") plane at position (uy,ux):
 * the sample in[uy/up_h][ux/up_w] when both are multiples of the factor and
 * fall inside the plane, else zero.  dwconv_kernel.cu:122-144 builds exactly
 * this view (floor_div of the mid coordinate and the zero fill of the tile). */
static double upsampled_at(const double *plane, int in_h, int in_w, int up_h,
                           int up_w, long uy, long ux)
{
    if (uy < 0 || ux < 0 || uy % up_h != 0 || ux % up_w != 0)
        return 0.0;
    long iy = uy / up_h, ix = ux / up_w;
    if (iy >= in_h || ix >= in_w)
        return 0.0;
    return plane[iy * in_w + ix];
}

/* dwconv_kernel.cu:69-181 (dwconv2d_kernel), any up/down/pad:
 *   out[n,c,oy,ox] = sum_{ty,tx} U[oy*down_h - pad_h0 + ty, ox*down_w - pad_w0 + tx] * f[ty,tx]
 * with U the zero-stuffed input and f = kernel (forward, :107-109) or the
 * kernel rotated by 180 degrees (backward, :111-113).
 * `out` must hold batch*channel*out_h*out_w doubles with out_* from
 * oracle_out_size. */
void oracle_dwconv2d_f64(const double *in, const double *kernel, double *out,
                         int batch, int channel, int in_h, int in_w,
                         int kernel_h, int kernel_w, int up_h, int up_w,
                         int down_h, int down_w, int pad_h0, int pad_h1,
                         int pad_w0, int pad_w1, int forward)
{
    const int out_h = oracle_out_size(in_h, up_h, down_h, pad_h0, pad_h1, kernel_h);
    const int out_w = oracle_out_size(in_w, up_w, down_w, pad_w0, pad_w1, kernel_w);
    const long planes = (long)batch * channel;
    if (out_h <= 0 || out_w <= 0)
        return;
#pragma omp parallel for schedule(static)
    for (long pl = 0; pl < planes; ++pl) {
        const double *src = in + pl * (long)in_h * in_w;
        const double *taps = kernel + (pl % channel) * (long)kernel_h * kernel_w;
        double *dst = out + pl * (long)out_h * out_w;
        for (int oy = 0; oy < out_h; ++oy)
            for (int ox = 0; ox < out_w; ++ox) {
                double acc = 0.0;
                for (int ty = 0; ty < kernel_h; ++ty)
                    for (int tx = 0; tx < kernel_w; ++tx) {
                        double f = forward
                            ? taps[ty * kernel_w + tx]
                            : taps[(kernel_h - 1 - ty) * kernel_w + (kernel_w - 1 - tx)];
                        acc += f * upsampled_at(src, in_h, in_w, up_h, up_w,
                                                (long)oy * down_h - pad_h0 + ty,
                                                (long)ox * down_w - pad_w0 + tx);
                    }
                dst[oy * out_w + ox] = acc;
            }
    }
}

/* dwconv_kernel.cu:308-442 (dwconv2d_small_kernel): stride-1, output the same
 * size as the input, leading pad (pad_h,pad_w); rows/columns past the plane
 * read as zero (:351-353); backward walks the taps in reverse (:412-425). */
void oracle_dwconv2d_small_f64(const double *in, const double *kernel,
                               double *out, int batch, int channel, int in_h,
                               int in_w, int kernel_h, int kernel_w, int pad_h,
                               int pad_w, int forward)
{
    const long planes = (long)batch * channel;
#pragma omp parallel for schedule(static)
    for (long pl = 0; pl < planes; ++pl) {
        const double *src = in + pl * (long)in_h * in_w;
        const double *taps = kernel + (pl % channel) * (long)kernel_h * kernel_w;
        double *dst = out + pl * (long)in_h * in_w;
        for (int y = 0; y < in_h; ++y)
            for (int x = 0; x < in_w; ++x) {
                double acc = 0.0;
                for (int r = 0; r < kernel_h; ++r)
                    for (int c = 0; c < kernel_w; ++c) {
                        int iy = y - pad_h + r, ix = x - pad_w + c;
                        if (iy < 0 || iy >= in_h || ix < 0 || ix >= in_w)
                            continue;
                        int t = r * kernel_w + c;
                        double f = forward ? taps[t]
                                           : taps[kernel_h * kernel_w - 1 - t];
                        acc += f * src[iy * in_w + ix];
                    }
                dst[y * in_w + x] = acc;
            }
    }
}

/* dwconv_kernel.cu:260-297 (dwconv2d_backward_kernel_kernel) and its
 * small-map twin :444-588 compute the same sum:
 *   gw[c,i,j] = sum_{n,oy,ox} gy[n,c,oy,ox] * x[n,c, oy*down_h - pad_h + i, ox*down_w - pad_w + j]
 * skipping taps that fall outside x (:280-286). */
void oracle_backward_kernel_f64(const double *in, const double *out_grad,
                                double *kernel_grad, int batch, int channel,
                                int in_h, int in_w, int out_h, int out_w,
                                int kernel_h, int kernel_w, int down_h,
                                int down_w, int pad_h, int pad_w)
{
#pragma omp parallel for schedule(static)
    for (int c = 0; c < channel; ++c)
        for (int i = 0; i < kernel_h; ++i)
            for (int j = 0; j < kernel_w; ++j) {
                double acc = 0.0;
                for (int n = 0; n < batch; ++n) {
                    const double *x = in + ((long)n * channel + c) * in_h * in_w;
                    const double *gy = out_grad + ((long)n * channel + c) * out_h * out_w;
                    for (int oy = 0; oy < out_h; ++oy) {
                        int iy = oy * down_h - pad_h + i;
                        if (iy < 0 || iy >= in_h)
                            continue;
                        for (int ox = 0; ox < out_w; ++ox) {
                            int ix = ox * down_w - pad_w + j;
                            if (ix < 0 || ix >= in_w)
                                continue;
                            acc += gy[oy * out_w + ox] * x[iy * in_w + ix];
                        }
                    }
                }
                kernel_grad[((long)c * kernel_h + i) * kernel_w + j] = acc;
            }
}
