// Whole-plane kernels for small feature maps (up to 32 elements wide, "same" column padding); element type fp32,
// fp16 or bf16, LDS and arithmetic fp32.
//
// Planes of a small map are tiny (196 B to 4 KiB) and sit back to back in memory,
// so the only way to move them at HBM speed is to treat a run of P planes as one
// flat stream: 128-bit loads of the run into LDS (same layout as in memory, no
// index arithmetic), arithmetic out of LDS, results back into LDS in their
// memory layout, 128-bit stores of the run.  One wavefront (a 64-lane workgroup,
// so no cross-wave barrier exists) owns a run; a CU holds about ten such
// wavefronts, each with several loads in flight.
//
// A lane owns BH full-width output rows of one plane.  Because it holds whole
// rows, which taps fall off the left/right edge is known at compile time (they
// are simply not emitted); rows above/below the plane are replaced by zeros
// with a select.  The reference's counterpart (torch_dwconv/dwconv_kernel.cu:308-442,
// :444-588) keeps a zero-filled padded tile in shared memory and re-reads every
// tap for every output; it takes any plane up to 32 x 32 (:652-671), and so does this family.
//
// The plane width is a template parameter in one of two ways.  Exact (RAG = false): rows are W elements and are
// read with vector reads where W allows.  Ragged (RAG = true): W is a capacity and the real width (1..W) arrives
// at run time; rows are read element by element, columns past the real width are zeroed by a wavefront-uniform
// select and their sums are never stored.  One translation unit per instance (dwconv_small_width.hip).
//
//   small_down_kernel : up = 1, decimation S; forward, and grad-input of stride-1 layers (FLIP)
//   small_up2_kernel  : up = 2, taps rotated; grad-input of stride-2 layers
// (grad-weight and the fused backward of these maps: dwconv_small_bwd.hpp)
#pragma once

#include "dwconv_small_common.hpp"

namespace dwconv {

namespace {

// out[oy,ox] = sum_{ty,tx} in[oy*S - pad_h + ty, ox*S - K/2 + tx] * f[ty,tx]
// D: dilation of the taps (both axes; the column padding is then D * (K/2)).
template <typename IO, int W, bool RAG, int K, int S, bool FLIP, int BH, int D = 1>
__global__ __launch_bounds__(kWave) void small_down_kernel(const SmallPlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int OW = (W - 1) / S + 1;  // output columns a lane computes (the real count when exact)
    constexpr int KE = (K - 1) * D + 1;  // rows and columns the dilated taps span
    constexpr int PW = D * (K / 2);
    constexpr int WIN_ROWS = (BH - 1) * S + KE;
    const int w_in = RAG ? p.in_w : W, w_out = RAG ? p.out_w : OW;

    const long plane0 = static_cast<long>(blockIdx.x) * p.planes_per_run;
    const int nplanes = static_cast<int>(min(static_cast<long>(p.planes_per_run), p.planes - plane0));
    const int in_plane = p.in_h * w_in, out_plane = p.out_h * w_out;
    // LDS row pitch: the width, or width + 1 for ragged even widths (see ragged_pitch)
    const int lp_in = RAG ? p.lp_in : W, lp_out = RAG ? p.lp_out : OW;
    const bool pad_in = RAG && p.magic_in != 0, pad_out = RAG && p.magic_out != 0;
    const int lin_plane = p.in_h * lp_in, lout_plane = p.out_h * lp_out;

    const int pl_raw = fast_div(threadIdx.x, p.lpp_magic);
    const int rb = threadIdx.x - pl_raw * p.lanes_per_plane;
    const bool active = pl_raw < nplanes;
    const int pl = active ? pl_raw : 0;

    // runs that start off a 4-element boundary are moved as the aligned span around them (see lds_to_run)
    const long in0 = plane0 * in_plane, out0 = plane0 * out_plane;
    const int hin = static_cast<int>(in0 & 3), hout = static_cast<int>(out0 & 3);

    float tapv[K * K];
    load_taps<K * K, FLIP>(static_cast<const IO *>(p.taps), static_cast<int>((plane0 + pl) % p.channel), tapv);
    if (pad_in)
        run_to_lds_rows(static_cast<const IO *>(p.in) + (in0 - hin), lds, nplanes * in_plane + hin, hin, p.magic_in, p.zero_off - 1);
    else
        run_to_lds(static_cast<const IO *>(p.in) + (in0 - hin), lds, nplanes * in_plane + hin);
    const float *zrow = lds + p.zero_off;  // stands in for the rows above and below the plane
    clear_zero_row<W>(lds + p.zero_off);
    __syncthreads();

    float acc[BH][OW];
#pragma unroll
    for (int b = 0; b < BH; ++b)
#pragma unroll
        for (int o = 0; o < OW; ++o) acc[b][o] = 0.f;

    const int oy0 = rb * BH;
    const float *plane = lds + (pad_in ? 0 : hin) + pl * lin_plane;
    // rows are read one ahead of their use and the sums pinned after every row (see pin_registers)
    auto row_at = [&](int iy) { return static_cast<unsigned>(iy) < static_cast<unsigned>(p.in_h) ? plane + iy * lp_in : zrow; };
    float nxt[W];
    lds_load_row_w<W, RAG>(row_at(oy0 * S - p.pad_h), nxt, w_in);
#pragma unroll
    for (int wr = 0; wr < WIN_ROWS; ++wr) {
        float row[W];
#pragma unroll
        for (int i = 0; i < W; ++i) row[i] = nxt[i];
        if (wr + 1 < WIN_ROWS) lds_load_row_w<W, RAG>(row_at(oy0 * S - p.pad_h + wr + 1), nxt, w_in);
#pragma unroll
        for (int b = 0; b < BH; ++b) {
            const int dy = wr - b * S;
            if (dy < 0 || dy >= KE || dy % D != 0) continue;
            const int ty = dy / D;
#pragma unroll
            for (int tx = 0; tx < K; ++tx)
#pragma unroll
                for (int o = 0; o < OW; ++o) {
                    const int ix = o * S - PW + tx * D;
                    if (ix < 0 || ix >= W) continue;
                    acc[b][o] = fmaf(row[ix], tapv[ty * K + tx], acc[b][o]);
                }
        }
        pin_registers(acc);
    }
    if constexpr (!FLIP) {
        if (p.epi.enabled()) {
            epilogue_apply_block<1>(acc, p.epi, static_cast<int>((plane0 + pl) % p.channel));
        }
    }
    __syncthreads();  // every lane has read its input rows: the run can be overwritten in place

    if (active) {
        float *dst = lds + (pad_out ? 0 : hout) + pl * lout_plane;
#pragma unroll
        for (int b = 0; b < BH; ++b)
            if (oy0 + b < p.out_h) lds_store_row_w<OW, RAG>(dst + (oy0 + b) * lp_out, acc[b], w_out);
    }
    __syncthreads();
    if (pad_out)
        lds_to_run_rows(static_cast<IO *>(p.out) + (out0 - hout), lds, nplanes * out_plane + hout, hout, p.magic_out);
    else
        lds_to_run(static_cast<IO *>(p.out) + (out0 - hout), lds, nplanes * out_plane + hout, hout);
}

// up = 2, taps rotated, "same" padding of the forward conv (leading pad of the transposed problem = K/2):
//   out[2q + r] = sum_a in[q - m + r + a] * g'[r + 2a],  g'[t] = g[t - E],  E = (K/2) & 1,  m = (K/2 + E) / 2.
// Input planes are W wide (or up to W, ragged), output planes 2W or 2W - 1 (the forward input had an odd extent);
// a lane owns output rows 2q, 2q+1.
template <typename IO, int W, bool RAG, int K>
__global__ __launch_bounds__(kWave) void small_up2_kernel(const SmallPlan p)
{
    extern __shared__ float4 lds_raw[];
    float *lds = reinterpret_cast<float *>(lds_raw);
    constexpr int OW = 2 * W;
    constexpr int E = (K / 2) & 1;
    constexpr int M = (K / 2 + E) / 2;
    constexpr int KA = (K + E + 1) / 2;
    constexpr int WIN_ROWS = KA + 1;
    const int w_in = RAG ? p.in_w : W, w_out = RAG ? p.out_w : OW;

    const long plane0 = static_cast<long>(blockIdx.x) * p.planes_per_run;
    const int nplanes = static_cast<int>(min(static_cast<long>(p.planes_per_run), p.planes - plane0));
    const int in_plane = p.in_h * w_in, out_plane = p.out_h * w_out;
    const int lp_in = RAG ? p.lp_in : W, lp_out = RAG ? p.lp_out : OW;
    const bool pad_in = RAG && p.magic_in != 0, pad_out = RAG && p.magic_out != 0;
    const int lin_plane = p.in_h * lp_in, lout_plane = p.out_h * lp_out;

    const int pl_raw = fast_div(threadIdx.x, p.lpp_magic);
    const int q = threadIdx.x - pl_raw * p.lanes_per_plane;
    const bool active = pl_raw < nplanes;
    const int pl = active ? pl_raw : 0;

    const long in0 = plane0 * in_plane, out0 = plane0 * out_plane;
    const int hin = static_cast<int>(in0 & 3), hout = static_cast<int>(out0 & 3);

    float tapv[K * K];
    load_taps<K * K, true>(static_cast<const IO *>(p.taps), static_cast<int>((plane0 + pl) % p.channel), tapv);
    if (pad_in)
        run_to_lds_rows(static_cast<const IO *>(p.in) + (in0 - hin), lds, nplanes * in_plane + hin, hin, p.magic_in, p.zero_off - 1);
    else
        run_to_lds(static_cast<const IO *>(p.in) + (in0 - hin), lds, nplanes * in_plane + hin);
    const float *zrow = lds + p.zero_off;  // stands in for the rows above and below the plane
    clear_zero_row<W>(lds + p.zero_off);
    __syncthreads();

    float acc[2][OW];
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int o = 0; o < OW; ++o) acc[r][o] = 0.f;

    const float *plane = lds + (pad_in ? 0 : hin) + pl * lin_plane;
    auto row_at = [&](int iy) { return static_cast<unsigned>(iy) < static_cast<unsigned>(p.in_h) ? plane + iy * lp_in : zrow; };
    float nxt[W];
    lds_load_row_w<W, RAG>(row_at(q - p.pad_h), nxt, w_in);
#pragma unroll
    for (int wr = 0; wr < WIN_ROWS; ++wr) {
        float row[W];
#pragma unroll
        for (int i = 0; i < W; ++i) row[i] = nxt[i];
        if (wr + 1 < WIN_ROWS) lds_load_row_w<W, RAG>(row_at(q - p.pad_h + wr + 1), nxt, w_in);
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int a = wr - r;
            if (a < 0 || a >= KA) continue;
            const int fy = r + 2 * a - E;
            if (fy < 0 || fy >= K) continue;
#pragma unroll
            for (int o = 0; o < OW; ++o) {
                const int xq = o / 2, rx = o % 2;
#pragma unroll
                for (int ax = 0; ax < KA; ++ax) {
                    const int fx = rx + 2 * ax - E;
                    const int ix = xq - M + rx + ax;
                    if (fx < 0 || fx >= K || ix < 0 || ix >= W) continue;
                    acc[r][o] = fmaf(row[ix], tapv[fy * K + fx], acc[r][o]);
                }
            }
        }
        pin_registers(acc);
    }
    __syncthreads();

    if (active) {
        float *dst = lds + (pad_out ? 0 : hout) + pl * lout_plane;
#pragma unroll
        for (int r = 0; r < 2; ++r)
            if (2 * q + r < p.out_h) lds_store_row_w<OW, RAG>(dst + (2 * q + r) * lp_out, acc[r], w_out);
    }
    __syncthreads();
    if (pad_out)
        lds_to_run_rows(static_cast<IO *>(p.out) + (out0 - hout), lds, nplanes * out_plane + hout, hout, p.magic_out);
    else
        lds_to_run(static_cast<IO *>(p.out) + (out0 - hout), lds, nplanes * out_plane + hout, hout);
}

// LDS of a run of `planes` planes (the larger of its input and output image, plus the up to three elements in front
// of a run that starts off a 4-element boundary) plus, for ragged widths, the spare floats that reads past the last
// row land in.
size_t small_lds_bytes(int planes, int in_plane, int out_plane, int spare)
{
    return (static_cast<size_t>(planes) * (in_plane > out_plane ? in_plane : out_plane) + 4 + spare) * 4;
}

// float offset of the row of zeros: behind the run image and the spare floats
int small_zero_off(int planes, int in_plane, int out_plane, int spare)
{
    return round_up(planes * (in_plane > out_plane ? in_plane : out_plane) + 4 + spare, 4);
}

// Planes per wavefront: as many as there are lane slots within the LDS budget; when a plane is not a multiple of 4
// elements a multiple of 4 of them if that costs less than half (every run then starts on a 4-element boundary).
int planes_per_run(int lanes_per_plane, int in_plane, int out_plane, int lin_plane, int lout_plane, long planes)
{
    int P = kWave / lanes_per_plane;
    while (P > 0 && small_lds_bytes(P, lin_plane, lout_plane, 0) > 16 * 1024 + 16) --P;
    if ((in_plane % 4 != 0 || out_plane % 4 != 0) && P >= 4) P -= P % 4;
    if (static_cast<long>(P) > planes && in_plane % 4 == 0 && out_plane % 4 == 0) P = static_cast<int>(planes);
    return P;
}

// Fills in the run shape of p (lanes_per_plane set); false when the geometry does not fit a wavefront.
bool finish_plan(SmallPlan &p, size_t &shmem, long &runs, int spare, int zero_floats, bool ragged)
{
    if (p.lanes_per_plane < 1 || p.lanes_per_plane > kWave) return false;
    const int in_plane = p.in_h * p.in_w, out_plane = p.out_h * p.out_w;
    p.lp_in = ragged ? ragged_pitch(p.in_w) : p.in_w;
    p.lp_out = ragged ? ragged_pitch(p.out_w) : p.out_w;
    p.magic_in = ragged ? ragged_magic(p.in_w) : 0;
    p.magic_out = ragged ? ragged_magic(p.out_w) : 0;
    const int lin_plane = p.in_h * p.lp_in, lout_plane = p.out_h * p.lp_out;
    p.planes_per_run = planes_per_run(p.lanes_per_plane, in_plane, out_plane, lin_plane, lout_plane, p.planes);
    if (p.planes_per_run < 1) return false;
    p.lpp_magic = magic_u16(p.lanes_per_plane);
    runs = (p.planes + p.planes_per_run - 1) / p.planes_per_run;
    if (runs > 0x7fffffffL) return false;
    p.zero_off = small_zero_off(p.planes_per_run, lin_plane, lout_plane, spare);
    shmem = static_cast<size_t>(p.zero_off + zero_floats) * 4;
    return true;
}

template <typename IO, int W, bool RAG, int K, int S, bool FLIP, int BH, int D = 1>
int launch_small_down(SmallPlan &p, hipStream_t stream)
{
    p.lanes_per_plane = ceil_div(p.out_h, BH);
    size_t shmem;
    long runs;
    if (!finish_plan(p, shmem, runs, RAG ? W : 0, zero_row_floats(W), RAG)) return -1;
    hipLaunchKernelGGL((small_down_kernel<IO, W, RAG, K, S, FLIP, BH, D>), dim3(static_cast<unsigned>(runs)), dim3(kWave),
                       shmem, stream, p);
    note_variant("small_down%s<%s%d,k%d,s%d,%s,bh%d%s> P%d", sizeof(IO) == 2 ? "16" : "", RAG ? "r" : "w", W, K, S,
                 FLIP ? "rot" : "fwd", BH, D == 2 ? ",d2" : "", p.planes_per_run);
    return check_launch("small_down_kernel");
}

template <typename IO, int W, bool RAG, int K>
int launch_small_up2(SmallPlan &p, hipStream_t stream)
{
    p.lanes_per_plane = ceil_div(p.out_h, 2);
    size_t shmem;
    long runs;
    if (!finish_plan(p, shmem, runs, RAG ? W : 0, zero_row_floats(W), RAG)) return -1;
    hipLaunchKernelGGL((small_up2_kernel<IO, W, RAG, K>), dim3(static_cast<unsigned>(runs)), dim3(kWave), shmem, stream, p);
    note_variant("small_up2%s<%s%d,k%d> P%d", sizeof(IO) == 2 ? "16" : "", RAG ? "r" : "w", W, K, p.planes_per_run);
    return check_launch("small_up2_kernel");
}

// Rows per lane, measured per width (fp32, batch 128 unless said):
//  * 7 wide: 3x3 filters a whole plane per lane (64 planes per wavefront) when there are enough planes to fill the
//    device that way, otherwise two rows; 5x5 and 7x7 filters four rows (C=1152 5x5 17.0 -> 14.8 us; N=256 C=1024
//    7x7 30.0 -> 27.4; two rows 17.4 / 30.0);
//  * 8 wide: four rows with 3x3 filters, two with larger ones (C=1152: whole planes 19.0 / 23.2 us, four rows
//    16.0 / 18.9, two rows 16.4 / 17.4);
//  * up to 16 wide: one row per lane (twice the lanes per plane, half the planes per wavefront, 80 instead of 140
//    registers) for fp32 with 3x3 and 5x5 filters (1-2 us per layer), two rows with 7x7 filters or 16-bit
//    elements (one row loses 1-3 us there);
//  * wider: one row (28x28 fp32 5x5 C=240 43.3 -> 39.0 us, 7x7 C=192 27.8 -> 20.4, bf16 5x5 30.7 -> 28.4);
//  * stride 2: one row.
// Ragged instances come with one choice each (two for the 16-wide class).
template <typename IO, int W, bool RAG, int K>
int launch_small_down_any(SmallPlan &p, int S, bool rot, hipStream_t stream)
{
#define DWCONV_DOWN(BHV)                                                                    \
    return rot ? launch_small_down<IO, W, RAG, K, 1, true, BHV>(p, stream)                  \
               : launch_small_down<IO, W, RAG, K, 1, false, BHV>(p, stream)
    if (S == 1) {
        if constexpr (W <= 8) {
            if constexpr (!RAG && W == 7 && K == 3) {
                if (p.planes >= 64l * 2048) { DWCONV_DOWN(7); }
            }
            if constexpr (!RAG && ((W == 7 && K >= 5) || (W == 8 && K == 3))) {
                DWCONV_DOWN(4);
            } else {
                DWCONV_DOWN(2);
            }
        } else if constexpr (W <= 16) {
            const bool one_row = sizeof(IO) == 4 && K <= 5;
            if (env_int("DWCONV_SMALL_BH", one_row ? 1 : 2) == 1) { DWCONV_DOWN(1); }
            DWCONV_DOWN(2);
        } else {
            DWCONV_DOWN(1);
        }
    }
#undef DWCONV_DOWN
    if (S == 2 && !rot) return launch_small_down<IO, W, RAG, K, 2, false, 1>(p, stream);
    return -1;
}

}  // namespace

template <int W, bool RAG, typename IO>
int small_fir_width(SmallPlan &p, int K, int S, int D, bool rot, bool up2, hipStream_t stream)
{
    if (D != 1) {
        // dilation 2: forward, stride 1, 3x3 and 5x5 taps; rows per lane as for the undilated filter of the same span
        if (D != 2 || S != 1 || rot || up2) return -1;
        constexpr int BHD = W <= 8 ? 2 : (W <= 16 ? 2 : 1);
        if (K == 3) return launch_small_down<IO, W, RAG, 3, 1, false, BHD, 2>(p, stream);
        if (K == 5) return launch_small_down<IO, W, RAG, 5, 1, false, BHD, 2>(p, stream);
        return -1;
    }
    if (up2) {
        if constexpr (W <= 16) {
            if (K == 3) return launch_small_up2<IO, W, RAG, 3>(p, stream);
            if (K == 5) return launch_small_up2<IO, W, RAG, 5>(p, stream);
            if (K == 7) return launch_small_up2<IO, W, RAG, 7>(p, stream);
        }
        return -1;
    }
    if (K == 3) return launch_small_down_any<IO, W, RAG, 3>(p, S, rot, stream);
    if (K == 5) return launch_small_down_any<IO, W, RAG, 5>(p, S, rot, stream);
    if (K == 7) return launch_small_down_any<IO, W, RAG, 7>(p, S, rot, stream);
    return -1;
}

}  // namespace dwconv
