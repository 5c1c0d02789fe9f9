// Gradients of the 2D convolution: with respect to the input (backward data), the filter
// (backward filter) and the bias.
//
// Replaces core::Conv2DBackwardData / core::Conv2DBackwardFilter (include/dlprim/core/conv.hpp:60-80,
// src/core/conv.cpp:113-220,299-434,512-669) and core::BiasBackwardFilter (src/core/bias.cpp) of
// dlprimitives; the arithmetic contract is the CPU one, src/ops/conv2d.cpp:411-435,475-498 and
// src/ops/bwd_bias.cpp:34-60: result = factor * old + gradient.
//
//  * backward data is a forward convolution of dy with the filter transposed within its group and
//    flipped in both axes, stride 1, padding dilate * (kernel - 1) - pad; it runs on the forward
//    operator of this library (every algorithm and tile shape of the forward path serves it).  For
//    stride > 1 the rows h = stride * i + a of dx (phase a) only meet the filter rows r with
//    a + pad - r * dilate divisible by the stride; over those the pass is again a stride-1 convolution of
//    dy (for a 3x3 filter at stride 2: filters of 1x1, 1x2, 2x1 and 2x2 taps), so every phase runs on the
//    forward operator into the workspace and one kernel interleaves the phases into dx.  No multiply
//    is spent on zeros.
//  * backward filter is a GEMM of its own: dW[Cout_g x Cin_g*KH*KW] = dy[Cout_g x B*OH*OW] *
//    cols[B*OH*OW x Cin_g*KH*KW], reduction over the pixels of all images.  Both operands are
//    contiguous along the reduction index in memory, so a workgroup stages 32 reduction indices of BM dy
//    rows (16 bytes per lane) and BN gathered x rows (lane = pixel, the padding test one bit of a tap mask)
//    in LDS and every lane fetches its four k values of a row with one 16-byte LDS read.  The reduction is cut into slices
//    across workgroups; the slices' partial tiles go to the workspace in output order and one small
//    kernel adds them up in slice order (deterministic).
#include <algorithm>
#include <new>
#include <string>

#include "dlp_internal.hpp"

namespace dlp {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int KC = 32;        // reduction indices (pixels of the batch, image after image) per staged chunk
constexpr int PITCH = KC + 4; // LDS row pitch in floats: 16-byte reads of 8 consecutive lanes cover all banks
constexpr uint32_t kOutOfRange = 0x80000000u;

struct WgradArgs {
    const float *x, *dy;
    float *out; // dW itself (one slice) or the partial sums [slice][Cout][Ncol]
    int Cin, Cin_g, Cout, Cout_g, groups, H, W, OW, OHW, KH, KW, sh, sw, ph, pw, dh, dw;
    int Ncol;   // Cin_g * KH * KW
    int Ktotal; // B * OH * OW
    int mtiles, ntiles, slices, chunks, cps; // chunks in all and per slice
    uint32_t x_bytes, dy_bytes;
    uint32_t ow_magic, ow_shift, ohw_magic, ohw_shift, khw_magic, khw_shift, kw_magic, kw_shift;
    float factor;
};

// dW tile of BM filters x BN (channel, tap) columns over the chunks of one slice.
// AVEC: OH * OW is a multiple of 4, dy rows are read 16 bytes per lane.
// MASKED: the padding test of a gathered element is one bit of a per-lane tap mask: 1 = KH * KW <= 31 (one word),
// 2 = KH * KW <= 63 (two words); 0 = row and column comparisons per element.
template <int BM, int BN, bool AVEC, int MASKED>
__global__ __launch_bounds__(256) void conv_wgrad_f32_kernel(WgradArgs a)
{
    constexpr int TM = BM / 64, TN = BN / 64; // 32x32 MFMA blocks per wavefront (wavefronts 2 x 2)
    constexpr int RB = BN / 8;                // gathered rows per thread: two rows per wavefront load
    constexpr int RA = AVEC ? BM / 32 : BM / 8;
    __shared__ __attribute__((aligned(16))) float As[BM * PITCH];
    __shared__ __attribute__((aligned(16))) float Bs[BN * PITCH];
    __shared__ __attribute__((aligned(16))) int rowtab[BN * 4]; // per column: x offset of the tap, tap bit (or 31), row and column shift

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, h = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;

    // tile fastest: workgroups that share a slice read the same dy / x data.  Workgroup ids are dealt round-robin
    // to the 8 XCDs, each with its own L2: renumber so that an XCD runs a contiguous range (whole slices).
    int t;
    {
        const int nb = gridDim.x, bid = blockIdx.x;
        const int q = nb >> 3, r = nb & 7;
        const int xcd = bid & 7, slot = bid >> 3;
        t = (xcd < r) ? xcd * (q + 1) + slot : r * (q + 1) + (xcd - r) * q + slot;
    }
    const int mt = t % a.mtiles;
    t /= a.mtiles;
    const int nt = t % a.ntiles;
    t /= a.ntiles;
    const int g = t % a.groups;
    const int slice = t / a.groups;
    const int m0 = mt * BM, n0 = nt * BN;
    const int ck_begin = slice * a.cps;
    const int ck_end = min(ck_begin + a.cps, a.chunks);

    if (tid < BN) {
        const int n = n0 + tid;
        const uint32_t c = fast_div((uint32_t)n, a.khw_magic, a.khw_shift);
        const int rs = n - (int)c * a.KH * a.KW;
        const int r = (int)fast_div((uint32_t)rs, a.kw_magic, a.kw_shift);
        const int s = rs - r * a.KW;
        const int dr = r * a.dh - a.ph, ds = s * a.dw - a.pw;
        const bool nv = n < a.Ncol;
        rowtab[tid * 4 + 0] = nv ? ((int)c * a.H + dr) * a.W + ds : 0;
        rowtab[tid * 4 + 1] = nv ? rs : (MASKED == 2 ? 63 : 31); // the last bit of a tap mask is never set
        rowtab[tid * 4 + 2] = nv ? dr : -(1 << 28); // far outside the image for the comparing path
        rowtab[tid * 4 + 3] = ds;
    }
    __syncthreads();

    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc((void *)a.dy, 0, a.dy_bytes, 0x00020000);

    float rb[RB];
    float ra[AVEC ? 1 : RA];
    f32x4 ra4[AVEC ? RA : 1];
    const int brow = wave * 2 + h;                              // gathered rows brow + 8 * i, pixel l32 of the chunk
    const int arow = AVEC ? wave * 8 + (lane >> 3) : brow;      // dy rows arow + 32 * i (16-byte pieces) or arow + 8 * i
    auto fetch = [&](int ck) {
        {
            const uint32_t kidx = (uint32_t)(ck * KC + l32);
            const bool pv = kidx < (uint32_t)a.Ktotal;
            const int b = (int)fast_div(kidx, a.ohw_magic, a.ohw_shift);
            const int pix = (int)kidx - b * a.OHW;
            const int oh = (int)fast_div((uint32_t)pix, a.ow_magic, a.ow_shift);
            const int ow = pix - oh * a.OW;
            const int ohs = oh * a.sh, ows = ow * a.sw;
            const int xbase = (b * a.Cin + g * a.Cin_g) * a.H * a.W + ohs * a.W + ows;
            if (MASKED == 1) {
                uint32_t cols = 0, taps = 0;
                for (int s = 0; s < a.KW; s++)
                    cols |= ((unsigned)(ows + s * a.dw - a.pw) < (unsigned)a.W ? 1u : 0u) << s;
                for (int r = 0; r < a.KH; r++)
                    taps |= ((unsigned)(ohs + r * a.dh - a.ph) < (unsigned)a.H ? cols : 0u) << (r * a.KW);
                const uint32_t bad = pv ? ~taps : 0xFFFFFFFFu;
#pragma unroll
                for (int i = 0; i < RB; i++) {
                    const int2 rt = *reinterpret_cast<const int2 *>(&rowtab[(brow + 8 * i) * 4]);
                    const uint32_t off = ((uint32_t)(xbase + rt.x) << 2) | (((bad >> rt.y) & 1u) << 31);
                    rb[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, off, 0, 0));
                }
            } else if (MASKED == 2) {
                uint64_t cols = 0, taps = 0;
                for (int s = 0; s < a.KW; s++)
                    cols |= (uint64_t)((unsigned)(ows + s * a.dw - a.pw) < (unsigned)a.W ? 1u : 0u) << s;
                for (int r = 0; r < a.KH; r++)
                    taps |= ((unsigned)(ohs + r * a.dh - a.ph) < (unsigned)a.H ? cols : 0ull) << (r * a.KW);
                const uint64_t bad = pv ? ~taps : ~0ull;
                const uint32_t bad_lo = (uint32_t)bad, bad_hi = (uint32_t)(bad >> 32);
#pragma unroll
                for (int i = 0; i < RB; i++) {
                    const int2 rt = *reinterpret_cast<const int2 *>(&rowtab[(brow + 8 * i) * 4]);
                    const uint32_t word = (rt.y & 32) ? bad_hi : bad_lo;
                    const uint32_t off = ((uint32_t)(xbase + rt.x) << 2) | (((word >> (rt.y & 31)) & 1u) << 31);
                    rb[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, off, 0, 0));
                }
            } else {
#pragma unroll
                for (int i = 0; i < RB; i++) {
                    const int4 rt = *reinterpret_cast<const int4 *>(&rowtab[(brow + 8 * i) * 4]);
                    const bool ok = pv && (unsigned)(ohs + rt.z) < (unsigned)a.H && (unsigned)(ows + rt.w) < (unsigned)a.W;
                    rb[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, ok ? (uint32_t)(xbase + rt.x) * 4u : kOutOfRange, 0, 0));
                }
            }
            if (!AVEC) {
                const uint32_t ybase = (uint32_t)((b * a.Cout + g * a.Cout_g + m0 + arow) * a.OHW + pix) * 4u;
#pragma unroll
                for (int i = 0; i < RA; i++) {
                    const bool ok = pv && (m0 + arow + 8 * i < a.Cout_g);
                    ra[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(yr, ok ? ybase : kOutOfRange, (uint32_t)(8 * i * a.OHW) * 4u, 0));
                }
            }
        }
        if (AVEC) { // four consecutive reduction indices of one dy row: never across two images, OH * OW being a multiple of 4
            const uint32_t kidx = (uint32_t)(ck * KC + 4 * (lane & 7));
            const bool pv = kidx < (uint32_t)a.Ktotal;
            const int b = (int)fast_div(kidx, a.ohw_magic, a.ohw_shift);
            const int pix = (int)kidx - b * a.OHW;
            const uint32_t ybase = (uint32_t)((b * a.Cout + g * a.Cout_g + m0 + arow) * a.OHW + pix) * 4u;
#pragma unroll
            for (int i = 0; i < RA; i++) {
                const bool ok = pv && (m0 + arow + 32 * i < a.Cout_g);
                ra4[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(yr, ok ? ybase : kOutOfRange, (uint32_t)(32 * i * a.OHW) * 4u, 0));
            }
        }
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[i][j][r] = 0.0f;

    if (ck_begin < ck_end)
        fetch(ck_begin);
    for (int ck = ck_begin; ck < ck_end; ck++) {
        __syncthreads(); // the previous chunk has been read
        if (AVEC) {
#pragma unroll
            for (int i = 0; i < RA; i++)
                *reinterpret_cast<f32x4 *>(&As[(arow + 32 * i) * PITCH + 4 * (lane & 7)]) = ra4[i];
        } else {
#pragma unroll
            for (int i = 0; i < RA; i++)
                As[(arow + 8 * i) * PITCH + l32] = ra[i];
        }
#pragma unroll
        for (int i = 0; i < RB; i++)
            Bs[(brow + 8 * i) * PITCH + l32] = rb[i];
        __syncthreads();
        if (ck + 1 < ck_end)
            fetch(ck + 1); // lands while this chunk is multiplied
        // k order inside a chunk: MFMA step 4*kq + e takes index 8*kq + e from the lower half-wave and
        // 8*kq + 4 + e from the upper one, for both operands alike
#pragma unroll
        for (int kq = 0; kq < KC / 8; kq++) {
            f32x4 av[TM], bv[TN];
#pragma unroll
            for (int i = 0; i < TM; i++)
                av[i] = *reinterpret_cast<const f32x4 *>(&As[(wm * (BM / 2) + i * 32 + l32) * PITCH + kq * 8 + h * 4]);
#pragma unroll
            for (int j = 0; j < TN; j++)
                bv[j] = *reinterpret_cast<const f32x4 *>(&Bs[(wn * (BN / 2) + j * 32 + l32) * PITCH + kq * 8 + h * 4]);
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i][e], bv[j][e], acc[i][j], 0, 0, 0);
        }
    }

    // accumulator element r of block (i, j): row 8 * (r / 4) + r % 4 + 4 * h, column l32
    const bool direct = a.slices == 1;
    float *dst = a.out + (direct ? (size_t)0 : (size_t)slice * a.Cout * a.Ncol);
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int n = n0 + wn * (BN / 2) + j * 32 + l32;
        if (n >= a.Ncol)
            continue;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + wm * (BM / 2) + i * 32 + 8 * (r >> 2) + (r & 3) + 4 * h;
                if (m < a.Cout_g) {
                    float *p = dst + (size_t)(g * a.Cout_g + m) * a.Ncol + n;
                    const float v = acc[i][j][r];
                    if (direct && a.factor != 0.0f)
                        *p = fmaf(*p, a.factor, v);
                    else
                        *p = v;
                }
            }
    }
}

// Depthwise 3x3 filter gradient (one input channel per group): every thread walks pixels of its
// channel's planes, multiplies dy by the nine taps it meets and the workgroup adds the nine sums up.
// Workgroup (k, slice) takes images slice, slice + slices, ...; partial sums [slice][Cout][9].
__global__ __launch_bounds__(256) void depthwise_wgrad3x3_kernel(const float *__restrict__ x, const float *__restrict__ dy, float *__restrict__ part,
                                                                int B, int Cin, int Cout, int mult, int H, int W, int OH, int OW, int sh, int sw, int ph,
                                                                int pw, int dh, int dw)
{
    __shared__ float red[4][9];
    const int k = blockIdx.x, slice = blockIdx.y, slices = gridDim.y;
    const int c = k / mult;
    const int ohw = OH * OW;
    float acc[9];
#pragma unroll
    for (int t = 0; t < 9; t++)
        acc[t] = 0.0f;
    for (int b = slice; b < B; b += slices) {
        const float *xp = x + ((size_t)b * Cin + c) * H * W;
        const float *yp = dy + ((size_t)b * Cout + k) * ohw;
        for (int pix = threadIdx.x; pix < ohw; pix += 256) {
            const float g = yp[pix];
            const int oh = pix / OW, ow = pix - oh * OW;
            const int ih0 = oh * sh - ph, iw0 = ow * sw - pw;
#pragma unroll
            for (int r = 0; r < 3; r++) {
                const int ih = ih0 + r * dh;
                const bool rv = (unsigned)ih < (unsigned)H;
#pragma unroll
                for (int q = 0; q < 3; q++) {
                    const int iw = iw0 + q * dw;
                    const float v = (rv && (unsigned)iw < (unsigned)W) ? xp[ih * W + iw] : 0.0f;
                    acc[r * 3 + q] = fmaf(g, v, acc[r * 3 + q]);
                }
            }
        }
    }
#pragma unroll
    for (int t = 0; t < 9; t++) {
        float v = acc[t];
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1)
            v += __shfl_down(v, off);
        if ((threadIdx.x & 63) == 0)
            red[threadIdx.x >> 6][t] = v;
    }
    __syncthreads();
    if (threadIdx.x < 9)
        part[((size_t)slice * Cout + k) * 9 + threadIdx.x] = (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
}

// out[i] = factor * out[i] + sum over slices.  A wavefront owns 64 consecutive outputs; the four wavefronts of a
// workgroup take every fourth slice each (slice order within a wavefront, then the four sums in wavefront order:
// the same bits every run), so a launch with few outputs and many slices still fills the chip.
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(const float *__restrict__ part, float *__restrict__ out, size_t n, int slices, float factor)
{
    __shared__ float sums[3][64];
    const int lane = threadIdx.x & 63, sub = threadIdx.x >> 6;
    for (size_t base = (size_t)blockIdx.x * 64; base < n; base += (size_t)gridDim.x * 64) {
        const size_t i = base + lane;
        float s = 0.0f;
        if (i < n) {
            int k = sub;
            for (; k + 12 < slices; k += 16) {
                const float v0 = part[(size_t)k * n + i], v1 = part[(size_t)(k + 4) * n + i], v2 = part[(size_t)(k + 8) * n + i],
                            v3 = part[(size_t)(k + 12) * n + i];
                s = (((s + v0) + v1) + v2) + v3;
            }
            for (; k < slices; k += 4)
                s += part[(size_t)k * n + i];
        }
        if (sub > 0)
            sums[sub - 1][lane] = s;
        __syncthreads();
        if (sub == 0 && i < n) {
            s = ((s + sums[0][lane]) + sums[1][lane]) + sums[2][lane];
            out[i] = factor != 0.0f ? fmaf(out[i], factor, s) : s;
        }
        __syncthreads();
    }
}

// wt[g][c][k][KH-1-r][KW-1-s] = w[g][k][c][r][s]: the filter of the stride-1 convolution that maps dy to dx
__global__ __launch_bounds__(256) void filter_transpose_flip_kernel(const float *__restrict__ w, float *__restrict__ wt, int groups, int cout_g, int cin_g,
                                                                    int khw)
{
    const size_t n = (size_t)groups * cout_g * cin_g * khw;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const int rs = (int)(i % khw);
        size_t q = i / khw;
        const int c = (int)(q % cin_g);
        q /= cin_g;
        const int k = (int)(q % cout_g);
        const int g = (int)(q / cout_g);
        wt[(((size_t)g * cin_g + c) * cout_g + k) * khw + (khw - 1 - rs)] = w[i];
    }
}

// One phase of a strided backward-data pass.  dx rows h = sh * i + a only meet the filter rows r with
// (a + ph - r * dh) divisible by sh; over those rows the pass is a stride-1 correlation of dy.
// wt[g][c][k][jh][jw] = w[g][k][c][rh(nh - 1 - jh)][rw(nw - 1 - jw)], r(j) = r0 + j * rstep.
struct PhaseFilterArgs {
    int groups, cout_g, cin_g, KH, KW;
    int nh, nw, rh0, rhstep, rw0, rwstep;
};
__global__ __launch_bounds__(256) void phase_filter_kernel(const float *__restrict__ w, float *__restrict__ wt, PhaseFilterArgs a)
{
    const int taps = a.nh * a.nw;
    const size_t n = (size_t)a.groups * a.cin_g * a.cout_g * taps;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const int jw = (int)(i % a.nw);
        size_t q = i / a.nw;
        const int jh = (int)(q % a.nh);
        q /= a.nh;
        const int k = (int)(q % a.cout_g);
        q /= a.cout_g;
        const int c = (int)(q % a.cin_g);
        const int g = (int)(q / a.cin_g);
        const int rh = a.rh0 + (a.nh - 1 - jh) * a.rhstep, rw = a.rw0 + (a.nw - 1 - jw) * a.rwstep;
        wt[i] = w[((((size_t)g * a.cout_g + k) * a.cin_g + c) * a.KH + rh) * a.KW + rw];
    }
}

// dx[p][sh * i + a][sw * j + b] = factor * dx + phase(a, b)[p][i + off_h][j + off_w] (0 for a phase without filter taps)
constexpr int kMaxPhases = 16;
struct InterleaveArgs {
    const float *buf[kMaxPhases];
    int out_h[kMaxPhases], out_w[kMaxPhases], off_h[kMaxPhases], off_w[kMaxPhases];
    int H, W, sh, sw;
    float factor;
};
__global__ __launch_bounds__(256) void phase_interleave_kernel(float *__restrict__ dx, size_t planes, InterleaveArgs a)
{
    const size_t n = planes * a.H * a.W;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += stride) {
        const int w = (int)(e % a.W);
        const size_t q = e / a.W;
        const int h = (int)(q % a.H);
        const size_t p = q / a.H;
        const int i = h / a.sh, j = w / a.sw;
        const int ph = (h - i * a.sh) * a.sw + (w - j * a.sw);
        const float *buf = a.buf[ph];
        float v = 0.0f;
        if (buf)
            v = buf[(p * a.out_h[ph] + i + a.off_h[ph]) * a.out_w[ph] + j + a.off_w[ph]];
        dx[e] = a.factor != 0.0f ? fmaf(dx[e], a.factor, v) : v;
    }
}

// db[f] = beta * db[f] + sum over batch and plane of dy[b][f][:]; one workgroup per feature
__global__ __launch_bounds__(256) void bias_backward_kernel(const float *__restrict__ dy, float *__restrict__ db, int batch, int features, int plane, float beta)
{
    __shared__ float partial[4];
    const int f = blockIdx.x;
    float s = 0.0f;
    for (int b = 0; b < batch; b++) {
        const float *p = dy + ((size_t)b * features + f) * plane;
        for (int i = threadIdx.x; i < plane; i += 256)
            s += p[i];
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1)
        s += __shfl_down(s, off);
    if ((threadIdx.x & 63) == 0)
        partial[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        const float v = (partial[0] + partial[1]) + (partial[2] + partial[3]);
        db[f] = beta != 0.0f ? fmaf(db[f], beta, v) : v;
    }
}

size_t round256(size_t v) { return (v + 255) / 256 * 256; }

unsigned reduce_grid_for(size_t n)
{
    return (unsigned)std::min<size_t>(std::max<size_t>((n + 63) / 64, 1), 256 * 64);
}

unsigned grid_for(size_t n)
{
    size_t blocks = (n + 255) / 256;
    return (unsigned)std::min<size_t>(std::max<size_t>(blocks, 1), 256 * 32);
}

struct WgradPlan {
    int BM, BN, mtiles, ntiles, chunks, cps, slices;
    bool depthwise; // depthwise_wgrad3x3_kernel: slices = workgroups per filter
    size_t part_bytes;
};

constexpr int kWgradSlots = 256 * 3; // workgroups resident at once: three per compute unit

// Slices: one full round of resident workgroups where the tiles allow it, at least two chunks each.
WgradPlan wgrad_plan(const dlp_conv2d_settings &c, int batch, int OH, int OW)
{
    WgradPlan p;
    const int cout_g = c.channels_out / c.groups, ncol = c.channels_in / c.groups * c.kernel[0] * c.kernel[1];
    p.depthwise = c.channels_in == c.groups && c.kernel[0] == 3 && c.kernel[1] == 3 && cout_g <= 4;
    if (p.depthwise) {
        p.BM = p.BN = p.mtiles = p.ntiles = p.chunks = p.cps = 0;
        p.slices = std::max(1, std::min(batch, (1024 + c.channels_out - 1) / c.channels_out));
        p.part_bytes = (size_t)p.slices * c.channels_out * 9 * sizeof(float);
        return p;
    }
    p.BM = cout_g > 64 ? 128 : 64;
    p.BN = ncol > 64 ? 128 : 64;
    if (p.BN == 128 && (ncol + 63) / 64 * 64 * 5 <= (ncol + 127) / 128 * 128 * 4)
        p.BN = 64; // the narrower tile wastes at least a fifth less of its columns on padding (conv1: 147 columns)
    p.mtiles = (cout_g + p.BM - 1) / p.BM;
    p.ntiles = (ncol + p.BN - 1) / p.BN;
    p.chunks = (int)(((long long)batch * OH * OW + KC - 1) / KC);
    const long long tiles = (long long)p.mtiles * p.ntiles * c.groups;
    long long want = std::max<long long>(1, kWgradSlots / tiles);
    want = std::min<long long>(want, std::max(1, p.chunks / 2));
    p.cps = (int)((p.chunks + want - 1) / want);
    p.slices = (p.chunks + p.cps - 1) / p.cps;
    p.part_bytes = p.slices > 1 ? (size_t)p.slices * c.channels_out * ncol * sizeof(float) : 0;
    return p;
}

} // namespace
} // namespace dlp

using namespace dlp;

// One axis of one phase: filter rows r0, r0 + rstep, ... (n of them), and the stride-1 convolution over dy
// that computes the phase: kernel extent n, dilation dil, symmetric padding pad; its output has `out`
// rows of which rows off .. off + len - 1 are the phase's rows of dx.
struct PhaseAxis {
    int n, r0, rstep, dil, pad, off, out, len;
};

struct BwdPhase {
    PhaseAxis h, w;
    dlp_conv2d_fwd *fwd;
    size_t wt_bytes, fwd_ws;
};

struct dlp_conv2d_bwd_data {
    dlp_conv2d_settings cfg;
    int OH, OW;
    bool strided;            // one stride-1 convolution per phase, then interleaved into dx
    dlp_conv2d_fwd *fwd;     // stride 1: the convolution dy -> dx on the transposed, flipped filter
    size_t wt_bytes, fwd_ws; // stride 1
    BwdPhase phase[kMaxPhases];
    int nphases;
};

struct dlp_conv2d_bwd_filter {
    dlp_conv2d_settings cfg;
    int OH, OW;
};

static int check_settings(const dlp_conv2d_settings *cfg, int out[4])
{
    DLP_REQUIRE(cfg != nullptr, "null argument");
    DLP_REQUIRE(cfg->channels_in > 0 && cfg->channels_out > 0 && cfg->groups > 0, "channels/groups must be positive");
    DLP_REQUIRE(cfg->channels_in % cfg->groups == 0 && cfg->channels_out % cfg->groups == 0, "channels not divisible by groups");
    if (cfg->dtype != DLP_FLOAT)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "convolution gradients: float_data is implemented");
    return dlp_conv2d_output_shape(cfg, cfg->shape, out);
}

extern "C" {

static PhaseAxis phase_axis(int a, int size, int osize, int k, int stride, int dilate, int pad)
{
    PhaseAxis x = {0, 0, 1, 1, 0, 0, 0, 0};
    x.len = a < size ? (size - a + stride - 1) / stride : 0;
    int qmax = 0, qmin = 0, r1 = -1;
    for (int r = 0; r < k; r++) {
        const int v = a + pad - r * dilate;
        if (((v % stride) + stride) % stride != 0)
            continue;
        const int q = (v - (((v % stride) + stride) % stride)) / stride; // exact
        if (x.n == 0) {
            x.r0 = r;
            qmax = q;
        } else if (x.n == 1)
            r1 = r;
        qmin = q;
        x.n++;
    }
    if (x.n == 0 || x.len == 0) {
        x.n = 0;
        return x;
    }
    if (x.n > 1) {
        x.rstep = r1 - x.r0;
        x.dil = dilate * x.rstep / stride;
    }
    x.pad = std::max(0, std::max(-qmin, x.len + qmax - osize));
    x.off = qmin + x.pad;
    x.out = osize + 2 * x.pad - x.dil * (x.n - 1);
    return x;
}

static void bwd_data_free(dlp_conv2d_bwd_data *op)
{
    dlp_conv2d_fwd_destroy(op->fwd);
    for (int i = 0; i < op->nphases; i++)
        dlp_conv2d_fwd_destroy(op->phase[i].fwd);
    delete op;
}

int dlp_conv2d_bwd_data_create(const dlp_conv2d_settings *cfg, const char *algo, dlp_conv2d_bwd_data **out)
{
    DLP_REQUIRE(out != nullptr, "null argument");
    *out = nullptr;
    int oshape[4];
    int rc = check_settings(cfg, oshape);
    if (rc != DLP_OK)
        return rc;
    dlp_conv2d_bwd_data *op = new (std::nothrow) dlp_conv2d_bwd_data();
    if (!op)
        return fail(DLP_ERR_RUNTIME, "out of host memory");
    op->cfg = *cfg;
    op->OH = oshape[2];
    op->OW = oshape[3];
    op->fwd = nullptr;
    op->nphases = 0;
    op->strided = cfg->stride[0] != 1 || cfg->stride[1] != 1;
    dlp_conv2d_settings t = *cfg;
    t.channels_in = cfg->channels_out;
    t.channels_out = cfg->channels_in;
    t.stride[0] = t.stride[1] = 1;
    t.shape[1] = cfg->channels_out;
    t.shape[2] = op->OH;
    t.shape[3] = op->OW;
    const size_t cin_g = cfg->channels_in / cfg->groups;
    if (!op->strided) {
        for (int i = 0; i < 2; i++) {
            t.pad[i] = cfg->dilate[i] * (cfg->kernel[i] - 1) - cfg->pad[i];
            if (t.pad[i] < 0) {
                delete op;
                return fail(DLP_ERR_NOT_IMPLEMENTED, "backward data: padding larger than dilate * (kernel - 1)");
            }
        }
        rc = dlp_conv2d_fwd_create(&t, 0, DLP_ACT_IDENTITY, algo, &op->fwd);
        if (rc != DLP_OK) {
            delete op;
            return rc;
        }
        op->wt_bytes = round256((size_t)cfg->channels_out * cin_g * cfg->kernel[0] * cfg->kernel[1] * sizeof(float));
        op->fwd_ws = round256(dlp_conv2d_fwd_workspace(op->fwd));
        *out = op;
        return DLP_OK;
    }
    if (cfg->stride[0] * cfg->stride[1] > kMaxPhases) {
        delete op;
        return fail(DLP_ERR_NOT_IMPLEMENTED, "backward data: more than 16 stride phases");
    }
    op->nphases = cfg->stride[0] * cfg->stride[1];
    for (int i = 0; i < op->nphases; i++)
        op->phase[i].fwd = nullptr;
    for (int a = 0; a < cfg->stride[0]; a++)
        for (int b = 0; b < cfg->stride[1]; b++) {
            BwdPhase &ph = op->phase[a * cfg->stride[1] + b];
            ph.h = phase_axis(a, cfg->shape[2], op->OH, cfg->kernel[0], cfg->stride[0], cfg->dilate[0], cfg->pad[0]);
            ph.w = phase_axis(b, cfg->shape[3], op->OW, cfg->kernel[1], cfg->stride[1], cfg->dilate[1], cfg->pad[1]);
            ph.wt_bytes = ph.fwd_ws = 0;
            if (ph.h.n == 0 || ph.w.n == 0)
                continue; // no filter tap meets this phase: its part of dx is zero
            dlp_conv2d_settings u = t;
            u.kernel[0] = ph.h.n;
            u.kernel[1] = ph.w.n;
            u.dilate[0] = ph.h.dil;
            u.dilate[1] = ph.w.dil;
            u.pad[0] = ph.h.pad;
            u.pad[1] = ph.w.pad;
            rc = dlp_conv2d_fwd_create(&u, 0, DLP_ACT_IDENTITY, algo, &ph.fwd);
            if (rc != DLP_OK) {
                bwd_data_free(op);
                return rc;
            }
            ph.wt_bytes = round256((size_t)cfg->channels_out * cin_g * ph.h.n * ph.w.n * sizeof(float));
            ph.fwd_ws = round256(dlp_conv2d_fwd_workspace(ph.fwd));
        }
    *out = op;
    return DLP_OK;
}

const char *dlp_conv2d_bwd_data_algo(const dlp_conv2d_bwd_data *op)
{
    if (!op)
        return "";
    if (!op->strided)
        return dlp_conv2d_fwd_algo(op->fwd);
    for (int i = 0; i < op->nphases; i++)
        if (op->phase[i].fwd)
            return dlp_conv2d_fwd_algo(op->phase[i].fwd);
    return "gemm";
}

// strided: [phase filters][phase outputs for `batch` images][largest forward workspace]
static size_t bwd_data_need(const dlp_conv2d_bwd_data *op, int batch, size_t *fwd_ws_out)
{
    if (!op->strided) {
        if (fwd_ws_out)
            *fwd_ws_out = op->fwd_ws;
        return op->wt_bytes + op->fwd_ws;
    }
    size_t total = 0, fws = 0;
    for (int i = 0; i < op->nphases; i++) {
        const BwdPhase &ph = op->phase[i];
        if (!ph.fwd)
            continue;
        total += ph.wt_bytes + round256((size_t)batch * op->cfg.channels_in * ph.h.out * ph.w.out * sizeof(float));
        fws = std::max(fws, ph.fwd_ws);
    }
    if (fwd_ws_out)
        *fwd_ws_out = fws;
    return total + fws;
}

size_t dlp_conv2d_bwd_data_workspace(const dlp_conv2d_bwd_data *op) { return op ? bwd_data_need(op, std::max(op->cfg.shape[0], 1), nullptr) : 0; }

int dlp_conv2d_bwd_data_enqueue(dlp_conv2d_bwd_data *op, const int x_shape[4], void *dx, const void *w, const void *dy, void *ws, size_t ws_bytes,
                                float factor, void *stream)
{
    DLP_REQUIRE(op != nullptr && x_shape != nullptr, "null argument");
    DLP_REQUIRE(x_shape[1] == op->cfg.channels_in && x_shape[2] == op->cfg.shape[2] && x_shape[3] == op->cfg.shape[3],
                "the operator was created for another input shape");
    const int batch = x_shape[0];
    DLP_REQUIRE(batch >= 0, "negative batch");
    if (batch == 0)
        return DLP_OK;
    DLP_REQUIRE(dx != nullptr && w != nullptr && dy != nullptr, "null tensor pointer");
    size_t fwd_ws = 0;
    const size_t need = bwd_data_need(op, batch, &fwd_ws);
    DLP_REQUIRE(ws != nullptr && ws_bytes >= need, "workspace smaller than workspace() for this batch");
    hipStream_t st = (hipStream_t)stream;
    const dlp_conv2d_settings &c = op->cfg;
    const int cout_g = c.channels_out / c.groups, cin_g = c.channels_in / c.groups, khw = c.kernel[0] * c.kernel[1];
    const int in_shape[4] = {batch, c.channels_out, op->OH, op->OW};
    if (!op->strided) {
        float *wt = (float *)ws;
        void *fws = (char *)ws + op->wt_bytes;
        {
            TimingScope ts("bwd_data_filter_transpose", st);
            hipLaunchKernelGGL(filter_transpose_flip_kernel, dim3(grid_for((size_t)c.channels_out * cin_g * khw)), dim3(256), 0, st, (const float *)w, wt,
                               c.groups, cout_g, cin_g, khw);
        }
        DLP_HIP_TRY(hipGetLastError());
        return dlp_conv2d_fwd_enqueue(op->fwd, in_shape, dy, wt, nullptr, dx, op->fwd_ws ? fws : nullptr, op->fwd_ws, factor, stream);
    }
    const size_t planes = (size_t)batch * c.channels_in;
    DLP_REQUIRE(planes * c.shape[2] * c.shape[3] < (1ull << 31) / 4, "tensor of 2 GiB or more");
    InterleaveArgs ia;
    ia.H = c.shape[2];
    ia.W = c.shape[3];
    ia.sh = c.stride[0];
    ia.sw = c.stride[1];
    ia.factor = factor;
    char *cursor = (char *)ws;
    void *fws = (char *)ws + (need - fwd_ws);
    for (int i = 0; i < kMaxPhases; i++) {
        ia.buf[i] = nullptr;
        ia.out_h[i] = ia.out_w[i] = 1;
        ia.off_h[i] = ia.off_w[i] = 0;
    }
    for (int i = 0; i < op->nphases; i++) {
        const BwdPhase &ph = op->phase[i];
        if (!ph.fwd)
            continue;
        float *wt = (float *)cursor;
        cursor += ph.wt_bytes;
        float *outp = (float *)cursor;
        cursor += round256(planes * ph.h.out * ph.w.out * sizeof(float));
        PhaseFilterArgs fa = {c.groups, cout_g, cin_g, c.kernel[0], c.kernel[1], ph.h.n, ph.w.n, ph.h.r0, ph.h.rstep, ph.w.r0, ph.w.rstep};
        {
            TimingScope ts("bwd_data_phase_filter", st);
            hipLaunchKernelGGL(phase_filter_kernel, dim3(grid_for((size_t)c.channels_out * cin_g * ph.h.n * ph.w.n)), dim3(256), 0, st, (const float *)w,
                               wt, fa);
        }
        DLP_HIP_TRY(hipGetLastError());
        int rc = dlp_conv2d_fwd_enqueue(ph.fwd, in_shape, dy, wt, nullptr, outp, ph.fwd_ws ? fws : nullptr, ph.fwd_ws, 0.0f, stream);
        if (rc != DLP_OK)
            return rc;
        ia.buf[i] = outp;
        ia.out_h[i] = ph.h.out;
        ia.out_w[i] = ph.w.out;
        ia.off_h[i] = ph.h.off;
        ia.off_w[i] = ph.w.off;
    }
    {
        TimingScope ts("bwd_data_interleave", st);
        hipLaunchKernelGGL(phase_interleave_kernel, dim3(grid_for(planes * c.shape[2] * c.shape[3])), dim3(256), 0, st, (float *)dx, planes, ia);
    }
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

void dlp_conv2d_bwd_data_destroy(dlp_conv2d_bwd_data *op)
{
    if (op)
        bwd_data_free(op);
}

int dlp_conv2d_bwd_filter_create(const dlp_conv2d_settings *cfg, const char *algo, dlp_conv2d_bwd_filter **out)
{
    DLP_REQUIRE(out != nullptr, "null argument");
    *out = nullptr;
    int oshape[4];
    int rc = check_settings(cfg, oshape);
    if (rc != DLP_OK)
        return rc;
    const std::string al = algo ? algo : "";
    DLP_REQUIRE(al == "" || al == "auto" || al == "gemm" || al == "winograd" || al == "depthwise_separable", "unknown algorithm name");
    DLP_REQUIRE(cfg->kernel[0] <= 31 && cfg->kernel[1] <= 31, "kernel extent above 31");
    dlp_conv2d_bwd_filter *op = new (std::nothrow) dlp_conv2d_bwd_filter();
    if (!op)
        return fail(DLP_ERR_RUNTIME, "out of host memory");
    op->cfg = *cfg;
    op->OH = oshape[2];
    op->OW = oshape[3];
    *out = op;
    return DLP_OK;
}

const char *dlp_conv2d_bwd_filter_algo(const dlp_conv2d_bwd_filter *) { return "gemm"; }

size_t dlp_conv2d_bwd_filter_workspace(const dlp_conv2d_bwd_filter *op)
{
    return op ? round256(wgrad_plan(op->cfg, std::max(op->cfg.shape[0], 1), op->OH, op->OW).part_bytes) : 0;
}

int dlp_conv2d_bwd_filter_enqueue(dlp_conv2d_bwd_filter *op, const int x_shape[4], const void *x, void *dw, const void *dy, void *ws, size_t ws_bytes,
                                  float factor, void *stream)
{
    DLP_REQUIRE(op != nullptr && x_shape != nullptr, "null argument");
    const dlp_conv2d_settings &c = op->cfg;
    DLP_REQUIRE(x_shape[1] == c.channels_in && x_shape[2] == c.shape[2] && x_shape[3] == c.shape[3], "the operator was created for another input shape");
    const int batch = x_shape[0];
    DLP_REQUIRE(batch >= 0, "negative batch");
    DLP_REQUIRE(dw != nullptr, "null tensor pointer");
    hipStream_t st = (hipStream_t)stream;
    const int cin_g = c.channels_in / c.groups, cout_g = c.channels_out / c.groups;
    const int ncol = cin_g * c.kernel[0] * c.kernel[1];
    const size_t n_out = (size_t)c.channels_out * ncol;
    if (batch == 0) { // the gradient is zero: dw = factor * dw
        TimingScope ts("wgrad_reduce", st);
        hipLaunchKernelGGL(wgrad_reduce_kernel, dim3(reduce_grid_for(n_out)), dim3(256), 0, st, (const float *)dw, (float *)dw, n_out, 0, factor);
        DLP_HIP_TRY(hipGetLastError());
        return DLP_OK;
    }
    DLP_REQUIRE(x != nullptr && dy != nullptr, "null tensor pointer");
    const size_t x_elems = (size_t)batch * c.channels_in * c.shape[2] * c.shape[3];
    const size_t y_elems = (size_t)batch * c.channels_out * op->OH * op->OW;
    if (x_elems >= (1ull << 31) / 4 || y_elems >= (1ull << 31) / 4)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "tensor of 2 GiB or more");
    WgradPlan p = wgrad_plan(c, batch, op->OH, op->OW);
    if (p.depthwise) {
        const size_t per_slice = n_out * sizeof(float);
        p.slices = (int)std::min<size_t>(ws ? ws_bytes / per_slice : 0, (size_t)p.slices);
        DLP_REQUIRE(p.slices >= 1, "workspace smaller than workspace()");
        DLP_REQUIRE(c.channels_out <= 0x7FFFFFFF && p.slices <= 65535, "grid");
        {
            TimingScope ts("wgrad_depthwise", st);
            hipLaunchKernelGGL(depthwise_wgrad3x3_kernel, dim3((unsigned)c.channels_out, (unsigned)p.slices), dim3(256), 0, st, (const float *)x,
                               (const float *)dy, (float *)ws, batch, c.channels_in, c.channels_out, cout_g, c.shape[2], c.shape[3], op->OH, op->OW,
                               c.stride[0], c.stride[1], c.pad[0], c.pad[1], c.dilate[0], c.dilate[1]);
        }
        TimingScope ts("wgrad_reduce", st);
        hipLaunchKernelGGL(wgrad_reduce_kernel, dim3(reduce_grid_for(n_out)), dim3(256), 0, st, (const float *)ws, (float *)dw, n_out, p.slices, factor);
        DLP_HIP_TRY(hipGetLastError());
        return DLP_OK;
    }
    if (p.slices > 1) {
        // fewer slices when the caller's workspace was sized for a smaller batch
        const size_t per_slice = n_out * sizeof(float);
        const int fit = (int)std::min<size_t>(ws ? ws_bytes / per_slice : 0, (size_t)p.slices);
        if (fit < p.slices) {
            const int want = std::max(fit, 1);
            p.cps = (p.chunks + want - 1) / want;
            p.slices = (p.chunks + p.cps - 1) / p.cps;
        }
        DLP_REQUIRE(p.slices == 1 || (ws != nullptr && (size_t)p.slices * per_slice <= ws_bytes), "workspace smaller than workspace()");
    }
    WgradArgs a;
    a.x = (const float *)x;
    a.dy = (const float *)dy;
    a.out = p.slices > 1 ? (float *)ws : (float *)dw;
    a.Cin = c.channels_in;
    a.Cin_g = cin_g;
    a.Cout = c.channels_out;
    a.Cout_g = cout_g;
    a.groups = c.groups;
    a.H = c.shape[2];
    a.W = c.shape[3];
    a.OW = op->OW;
    a.OHW = op->OH * op->OW;
    a.KH = c.kernel[0];
    a.KW = c.kernel[1];
    a.sh = c.stride[0];
    a.sw = c.stride[1];
    a.ph = c.pad[0];
    a.pw = c.pad[1];
    a.dh = c.dilate[0];
    a.dw = c.dilate[1];
    a.Ncol = ncol;
    a.mtiles = p.mtiles;
    a.ntiles = p.ntiles;
    a.slices = p.slices;
    a.Ktotal = batch * op->OH * op->OW;
    a.chunks = p.chunks;
    a.cps = p.cps;
    a.x_bytes = (uint32_t)(x_elems * 4);
    a.dy_bytes = (uint32_t)(y_elems * 4);
    make_magic((uint32_t)a.OW, a.ow_magic, a.ow_shift);
    make_magic((uint32_t)(a.KH * a.KW), a.khw_magic, a.khw_shift);
    make_magic((uint32_t)a.KW, a.kw_magic, a.kw_shift);
    make_magic((uint32_t)a.OHW, a.ohw_magic, a.ohw_shift);
    a.factor = factor;
    const long long wgs = (long long)p.mtiles * p.ntiles * c.groups * p.slices;
    DLP_REQUIRE(wgs < (1ll << 31), "too many workgroups");
    {
        TimingScope ts("wgrad", st);
        const dim3 grid((unsigned)wgs), block(256);
        const bool avec = a.OHW % 4 == 0 && ((uintptr_t)dy & 15) == 0;
        const int taps = a.KH * a.KW;
        const int masked = taps <= 31 ? 1 : taps <= 63 ? 2 : 0;
#define DLP_WGRAD_LAUNCH_M(BM_, BN_, AV_)                                                                      \
    do {                                                                                                       \
        if (masked == 1)                                                                                       \
            hipLaunchKernelGGL((conv_wgrad_f32_kernel<BM_, BN_, AV_, 1>), grid, block, 0, st, a);              \
        else if (masked == 2)                                                                                  \
            hipLaunchKernelGGL((conv_wgrad_f32_kernel<BM_, BN_, AV_, 2>), grid, block, 0, st, a);              \
        else                                                                                                   \
            hipLaunchKernelGGL((conv_wgrad_f32_kernel<BM_, BN_, AV_, 0>), grid, block, 0, st, a);              \
    } while (0)
#define DLP_WGRAD_LAUNCH(BM_, BN_)                                                                             \
    do {                                                                                                       \
        if (avec)                                                                                              \
            DLP_WGRAD_LAUNCH_M(BM_, BN_, true);                                                                \
        else                                                                                                   \
            DLP_WGRAD_LAUNCH_M(BM_, BN_, false);                                                               \
    } while (0)
        if (p.BM == 128 && p.BN == 128)
            DLP_WGRAD_LAUNCH(128, 128);
        else if (p.BM == 128)
            DLP_WGRAD_LAUNCH(128, 64);
        else if (p.BN == 128)
            DLP_WGRAD_LAUNCH(64, 128);
        else
            DLP_WGRAD_LAUNCH(64, 64);
#undef DLP_WGRAD_LAUNCH
#undef DLP_WGRAD_LAUNCH_M
    }
    if (p.slices > 1) {
        TimingScope ts("wgrad_reduce", st);
        hipLaunchKernelGGL(wgrad_reduce_kernel, dim3(reduce_grid_for(n_out)), dim3(256), 0, st, (const float *)ws, (float *)dw, n_out, p.slices, factor);
    }
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

void dlp_conv2d_bwd_filter_destroy(dlp_conv2d_bwd_filter *op) { delete op; }

// ---- TransposedConvolution2D forward (src/ops/conv2d.cpp:559-805): the gradient-of-data pass of the convolution whose
//      input and output channels are swapped (:588-590), then bias (core::add_bias) and activation ----
struct dlp_tconv2d_fwd {
    dlp_conv2d_settings cfg; // of the transposed operator: shape = its input shape
    int output_pad[2];
    int out_shape[4];
    bool bias;
    int activation;
    dlp_conv2d_bwd_data *bwd;
};

int dlp_conv2d_transposed_output_shape(const dlp_conv2d_settings *cfg, const int in_shape[4], const int output_pad[2], int out_shape[4])
{
    DLP_REQUIRE(cfg != nullptr && in_shape != nullptr && output_pad != nullptr && out_shape != nullptr, "null argument");
    DLP_REQUIRE(in_shape[1] == cfg->channels_in, "input channels differ from channels_in");
    for (int i = 0; i < 2; i++) {
        DLP_REQUIRE(cfg->kernel[i] > 0 && cfg->stride[i] > 0 && cfg->dilate[i] > 0 && cfg->pad[i] >= 0 && output_pad[i] >= 0, "kernel/stride/dilate/pad");
        const int o = (in_shape[2 + i] - 1) * cfg->stride[i] - 2 * cfg->pad[i] + cfg->dilate[i] * (cfg->kernel[i] - 1) + output_pad[i] + 1;
        DLP_REQUIRE(o > 0, "empty output");
        out_shape[2 + i] = o;
    }
    out_shape[0] = in_shape[0];
    out_shape[1] = cfg->channels_out;
    return DLP_OK;
}

int dlp_tconv2d_fwd_create(const dlp_conv2d_settings *cfg, const int output_pad[2], int bias, int activation, const char *algo, dlp_tconv2d_fwd **out)
{
    DLP_REQUIRE(cfg != nullptr && output_pad != nullptr && out != nullptr, "null argument");
    *out = nullptr;
    DLP_REQUIRE(cfg->channels_in > 0 && cfg->channels_out > 0 && cfg->groups > 0, "channels/groups must be positive");
    DLP_REQUIRE(cfg->channels_in % cfg->groups == 0 && cfg->channels_out % cfg->groups == 0, "channels not divisible by groups");
    DLP_REQUIRE(activation >= DLP_ACT_IDENTITY && activation <= DLP_ACT_RELU6, "unknown activation");
    if (cfg->dtype != DLP_FLOAT) // src/ops/conv2d.cpp:584
        return fail(DLP_ERR_NOT_IMPLEMENTED, "TransposedConvolution2D: float_data is implemented");
    int oshape[4];
    int rc = dlp_conv2d_transposed_output_shape(cfg, cfg->shape, output_pad, oshape);
    if (rc != DLP_OK)
        return rc;
    // the convolution it is the data gradient of: channels swapped, input = this operator's output (:588-590, :693-699)
    dlp_conv2d_settings conv = *cfg;
    conv.channels_in = cfg->channels_out;
    conv.channels_out = cfg->channels_in;
    for (int i = 0; i < 4; i++)
        conv.shape[i] = oshape[i];
    int back[4];
    rc = dlp_conv2d_output_shape(&conv, conv.shape, back);
    if (rc != DLP_OK)
        return rc;
    // an output_pad of a whole stride or more would describe the next larger input
    DLP_REQUIRE(back[2] == cfg->shape[2] && back[3] == cfg->shape[3], "output_pad must be smaller than the stride");
    dlp_tconv2d_fwd *op = new (std::nothrow) dlp_tconv2d_fwd();
    if (!op)
        return fail(DLP_ERR_RUNTIME, "out of host memory");
    op->cfg = *cfg;
    op->output_pad[0] = output_pad[0];
    op->output_pad[1] = output_pad[1];
    for (int i = 0; i < 4; i++)
        op->out_shape[i] = oshape[i];
    op->bias = bias != 0;
    op->activation = activation;
    op->bwd = nullptr;
    rc = dlp_conv2d_bwd_data_create(&conv, algo, &op->bwd);
    if (rc != DLP_OK) {
        delete op;
        return rc;
    }
    *out = op;
    return DLP_OK;
}

const char *dlp_tconv2d_fwd_algo(const dlp_tconv2d_fwd *op) { return op ? dlp_conv2d_bwd_data_algo(op->bwd) : ""; }

size_t dlp_tconv2d_fwd_workspace(const dlp_tconv2d_fwd *op) { return op ? dlp_conv2d_bwd_data_workspace(op->bwd) : 0; }

int dlp_tconv2d_fwd_enqueue(dlp_tconv2d_fwd *op, const int x_shape[4], const void *x, const void *w, const void *bias, void *y, void *ws,
                            size_t ws_bytes, void *stream)
{
    DLP_REQUIRE(op != nullptr && x_shape != nullptr, "null argument");
    DLP_REQUIRE(x_shape[0] >= 0, "negative batch");
    DLP_REQUIRE(x_shape[1] == op->cfg.channels_in && x_shape[2] == op->cfg.shape[2] && x_shape[3] == op->cfg.shape[3],
                "input shape differs from the shape given at create (only the batch may change)");
    DLP_REQUIRE((bias != nullptr) == op->bias, "bias pointer must be given exactly when the op was created with bias");
    if (x_shape[0] == 0)
        return DLP_OK;
    const int y_shape[4] = {x_shape[0], op->out_shape[1], op->out_shape[2], op->out_shape[3]};
    int rc = dlp_conv2d_bwd_data_enqueue(op->bwd, y_shape, y, w, x, ws, ws_bytes, 0.0f, stream); // :782
    if (rc != DLP_OK)
        return rc;
    if (op->bias || op->activation != DLP_ACT_IDENTITY) // :783-790; one pass for both
        rc = channel_affine_launch(DLP_FLOAT, op->activation, y_shape[0], y_shape[1], y_shape[2] * y_shape[3], y, nullptr, (const float *)bias, y,
                                   (hipStream_t)stream);
    return rc;
}

void dlp_tconv2d_fwd_destroy(dlp_tconv2d_fwd *op)
{
    if (!op)
        return;
    dlp_conv2d_bwd_data_destroy(op->bwd);
    delete op;
}

int dlp_bias_bwd_enqueue(int dtype, int batch, int features, int plane, const void *dy, float *db, float beta, void *stream)
{
    if (dtype != DLP_FLOAT)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "bias gradient: float_data is implemented");
    DLP_REQUIRE(batch >= 0 && features > 0 && plane > 0, "shape");
    DLP_REQUIRE(db != nullptr && (batch == 0 || dy != nullptr), "null tensor pointer");
    TimingScope ts("bias_backward", (hipStream_t)stream);
    hipLaunchKernelGGL(bias_backward_kernel, dim3((unsigned)features), dim3(256), 0, (hipStream_t)stream, (const float *)dy, db, batch, features, plane, beta);
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

} // extern "C"
