// Strided convolutions with very few input channels (the 7x7 / stride 2 / 3-channel stem of the
// ResNet family): conv_stem_f32_kernel.
//
// With 3 input channels the reduction index of the implicit GEMM runs over filter taps, so the
// gathering kernel of conv_gemm.hip spends vector-ALU work on every gathered element and a K loop
// of ten tiles never amortises its prologue.  Here a workgroup owns a band of R output rows of one
// image and all 64 output channels of an m tile:
//   * the input rows the band touches (CIN x (STRIDE*(R-1)+KH) rows) are copied to LDS once, with
//     coalesced 16-byte loads, zero padded on every side, at a compile-time row pitch;
//   * the filter rows of the m tile are copied to LDS as they lie in memory ([m][k], odd pitch), so
//     nothing is packed beforehand;
//   * a wavefront takes 32 consecutive output pixels of the band at a time (the pixels of a band are
//     contiguous in NCHW) and walks the whole reduction with every address fixed beforehand: the
//     operand of tap (c, r, s) is a ds_read at lane base + compile-time offset.  The two k of a
//     v_mfma_f32_32x32x2_f32 belong to the two halves of the wavefront, so the lane base carries
//     half * (distance of the two taps); consecutive taps are 1 element apart, PITCH - (KW-1) at the
//     end of a filter row, and a third constant at the end of a channel: three lane bases cover
//     all pairs.  The loop body is matrix instructions and LDS reads only;
//   * blocks of 32 pixels are handed out through an LDS counter, so wavefronts on a less loaded
//     SIMD take more of them.
// Accumulators start from the bias; activation and factor as in the other kernels
// (src/kernels/sgemm.cl:658-672,707-710 of the reference describe the fused epilogue).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>
#include <type_traits>
#include <utility>

#include "dlp_internal.hpp"

namespace dlp {

typedef float stem_f32x16 __attribute__((ext_vector_type(16)));
typedef float stem_f32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int kStemThreads = 512;
constexpr int kStemPadL = 4;                    // zero columns left of an input row in LDS (keeps 16-byte stores aligned)
constexpr uint32_t kStemOutOfRange = 0x80000000u; // >= num_records of every buffer we accept

struct StemArgs {
    const float *x, *w, *bias;
    float *y;
    int B, H, W, Cout, OH, OW, OHW;
    int ph, pw;
    int bands, mtiles, total; // bands of R output rows per image, m tiles of 64 channels, workgroups with work
    int chunk;                // workgroups per XCD
    uint32_t x_img_bytes, y_img_bytes, w_bytes;
    uint32_t upr, upr_magic, upr_shift; // load units (16 bytes or one float) per input row
    uint32_t ow_magic, ow_shift;
    uint32_t padw, padw_magic, padw_shift; // PITCH - W zero columns per LDS row
    float factor;
    int pre, act;
    float clamp_lo, clamp_hi;
};

template <class F, int... I>
__device__ __forceinline__ void stem_for_seq(F &&f, std::integer_sequence<int, I...>)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void stem_for(F &&f)
{
    stem_for_seq(f, std::make_integer_sequence<int, N>{});
}

template <int CIN, int KH, int KW, int STRIDE, int R, int PITCH, bool VEC, bool GENERIC_ACT>
__global__ __launch_bounds__(kStemThreads, 4) void conv_stem_f32_kernel(StemArgs a)
{
    constexpr int K = CIN * KH * KW, KP = (K + 1) / 2 * 2, NJ = KP / 2;
    constexpr int ROWS = STRIDE * (R - 1) + KH; // input rows of a band
    constexpr int APITCH = KP + 1;              // odd: rows of the filter tile fall on different LDS banks
    constexpr int QROWS = CIN * ROWS;
    constexpr int D1 = PITCH - (KW - 1);                       // last tap of a filter row -> first of the next
    constexpr int D2 = (ROWS - KH + 1) * PITCH - (KW - 1);     // last tap of a channel -> first of the next
    constexpr int UNITS_MAX = QROWS * (VEC ? (PITCH - 2 * kStemPadL) / 4 : PITCH - 2 * kStemPadL);
    constexpr int NLOAD = (UNITS_MAX + kStemThreads - 1) / kStemThreads;
    constexpr int WU = VEC ? 4 : 1; // floats per filter load
    constexpr int NWLOAD = (64 * K / WU + kStemThreads - 1) / kStemThreads;
    static_assert((64 * K) % 4 == 0, "filter tile in 16-byte units");
    static_assert(PITCH % 4 == 0 && KP % 2 == 0, "shape");

    __shared__ __attribute__((aligned(16))) float As[64 * APITCH];
    __shared__ __attribute__((aligned(16))) float Ps[QROWS * PITCH];
    __shared__ __attribute__((aligned(16))) float Bs[64];
    __shared__ int next_block;

    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, h = lane >> 5;

    // each XCD (workgroup id mod 8) walks a contiguous range of bands, so that the rows two
    // neighbouring bands share are fetched into one L2
    const int logical = (int)(blockIdx.x & 7) * a.chunk + (int)(blockIdx.x >> 3);
    if (logical >= a.total)
        return;
    const int mt = logical % a.mtiles, rest = logical / a.mtiles;
    const int band = rest % a.bands, n = rest / a.bands;
    const int r0 = band * R, rb = min(R, a.OH - r0), iy0 = STRIDE * r0 - a.ph, m0 = mt * 64;

    // ---- global -> registers: input rows of the band, filter rows of the m tile, bias ----
    const __amdgpu_buffer_rsrc_t xr =
        __builtin_amdgcn_make_buffer_rsrc((void *)(a.x + (size_t)n * CIN * a.H * a.W), 0, a.x_img_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, a.w_bytes, 0x00020000);
    typedef typename std::conditional<VEC, stem_f32x4, float>::type unit_t;
    unit_t xv[NLOAD];
    int xdst[NLOAD];
#pragma unroll
    for (int i = 0; i < NLOAD; i++) {
        const uint32_t unit = (uint32_t)(tid + i * kStemThreads);
        const uint32_t q = fast_div(unit, a.upr_magic, a.upr_shift), u = unit - q * a.upr;
        const int c = (int)q / ROWS, pr = (int)q - c * ROWS, iy = iy0 + pr;
        const bool row = q < (uint32_t)QROWS;
        const bool ok = row && (unsigned)iy < (unsigned)a.H;
        const uint32_t voff = ok ? (uint32_t)(((c * a.H + iy) * a.W + (int)u * (VEC ? 4 : 1)) * 4) : kStemOutOfRange;
        if constexpr (VEC)
            xv[i] = __builtin_bit_cast(stem_f32x4, __builtin_amdgcn_raw_buffer_load_b128(xr, voff, 0, 0));
        else
            xv[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, voff, 0, 0));
        xdst[i] = row ? (int)q * PITCH + kStemPadL + (int)u * (VEC ? 4 : 1) : -1;
    }
    // the filter rows of an m tile are one contiguous run of 64*K floats, 16-byte aligned when the tensor is
    unit_t wv[NWLOAD];
#pragma unroll
    for (int i = 0; i < NWLOAD; i++) {
        const uint32_t f = (uint32_t)(tid + i * kStemThreads) * WU;
        // rows past Cout read as zero: the offset is past the end of the tensor
        const uint32_t voff = f < 64u * K ? ((uint32_t)m0 * K + f) * 4u : kStemOutOfRange;
        if constexpr (VEC)
            wv[i] = __builtin_bit_cast(stem_f32x4, __builtin_amdgcn_raw_buffer_load_b128(wr, voff, 0, 0));
        else
            wv[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(wr, voff, 0, 0));
    }
    if (tid < 64)
        Bs[tid] = (a.bias != nullptr && m0 + tid < a.Cout) ? a.bias[m0 + tid] : 0.0f;

    // ---- registers -> LDS ----
    if (tid == 0)
        next_block = 0;
    for (uint32_t idx = (uint32_t)tid; idx < (uint32_t)QROWS * a.padw; idx += kStemThreads) { // the zero columns
        const uint32_t q = fast_div(idx, a.padw_magic, a.padw_shift), j = idx - q * a.padw;
        Ps[q * PITCH + (j < (uint32_t)kStemPadL ? j : (uint32_t)a.W + j)] = 0.0f;
    }
    if (K != KP && tid < 64)
        As[tid * APITCH + K] = 0.0f;
#pragma unroll
    for (int i = 0; i < NLOAD; i++)
        if (xdst[i] >= 0) {
            if constexpr (VEC)
                *(stem_f32x4 *)&Ps[xdst[i]] = xv[i];
            else
                Ps[xdst[i]] = xv[i];
        }
#pragma unroll
    for (int i = 0; i < NWLOAD; i++) {
        const int f = (tid + i * kStemThreads) * WU;
        if (f < 64 * K) {
            int m = f / K, k = f - m * K;
            if constexpr (VEC) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    As[m * APITCH + k] = wv[i][e];
                    if (++k == K) {
                        k = 0;
                        m++;
                    }
                }
            } else
                As[m * APITCH + k] = wv[i];
        }
    }
    __syncthreads();

    // ---- blocks of 32 pixels ----
    const int npix = rb * a.OW, nblk = (npix + 31) >> 5;
    const __amdgpu_buffer_rsrc_t yr =
        __builtin_amdgcn_make_buffer_rsrc((void *)(a.y + (size_t)n * a.Cout * a.OHW), 0, a.y_img_bytes, 0x00020000);
    const float *Ab = As + l32 * APITCH + h;
    // accumulator register r of a 32x32 block holds row 8*(r/4) + 4*h + r%4, column l32
    float bv[32];
#pragma unroll
    for (int r = 0; r < 32; r += 4) {
        const stem_f32x4 b4 = *(const stem_f32x4 *)&Bs[(r >> 4) * 32 + 8 * ((r & 15) >> 2) + 4 * h];
        bv[r] = b4[0];
        bv[r + 1] = b4[1];
        bv[r + 2] = b4[2];
        bv[r + 3] = b4[3];
    }
    const bool use_old = a.factor != 0.0f, pre = a.pre != 0;
    for (;;) {
        int blk = 0;
        if (lane == 0)
            blk = atomicAdd(&next_block, 1);
        blk = __builtin_amdgcn_readfirstlane(blk);
        if (blk >= nblk)
            break;
        const int p = blk * 32 + l32;
        const bool valid = p < npix;
        const uint32_t pc = valid ? (uint32_t)p : 0u;
        const int ro = (int)fast_div(pc, a.ow_magic, a.ow_shift), co = (int)pc - ro * a.OW;
        const int lb = STRIDE * (ro * PITCH + co) + kStemPadL - a.pw;
        const float *P0 = Ps + lb + h, *P1 = Ps + lb + h * D1, *P2 = Ps + lb + h * D2;

        stem_f32x16 acc0, acc1;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            acc0[r] = bv[r];
            acc1[r] = bv[16 + r];
        }
        auto fetch = [&](auto jc, float &fa0, float &fa1, float &fb) {
            constexpr int j = decltype(jc)::value;
            constexpr int k0 = 2 * j, k1 = 2 * j + 1;
            constexpr int o0 = ((k0 / (KH * KW)) * ROWS + (k0 % (KH * KW)) / KW) * PITCH + k0 % KW;
            constexpr int o1 = ((k1 / (KH * KW)) * ROWS + (k1 % (KH * KW)) / KW) * PITCH + k1 % KW;
            constexpr int d = k1 < K ? o1 - o0 : 1; // the spare k of an odd K has zero weights: any finite value will do
            static_assert(d == 1 || d == D1 || d == D2, "tap distance");
            fa0 = Ab[k0];
            fa1 = Ab[32 * APITCH + k0];
            fb = (d == 1 ? P0 : d == D1 ? P1 : P2)[o0];
        };
        float ca0, ca1, cb;
        fetch(std::integral_constant<int, 0>{}, ca0, ca1, cb);
        stem_for<NJ>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            float na0 = 0.0f, na1 = 0.0f, nb = 0.0f;
            if constexpr (j + 1 < NJ)
                fetch(std::integral_constant<int, j + 1>{}, na0, na1, nb);
            acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(ca0, cb, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(ca1, cb, acc1, 0, 0, 0);
            ca0 = na0;
            ca1 = na1;
            cb = nb;
        });

        // ---- epilogue: activation, factor, NCHW store (the pixels of a band are contiguous) ----
        const uint32_t voff = valid ? (uint32_t)((4 * h * a.OHW + r0 * a.OW + p) * 4) : kStemOutOfRange;
#pragma unroll
        for (int r = 0; r < 32; r++) {
            const int mrow = m0 + (r >> 4) * 32 + 8 * ((r & 15) >> 2); // + 4*h + r%4 < Cout as Cout is a multiple of 8
            if (mrow >= a.Cout)
                continue;
            const uint32_t soff = (uint32_t)((mrow + (r & 3)) * a.OHW * 4);
            float v = r < 16 ? acc0[r & 15] : acc1[r & 15];
            float old = 0.0f;
            if (use_old)
                old = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(yr, voff, soff, 0));
            if (use_old && pre)
                v = fmaf(old, a.factor, v);
            if constexpr (GENERIC_ACT)
                v = apply_act(v, a.act);
            else if (a.act != DLP_ACT_IDENTITY) // identity must keep NaNs: no min/max
                v = fminf(fmaxf(v, a.clamp_lo), a.clamp_hi);
            if (use_old && !pre)
                v = fmaf(old, a.factor, v);
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), yr, voff, soff, 0);
        }
    }
}

constexpr int kStemR = 4, kStemPitch = 240;

bool generic_activation(int act) { return act == DLP_ACT_TANH || act == DLP_ACT_SIGMOID; }

} // namespace

bool conv_stem_supported(const ConvGeom &g)
{
    if (g.dtype != DLP_FLOAT || g.groups != 1 || g.Cin != 3 || g.KH != 7 || g.KW != 7 || g.sh != 2 || g.sw != 2 || g.dh != 1 || g.dw != 1)
        return false;
    if (g.pw < 0 || g.pw > kStemPadL || g.ph < 0 || g.Cout % 8 != 0 || g.OH <= 0 || g.OW <= 0)
        return false;
    // rightmost LDS column a lane may read: last tap of the last output column, plus the spare k
    if (2 * (g.OW - 1) - g.pw + 6 + kStemPadL + 1 >= kStemPitch || g.W + 2 * kStemPadL > kStemPitch)
        return false;
    return (long long)g.Cin * g.H * g.W * 4 < 0x7fffffffLL && (long long)g.Cout * g.OH * g.OW * 4 < 0x7fffffffLL &&
           (long long)g.Cout * 147 * 4 < 0x7fffffffLL;
}

int conv_stem_launch(const ConvGeom &g, const void *x, const void *w, void *y, const Epilogue &ep, hipStream_t stream)
{
    if (!conv_stem_supported(g))
        return fail(DLP_ERR_NOT_IMPLEMENTED, "conv_stem: unsupported geometry");
    if (g.B == 0)
        return DLP_OK;
    StemArgs a;
    a.x = (const float *)x;
    a.w = (const float *)w;
    a.bias = ep.bias;
    a.y = (float *)y;
    a.B = g.B; a.H = g.H; a.W = g.W; a.Cout = g.Cout; a.OH = g.OH; a.OW = g.OW; a.OHW = g.OH * g.OW;
    a.ph = g.ph; a.pw = g.pw;
    a.bands = (g.OH + kStemR - 1) / kStemR;
    a.mtiles = (g.Cout + 63) / 64;
    const long long total = (long long)g.B * a.bands * a.mtiles;
    if (total > 0x7fffffffLL - 8)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "convolution too large for a single launch");
    a.total = (int)total;
    a.chunk = (int)((total + 7) / 8);
    a.x_img_bytes = (uint32_t)((size_t)g.Cin * g.H * g.W * 4);
    a.y_img_bytes = (uint32_t)((size_t)g.Cout * g.OH * g.OW * 4);
    a.w_bytes = (uint32_t)((size_t)g.Cout * 147 * 4);
    // 16-byte loads: every input row and the filter rows of every m tile then start 16-byte aligned
    const bool vec = g.W % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0;
    a.upr = (uint32_t)(vec ? g.W / 4 : g.W);
    make_magic(a.upr, a.upr_magic, a.upr_shift);
    make_magic((uint32_t)g.OW, a.ow_magic, a.ow_shift);
    a.padw = (uint32_t)(kStemPitch - g.W);
    make_magic(a.padw, a.padw_magic, a.padw_shift);
    a.factor = ep.factor;
    a.pre = ep.accumulate_first;
    a.act = ep.activation;
    a.clamp_lo = -__builtin_huge_valf();
    a.clamp_hi = __builtin_huge_valf();
    if (ep.activation == DLP_ACT_RELU || ep.activation == DLP_ACT_RELU6)
        a.clamp_lo = 0.0f;
    if (ep.activation == DLP_ACT_RELU6)
        a.clamp_hi = 6.0f;
    const dim3 grid((unsigned)(8 * a.chunk)), block(kStemThreads);
    TimingScope ts("conv_gemm", stream);
    const bool gen = generic_activation(ep.activation);
    if (vec && !gen)
        hipLaunchKernelGGL((conv_stem_f32_kernel<3, 7, 7, 2, kStemR, kStemPitch, true, false>), grid, block, 0, stream, a);
    else if (vec)
        hipLaunchKernelGGL((conv_stem_f32_kernel<3, 7, 7, 2, kStemR, kStemPitch, true, true>), grid, block, 0, stream, a);
    else if (!gen)
        hipLaunchKernelGGL((conv_stem_f32_kernel<3, 7, 7, 2, kStemR, kStemPitch, false, false>), grid, block, 0, stream, a);
    else
        hipLaunchKernelGGL((conv_stem_f32_kernel<3, 7, 7, 2, kStemR, kStemPitch, false, true>), grid, block, 0, stream, a);
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

} // namespace dlp
