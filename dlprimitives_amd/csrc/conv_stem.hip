// Strided convolutions with very few input channels (the 7x7 / stride 2 / 3-channel stem of the
// ResNet family): conv_stem_f32_kernel and, for bfloat16 tensors, conv_stem_bf16_kernel (described at the kernel).
//
// With 3 input channels the reduction index of the implicit GEMM runs over filter taps, so the
// gathering kernel of conv_gemm.hip spends vector-ALU work on every gathered element and a K loop
// of ten tiles never amortises its prologue.  Here one workgroup of 16 wavefronts per CU walks a
// contiguous range of output rows in bands of up to R rows, for all 64 output channels of an m tile:
//   * the input rows a band touches (CIN x (STRIDE*(R-1)+KH) rows) are copied to LDS once, with
//     coalesced 16-byte loads, zero padded on every side, at a compile-time row pitch; the rows of
//     the next band are loaded into registers while the current band is computed;
//   * the filter rows of the m tile are copied to LDS as they lie in memory ([m][k], odd pitch), so
//     nothing is packed beforehand;
//   * a wavefront takes 32 consecutive output pixels of the band at a time (the pixels of a band are
//     contiguous in NCHW) and walks the whole reduction with every address fixed beforehand: the
//     operand of tap (c, r, s) is a ds_read at lane base + compile-time offset.  The two k of a
//     v_mfma_f32_32x32x2_f32 belong to the two halves of the wavefront, so the lane base carries
//     half * (distance of the two taps); consecutive taps are 1 element apart, PITCH - (KW-1) at the
//     end of a filter row, and a third constant at the end of a channel: three lane bases cover
//     all pairs.  The loop body is matrix instructions and LDS reads only.
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

constexpr int kStemThreads = 1024;
constexpr int kStemPadL = 4;                    // zero columns left of an input row in LDS (keeps 16-byte stores aligned)
constexpr uint32_t kStemOutOfRange = 0x80000000u; // >= num_records of every buffer we accept

struct StemArgs {
    const void *x, *w; // float or bfloat16, as the kernel says
    const float *bias;
    void *y;
    int B, H, W, Cout, OH, OW, OHW;
    int ph, pw;
    int total_rows, rows_per_wg; // output rows of the launch, numbered (m tile, image, row); rows per workgroup
    uint32_t x_img_bytes, y_img_bytes, w_bytes;
    uint32_t ow_magic, ow_shift;
    uint32_t padw, padw_magic, padw_shift; // PITCH - W zero columns per LDS row
    int e0;                                // bf16 kernel: LDS column of the first of a lane's eight k for output column 0
    float factor;
    int pre, act;
    float clamp_lo, clamp_hi;
    int PH, PW, upi; // max pooling inside the bf16 kernel: pooled size, units (pairs of pooled rows) per image
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
__global__ __launch_bounds__(kStemThreads) void conv_stem_f32_kernel(StemArgs a)
{
    constexpr int K = CIN * KH * KW, KP = (K + 1) / 2 * 2, NJ = KP / 2;
    constexpr int ROWS = STRIDE * (R - 1) + KH; // input rows of a full band
    constexpr int APITCH = KP + 1;              // odd: rows of the filter tile fall on different LDS banks
    constexpr int QROWS = CIN * ROWS;
    constexpr int D1 = PITCH - (KW - 1);                       // last tap of a filter row -> first of the next
    constexpr int D2 = (ROWS - KH + 1) * PITCH - (KW - 1);     // last tap of a channel -> first of the next
    constexpr int XU = VEC ? 4 : 1;                            // floats per load
    constexpr int NROWIT = (QROWS + kStemThreads / 64 - 1) / (kStemThreads / 64);            // LDS rows per wavefront
    constexpr int NCH = ((PITCH - 2 * kStemPadL) / XU + 63) / 64;                              // loads per lane and row
    constexpr int NWLOAD = (64 * K / XU + kStemThreads - 1) / kStemThreads;
    static_assert(PITCH % 4 == 0 && KP % 2 == 0 && (64 * K) % 4 == 0, "shape");

    __shared__ __attribute__((aligned(16))) float As[64 * APITCH];
    __shared__ __attribute__((aligned(16))) float Ps[QROWS * PITCH];
    __shared__ __attribute__((aligned(16))) float Bs[64];

    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // The wavefronts that share a SIMD get different priorities: they would otherwise advance in step and reach their
    // epilogues (32 stores each) together, with the matrix pipe idle meanwhile; now one finishes its block first and
    // stores while the next one computes.
    switch ((wave >> 2) & 3) {
    case 0: __builtin_amdgcn_s_setprio(3); break;
    case 1: __builtin_amdgcn_s_setprio(2); break;
    case 2: __builtin_amdgcn_s_setprio(1); break;
    default: __builtin_amdgcn_s_setprio(0); break;
    }
    typedef typename std::conditional<VEC, stem_f32x4, float>::type unit_t;

    // this workgroup's share: a contiguous range of the output rows of the whole launch, numbered (m tile, image, row)
    const int first = (int)blockIdx.x * a.rows_per_wg, last = min(first + a.rows_per_wg, a.total_rows);
    if (first >= last)
        return;
    const int boh = a.B * a.OH;
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, a.w_bytes, 0x00020000);

    // the zero columns left and right of every LDS row are written once
    for (uint32_t idx = (uint32_t)tid; idx < (uint32_t)QROWS * a.padw; idx += kStemThreads) {
        const uint32_t q = fast_div(idx, a.padw_magic, a.padw_shift), j = idx - q * a.padw;
        Ps[q * PITCH + (j < (uint32_t)kStemPadL ? j : (uint32_t)a.W + j)] = 0.0f;
    }
    if (K != KP && tid < 64)
        As[tid * APITCH + K] = 0.0f;

    // Copy of a band's input rows: wavefront w moves LDS rows w, w + 16, ... and a lane one 16-byte unit (or, for
    // tensors that do not allow 16-byte loads, every 64th element) of each, so that the row arithmetic is scalar.
    // Rows above / below the image and the lanes past the end of a row read as zero: out-of-range offsets.
    uint32_t lane_off[NCH];
#pragma unroll
    for (int j = 0; j < NCH; j++) {
        const int col = (lane + 64 * j) * XU;
        lane_off[j] = col < a.W ? (uint32_t)col * 4u : kStemOutOfRange;
    }
    auto load_band = [&](int n, int iy0, unit_t (&xv)[NROWIT * NCH]) {
        const __amdgpu_buffer_rsrc_t xr =
            __builtin_amdgcn_make_buffer_rsrc((void *)((const float *)a.x + (size_t)n * CIN * a.H * a.W), 0, a.x_img_bytes, 0x00020000);
#pragma unroll
        for (int i = 0; i < NROWIT; i++) {
            const int q = wave + (kStemThreads / 64) * i;
            const int c = q / ROWS, pr = q - c * ROWS, iy = iy0 + pr;
            const bool ok = q < QROWS && (unsigned)iy < (unsigned)a.H; // uniform
            const uint32_t soff = ok ? (uint32_t)((c * a.H + iy) * a.W * 4) : 0u;
#pragma unroll
            for (int j = 0; j < NCH; j++) {
                const uint32_t voff = ok ? lane_off[j] : kStemOutOfRange;
                if constexpr (VEC)
                    xv[i * NCH + j] = __builtin_bit_cast(stem_f32x4, __builtin_amdgcn_raw_buffer_load_b128(xr, voff, soff, 0));
                else
                    xv[i * NCH + j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, voff, soff, 0));
            }
        }
    };
    auto store_band = [&](const unit_t (&xv)[NROWIT * NCH]) {
#pragma unroll
        for (int i = 0; i < NROWIT; i++) {
            const int q = wave + (kStemThreads / 64) * i;
            if (q >= QROWS)
                continue;
#pragma unroll
            for (int j = 0; j < NCH; j++) {
                const int col = (lane + 64 * j) * XU;
                if (col < a.W) {
                    if constexpr (VEC)
                        *(stem_f32x4 *)&Ps[q * PITCH + kStemPadL + col] = xv[i * NCH + j];
                    else
                        Ps[q * PITCH + kStemPadL + col] = xv[i * NCH + j];
                }
            }
        }
    };
    // the band that starts at output row `row` of the launch: m tile, image, first row, rows
    auto decode = [&](int row, int &mt, int &n, int &oy, int &rb) {
        mt = row / boh;
        const int rem = row - mt * boh;
        n = rem / a.OH;
        oy = rem - n * a.OH;
        rb = min(min(R, a.OH - oy), last - row);
    };

    int cur = first, mt, n, oy, rb, loaded_mt = -1;
    decode(cur, mt, n, oy, rb);
    unit_t xv[NROWIT * NCH];
    load_band(n, STRIDE * oy - a.ph, xv);
    const float *Ab = As + l32 * APITCH + h;
    const bool use_old = a.factor != 0.0f, pre = a.pre != 0;

    for (;;) {
        const int m0 = mt * 64;
        const bool new_tile = mt != loaded_mt; // uniform
        unit_t wv[NWLOAD];
        float bias_v = 0.0f;
        if (new_tile) {
            // the filter rows of an m tile are one contiguous run of 64*K floats, 16-byte aligned when the tensor is;
            // rows past Cout read as zero: their offsets are past the end of the tensor
#pragma unroll
            for (int i = 0; i < NWLOAD; i++) {
                const uint32_t f = (uint32_t)(tid + i * kStemThreads) * XU;
                const uint32_t voff = f < 64u * K ? ((uint32_t)m0 * K + f) * 4u : kStemOutOfRange;
                if constexpr (VEC)
                    wv[i] = __builtin_bit_cast(stem_f32x4, __builtin_amdgcn_raw_buffer_load_b128(wr, voff, 0, 0));
                else
                    wv[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(wr, voff, 0, 0));
            }
            if (tid < 64)
                bias_v = (a.bias != nullptr && m0 + tid < a.Cout) ? a.bias[m0 + tid] : 0.0f;
        }
        __syncthreads(); // every wavefront has finished the previous band: LDS may be overwritten
        store_band(xv);
        if (new_tile) {
#pragma unroll
            for (int i = 0; i < NWLOAD; i++) {
                const int f = (tid + i * kStemThreads) * XU;
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
            if (tid < 64)
                Bs[tid] = bias_v;
        }
        __syncthreads();
        loaded_mt = mt;
        // the next band's rows travel while this one is computed
        const int next = cur + rb;
        int nmt = mt, nn = n, noy = oy, nrb = 0;
        if (next < last) {
            decode(next, nmt, nn, noy, nrb);
            load_band(nn, STRIDE * noy - a.ph, xv);
        }

        // ---- blocks of 32 pixels of the band ----
        const int npix = rb * a.OW, nblk = (npix + 31) >> 5;
        const __amdgpu_buffer_rsrc_t yr =
            __builtin_amdgcn_make_buffer_rsrc((void *)((float *)a.y + (size_t)n * a.Cout * a.OHW), 0, a.y_img_bytes, 0x00020000);
        // blocks are dealt round-robin: with wavefront w on SIMD w % 4 every SIMD gets the same number (+-1)
        for (int blk = wave; blk < nblk; blk += kStemThreads / 64) {
            const int p = blk * 32 + l32;
            const bool valid = p < npix;
            const uint32_t pc = valid ? (uint32_t)p : 0u;
            const int ro = (int)fast_div(pc, a.ow_magic, a.ow_shift), co = (int)pc - ro * a.OW;
            const int lb = STRIDE * (ro * PITCH + co) + kStemPadL - a.pw;
            const float *P0 = Ps + lb + h, *P1 = Ps + lb + h * D1, *P2 = Ps + lb + h * D2;

            // accumulator register r of a 32x32 block holds row 8*(r/4) + 4*h + r%4, column l32: it starts from that row's bias
            stem_f32x16 acc0, acc1;
#pragma unroll
            for (int r = 0; r < 16; r += 4) {
                const stem_f32x4 b0 = *(const stem_f32x4 *)&Bs[2 * r + 4 * h], b1 = *(const stem_f32x4 *)&Bs[32 + 2 * r + 4 * h];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    acc0[r + e] = b0[e];
                    acc1[r + e] = b1[e];
                }
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
            // operands are read DEPTH steps ahead of the matrix instructions that use them
            constexpr int DEPTH = 3;
            float oa0[DEPTH + 1], oa1[DEPTH + 1], ob[DEPTH + 1];
            stem_for<DEPTH>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                if constexpr (j < NJ)
                    fetch(jc, oa0[j], oa1[j], ob[j]);
            });
            stem_for<NJ>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                if constexpr (j + DEPTH < NJ)
                    fetch(std::integral_constant<int, j + DEPTH>{}, oa0[(j + DEPTH) % (DEPTH + 1)], oa1[(j + DEPTH) % (DEPTH + 1)],
                          ob[(j + DEPTH) % (DEPTH + 1)]);
                __builtin_amdgcn_sched_barrier(0); // keep this order: the scheduler would sink the operand reads to their uses
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(oa0[j % (DEPTH + 1)], ob[j % (DEPTH + 1)], acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(oa1[j % (DEPTH + 1)], ob[j % (DEPTH + 1)], acc1, 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            });

            // ---- epilogue: activation, factor, NCHW store (the pixels of a band are contiguous) ----
            const uint32_t voff = valid ? (uint32_t)((4 * h * a.OHW + oy * a.OW + p) * 4) : kStemOutOfRange;
            // every vector-ALU instruction here takes issue cycles from the matrix pipe of the SIMD, so the common case
            // (no old value; identity, ReLU or ReLU6) is one v_med3_f32 per value at most
            auto finish = [&](auto mode_c) {
                constexpr int MODE = decltype(mode_c)::value; // 0 store as is, 1 clamp, 2 general
#pragma unroll
                for (int r = 0; r < 32; r++) {
                    const int mrow = m0 + (r >> 4) * 32 + 8 * ((r & 15) >> 2); // + 4*h + r%4 < Cout as Cout is a multiple of 8
                    if (mrow >= a.Cout)
                        continue;
                    const uint32_t soff = (uint32_t)((mrow + (r & 3)) * a.OHW * 4);
                    float v = r < 16 ? acc0[r & 15] : acc1[r & 15];
                    if constexpr (MODE == 1)
                        v = clamp_med3(v, a.clamp_lo, a.clamp_hi);
                    if constexpr (MODE == 2) {
                        float old = 0.0f;
                        if (use_old)
                            old = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(yr, voff, soff, 0));
                        if (use_old && pre)
                            v = fmaf(old, a.factor, v);
                        if constexpr (GENERIC_ACT)
                            v = apply_act(v, a.act);
                        else if (a.act != DLP_ACT_IDENTITY) // identity must keep NaNs: no min/max
                            v = clamp_med3(v, a.clamp_lo, a.clamp_hi);
                        if (use_old && !pre)
                            v = fmaf(old, a.factor, v);
                    }
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), yr, voff, soff, 0);
                }
            };
            if (GENERIC_ACT || use_old)
                finish(std::integral_constant<int, 2>{});
            else if (a.act != DLP_ACT_IDENTITY)
                finish(std::integral_constant<int, 1>{});
            else
                finish(std::integral_constant<int, 0>{});
        }
        if (next >= last)
            break;
        cur = next;
        mt = nmt;
        n = nn;
        oy = noy;
        rb = nrb;
    }
}

// ---- bfloat16 tensors ----------------------------------------------------------------------------------------------
// The same walk (one workgroup per CU, bands of R output rows, the next band's input rows in flight while this one is
// computed) around v_mfma_f32_32x32x16_bf16, whose lanes hold EIGHT consecutive k each: one filter row of seven taps
// and a leading zero.  The reduction therefore runs over the CIN * KH filter rows, two per instruction (one per half of
// the wavefront), and an operand is 16 contiguous bytes on both sides:
//   * pixels are the M side: lane (pixel p, half h) reads the eight input values left of and under filter row
//     2j + h from the band in LDS, starting one element left of the window so that the address is a multiple of four
//     bytes (even column: the kernel takes odd paddings only); the spare first element meets a zero weight;
//   * filters are the N side: the tile's filters lie in LDS as [filter][filter row][8] with the zero in front.
// With 21 filter rows that is 11 matrix instructions per 32 pixels x 32 filters -- some 15 us of matrix time for
// ResNet-50's stem at batch 128 -- so the kernel is bound by its stores: the accumulators (lane = filter, register =
// pixel, four consecutive pixels per register quad) are rounded, staged through LDS as [filter][pixel] and leave as
// 16-byte stores, four lanes per 64-byte run of a filter's row.  Accumulation with an old y, and images whose rows are
// not multiples of eight pixels, take 2-byte accesses straight from the accumulators.
// As in the fp32 kernel, input values that are not finite may spread to the neighbouring output column through the
// spare element (0 * inf).
typedef __bf16 stem_bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t stem_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t stem_u32x2 __attribute__((ext_vector_type(2)));

constexpr int kStemPadL16 = 8;     // zero columns left of an input row (keeps the 16-byte LDS stores aligned)
constexpr int kStemPoolPitch = 120;  // elements per row of convolution results kept for the pooling: 8 to the left, up to 112 columns
constexpr int kStemStagePitch = 80; // bytes per filter of a wavefront's staged 32 x 32 output block (64 + 16: 16-byte rows)

template <int CIN, int KH, int KW, int STRIDE, int R, int PITCH, int NT, bool POOL = false>
constexpr int stem_bf16_lds_bytes()
{
    constexpr int ROWS = STRIDE * (R - 1) + KH, QP = (CIN * KH + 1) / 2 * 2;
    return CIN * ROWS * PITCH * 2 + 64 * (QP * 8 + 8) * 2 + 64 * 4 + (POOL ? 64 * R * kStemPoolPitch * 2 : (NT / 64) * 32 * kStemStagePitch);
}

// POOL: the 3x3 stride-2 pad-1 max pooling that follows the stem of every ResNet runs inside the kernel.  The workgroup walks units
// of two pooled rows instead of bands: pooled rows 2u and 2u + 1 look at convolution rows 4u - 1 .. 4u + 3.  Results go to LDS as bf16
// [filter][row % 5][column] -- eight columns of -inf to the left stand for column -1 -- so row 4u - 1 is still there from the unit
// before and a unit computes four rows; only the first unit of a workgroup's range, when it is not the top of an image, computes
// all five (R = 5).  The pooled rows leave as 16-byte stores: a quarter of the convolution's bytes, and the pooling operator's pass
// over them (as long again as the convolution) is gone.  Values equal those of the two operators run one after the other bit for bit.
template <int CIN, int KH, int KW, int STRIDE, int R, int PITCH, bool VEC, int NT, bool POOL = false>
__global__ __launch_bounds__(NT) void conv_stem_bf16_kernel(StemArgs a)
{
    static_assert(!POOL || (VEC && R == 5), "the pooled form: five rows at most and 16-byte input loads");
    constexpr int OBP = kStemPoolPitch; // POOL: elements per row of the results in LDS
    static_assert(KW <= 7, "a filter row and its leading zero are the eight k of a lane");
    constexpr int K = CIN * KH * KW;
    constexpr int Q = CIN * KH, QP = (Q + 1) / 2 * 2, NJ = QP / 2; // filter rows, two per matrix instruction
    constexpr int ROWS = STRIDE * (R - 1) + KH;                   // input rows of a full band
    constexpr int QROWS = CIN * ROWS;
    constexpr int WPITCH = QP * 8 + 8;                            // elements per filter in LDS (16-byte rows, off the powers of two)
    constexpr int D1 = PITCH;                                     // filter row -> the next of the same channel
    constexpr int D2 = (ROWS - KH + 1) * PITCH;                   // last filter row of a channel -> first of the next
    constexpr int XU = VEC ? 8 : 1;                               // elements per load
    constexpr int NROWIT = (QROWS + NT / 64 - 1) / (NT / 64);
    constexpr int NCH = ((PITCH - 2 * kStemPadL16) / XU + 63) / 64;
    constexpr int NWLOAD = (64 * K + NT - 1) / NT;
    constexpr int YP = kStemStagePitch;
    static_assert(PITCH % 8 == 0 && (QROWS * PITCH * 2) % 16 == 0 && (WPITCH * 2) % 16 == 0, "16-byte LDS rows");

    extern __shared__ __attribute__((aligned(16))) unsigned char stem_lds[];
    uint16_t *Ps = (uint16_t *)stem_lds;     // [QROWS][PITCH] input rows of the band
    uint16_t *Ws = Ps + QROWS * PITCH;       // [64][WPITCH] filters of the tile
    float *Bs = (float *)(Ws + 64 * WPITCH); // [64] bias
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    unsigned char *Ys = (unsigned char *)(Bs + 64) + (POOL ? 0 : wave * (32 * YP)); // this wavefront's staged block
    uint16_t *Ob = (uint16_t *)(Bs + 64);                                            // POOL: [64][5][OBP] results, row r in slot r % 5
    typedef typename std::conditional<VEC, stem_u32x4, uint16_t>::type unit_t;

    const int first = (int)blockIdx.x * a.rows_per_wg, last = min(first + a.rows_per_wg, a.total_rows);
    if (first >= last)
        return;
    const int boh = a.B * a.OH;
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, a.w_bytes, 0x00020000);

    // written once: the zero columns left and right of every input row, and the filter tile's zeros (leading element
    // of every filter row, the spare filter row)
    for (uint32_t idx = (uint32_t)tid; idx < (uint32_t)QROWS * a.padw; idx += NT) {
        const uint32_t q = fast_div(idx, a.padw_magic, a.padw_shift), j = idx - q * a.padw;
        Ps[q * PITCH + (j < (uint32_t)kStemPadL16 ? j : (uint32_t)a.W + j)] = 0;
    }
    for (int i = tid; i < 64 * WPITCH / 2; i += NT)
        ((uint32_t *)Ws)[i] = 0u;
    if constexpr (POOL)
        for (int i = tid; i < 64 * R * 8; i += NT) // left of column 0: never the maximum
            Ob[(i >> 3) * OBP + (i & 7)] = 0xFF80u;

    uint32_t lane_off[NCH];
#pragma unroll
    for (int j = 0; j < NCH; j++) {
        const int col = (lane + 64 * j) * XU;
        lane_off[j] = col < a.W ? (uint32_t)col * 2u : kStemOutOfRange;
    }
    auto load_band = [&](int n, int iy0, unit_t (&xv)[NROWIT * NCH]) {
        const __amdgpu_buffer_rsrc_t xr =
            __builtin_amdgcn_make_buffer_rsrc((void *)((const uint16_t *)a.x + (size_t)n * CIN * a.H * a.W), 0, a.x_img_bytes, 0x00020000);
#pragma unroll
        for (int i = 0; i < NROWIT; i++) {
            const int q = wave + (NT / 64) * i;
            const int c = q / ROWS, pr = q - c * ROWS, iy = iy0 + pr;
            const bool ok = q < QROWS && (unsigned)iy < (unsigned)a.H; // uniform
            const uint32_t soff = ok ? (uint32_t)((c * a.H + iy) * a.W * 2) : 0u;
#pragma unroll
            for (int j = 0; j < NCH; j++) {
                const uint32_t voff = ok ? lane_off[j] : kStemOutOfRange;
                if constexpr (VEC)
                    xv[i * NCH + j] = __builtin_amdgcn_raw_buffer_load_b128(xr, voff, soff, 0);
                else
                    xv[i * NCH + j] = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(xr, voff, soff, 0);
            }
        }
    };
    auto store_band = [&](const unit_t (&xv)[NROWIT * NCH]) {
#pragma unroll
        for (int i = 0; i < NROWIT; i++) {
            const int q = wave + (NT / 64) * i;
            if (q >= QROWS)
                continue;
#pragma unroll
            for (int j = 0; j < NCH; j++) {
                const int col = (lane + 64 * j) * XU;
                if (col < a.W) {
                    if constexpr (VEC)
                        *(stem_u32x4 *)&Ps[q * PITCH + kStemPadL16 + col] = xv[i * NCH + j];
                    else
                        Ps[q * PITCH + kStemPadL16 + col] = xv[i * NCH + j];
                }
            }
        }
    };
    int unit_u = 0; // POOL: the pair of pooled rows in hand
    auto decode = [&](int row, int &mt, int &n, int &oy, int &rb) {
        if constexpr (POOL) { // `row` numbers units: (m tile, image, pair of pooled rows)
            const int per_tile = a.B * a.upi;
            mt = row / per_tile;
            const int rem = row - mt * per_tile;
            n = rem / a.upi;
            const int u = rem - n * a.upi;
            oy = (u > 0 && row == first) ? 4 * u - 1 : 4 * u; // row 4u - 1 is in LDS unless the range starts here
            rb = max(min(4 * u + 4, a.OH) - oy, 0);
        } else {
            mt = row / boh;
            const int rem = row - mt * boh;
            n = rem / a.OH;
            oy = rem - n * a.OH;
            rb = min(min(R, a.OH - oy), last - row);
        }
    };

    int cur = first, mt, n, oy, rb, loaded_mt = -1;
    decode(cur, mt, n, oy, rb);
    unit_t xv[NROWIT * NCH];
    load_band(n, STRIDE * oy - a.ph, xv);
    const uint16_t *Wb = Ws + l32 * WPITCH + h * 8;
    const bool use_old = a.factor != 0.0f, pre = a.pre != 0;
    const bool generic = a.act == DLP_ACT_TANH || a.act == DLP_ACT_SIGMOID;
    // 16-byte stores: rows of whole 8-pixel runs, every run 16-byte aligned
    const bool wide = !use_old && a.OW % 8 == 0 && ((uintptr_t)a.y & 15) == 0;
    auto activate = [&](float v) {
        if (generic)
            return apply_act(v, a.act);
        return a.act != DLP_ACT_IDENTITY ? clamp_med3(v, a.clamp_lo, a.clamp_hi) : v; // identity must keep NaNs: no min/max
    };

    for (;;) {
        const int m0 = mt * 64;
        const bool new_tile = mt != loaded_mt; // uniform
        __syncthreads(); // every wavefront has finished the previous band: LDS may be overwritten
        store_band(xv);
        if (new_tile) {
            // filter m of the tile: K contiguous elements [c][r][s] -> LDS [c * KH + r][1 + s]; filters past Cout read as zero
#pragma unroll
            for (int i = 0; i < NWLOAD; i++) {
                const int f = tid + i * NT;
                const uint32_t voff = f < 64 * K ? ((uint32_t)m0 * K + (uint32_t)f) * 2u : kStemOutOfRange;
                const uint16_t v = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(wr, voff, 0, 0);
                if (f < 64 * K) {
                    const int m = f / K, k = f - m * K, q = k / KW, s_ = k - q * KW;
                    Ws[m * WPITCH + q * 8 + 1 + s_] = v;
                }
            }
            if (tid < 64)
                Bs[tid] = (a.bias != nullptr && m0 + tid < a.Cout) ? a.bias[m0 + tid] : 0.0f;
        }
        __syncthreads();
        loaded_mt = mt;
        const int next = POOL ? cur + 1 : cur + rb;
        if constexpr (POOL)
            unit_u = (cur - mt * a.B * a.upi) % a.upi;
        int nmt = mt, nn = n, noy = oy, nrb = 0;
        if (next < last) {
            decode(next, nmt, nn, noy, nrb);
            load_band(nn, STRIDE * noy - a.ph, xv);
        }

        // ---- blocks of 32 pixels of the band ----
        const int npix = rb * a.OW, nblk = (npix + 31) >> 5;
        const __amdgpu_buffer_rsrc_t yr =
            __builtin_amdgcn_make_buffer_rsrc((void *)((uint16_t *)a.y + (size_t)n * a.Cout * a.OHW), 0, a.y_img_bytes, 0x00020000);
        for (int blk = wave; blk < nblk; blk += NT / 64) {
            const int p = blk * 32 + l32;
            const uint32_t pc = p < npix ? (uint32_t)p : 0u;
            const int ro = (int)fast_div(pc, a.ow_magic, a.ow_shift), co = (int)pc - ro * a.OW;
            const int lb = STRIDE * (ro * PITCH + co) + a.e0; // even
            const uint32_t *P0 = (const uint32_t *)(Ps + lb), *P1 = (const uint32_t *)(Ps + lb + h * D1), *P2 = (const uint32_t *)(Ps + lb + h * D2);

            stem_f32x16 acc[2];
#pragma unroll
            for (int cb = 0; cb < 2; cb++) {
                const float b = Bs[cb * 32 + l32];
#pragma unroll
                for (int r = 0; r < 16; r++)
                    acc[cb][r] = b;
            }
            // operands of step j + DEPTH are asked for before the matrix instructions of step j: left to itself the compiler reads
            // each step's operands right in front of their use and every step waits for a whole trip to LDS (deeper than one step
            // ahead the 128 registers of a 1024-thread workgroup run out, and the block is bound by LDS reads anyway: 3 KB a step)
            constexpr int DEPTH = 1;
            stem_u32x4 px[DEPTH + 1];
            stem_bf16x8 w0[DEPTH + 1], w1[DEPTH + 1];
            auto fetch = [&](auto jc) {
                constexpr int j = decltype(jc)::value, slot = j % (DEPTH + 1);
                constexpr int q0 = 2 * j, q1 = 2 * j + 1;
                constexpr int o0 = ((q0 / KH) * ROWS + q0 % KH) * PITCH, o1 = ((q1 / KH) * ROWS + q1 % KH) * PITCH;
                constexpr int d = q1 < Q ? o1 - o0 : 0; // the spare filter row has zero weights: the other half's values do
                static_assert(d == 0 || d == D1 || d == D2, "filter row distance");
                static_assert(o0 % 2 == 0, "dword aligned");
                const uint32_t *pp = (d == D1 ? P1 : d == D2 ? P2 : P0) + o0 / 2;
                px[slot][0] = pp[0], px[slot][1] = pp[1], px[slot][2] = pp[2], px[slot][3] = pp[3];
                w0[slot] = *(const stem_bf16x8 *)(Wb + j * 16);
                w1[slot] = *(const stem_bf16x8 *)(Wb + 32 * WPITCH + j * 16);
            };
            stem_for<DEPTH>([&](auto jc) {
                if constexpr (decltype(jc)::value < NJ)
                    fetch(jc);
            });
            stem_for<NJ>([&](auto jc) {
                constexpr int j = decltype(jc)::value, slot = j % (DEPTH + 1);
                if constexpr (j + DEPTH < NJ)
                    fetch(std::integral_constant<int, j + DEPTH>{});
                __builtin_amdgcn_sched_barrier(0); // keep this order: the scheduler would sink the operand reads to their uses
                const stem_bf16x8 xa = __builtin_bit_cast(stem_bf16x8, px[slot]);
                acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa, w0[slot], acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa, w1[slot], acc[1], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            });

            // accumulator register r of filter block cb: filter m0 + 32 * cb + l32, pixel blk * 32 + 8 * (r / 4) + 4 * h + r % 4
            if constexpr (POOL) {
                // a register quad is four consecutive pixels of one row (rows are multiples of eight pixels): one 8-byte LDS store
#pragma unroll
                for (int rq = 0; rq < 4; rq++) {
                    const int p4 = blk * 32 + 8 * rq + 4 * h;
                    const uint32_t p4c = p4 < npix ? (uint32_t)p4 : 0u;
                    const int r4 = (int)fast_div(p4c, a.ow_magic, a.ow_shift), c4 = (int)p4c - r4 * a.OW;
                    const int slot = (oy + r4) % 5;
#pragma unroll
                    for (int cb = 0; cb < 2; cb++) {
                        stem_u32x2 o;
#pragma unroll
                        for (int e = 0; e < 2; e++) {
                            const float lo = activate(acc[cb][4 * rq + 2 * e]), hi = activate(acc[cb][4 * rq + 2 * e + 1]);
                            o[e] = (uint32_t)to_bf16(lo).bits | ((uint32_t)to_bf16(hi).bits << 16);
                        }
                        if (p4 < npix)
                            *(stem_u32x2 *)(Ob + ((cb * 32 + l32) * 5 + slot) * OBP + 8 + c4) = o;
                    }
                }
            } else if (wide) {
#pragma unroll
                for (int cb = 0; cb < 2; cb++) {
                    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront"); // the block's previous reads are done
                    __builtin_amdgcn_wave_barrier();
#pragma unroll
                    for (int rq = 0; rq < 4; rq++) {
                        stem_u32x2 o;
#pragma unroll
                        for (int e = 0; e < 2; e++) {
                            const float lo = activate(acc[cb][4 * rq + 2 * e]), hi = activate(acc[cb][4 * rq + 2 * e + 1]);
                            o[e] = (uint32_t)to_bf16(lo).bits | ((uint32_t)to_bf16(hi).bits << 16);
                        }
                        *(stem_u32x2 *)(Ys + l32 * YP + (8 * rq + 4 * h) * 2) = o;
                    }
                    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                    __builtin_amdgcn_wave_barrier();
#pragma unroll
                    for (int t = 0; t < 2; t++) {
                        const int fl = t * 16 + (lane >> 2), seg = lane & 3; // filter of the block, run of eight pixels
                        const stem_u32x4 o = *(const stem_u32x4 *)(Ys + fl * YP + seg * 16);
                        const int m = m0 + cb * 32 + fl, p0 = blk * 32 + seg * 8;
                        const uint32_t voff = (m < a.Cout && p0 < npix) ? (uint32_t)((m * a.OHW + oy * a.OW + p0) * 2) : kStemOutOfRange;
                        __builtin_amdgcn_raw_buffer_store_b128(o, yr, voff, 0, 0);
                    }
                }
            } else {
#pragma unroll
                for (int cb = 0; cb < 2; cb++) {
                    const int m = m0 + cb * 32 + l32;
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int pp = blk * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                        const uint32_t voff = (m < a.Cout && pp < npix) ? (uint32_t)((m * a.OHW + oy * a.OW + pp) * 2) : kStemOutOfRange;
                        float v = acc[cb][r], old = 0.0f;
                        if (use_old)
                            old = __builtin_bit_cast(float, (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(yr, voff, 0, 0) << 16);
                        if (use_old && pre)
                            v = fmaf(old, a.factor, v);
                        v = activate(v);
                        if (use_old && !pre)
                            v = fmaf(old, a.factor, v);
                        __builtin_amdgcn_raw_buffer_store_b16((short)to_bf16(v).bits, yr, voff, 0, 0);
                    }
                }
            }
        }
        if constexpr (POOL) {
            // ---- the unit's pooled rows: a thread takes eight pooled columns of a (filter, row): 17 columns of up to three rows ----
            __syncthreads();
            constexpr float kLowest = -3.402823466e+38f;
            const int pw8 = a.PW >> 3, prs = min(2, a.PH - 2 * unit_u), per_m = prs * pw8;
            const __amdgpu_buffer_rsrc_t pyr =
                __builtin_amdgcn_make_buffer_rsrc((void *)((uint16_t *)a.y + (size_t)n * a.Cout * a.PH * a.PW), 0, a.y_img_bytes, 0x00020000);
            for (int t = tid; t < 64 * per_m; t += NT) {
                const int m = t / per_m, r2 = t - m * per_m, pr = r2 / pw8, k = r2 - pr * pw8;
                const int prow = 2 * unit_u + pr;
                float rowmax[3][8];
#pragma unroll
                for (int dr = 0; dr < 3; dr++) {
                    const int row = 2 * prow - 1 + dr;
                    const bool ok = row >= 0 && row < a.OH;
                    const uint16_t *src = Ob + (m * 5 + (ok ? row % 5 : 0)) * OBP + 8 + 16 * k;
                    float e[17];
                    e[0] = __builtin_bit_cast(float, (uint32_t)src[-1] << 16);
                    const stem_u32x4 v0 = *(const stem_u32x4 *)src, v1 = *(const stem_u32x4 *)(src + 8);
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        e[1 + 2 * q] = __builtin_bit_cast(float, v0[q] << 16);
                        e[2 + 2 * q] = __builtin_bit_cast(float, v0[q] & 0xffff0000u);
                        e[9 + 2 * q] = __builtin_bit_cast(float, v1[q] << 16);
                        e[10 + 2 * q] = __builtin_bit_cast(float, v1[q] & 0xffff0000u);
                    }
#pragma unroll
                    for (int j = 0; j < 8; j++)
                        rowmax[dr][j] = ok ? fmaxf(fmaxf(e[2 * j], e[2 * j + 1]), e[2 * j + 2]) : kLowest;
                }
                float best[8];
#pragma unroll
                for (int j = 0; j < 8; j++)
                    best[j] = fmaxf(fmaxf(rowmax[0][j], rowmax[1][j]), rowmax[2][j]);
                stem_u32x4 o;
#pragma unroll
                for (int q = 0; q < 4; q++) // maxima of stored values are bf16 already: the upper halves are the results
                    o[q] = (__builtin_bit_cast(uint32_t, best[2 * q]) >> 16) | (__builtin_bit_cast(uint32_t, best[2 * q + 1]) & 0xffff0000u);
                const uint32_t voff = (m0 + m < a.Cout) ? (uint32_t)((((m0 + m) * a.PH + prow) * a.PW + 8 * k) * 2) : kStemOutOfRange;
                __builtin_amdgcn_raw_buffer_store_b128(o, pyr, voff, 0, 0);
            }
        }
        if (next >= last)
            break;
        cur = next;
        mt = nmt;
        n = nn;
        oy = noy;
        rb = nrb;
    }
}

constexpr int kStemR = 8, kStemPitch = 240, kStemPoolR = 5;
constexpr int kStemPitchBf16 = 240; // 320 (rows of the two lane halves on different LDS banks) measured the same

bool generic_activation(int act) { return act == DLP_ACT_TANH || act == DLP_ACT_SIGMOID; }

} // namespace

bool conv_stem_supported(const ConvGeom &g)
{
    if ((g.dtype != DLP_FLOAT && g.dtype != DLP_BFLOAT16) || g.groups != 1 || g.Cin != 3 || g.KH != 7 || g.KW != 7 || g.sh != 2 || g.sw != 2 || g.dh != 1 ||
        g.dw != 1)
        return false;
    if (g.pw < 0 || g.ph < 0 || g.OH <= 0 || g.OW <= 0)
        return false;
    const long long esize = g.dtype == DLP_FLOAT ? 4 : 2;
    if ((long long)g.Cin * g.H * g.W * esize >= 0x7fffffffLL || (long long)g.Cout * g.OH * g.OW * esize >= 0x7fffffffLL || (long long)g.Cout * 147 * esize >= 0x7fffffffLL)
        return false;
    if (g.dtype == DLP_BFLOAT16) {
        // a lane's eight k start one element left of the window, on an even LDS column: odd paddings only;
        // rightmost column read: the eighth element of the last output column
        const int e0 = kStemPadL16 - g.pw - 1;
        return e0 >= 0 && e0 % 2 == 0 && 2 * (g.OW - 1) + e0 + 7 < kStemPitchBf16 && g.W + 2 * kStemPadL16 <= kStemPitchBf16;
    }
    if (g.pw > kStemPadL || g.Cout % 8 != 0)
        return false;
    // rightmost LDS column a lane may read: last tap of the last output column, plus the spare k
    return 2 * (g.OW - 1) - g.pw + 6 + kStemPadL + 1 < kStemPitch && g.W + 2 * kStemPadL <= kStemPitch;
}

bool conv_stem_pool_supported(const ConvGeom &g, int PH, int PW)
{
    // whole runs of eight pixels in convolution and pooled rows; the last pooling window ends inside the row (the columns
    // right of it are not initialised in LDS) and starts inside the image
    return g.dtype == DLP_BFLOAT16 && conv_stem_supported(g) && g.W % 8 == 0 && g.OW % 8 == 0 && PW % 8 == 0 && PW >= 8 && 2 * PW == g.OW &&
           PH >= 1 && 2 * (PH - 1) - 1 < g.OH && 8 + g.OW <= kStemPoolPitch && (long long)g.Cout * PH * PW * 2 < 0x7fffffffLL;
}

int conv_stem_launch(const ConvGeom &g, const void *x, const void *w, void *y, const Epilogue &ep, hipStream_t stream, int PH, int PW)
{
    if (!conv_stem_supported(g))
        return fail(DLP_ERR_NOT_IMPLEMENTED, "conv_stem: unsupported geometry");
    const bool pool = PH > 0;
    if (pool && (!conv_stem_pool_supported(g, PH, PW) || ep.factor != 0.0f || ((uintptr_t)x & 15) != 0 || ((uintptr_t)y & 15) != 0))
        return fail(DLP_ERR_NOT_IMPLEMENTED, "conv_stem: the max pooling cannot run inside the kernel for this geometry, alignment or scale of the old y");
    if (g.B == 0)
        return DLP_OK;
    StemArgs a;
    const bool bf16 = g.dtype == DLP_BFLOAT16;
    const size_t esize = bf16 ? 2 : 4;
    a.x = x;
    a.w = w;
    a.bias = ep.bias;
    a.y = y;
    a.B = g.B; a.H = g.H; a.W = g.W; a.Cout = g.Cout; a.OH = g.OH; a.OW = g.OW; a.OHW = g.OH * g.OW;
    a.ph = g.ph; a.pw = g.pw;
    const int mtiles = (g.Cout + 63) / 64;
    a.PH = PH; a.PW = PW; a.upi = (PH + 1) / 2;
    const long long total = (long long)mtiles * g.B * (pool ? a.upi : g.OH); // rows, or pairs of pooled rows
    if (total > 0x7fffffffLL - 65536)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "convolution too large for a single launch");
    // one workgroup per CU walks a contiguous range of output rows in bands of up to R rows
    const int wgs = (int)std::min<long long>(dlp_cu_count(), (total + 1) / 2);
    a.total_rows = (int)total;
    a.rows_per_wg = (int)((total + wgs - 1) / wgs);
    a.x_img_bytes = (uint32_t)((size_t)g.Cin * g.H * g.W * esize);
    a.y_img_bytes = pool ? (uint32_t)((size_t)g.Cout * PH * PW * esize) : (uint32_t)((size_t)g.Cout * g.OH * g.OW * esize);
    a.w_bytes = (uint32_t)((size_t)g.Cout * 147 * esize);
    // 16-byte loads: every input row and (fp32) the filter rows of every m tile then start 16-byte aligned
    const bool vec = bf16 ? g.W % 8 == 0 && ((uintptr_t)x & 15) == 0 : g.W % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0;
    make_magic((uint32_t)g.OW, a.ow_magic, a.ow_shift);
    a.padw = (uint32_t)((bf16 ? kStemPitchBf16 : kStemPitch) - g.W);
    a.e0 = kStemPadL16 - g.pw - 1;
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
    const dim3 grid((unsigned)((a.total_rows + a.rows_per_wg - 1) / a.rows_per_wg)), block(kStemThreads);
    TimingScope ts("conv_gemm", stream);
    if (pool) {
        constexpr int lds = stem_bf16_lds_bytes<3, 7, 7, 2, kStemPoolR, kStemPitchBf16, kStemThreads, true>();
        auto kernel = conv_stem_bf16_kernel<3, 7, 7, 2, kStemPoolR, kStemPitchBf16, true, kStemThreads, true>;
        static bool asked[64] = {}; // per device
        int dev = 0;
        DLP_HIP_TRY(hipGetDevice(&dev));
        if (dev < 0 || dev >= 64 || !asked[dev]) {
            DLP_HIP_TRY(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
            if (dev >= 0 && dev < 64)
                asked[dev] = true;
        }
        DLP_LAUNCH_TIMED(ts, kernel, grid, block, lds, stream, a);
        DLP_HIP_TRY(hipGetLastError());
        return DLP_OK;
    }
    if (bf16) {
        constexpr int lds = stem_bf16_lds_bytes<3, 7, 7, 2, kStemR, kStemPitchBf16, kStemThreads>();
        auto kernel = vec ? conv_stem_bf16_kernel<3, 7, 7, 2, kStemR, kStemPitchBf16, true, kStemThreads> : conv_stem_bf16_kernel<3, 7, 7, 2, kStemR, kStemPitchBf16, false, kStemThreads>;
        // more than 64 KB of LDS has to be asked for (bands of 16 rows, or two workgroups of 8 wavefronts per CU, were no faster)
        static bool asked[2][64] = {}; // per kernel and device
        int dev = 0;
        DLP_HIP_TRY(hipGetDevice(&dev));
        if (dev < 0 || dev >= 64 || !asked[vec][dev]) {
            DLP_HIP_TRY(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
            if (dev >= 0 && dev < 64)
                asked[vec][dev] = true;
        }
        DLP_LAUNCH_TIMED(ts, kernel, grid, block, lds, stream, a);
        DLP_HIP_TRY(hipGetLastError());
        return DLP_OK;
    }
    const bool gen = generic_activation(ep.activation);
    if (vec && !gen)
        DLP_LAUNCH_TIMED(ts, (conv_stem_f32_kernel<3, 7, 7, 2, kStemR, kStemPitch, true, false>), grid, block, 0, stream, a);
    else if (vec)
        DLP_LAUNCH_TIMED(ts, (conv_stem_f32_kernel<3, 7, 7, 2, kStemR, kStemPitch, true, true>), grid, block, 0, stream, a);
    else if (!gen)
        DLP_LAUNCH_TIMED(ts, (conv_stem_f32_kernel<3, 7, 7, 2, kStemR, kStemPitch, false, false>), grid, block, 0, stream, a);
    else
        DLP_LAUNCH_TIMED(ts, (conv_stem_f32_kernel<3, 7, 7, 2, kStemR, kStemPitch, false, true>), grid, block, 0, stream, a);
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

} // namespace dlp
