// Pointwise (1x1, stride 1, no padding, one group) convolutions with at most 32 output channels over many pixels, fp32:
//   Y_b[M x HW] = act(W[M x K] * X_b[K x HW] + bias),  M = Cout <= 32, K = Cin a multiple of 16, H * W a multiple of 4,
//   at least 1024 tiles of 128 pixels (MobileNet's 144 -> 24 at 56 x 56 from batch 42 on).
//
// Replaces, for these shapes, the generic path of conv_gemm.hip (reference: the 1x1 fast path of sgemm.cl,
// src/kernels/sgemm.cl:78-93, under Conv2DForwardGEMM, src/core/conv.cpp:45-111).  Such a layer reads six times more than it
// writes and sits on the bandwidth leg of the roofline: what counts is that X is read once, in wide pieces, with many loads in flight.
//  * NCHW keeps the pixels of a channel contiguous, which is the operand layout of v_mfma_f32_32x32x2_f32: lane
//    (column n, half h) holds B[k = h][n].  A wavefront therefore loads X straight from memory into operand registers:
//    one 16-byte buffer load per pair of channels (lanes 0-31 channel 2p, lanes 32-63 channel 2p + 1) feeds four matrix
//    instructions, the MFMA block j taking pixel 4 n + j; eight pairs (8 KB) are in flight per wavefront.  No LDS traffic, no barrier
//    and no vector-ALU instruction for the big operand; the output leaves in 16-byte stores.
//  * The filter is small: it goes through LDS in chunks of 64 channels, transposed to [k][m] on the way in (an operand fetch is
//    then a conflict-free ds_read_b32), double buffered, one barrier per chunk; operands are read eight pairs at a time.
//  * The kernel is written for any split of a workgroup's four wavefronts into MS slices of the output channels times 4 / MS pixel
//    tiles, MTW blocks of 32 rows per wavefront and 1 or 4 pixels per lane.  Measured alone on cold tensors at batch 64, only the
//    shape above beats the LDS-tiled kernel (144->24 at 56x56: 30.7 against 33.7 us; 144->32 at 28x28 with one pixel per lane 14.0
//    against 12.4; 192->64 at 14x14 11.8 against 9.3; 64->64 at 56x56 with two blocks per wavefront 42.8 against 34.2): the small layers
//    are bound by the fixed 2 us each of prologue (first filter chunk) and epilogue, not by how X arrives.  Only that variant is built.
// The sum over k runs in channel order, two channels per matrix instruction, accumulated in fp32.
#include "dlp_internal.hpp"
// the output runs are whole cache lines that this launch does not read again: non-temporal stores (144->24 at 56x56, batch 64: 31.5 -> 28.9 us)
#ifndef PW_STORE_AUX
#define PW_STORE_AUX 2
#endif

#include <algorithm>
#include <type_traits>

namespace dlp {

typedef float pw_f32x16 __attribute__((ext_vector_type(16)));
typedef float pw_f32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int kPwThreads = 256;
constexpr int kPwChunk = 64;  // channels of a filter chunk in LDS
#ifndef DLP_PW_DEPTH1
#define DLP_PW_DEPTH1 32
#endif
#ifndef DLP_PW_DEPTH4
#define DLP_PW_DEPTH4 8
#endif
constexpr uint32_t kPwOutOfRange = 0x80000000u;

struct PwArgs {
    const float *x, *w, *bias;
    float *y;
    int M, K, HW, N;      // output channels, input channels, pixels per image, pixels in all (batch * HW)
    int mpad;             // rows of the LDS filter chunk: M rounded up to 32 * MS * MTW
    uint32_t x_bytes, y_bytes, w_bytes;
    uint32_t hw_magic, hw_shift;
    float factor;
    int pre;              // y = act(conv + bias + factor * y) (Epilogue::accumulate_first)
    int clamp;            // 0: identity
    float clamp_lo, clamp_hi;
};

template <int PX>
struct PwB {
    float v[PX];
};

template <int PX>
__device__ __forceinline__ PwB<PX> pw_load(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff)
{
    PwB<PX> b;
    if constexpr (PX == 4) {
        const pw_f32x4 t = __builtin_bit_cast(pw_f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
        b.v[0] = t[0], b.v[1] = t[1], b.v[2] = t[2], b.v[3] = t[3];
    } else
        b.v[0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
    return b;
}

// PX: pixels per lane (1, 4); MTW: 32-row blocks per wavefront; MS: slices of the output channels among the wavefronts
template <int PX, int MTW, int MS>
__global__ __launch_bounds__(kPwThreads) void conv_pointwise_f32_kernel(PwArgs a)
{
    static_assert(MS == 1 || MS == 2 || MS == 4, "wavefront split");
    constexpr int MPAD = 32 * MTW * MS;             // rows of the filter chunk
    constexpr int PT = 4 / MS;                       // pixel tiles per workgroup
    constexpr int TILE = 32 * PX;                    // pixels per pixel tile
    constexpr int A_F4 = MPAD * kPwChunk / 4;        // 16-byte pieces of a filter chunk
    constexpr int A_LD = (A_F4 + kPwThreads - 1) / kPwThreads;
    constexpr int kPwDepth = PX == 1 ? DLP_PW_DEPTH1 : DLP_PW_DEPTH4; // channel pairs in flight per wavefront
    __shared__ float As[2][kPwChunk][MPAD];
    __shared__ float bias_s[MPAD];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, h = lane >> 5;
    const int ms = wave % MS, pt = wave / MS;
    const int n0 = ((int)blockIdx.x * PT + pt) * TILE + l32 * PX; // this lane's first pixel

    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, a.w_bytes, 0x00020000);

    // ---- X: byte offset of (image, channel h, pixel) for this lane; a pair of channels further is 2 * HW * 4 bytes on ----
    const int b_img = (int)fast_div((uint32_t)n0, a.hw_magic, a.hw_shift);
    const int pix = n0 - b_img * a.HW;
    const uint32_t xvoff = n0 < a.N ? (uint32_t)(((b_img * a.K + h) * a.HW + pix) * 4) : kPwOutOfRange;
    const uint32_t pair_bytes = (uint32_t)(2 * a.HW * 4);
    const int npairs = a.K / 2;

    // ---- filter chunk loader: thread (m = t % MPAD, c4 = t / MPAD) takes W[m][c0 + 4 c4 .. + 3] and scatters the four values down
    //      a column of the [k][m] chunk (consecutive lanes, consecutive m: no bank conflicts) ----
    pw_f32x4 ra[A_LD];
    auto load_chunk = [&](int c0) {
#pragma unroll
        for (int q = 0; q < A_LD; q++) {
            const int t = tid + q * kPwThreads;
            const int m = t % MPAD, c = c0 + 4 * (t / MPAD);
            const bool ok = (A_F4 % kPwThreads == 0 || t < A_F4) && m < a.M && c < a.K;
            ra[q] = __builtin_bit_cast(pw_f32x4, __builtin_amdgcn_raw_buffer_load_b128(wr, ok ? (uint32_t)((m * a.K + c) * 4) : kPwOutOfRange, 0, 0));
        }
    };
    auto store_chunk = [&](int buf) {
#pragma unroll
        for (int q = 0; q < A_LD; q++) {
            const int t = tid + q * kPwThreads;
            if (A_F4 % kPwThreads == 0 || t < A_F4) {
                const int m = t % MPAD, k4 = 4 * (t / MPAD);
#pragma unroll
                for (int e = 0; e < 4; e++)
                    As[buf][k4 + e][m] = ra[q][e];
            }
        }
    };

    pw_f32x16 acc[MTW][PX];
#pragma unroll
    for (int i = 0; i < MTW; i++)
#pragma unroll
        for (int j = 0; j < PX; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[i][j][r] = 0.0f;

    // ---- prologue: the first channel pairs of X and the first filter chunk ----
    PwB<PX> fb[kPwDepth];
#pragma unroll
    for (int d = 0; d < kPwDepth; d++)
        fb[d] = pw_load<PX>(xr, xvoff, (uint32_t)min(d, npairs - 1) * pair_bytes);
    load_chunk(0);
    if (tid < MPAD) // the bias waits in LDS for the epilogue: a global load per output row there would cost its latency sixteen times
        bias_s[tid] = (a.bias && tid < a.M) ? a.bias[tid] : 0.0f;
    store_chunk(0);
    __syncthreads();

    const int nchunks = (a.K + kPwChunk - 1) / kPwChunk;
    for (int ch = 0; ch < nchunks; ch++) {
        const int buf = ch & 1;
        const int c0 = ch * kPwChunk;
        const int pairs = min(kPwChunk, a.K - c0) / 2; // a multiple of 8: K is a multiple of 16
        if (ch + 1 < nchunks)
            load_chunk(c0 + kPwChunk);
        // The filter operands are read from LDS eight pairs at a time: a ds_read right in front of its matrix instruction exposes the LDS
        // latency in every step (measured: 170 to 210 instead of 64 clocks per step), eight in flight expose it once per eight steps.
        constexpr int G = 8;
        float fa[G][MTW];
        for (int p0 = 0; p0 < pairs; p0 += kPwDepth) {
#pragma unroll
            for (int d = 0; d < kPwDepth; d++) {
                const int p = p0 + d;           // pair inside the chunk: channels c0 + 2 p, c0 + 2 p + 1
                if (d % G == 0) {
                    if (p >= pairs)             // uniform: only the last chunk of a K that is no multiple of 2 * kPwDepth stops early (pairs % 8 == 0)
                        break;
#pragma unroll
                    for (int e = 0; e < G; e++)
#pragma unroll
                        for (int i = 0; i < MTW; i++)
                            fa[e][i] = As[buf][2 * (p + e) + h][(ms * MTW + i) * 32 + l32];
                }
                const int gp = c0 / 2 + p;      // pair of the tensor
                const PwB<PX> cur = fb[d];
                // the pair kPwDepth further on takes this register (pairs past the end re-read the last one and are never multiplied)
                fb[d] = pw_load<PX>(xr, xvoff, (uint32_t)min(gp + kPwDepth, npairs - 1) * pair_bytes);
#pragma unroll
                for (int i = 0; i < MTW; i++)
#pragma unroll
                    for (int j = 0; j < PX; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[d % G][i], cur.v[j], acc[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0); // keep every load where it is: right behind the use of its register, kPwDepth pairs ahead of its own
            }
        }
        if (ch + 1 < nchunks) {
            store_chunk(buf ^ 1); // nobody reads that buffer: its chunk was finished before the previous barrier
            __syncthreads();
        }
    }

    // ---- epilogue: accumulator register r of block (i, j) is row 32 * (ms * MTW + i) + 8 * (r / 4) + 4 * h + r % 4, pixel n0 + j ----
    const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc(a.y, 0, a.y_bytes, 0x00020000);
    const bool use_old = a.factor != 0.0f;
    const bool pre = a.pre != 0 && use_old;
    const uint32_t yvoff = n0 < a.N ? (uint32_t)((b_img * a.M * a.HW + pix) * 4) : kPwOutOfRange;
#pragma unroll
    for (int i = 0; i < MTW; i++) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int m = (ms * MTW + i) * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
            if (m >= a.M)
                continue;
            const float bias = bias_s[m];
            const uint32_t voff = yvoff == kPwOutOfRange ? kPwOutOfRange : yvoff + (uint32_t)(m * a.HW * 4);
            PwB<PX> old;
            if (use_old)
                old = pw_load<PX>(yr, voff, 0);
            float v[PX];
#pragma unroll
            for (int j = 0; j < PX; j++) {
                v[j] = acc[i][j][r] + bias;
                if (pre)
                    v[j] = fmaf(old.v[j], a.factor, v[j]);
                const float c = clamp_med3(v[j], a.clamp_lo, a.clamp_hi);
                v[j] = a.clamp ? c : v[j]; // identity keeps NaNs: no clamp
                if (use_old && !pre)
                    v[j] = fmaf(old.v[j], a.factor, v[j]);
            }
            if constexpr (PX == 4)
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(__attribute__((ext_vector_type(4))) uint32_t, (pw_f32x4){v[0], v[1], v[2], v[3]}), yr,
                                                       voff, 0, PW_STORE_AUX);
            else
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v[0]), yr, voff, 0, 0);
        }
    }
}

struct PwShape {
    int px, mtw, ms;
};

// How the wavefronts are cut for a layer: enough wavefront tasks for the chip (about one per SIMD), wide loads when there are
// pixels to spare.
PwShape pw_shape(const ConvGeom &g)
{
    const long long N = (long long)g.B * g.H * g.W;
    const int mblocks = (g.Cout + 31) / 32;
    PwShape s;
    s.px = ((g.H * g.W) % 4 == 0 && N / 128 >= 1024) ? 4 : 1;
    if (mblocks == 1) {
        s.ms = 1;
        s.mtw = 1;
    } else if (N / (32 * s.px) * 1 >= 1536) { // many pixel tiles: every wavefront takes all rows of its own
        s.ms = 1;
        s.mtw = mblocks;
    } else { // few pixel tiles: the wavefronts share one and split the rows
        s.ms = mblocks <= 2 ? 2 : 4;
        s.mtw = 1;
    }
    return s;
}

} // namespace

bool conv_pointwise_supported(const ConvGeom &g, int activation)
{
    if (g.dtype != DLP_FLOAT || g.KH != 1 || g.KW != 1 || g.sh != 1 || g.sw != 1 || g.ph != 0 || g.pw != 0 || g.groups != 1)
        return false;
    if (activation == DLP_ACT_TANH || activation == DLP_ACT_SIGMOID)
        return false;
    if (g.Cin % 16 != 0 || g.Cout > 128)
        return false;
    const PwShape s = pw_shape(g);
    return s.px == 4 && s.mtw == 1 && s.ms == 1;
}

int conv_pointwise_launch(const ConvGeom &g, const void *x, const void *w, void *y, const Epilogue &ep, hipStream_t stream)
{
    DLP_REQUIRE(conv_pointwise_supported(g, ep.activation), "geometry is not served by the pointwise kernel");
    DLP_REQUIRE((((uintptr_t)x | (uintptr_t)w | (uintptr_t)y) & 15) == 0, "pointwise kernel: tensors must be 16-byte aligned");
    if (g.B == 0)
        return DLP_OK;
    const size_t HW = (size_t)g.H * g.W;
    const size_t x_bytes = (size_t)g.B * g.Cin * HW * 4, y_bytes = (size_t)g.B * g.Cout * HW * 4;
    if (x_bytes >= kPwOutOfRange || y_bytes >= kPwOutOfRange)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "tensors of 2 GiB or more are not supported by the 32-bit buffer addressing");
    const PwShape s = pw_shape(g);
    PwArgs a;
    a.x = (const float *)x;
    a.w = (const float *)w;
    a.bias = ep.bias;
    a.y = (float *)y;
    a.M = g.Cout;
    a.K = g.Cin;
    a.HW = (int)HW;
    a.N = (int)(g.B * HW);
    a.mpad = 32 * s.mtw * s.ms;
    a.x_bytes = (uint32_t)x_bytes;
    a.y_bytes = (uint32_t)y_bytes;
    a.w_bytes = (uint32_t)((size_t)g.Cout * g.Cin * 4);
    make_magic((uint32_t)HW, a.hw_magic, a.hw_shift);
    a.factor = ep.factor;
    a.pre = ep.accumulate_first;
    a.clamp = ep.activation != DLP_ACT_IDENTITY;
    a.clamp_lo = 0.0f;
    a.clamp_hi = ep.activation == DLP_ACT_RELU6 ? 6.0f : __builtin_huge_valf();
    const int per_wg = 32 * s.px * (4 / s.ms); // pixels per workgroup
    const dim3 grid((unsigned)((a.N + per_wg - 1) / per_wg)), block(kPwThreads);
    TimingScope ts("conv_gemm", stream);
#define DLP_PW_CASE(PX, MTW, MS)                                                                                         \
    if (s.px == PX && s.mtw == MTW && s.ms == MS) {                                                                      \
        DLP_LAUNCH_TIMED(ts, (conv_pointwise_f32_kernel<PX, MTW, MS>), grid, block, 0, stream, a);                       \
        DLP_HIP_TRY(hipGetLastError());                                                                                  \
        return DLP_OK;                                                                                                   \
    }
    DLP_PW_CASE(4, 1, 1)
#undef DLP_PW_CASE
    return fail(DLP_ERR_RUNTIME, "pointwise kernel: no instantiation for this shape");
}

} // namespace dlp
