// Depthwise 3x3 convolution followed by a pointwise (1x1) convolution in ONE launch, fp32:
//   t[b][c]   = act1(depthwise3x3(x[b][c]) + bd[c])            (stride 1 or 2, padding 1, never written to memory)
//   y[b][m]   = act2(sum_c wp[m][c] * t[b][c] + bp[m])          (M <= 128 filters)
// the pair of layers a MobileNet block ends in (reference: two operators, Conv2DForward "depthwise_separable",
// src/core/conv.cpp:436-510 with depthwise_separable_conv.cl:20-105, then the 1x1 fast path of the GEMM, src/core/conv.cpp:45-111).
// Run separately both layers sit on the bandwidth leg of the roofline and the tensor between them, as large as x,
// is written once and read once; fused, that tensor never leaves the compute unit.
//
//  * A workgroup takes a band of R output rows of one image and walks the channels in chunks of CK.  The input rows of a chunk
//    that the band needs ((R - 1) * stride + 3 rows per channel) travel global -> registers -> LDS in 16-byte pieces; a chunk
//    stays in registers for two iterations, so its loads have two iterations to arrive.  An LDS row has four zero columns in
//    front of the image row (pitch = compile-time constant >= W + 4): the left padding of one row and the right padding of the
//    row before it, so the taps need no column test; padding rows arrive as zeros because their loads are sent out of range.
//  * Every iteration runs two stages on different chunks, with one barrier: the depthwise stage (all threads; a work item is 4
//    neighbouring outputs of one channel: three LDS reads per input row, 36 multiply-adds in the reference's order -- bias first,
//    then the taps row by row -- so t is bit for bit what the depthwise operator alone writes) leaves chunk c + 1 in LDS as
//    [channel][pixel of the band]; the matrix stage multiplies chunk c: that layout IS the B operand of v_mfma_f32_32x32x2_f32
//    (lane (pixel n, half h) reads t[2p + h][n]), the A operand is the pointwise filter, transposed to [c][m] in LDS chunk by
//    chunk.  The pointwise sum runs over channel pairs in order, accumulated in fp32 on the matrix cores.
//  * Small images leave few pixels per compute unit: KS wavefronts then share a set of 32 pixels and split the channel pairs of a
//    chunk among them; their accumulators are added in wavefront order through LDS at the end (deterministic).
#include "dlp_internal.hpp"

#include <algorithm>
#include <type_traits>

namespace dlp {

typedef float dp_f32x16 __attribute__((ext_vector_type(16)));
typedef float dp_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t dp_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t dp_u32x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr uint32_t kDpOutOfRange = 0x80000000u;
constexpr int kDpKw = 12; // floats per channel of the depthwise filter table in LDS: 9 taps, bias, 2 unused (three 16-byte reads)

struct DwPwArgs {
    const float *x, *wd, *bd, *wp, *bp; // input, depthwise filter [C][3][3], its bias or null, pointwise filter [M][C], its bias or null
    float *y;
    int C, H, W, OH, OW, M;
    int nbands, ntiles;                 // bands per image, bands in all
    uint32_t x_img_bytes, y_img_bytes, wp_bytes;
    uint32_t nb_magic, nb_shift;        // divisions by launch-time constants: bands per image,
    uint32_t pc_magic, pc_shift;        // pieces per channel of a patch (rows x pieces per row),
    uint32_t wp_magic, wp_shift;        // pieces per row,
    uint32_t ic_magic, ic_shift;        // depthwise work items per channel (R x items per row),
    uint32_t qw_magic, qw_shift;        // items per row
    int clamp1;
    float lo1, hi1;                     // activation of the depthwise layer as a clamp (clamp1 = 0: identity)
    int clamp2;
    float lo2, hi2;                     // activation of the pointwise layer
    float factor;
    int pre;                            // y = act2(conv + bias + factor * y)
};

template <int PB>
struct DpPiece;
template <>
struct DpPiece<16> {
    typedef dp_u32x4 type;
    static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, uint32_t v, uint32_t s) { return __builtin_bit_cast(type, __builtin_amdgcn_raw_buffer_load_b128(r, v, s, 0)); }
};
// S: stride; PITCH: floats per LDS row of the input patch; R: output rows per band; CK: channels per chunk; NSG x NS sets of 32
// pixels per band (NS per wavefront); KS: wavefronts that share a set and split the channel pairs; MTW: blocks of 32 filters;
// PB: bytes per global load; PXI: output pixels per depthwise work item (4 or 2 neighbours in a row)
template <int S, int PITCH, int R, int CK, int NSG, int NS, int KS, int MTW, int PB, int PXI>
__global__ __launch_bounds__(NSG *KS * 64) void conv_dwpw_f32_kernel(DwPwArgs a)
{
    constexpr int NW = NSG * KS, NT = NW * 64;
    constexpr int PR = (R - 1) * S + 3;  // patch rows per channel
    constexpr int CHS = PR * PITCH;      // floats per channel of a patch
    constexpr int PATCH = CK * CHS;      // floats per patch buffer
    constexpr int TP = NSG * NS * 32;    // floats per channel of the depthwise result
    constexpr int TBUF = CK * TP;
    constexpr int MPAD = 32 * MTW;
    constexpr int WPMAX = (PITCH - 4) * 4 / PB;
    constexpr int NP = (CK * PR * WPMAX + NT - 1) / NT; // pieces per thread and chunk, at most
    constexpr int QWMAX = (((PITCH - 4) + S - 1) / S + PXI - 1) / PXI;
    constexpr int NI = (CK * R * QWMAX + NT - 1) / NT;  // depthwise work items per thread and chunk, at most
    constexpr int NIN = (PXI - 1) * S + 3;              // input columns of a work item
    constexpr int NSTEP = CK / 2 / KS;                  // channel pairs per wavefront and chunk
    constexpr int RED = KS > 1 ? NSG * (KS - 1) * 16 * 64 : 0;
    constexpr int PATCH_ALL = (2 * PATCH + 4 > RED ? 2 * PATCH + 4 : RED);
    static_assert((PXI == 4 || (PXI == 2 && S == 2)) && PB == 16, "depthwise work items of 4 pixels, or of 2 at stride 2; 16-byte loads");
    static_assert(CK % (2 * KS) == 0, "the wavefronts of a set split the channel pairs of a chunk evenly");
    static_assert(CK * 10 <= NT, "depthwise filter chunk: one load per thread");
    static_assert((2 * PATCH + 4 + 2 * TBUF + 3 * CK * MPAD + 2 * CK * kDpKw) * 4 < 65536, "LDS offsets must fit the 16-bit immediate field");
    typedef typename DpPiece<PB>::type piece_t;

    __shared__ __attribute__((aligned(16))) float lds_patch[PATCH_ALL];  // two input patches [channel][row][PITCH] (later: the accumulator exchange)
    __shared__ __attribute__((aligned(16))) float lds_t[2 * TBUF];       // two depthwise results [channel][pixel of the band]
    __shared__ __attribute__((aligned(16))) float lds_a[3 * CK * MPAD];  // three pointwise filter chunks [channel][filter]
    __shared__ __attribute__((aligned(16))) float lds_k[2 * CK * kDpKw]; // two depthwise filter chunks [channel][9 taps, bias, -, -]
    __shared__ float bias_s[MPAD];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, h = lane >> 5;
    const int wk = wave % KS, wsg = wave / KS;

    // bands in (image, band) order; each XCD (workgroup id modulo 8) walks one contiguous eighth of them, so the bands of an
    // image, which share halo rows, meet in one L2
    const int per = (a.ntiles + 7) >> 3;
    const int tile = ((int)blockIdx.x & 7) * per + ((int)blockIdx.x >> 3);
    if (tile >= a.ntiles)
        return;
    const int b = (int)fast_div((uint32_t)tile, a.nb_magic, a.nb_shift);
    const int band = tile - b * a.nbands;
    const int oy0 = band * R;
    const int rows = min(R, a.OH - oy0);
    const int npx = rows * a.OW;
    const int iy0 = oy0 * S - 1;
    const int prows = (rows - 1) * S + 3;
    const int OHW = a.OH * a.OW;

    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void *)(a.x + (size_t)b * a.C * a.H * a.W), 0, a.x_img_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)a.wp, 0, a.wp_bytes, 0x00020000);

    // ---- this thread's pieces of a chunk: offsets inside the image (chunk-invariant), position in the LDS patch ----
    uint32_t gv[NP];
    int lo[NP];
    {
        const int WP = a.W * 4 / PB, per_ch = PR * WP;
#pragma unroll
        for (int i = 0; i < NP; i++) {
            const int q = tid + i * NT;
            const int ch = (int)fast_div((uint32_t)q, a.pc_magic, a.pc_shift), rem = q - ch * per_ch;
            const int row = (int)fast_div((uint32_t)rem, a.wp_magic, a.wp_shift), cp = rem - row * WP;
            const int iy = iy0 + row;
            const bool valid = ch < CK;
            const bool in = valid && row < prows && iy >= 0 && iy < a.H;
            gv[i] = in ? (uint32_t)(((ch * a.H + iy) * a.W) * 4 + cp * PB) : kDpOutOfRange;
            lo[i] = valid ? ((ch * PR + row) * PITCH + 4) * 4 + cp * PB : -1;
        }
    }
    const uint32_t ch_bytes = (uint32_t)(a.H * a.W * 4);
    // pointwise filter chunk: thread (m = t % MPAD, k4 = t / MPAD) takes wp[m][c0 + 4 k4 ..], scattered down a column of [c][m]
    constexpr int A_F4 = MPAD * CK / 4, A_LD = (A_F4 + NT - 1) / NT;
    uint32_t av[A_LD];
#pragma unroll
    for (int q = 0; q < A_LD; q++) {
        const int t = tid + q * NT, am = t % MPAD, ak = (t / MPAD) * 4;
        av[q] = (t < A_F4 && am < a.M) ? (uint32_t)((am * a.C + ak) * 4) : kDpOutOfRange;
    }
    // depthwise filter chunk: thread (channel t / 10, j = t % 10): tap j or the bias
    const int kc = tid / 10, kj = tid - kc * 10;
    const bool k_thread = tid < CK * 10;

    // two register sets: a chunk is in flight for two iterations before it is stored to LDS
    piece_t pr[2][NP];
    dp_f32x4 ra[2][A_LD];
    float rk[2];
    auto load_chunk = [&](auto set_c, int c0) {
        constexpr int SET = decltype(set_c)::value;
        const uint32_t soff = (uint32_t)c0 * ch_bytes;
#pragma unroll
        for (int i = 0; i < NP; i++)
            pr[SET][i] = DpPiece<PB>::load(xr, gv[i], soff);
#pragma unroll
        for (int q = 0; q < A_LD; q++)
            ra[SET][q] = __builtin_bit_cast(dp_f32x4, __builtin_amdgcn_raw_buffer_load_b128(wr, av[q], (uint32_t)c0 * 4u, 0));
        rk[SET] = 0.0f;
        if (k_thread)
            rk[SET] = kj < 9 ? a.wd[(c0 + kc) * 9 + kj] : (a.bd ? a.bd[c0 + kc] : 0.0f);
    };
    // SET: register set = patch and depthwise filter buffer (0, 1); abuf: pointwise filter buffer (0, 1, 2)
    auto store_chunk = [&](auto set_c, int abuf) {
        constexpr int SET = decltype(set_c)::value;
        char *pb = reinterpret_cast<char *>(lds_patch + SET * PATCH);
#pragma unroll
        for (int i = 0; i < NP; i++)
            if (lo[i] >= 0)
                *reinterpret_cast<piece_t *>(pb + lo[i]) = pr[SET][i];
#pragma unroll
        for (int q = 0; q < A_LD; q++) {
            const int t = tid + q * NT, am = t % MPAD, ak = (t / MPAD) * 4;
            if (A_F4 % NT == 0 || t < A_F4) {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    lds_a[(abuf * CK + ak + e) * MPAD + am] = ra[SET][q][e];
            }
        }
        if (k_thread)
            lds_k[(SET * CK + kc) * kDpKw + kj] = rk[SET];
    };

    // ---- depthwise work items of this thread: (channel of the chunk, row of the band, group of PXI columns), chunk-invariant ----
    int it_in[NI], it_out[NI], it_k[NI];
    {
        const int QW = a.OW / PXI, per_ch = R * QW;
#pragma unroll
        for (int i = 0; i < NI; i++) {
            const int it = tid + i * NT;
            const int ch = (int)fast_div((uint32_t)it, a.ic_magic, a.ic_shift), rem = it - ch * per_ch;
            const int r = (int)fast_div((uint32_t)rem, a.qw_magic, a.qw_shift), q = rem - r * QW;
            const bool valid = ch < CK && r < rows;
            it_in[i] = valid ? (ch * PR + r * S) * PITCH + q * PXI * S + 3 : -1;
            it_out[i] = ch * TP + r * a.OW + q * PXI;
            it_k[i] = ch * kDpKw;
        }
    }
    const bool clamp1 = a.clamp1 != 0;
    // the depthwise convolution of the chunk in patch buffer BUF -> lds_t[BUF]; the reference's operation order
    auto depthwise = [&](auto buf_c) {
        constexpr int BUF = decltype(buf_c)::value;
#pragma unroll
        for (int i = 0; i < NI; i++) {
            if (it_in[i] < 0)
                continue;
            const float *kp = lds_k + BUF * CK * kDpKw + it_k[i];
            const dp_f32x4 k0 = *reinterpret_cast<const dp_f32x4 *>(kp), k1 = *reinterpret_cast<const dp_f32x4 *>(kp + 4),
                           k2 = *reinterpret_cast<const dp_f32x4 *>(kp + 8);
            const float k[9] = {k0[0], k0[1], k0[2], k0[3], k1[0], k1[1], k1[2], k1[3], k2[0]};
            const float *p = lds_patch + BUF * PATCH + it_in[i];
            float v[3][NIN];
#pragma unroll
            for (int dr = 0; dr < 3; dr++) {
                const float *row = p + dr * PITCH;
                v[dr][0] = row[0];
#pragma unroll
                for (int g = 0; g < (NIN - 1) / 4; g++) { // aligned groups of four
                    const dp_f32x4 m = *reinterpret_cast<const dp_f32x4 *>(row + 1 + 4 * g);
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        v[dr][1 + 4 * g + e] = m[e];
                }
                if constexpr ((NIN - 1) % 4 != 0)
                    v[dr][NIN - 1] = row[NIN - 1];
            }
            float o[PXI];
#pragma unroll
            for (int e = 0; e < PXI; e++) {
                float sum = k2[1]; // the bias
#pragma unroll
                for (int dr = 0; dr < 3; dr++)
#pragma unroll
                    for (int dc = 0; dc < 3; dc++)
                        sum = fmaf(k[dr * 3 + dc], v[dr][e * S + dc], sum);
                const float clamped = clamp_med3(sum, a.lo1, a.hi1);
                o[e] = clamp1 ? clamped : sum; // identity keeps NaNs: no clamp
            }
            float *out = lds_t + BUF * TBUF + it_out[i];
            if constexpr (PXI == 4)
                *reinterpret_cast<dp_f32x4 *>(out) = (dp_f32x4){o[0], o[1], o[2], o[3]};
            else
                *reinterpret_cast<float2 *>(out) = make_float2(o[0], o[1]);
        }
    };

    // ---- this lane's pixels in the matrix stage: set (wsg * NS + j), pixel l32 of it ----
    bool pvalid[NS];
#pragma unroll
    for (int j = 0; j < NS; j++)
        pvalid[j] = (wsg * NS + j) * 32 + l32 < npx;
    const int tbase = (2 * wk + h) * TP + wsg * NS * 32 + l32;
    const int abase = (2 * wk + h) * MPAD + l32;

    dp_f32x16 acc[NS][MTW];
#pragma unroll
    for (int j = 0; j < NS; j++)
#pragma unroll
        for (int i = 0; i < MTW; i++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[j][i][r] = 0.0f;

    // the pointwise product of the chunk whose depthwise result is in lds_t[BUF] and whose filter chunk is lds_a[abuf]
    auto pointwise = [&](auto buf_c, int abuf) {
        constexpr int BUF = decltype(buf_c)::value;
        const float *ap = lds_a + abase + abuf * CK * MPAD;
#pragma unroll
        for (int s = 0; s < NSTEP; s++) {
            float fa[MTW];
#pragma unroll
            for (int i = 0; i < MTW; i++)
                fa[i] = ap[2 * KS * s * MPAD + i * 32];
#pragma unroll
            for (int j = 0; j < NS; j++) {
                const float t = lds_t[tbase + BUF * TBUF + 2 * KS * s * TP + j * 32];
#pragma unroll
                for (int i = 0; i < MTW; i++)
                    acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], t, acc[j][i], 0, 0, 0);
            }
        }
    };

    // ---- prologue: chunk 0 through the depthwise stage, chunk 1 in its patch buffer, chunk 2 on its way ----
    const int nch = a.C / CK;
    using B0 = std::integral_constant<int, 0>;
    using B1 = std::integral_constant<int, 1>;
    load_chunk(B0{}, 0);
    if (nch > 1)
        load_chunk(B1{}, CK);
    for (int i = tid; i < (2 * PATCH + 4) / 4; i += NT)
        reinterpret_cast<dp_f32x4 *>(lds_patch)[i] = (dp_f32x4){0.0f, 0.0f, 0.0f, 0.0f};
    if (tid < MPAD)
        bias_s[tid] = (a.bp && tid < a.M) ? a.bp[tid] : 0.0f;
    __syncthreads();
    store_chunk(B0{}, 0);
    if (nch > 2)
        load_chunk(B0{}, 2 * CK);
    __syncthreads();
    depthwise(B0{});
    if (nch > 1)
        store_chunk(B1{}, 1);
    __syncthreads();

    // ---- iteration c: chunk c + 3 leaves memory, chunk c + 2 (loaded an iteration ago) goes to LDS at the end, chunk c + 1 goes
    //      through the depthwise stage, chunk c through the matrix stage; one barrier.  Register sets, patch, depthwise-filter and
    //      result buffers alternate; the pointwise filter chunk lives three iterations ----
    int abuf = 0; // c % 3
    auto iteration = [&](int c, auto buf_c) {
        constexpr int BUF = decltype(buf_c)::value; // c & 1
        using Other = std::integral_constant<int, BUF ^ 1>;
        if (c + 3 < nch)
            load_chunk(Other{}, (c + 3) * CK);
        if (c + 1 < nch)
            depthwise(Other{});
        pointwise(buf_c, abuf);
        if (c + 2 < nch)
            store_chunk(buf_c, abuf == 0 ? 2 : abuf - 1); // (c + 2) % 3
        if (c + 1 < nch)
            __syncthreads();
        abuf = abuf == 2 ? 0 : abuf + 1;
    };
    for (int c = 0; c < nch; c += 2) {
        iteration(c, B0{});
        if (c + 1 < nch)
            iteration(c + 1, B1{});
    }

    // ---- the wavefronts of a set add their accumulators: one 32 x 32 block at a time through LDS, in wavefront order ----
    if constexpr (KS > 1) {
#pragma unroll
        for (int j = 0; j < NS; j++)
#pragma unroll
            for (int i = 0; i < MTW; i++) {
                __syncthreads(); // the patch (first round) or the previous block has been read by everybody
                if (wk > 0) {
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        lds_patch[((wsg * (KS - 1) + wk - 1) * 16 + r) * 64 + lane] = acc[j][i][r];
                }
                __syncthreads();
                if (wk == 0) {
#pragma unroll
                    for (int q = 0; q < KS - 1; q++)
#pragma unroll
                        for (int r = 0; r < 16; r++)
                            acc[j][i][r] += lds_patch[((wsg * (KS - 1) + q) * 16 + r) * 64 + lane];
                }
            }
        if (wk > 0)
            return;
    }

    // ---- epilogue: accumulator register r of block (j, i) is filter 32 i + 8 (r / 4) + 4 h + r % 4 at pixel (set j, l32) ----
    const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc(a.y + (size_t)b * a.M * OHW, 0, a.y_img_bytes, 0x00020000);
    const bool use_old = a.factor != 0.0f;
    const bool pre = a.pre != 0 && use_old;
    const bool clamp2 = a.clamp2 != 0;
#pragma unroll
    for (int j = 0; j < NS; j++) {
        const int p = (wsg * NS + j) * 32 + l32;
        const uint32_t pv = pvalid[j] ? (uint32_t)((oy0 * a.OW + p) * 4) : kDpOutOfRange;
#pragma unroll
        for (int i = 0; i < MTW; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = i * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                const uint32_t voff = (m < a.M && pvalid[j]) ? pv + (uint32_t)(m * OHW * 4) : kDpOutOfRange;
                float v = acc[j][i][r] + bias_s[m];
                float old = 0.0f;
                if (use_old)
                    old = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(yr, voff, 0, 0));
                if (pre)
                    v = fmaf(old, a.factor, v);
                const float c = clamp_med3(v, a.lo2, a.hi2);
                v = clamp2 ? c : v;
                if (use_old && !pre)
                    v = fmaf(old, a.factor, v);
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), yr, voff, 0, 0);
            }
        }
    }
}

// LDS bytes of a kernel instance (the same sum as in the kernel)
constexpr int dp_lds_bytes(int S, int PITCH, int R, int CK, int NSG, int NS, int MTW)
{
    return (2 * CK * ((R - 1) * S + 3) * PITCH + 4 + 2 * CK * NSG * NS * 32 + 3 * CK * 32 * MTW + 2 * CK * kDpKw + 32 * MTW) * 4;
}

// How a geometry is cut: one row per kernel variant
struct DpVariant {
    int S, PITCH, R, CK, NSG, NS, KS, PB, PXI;
};
// index, S, PITCH, R, CK, NSG, NS, KS, PB, PXI; the first row that fits is taken.  Chosen by timing the MobileNet pairs at batch 64
// (cold tensors, back-to-back launches): bands of few rows and several wavefronts per set keep enough workgroups on every CU.
#define DLP_DP_ROWS(X) \
    X(0, 1, 32, 4, 16, 4, 1, 2, 16, 4) /* stride 1, images up to 28 wide (192 -> 32 at 28 x 28: 23 us, the two operators 30 us) */ \
    X(1, 1, 32, 4, 8, 4, 1, 2, 16, 4)  /* ... channels a multiple of 8 only, or more than 96 filters */ \
    X(2, 1, 60, 8, 4, 7, 2, 1, 16, 4)  /* stride 1, up to 56 wide (144 -> 24 at 56 x 56: 53 us against 75 us) */ \
    X(3, 2, 32, 4, 16, 2, 1, 8, 16, 2) /* stride 2, up to 28 wide (192 -> 64 at 28 x 28: 22 us against 23 us) */ \
    X(4, 2, 32, 4, 8, 2, 1, 4, 16, 2)  /* ... channels a multiple of 8 only, or more than 96 filters */ \
    X(5, 2, 60, 4, 8, 4, 1, 2, 16, 4)  /* stride 2, up to 56 wide (144 -> 32 at 56 x 56: 30 us against 43 us) */
#define DLP_DP_TABLE_ROW(V_, S_, PITCH_, R_, CK_, NSG_, NS_, KS_, PB_, PXI_) {S_, PITCH_, R_, CK_, NSG_, NS_, KS_, PB_, PXI_},
constexpr DpVariant kDpVariants[] = {DLP_DP_ROWS(DLP_DP_TABLE_ROW)};
#undef DLP_DP_TABLE_ROW
constexpr int kDpNumVariants = (int)(sizeof(kDpVariants) / sizeof(kDpVariants[0]));

int dp_variant(const ConvGeom &g, int M)
{
    const int mtw = (M + 31) / 32;
    for (int v = 0; v < kDpNumVariants; v++) {
        const DpVariant &d = kDpVariants[v];
        if (g.sh != d.S || g.W + 4 > d.PITCH)
            continue;
        if ((g.W * 4) % d.PB != 0 || ((long long)g.H * g.W * 4) % d.PB != 0)
            continue;
        if (g.Cin % d.CK != 0 || g.OW % d.PXI != 0)
            continue;
        if (dp_lds_bytes(d.S, d.PITCH, d.R, d.CK, d.NSG, d.NS, mtw) >= 65536)
            continue;
        if (std::min(d.R, g.OH) * g.OW > d.NSG * d.NS * 32)
            continue;
        return v;
    }
    return -1;
}

template <int S, int PITCH, int R, int CK, int NSG, int NS, int KS, int MTW, int PB, int PXI>
int dp_launch(TimingScope &ts, dim3 grid, dim3 block, hipStream_t stream, const DwPwArgs &a)
{
    if constexpr (dp_lds_bytes(S, PITCH, R, CK, NSG, NS, MTW) < 65536) {
        DLP_LAUNCH_TIMED(ts, (conv_dwpw_f32_kernel<S, PITCH, R, CK, NSG, NS, KS, MTW, PB, PXI>), grid, block, 0, stream, a);
        DLP_HIP_TRY(hipGetLastError());
        return DLP_OK;
    } else
        return fail(DLP_ERR_RUNTIME, "fused depthwise + pointwise kernel: this variant does not fit the LDS with so many filters");
}

bool clamp_act(int act) { return act == DLP_ACT_IDENTITY || act == DLP_ACT_RELU || act == DLP_ACT_RELU6; }

} // namespace

// g: the depthwise layer (groups = Cin = Cout); M: filters of the pointwise layer
bool conv_dwpw_supported(const ConvGeom &g, int M, int act1, int act2)
{
    if (g.dtype != DLP_FLOAT || g.KH != 3 || g.KW != 3 || g.ph != 1 || g.pw != 1 || g.dh != 1 || g.dw != 1 || g.sh != g.sw)
        return false;
    if (g.groups != g.Cin || g.Cout != g.Cin || M < 1 || M > 128)
        return false;
    if (!clamp_act(act1) || !clamp_act(act2))
        return false;
    // small planes leave a band too little to do per channel chunk: 384 -> 64 at 14 x 14 takes 30 us here, 26 us as two operators
    if (g.H * g.W < 512)
        return false;
    return dp_variant(g, M) >= 0;
}

int conv_dwpw_launch(const ConvGeom &g, int M, const void *x, const void *wd, const float *bd, int act1, const void *wp, void *y, const Epilogue &ep,
                     hipStream_t stream)
{
    DLP_REQUIRE(conv_dwpw_supported(g, M, act1, ep.activation), "geometry is not served by the fused depthwise + pointwise kernel");
    DLP_REQUIRE((((uintptr_t)x | (uintptr_t)wp) & 15) == 0 && ((uintptr_t)y & 3) == 0, "fused depthwise + pointwise kernel: x and the pointwise filter must be 16-byte aligned");
    if (g.B == 0)
        return DLP_OK;
    const size_t x_img = (size_t)g.Cin * g.H * g.W * 4, y_img = (size_t)M * g.OH * g.OW * 4;
    if (x_img >= kDpOutOfRange || y_img >= kDpOutOfRange)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "images of 2 GiB or more are not supported by the 32-bit buffer addressing");
    const int v = dp_variant(g, M);
    const DpVariant &d = kDpVariants[v];
    DwPwArgs a;
    a.x = (const float *)x;
    a.wd = (const float *)wd;
    a.bd = bd;
    a.wp = (const float *)wp;
    a.bp = ep.bias;
    a.y = (float *)y;
    a.C = g.Cin;
    a.H = g.H;
    a.W = g.W;
    a.OH = g.OH;
    a.OW = g.OW;
    a.M = M;
    a.nbands = (g.OH + d.R - 1) / d.R;
    const long long ntiles = (long long)g.B * a.nbands;
    if (ntiles > 0x0fffffff)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "too many bands for one launch");
    a.ntiles = (int)ntiles;
    a.x_img_bytes = (uint32_t)x_img;
    a.y_img_bytes = (uint32_t)y_img;
    a.wp_bytes = (uint32_t)((size_t)M * g.Cin * 4);
    make_magic((uint32_t)a.nbands, a.nb_magic, a.nb_shift);
    const int n_wp = g.W * 4 / d.PB, n_qw = g.OW / d.PXI;
    make_magic((uint32_t)(((d.R - 1) * d.S + 3) * n_wp), a.pc_magic, a.pc_shift);
    make_magic((uint32_t)n_wp, a.wp_magic, a.wp_shift);
    make_magic((uint32_t)(d.R * n_qw), a.ic_magic, a.ic_shift);
    make_magic((uint32_t)n_qw, a.qw_magic, a.qw_shift);
    a.clamp1 = act1 != DLP_ACT_IDENTITY;
    a.lo1 = 0.0f;
    a.hi1 = act1 == DLP_ACT_RELU6 ? 6.0f : __builtin_huge_valf();
    a.clamp2 = ep.activation != DLP_ACT_IDENTITY;
    a.lo2 = 0.0f;
    a.hi2 = ep.activation == DLP_ACT_RELU6 ? 6.0f : __builtin_huge_valf();
    a.factor = ep.factor;
    a.pre = ep.accumulate_first;
    const int mtw = (M + 31) / 32;
    const dim3 grid((unsigned)(((a.ntiles + 7) / 8) * 8)), block((unsigned)(d.NSG * d.KS * 64));
    TimingScope ts("dwpw_fused", stream);
#define DLP_DP_CASE(V_, S_, PITCH_, R_, CK_, NSG_, NS_, KS_, PB_, PXI_, MTW_)                                                       \
    if (v == V_ && mtw == MTW_)                                                                                                     \
        return dp_launch<S_, PITCH_, R_, CK_, NSG_, NS_, KS_, MTW_, PB_, PXI_>(ts, grid, block, stream, a);
#define DLP_DP_VARIANT(V_, S_, PITCH_, R_, CK_, NSG_, NS_, KS_, PB_, PXI_)                                                          \
    DLP_DP_CASE(V_, S_, PITCH_, R_, CK_, NSG_, NS_, KS_, PB_, PXI_, 1)                                                              \
    DLP_DP_CASE(V_, S_, PITCH_, R_, CK_, NSG_, NS_, KS_, PB_, PXI_, 2)                                                              \
    DLP_DP_CASE(V_, S_, PITCH_, R_, CK_, NSG_, NS_, KS_, PB_, PXI_, 3)                                                              \
    DLP_DP_CASE(V_, S_, PITCH_, R_, CK_, NSG_, NS_, KS_, PB_, PXI_, 4)
    DLP_DP_ROWS(DLP_DP_VARIANT)
#undef DLP_DP_VARIANT
#undef DLP_DP_CASE
    return fail(DLP_ERR_RUNTIME, "fused depthwise + pointwise kernel: no instantiation for this shape");
}

} // namespace dlp
