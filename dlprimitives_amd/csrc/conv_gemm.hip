// Implicit-GEMM convolution forward for gfx950 (fp32 MFMA).
//
// Replaces the reference's ConvSGEMM / sgemm.cl CONVGEMM=1 path
// (src/core/conv.cpp:45-111, src/gemm.cpp:429-565, src/kernels/sgemm.cl:75-133,296-715):
//   C[M x N] = W[M x K] * im2col(X)[K x N],  M = Cout/groups, N = B*OH*OW, K = Cin/groups*KH*KW
// with the im2col gather fused into the B-tile load, and bias + activation +
// factor applied in registers before the NCHW store.
//
// Mapping to the hardware:
//  * one workgroup = 4 wavefronts of 64 lanes; each wavefront owns a register
//    tile made of 32x32 v_mfma_f32_32x32x2_f32 blocks.  The pixel dimension N is
//    put on the MFMA column axis, so that the 32 lanes of a half-wave hold 32
//    consecutive output pixels and every store is a 128-byte run in NCHW.
//  * A (weights) and B (gathered input) tiles are staged through LDS in [k][m]
//    and [k][n] order: an MFMA operand fetch is a conflict-free ds_read.
//  * on this chip a vector-ALU instruction takes issue cycles away from the matrix
//    pipe of its SIMD (measured: MFMA time and VALU time add up), so the main loop
//    is built to need almost no VALU work:
//      - every global load is a buffer load whose address is
//        resource base + per-thread VGPR offset (loop invariant) + SGPR offset (per k),
//        the SGPR part coming from a small table read through the scalar unit;
//      - padding and tile tails are handled by swapping the VGPR offset for an
//        out-of-range one, which the buffer load returns as 0.0 (no branches);
//      - K is walked tap-major whenever Cin/groups is a multiple of 16: one K tile =
//        one filter tap x 16 input channels, so the in-image test is one bit test
//        per K tile instead of one per element (the sum over K is order-free).
//        Other shapes (e.g. the 3-channel stem) use a per-element table;
//      - the weights are repacked once per call (a small kernel, like the reference's
//        Winograd filter transform) into the exact [m tile][K tile][k][m] image of the
//        LDS A tile, zero padded: the A load is one coalesced 16-byte load per thread
//        with no masks, whatever the K order.
//  * software pipeline of distance two: tile kt+2 is in flight from memory to
//    registers while tile kt+1 moves registers -> LDS and tile kt feeds the MFMAs.
//  * layers with too few output tiles for 256 CUs split K over several
//    workgroups; partial sums go through the workspace and are reduced in a
//    fixed order by a second kernel (deterministic).
#include "dlp_internal.hpp"

#include <algorithm>
#include <atomic>
#include <type_traits>

namespace dlp {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr int kThreads = 256;
constexpr int BK = 16;
constexpr uint32_t kOutOfRange = 0x80000000u; // >= num_records of every buffer we accept
constexpr int kPatchPitch = 192;               // LDS patch rows of conv_patch_f32_kernel
constexpr int kPatchPitchBf16_128 = 320;       // ... of conv_patch_bf16_kernel with 128-pixel tiles
constexpr int kPatchPitchBf16_256 = 448;       // ... with 256-pixel tiles

enum { ACT_CLAMP = 0, ACT_GENERIC = 1 };

struct GemmArgs {
    const void *x;   // storage type T (float or bf16_t)
    const float *wp; // packed weights, always fp32
    const float *bias;
    void *y;         // storage type T
    const int32_t *ktab;
    int M, N, K, nkt;
    int mtiles, ntiles;
    int splitk, kt_per_slice; // K tiles are dealt to `splitk` slices of kt_per_slice (even) tiles
    // conv_gemm_f32_kernel: the last tail_tiles tiles (m tile fastest, then n tile, then group) are cut into tail_splitk
    // finer slices of tail_kt K tiles, launched as the last workgroups, so that the partial last round of workgroups
    // becomes about one small piece per CU; main_wgs = (tiles - tail_tiles) * splitk workgroups run the other tiles
    int tail_tiles, tail_splitk, tail_kt, main_wgs;
    float *part;              // split-K partial sums [slice][Cout][N]
    int sk_units;             // stream-K (conv_patch_f32_kernel): tiles * stages
    float *sk_part;           // two 64x64 accumulator images per workgroup
    uint32_t sk_part_bytes;
    int *sk_cnt;              // pieces arrived, per tile (zero at launch)
    int sk_tpw, sk_mb;        // tile order of the stream: tiles per workgroup (transposition), m tiles per pixel tile run
    int sk_tiles;             // tiles of the stream (sk_units / stages per tile)
    // divisions of the per-tile decode, as magic numbers (fast_div): they are uniform, and a uniform integer division
    // would otherwise run as some forty vector instructions in every wavefront, next to the matrix instructions
    uint32_t ncb_magic, ncb_shift, nt_magic, nt_shift, tpw_magic, tpw_shift, pg_magic, pg_shift, mbnt_magic, mbnt_shift, mb_magic, mb_shift;
    int pxv;                  // bf16 matrix-instruction kernels: pixels per output store (0 = one element per store)
    int pp_nbr;               // conv_patch_bf16_kernel: blocks of PXP rows in the largest patch of the launch
    int wdirect;              // conv_gemm_bf16_kernel: wp is the weight tensor itself (1x1 convolution), not packed tiles
    int y_cl;                 // bf16 matrix-instruction kernels: y is [image][pixel][channel]
    int Cin, Cin_g, H, W, Cout, OW, OHW, groups;
    int sh, sw, ph, pw, dh, dw, KH, KW;
    uint32_t x_bytes, wp_bytes;
    uint32_t y_bytes; // size of y when it is below 2 GiB (buffer stores), else 0
    uint32_t part_bytes; // likewise for the split-K partial sums
    uint32_t x_shift; // bytes by which the X resource base is moved back (padding offset)
    uint32_t hw4;     // H*W*sizeof(T): byte stride between input channels
    uint32_t ohw_magic, ohw_shift, ow_magic, ow_shift;
    // divisions of the tile decode: by mtiles, ntiles, groups, by the tiles of the main part and of the tail of a split launch
    // (an integer division by a run-time value costs some forty vector instructions, per wavefront, before the first load)
    uint32_t mt_magic, mt_shift, ntl_magic, ntl_shift, gr_magic, gr_shift, tm_magic, tm_shift, tt_magic, tt_shift;
    float factor;
    int pre; // the old value of y is added before the activation (Epilogue::accumulate_first)
    int act;
    float clamp_lo, clamp_hi;
};

typedef __attribute__((address_space(4))) const int32_t ConstInt;

// one storage element, widened to fp32 (bf16 -> fp32 is a 16-bit shift)
template <class T>
__device__ __forceinline__ float buf_load(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff);
template <>
__device__ __forceinline__ float buf_load<float>(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}
template <>
__device__ __forceinline__ float buf_load<bf16_t>(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff)
{
    return __builtin_bit_cast(float, (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, 0) << 16);
}

__device__ __forceinline__ f32x4 buf_load4(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff)
{
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
}

// keep a selected offset one opaque value, so that the select stays a v_cndmask
// instead of being turned into two loads under divergent branches
__device__ __forceinline__ uint32_t opaque(uint32_t v)
{
    asm("" : "+v"(v));
    return v;
}

// call f(integral_constant<int, kk>) for the compile-time value matching the unrolled kk
template <class F>
__device__ __forceinline__ void static_for_slice(int kk, F &&f)
{
    switch (kk) {
    case 0: f(std::integral_constant<int, 0>{}); break;
    case 1: f(std::integral_constant<int, 1>{}); break;
    case 2: f(std::integral_constant<int, 2>{}); break;
    case 3: f(std::integral_constant<int, 3>{}); break;
    case 4: f(std::integral_constant<int, 4>{}); break;
    case 5: f(std::integral_constant<int, 5>{}); break;
    case 6: f(std::integral_constant<int, 6>{}); break;
    default: f(std::integral_constant<int, 7>{}); break;
    }
}
template <class F>
__device__ __forceinline__ void static_for_all(F &&f)
{
    f(std::integral_constant<int, 0>{});
    f(std::integral_constant<int, 1>{});
    f(std::integral_constant<int, 2>{});
    f(std::integral_constant<int, 3>{});
    f(std::integral_constant<int, 4>{});
    f(std::integral_constant<int, 5>{});
    f(std::integral_constant<int, 6>{});
    f(std::integral_constant<int, 7>{});
}

template <class T, int BM, int BN, int WM, int WN, int ACT>
__device__ __forceinline__ void gemm_tile_output(const GemmArgs &a, f32x16 (&acc)[BM / WM / 32][BN / WN / 32], float *lds, int m0, int n0,
                                                 int g, int slice, int splitk, uint32_t image0, int wm, int wn, int h, int l32, int tid,
                                                 const float *bias_s);

// NSET: register sets of tiles in flight = how many K tiles ahead of the matrix instructions the loads are issued.  Two is
// enough when eight workgroups share a CU and cover each other's waits; launches with few workgroups per CU (small layers,
// short K) run four, so that one workgroup alone has four K tiles on their way.
template <class T, int BM, int BN, int WM, int WN, int ORDER, int MASK, int ACT, int NSET = 2>
__global__ __launch_bounds__(kThreads) void conv_gemm_f32_kernel(GemmArgs a)
{
    static_assert(NSET == 2 || NSET == 4, "register sets");
    static_assert(BK == 16, "the slice helpers assume 8 MFMA steps per K tile");
    static_assert(WM * WN == 4, "four wavefronts per workgroup");
    constexpr int WTM = BM / WM, WTN = BN / WN; // wavefront tile
    constexpr int TM = WTM / 32, TN = WTN / 32; // MFMA blocks per wavefront
    static_assert(TM >= 1 && TN >= 1 && WTM % 32 == 0 && WTN % 32 == 0, "tile shape");
    // Unpadded rows: two k steps are then a multiple of 256 bytes apart, so every operand fetch is a
    // ds_read2st64 with immediate offsets (a padded row cost one VALU address add per pair of
    // fetches; the two half-waves of a fetch read different rows in different cycles: no conflicts)
    constexpr int LDA = BM;
    constexpr int LDB = BN;
    constexpr int KSPLIT = kThreads / BN;    // k slices among the B loader threads
    static_assert(KSPLIT >= 1 && BN % 64 == 0 && BK % KSPLIT == 0, "B loader shape");
    constexpr int B_LD = BK / KSPLIT;        // gathered elements per thread per K step (contiguous k)
    constexpr int A_V4 = BM * BK / 4;        // 16-byte pieces of a packed A tile
    constexpr int A_LD = (A_V4 + kThreads - 1) / kThreads; // ... per thread
    static_assert(BM % 4 == 0, "packed A rows are read in 16-byte pieces");

    __shared__ __attribute__((aligned(16))) float As[2][BK][LDA];
    __shared__ float Bs[2][BK][LDB];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int h = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;

    // Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.  Renumber
    // them so that every XCD walks one contiguous range of tiles: the m tiles of one pixel
    // tile, and neighbouring pixel tiles (which share input rows), then hit the same L2.
    int t, slice, splitk = a.splitk, kt_per_slice = a.kt_per_slice;
    uint32_t image0; // index of the tile's first accumulator image in the split-K workspace
    {
        const int tiles = a.mtiles * a.ntiles * a.groups, tiles_main = tiles - a.tail_tiles;
        const int bid = blockIdx.x;
        if (bid < a.main_wgs) {
            const int nb = a.main_wgs;
            const int q = nb >> 3, r = nb & 7;
            const int xcd = bid & 7, slot = bid >> 3;
            t = (xcd < r) ? xcd * (q + 1) + slot : r * (q + 1) + (xcd - r) * q + slot;
            slice = (int)fast_div((uint32_t)t, a.tm_magic, a.tm_shift); // t / tiles_main
            t -= slice * tiles_main;
            image0 = (uint32_t)(t * splitk);
        } else { // finer slices of the last tiles
            t = bid - a.main_wgs;
            slice = (int)fast_div((uint32_t)t, a.tt_magic, a.tt_shift); // t / tail_tiles
            t -= slice * a.tail_tiles;
            image0 = (uint32_t)((splitk > 1 ? tiles_main * splitk : 0) + t * a.tail_splitk);
            t += tiles_main;
            splitk = a.tail_splitk;
            kt_per_slice = a.tail_kt;
        }
    }
    // tile decode: m tile fastest, then n tile, then group
    const int tm = (int)fast_div((uint32_t)t, a.mt_magic, a.mt_shift);
    const int mt = t - tm * a.mtiles;
    const int g = (int)fast_div((uint32_t)tm, a.ntl_magic, a.ntl_shift);
    const int nt = tm - g * a.ntiles;
    const int m0 = mt * BM, n0 = nt * BN;
    const int kt_begin = slice * kt_per_slice;
    const int kt_end = min(kt_begin + kt_per_slice, a.nkt);
    // the bias of the tile's rows, for the epilogue: in LDS long before it is wanted (the barriers of the main loop lie between)
    __shared__ float bias_early[BM];
    if (tid < BM)
        bias_early[tid] = (a.bias && m0 + tid < a.M) ? a.bias[g * a.M + m0 + tid] : 0.0f;

    // The X resource starts one padding offset before the tensor, so that the
    // per-pixel window origin is a non-negative offset; taps that the masks let
    // through never address below the tensor.
    const __amdgpu_buffer_rsrc_t xr =
        __builtin_amdgcn_make_buffer_rsrc((void *)((const char *)a.x - a.x_shift), 0, a.x_bytes + a.x_shift, 0x00020000);
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)a.wp, 0, a.wp_bytes, 0x00020000);
    ConstInt *ktab = (ConstInt *)a.ktab; // read-only, wavefront-uniform index: scalar loads

    // ---- per-thread gather state (one output pixel per thread) ----
    const int p = tid % BN;
    const int ks = (KSPLIT == 1) ? 0 : __builtin_amdgcn_readfirstlane(tid / BN);
    uint32_t vbase;          // byte offset of the window origin from the shifted base
    uint32_t my = 0, mx = 0; // MASK_TAPS: my = tap mask; MASK_ROWCOL: row / column masks
    {
        const int n = n0 + p;
        const bool vn = n < a.N;
        const int b = (int)fast_div((uint32_t)n, a.ohw_magic, a.ohw_shift);
        const int pix = n - b * a.OHW;
        const int oy = (int)fast_div((uint32_t)pix, a.ow_magic, a.ow_shift);
        const int ox = pix - oy * a.OW;
        const int iy0 = oy * a.sh - a.ph;
        const int ix0 = ox * a.sw - a.pw;
        vbase = (uint32_t)((((b * a.Cin + g * a.Cin_g) * a.H + oy * a.sh) * a.W + ox * a.sw) * (int)sizeof(T));
        if (vn) {
            uint32_t ry = 0, rx = 0;
            for (int ky = 0; ky < a.KH; ky++) {
                int yy = iy0 + ky * a.dh;
                if (yy >= 0 && yy < a.H)
                    ry |= 1u << ky;
            }
            for (int kx = 0; kx < a.KW; kx++) {
                int xx = ix0 + kx * a.dw;
                if (xx >= 0 && xx < a.W)
                    rx |= 1u << kx;
            }
            if (MASK == GEMM_MASK_TAPS) {
                for (int ky = 0; ky < a.KH; ky++)
                    if ((ry >> ky) & 1u)
                        my |= rx << (ky * a.KW);
            } else {
                my = ry;
                mx = rx;
            }
        }
    }

    // ---- weight loader: 16-byte pieces of the packed tile, in tile order; or (a.wdirect: 1x1 convolutions, whose K tile
    // is 16 consecutive input channels) of the weight tensor itself: lane m of wavefront q takes channels 4q..4q+3 of
    // filter row m, and the four values go to LDS one by one ----
    const uint32_t a_tile_bytes = BK * BM * 4;
    const bool wdirect = a.wdirect != 0; // uniform
    const uint32_t a_step = wdirect ? (uint32_t)(BK * 4) : a_tile_bytes;                                       // SGPR
    const uint32_t a_row_base = wdirect ? 0u : (uint32_t)((g * a.mtiles + mt) * a.nkt) * a_tile_bytes;         // SGPR
    const bool a_active = (A_V4 >= kThreads) || (tid < A_V4);
    uint32_t a_voff0 = a_active ? (uint32_t)(tid * 16) : kOutOfRange;
    if (wdirect) {
        const int m = tid % BM, kq = tid / BM;
        a_voff0 = (a_active && m0 + m < a.M) ? (uint32_t)(((g * a.M + m0 + m) * a.K + 4 * kq) * 4) : kOutOfRange;
    }

    // Two register sets for staged tiles: tile kt+2 is being fetched from memory
    // into one set while tile kt+1 moves from the other set into LDS and tile kt
    // (already in LDS) feeds the matrix cores.  A global load therefore has a whole
    // K step to land before anything waits on it.
    f32x4 ra[NSET][A_LD];
    float rb[NSET][B_LD];
    uint32_t vsel[NSET]; // GEMM_ORDER_TAP: this tile's (masked) pixel offset
#pragma unroll
    for (int i = 0; i < NSET; i++)
        vsel[i] = kOutOfRange;

    // one slice of the loads of tile kt into register set S: called once per MFMA
    // group so that vector-memory issue is spread under the MFMAs
    auto load_slice = [&](auto set, int kt, auto slice_q) {
        constexpr int S = decltype(set)::value;
        constexpr int Q = decltype(slice_q)::value;
        // tiles fetched past the end of K are never multiplied: re-read the last tile
        const uint32_t a_soff = a_row_base + (uint32_t)min(kt, a.nkt - 1) * a_step;
#pragma unroll
        for (int j = 0; j < A_LD; j++)
            if (j % (BK / 2) == Q)
                ra[S][j] = buf_load4(wr, j == 0 ? a_voff0 : (a_active ? (uint32_t)(tid * 16 + j * kThreads * 16) : kOutOfRange), a_soff);
        // (tiles fetched past the end of K are never multiplied; their table entries are the spare ones behind the last tile)
        const int ktt = min(kt, a.nkt + 1);
        if (ORDER == GEMM_ORDER_TAP) {
            // table entry of a K tile: {x byte offset of (channel block, tap), tap bit, -, -}
            ConstInt *e = ktab + ktt * 4;
            const uint32_t xoff = (uint32_t)e[0], tap = (uint32_t)e[1];
            if (Q == 0) {
                // bit `tap` of the pixel's tap mask, spread over a word, picks the offset (two VALU operations)
                const uint32_t m = (uint32_t)__builtin_amdgcn_sbfe((int)my, tap, 1u);
                vsel[S] = opaque((vbase & m) | (kOutOfRange & ~m));
            }
#pragma unroll
            for (int i = 0; i < B_LD; i++)
                if (i % (BK / 2) == Q)
                    rb[S][i] = buf_load<T>(xr, vsel[S], xoff + (uint32_t)(ks * B_LD + i) * a.hw4);
        } else {
            // table entry of a k: {x byte offset of (c,ky,kx), tap bit or ky|kx<<8}
            ConstInt *e = ktab + (ktt * BK + ks * B_LD) * 2;
#pragma unroll
            for (int i = 0; i < B_LD; i++) {
                if (i % (BK / 2) != Q)
                    continue;
                const uint32_t xoff = (uint32_t)e[2 * i], tap = (uint32_t)e[2 * i + 1];
                bool ok;
                if (MASK == GEMM_MASK_TAPS)
                    ok = (my & tap) != 0;
                else
                    ok = ((my >> (tap & 0xff)) & (mx >> (tap >> 8)) & 1u) != 0;
                rb[S][i] = buf_load<T>(xr, opaque(ok ? vbase : kOutOfRange), xoff);
            }
        }
    };
    auto store_slice = [&](auto set, auto buf_c, auto slice_q) {
        constexpr int S = decltype(set)::value;
        constexpr int BUF = decltype(buf_c)::value;
        constexpr int Q = decltype(slice_q)::value;
#pragma unroll
        for (int j = 0; j < A_LD; j++)
            if (j % (BK / 2) == Q) {
                const int idx = (tid + j * kThreads) * 4; // float index inside the [BK][BM] tile
                if (a_active) {
                    if (A_LD == 1 && wdirect) {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            As[BUF][4 * (tid / BM) + e][tid % BM] = ra[S][j][e];
                    } else
                        *(f32x4 *)&As[BUF][idx / BM][idx % BM] = ra[S][j];
                }
            }
#pragma unroll
        for (int i = 0; i < B_LD; i++)
            if (i % (BK / 2) == Q)
                Bs[BUF][ks * B_LD + i][p] = rb[S][i];
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[i][j][r] = 0.0f;

    float fa[2][TM], fb[2][TN]; // MFMA operands, double buffered across the kk steps
    auto read_operands = [&](auto buf_c, int kk, int slot) {
        constexpr int BUF = decltype(buf_c)::value;
        const int k = 2 * kk + h;
#pragma unroll
        for (int i = 0; i < TM; i++)
            fa[slot][i] = As[BUF][k][wm * WTM + i * 32 + l32];
#pragma unroll
        for (int j = 0; j < TN; j++)
            fb[slot][j] = Bs[BUF][k][wn * WTN + j * 32 + l32];
    };

    // One K step on tile kt, resident in LDS[BUF]: register set SN (tile kt+1) goes to
    // LDS[BUF^1]; tile kt+2 is fetched into register set SL.  Operands of step kk+1
    // are read from LDS before the MFMAs of step kk are issued.
    auto k_step = [&](auto buf_c, auto set_next, auto set_load, int kt) {
        constexpr int BUF = decltype(buf_c)::value;
        using NextBuf = std::integral_constant<int, BUF ^ 1>;
        // channel-major order: K need not be a multiple of the K tile; the MFMA steps of the last tile
        // whose two k rows are both padding are skipped (the 7x7x3 stem: 147 = 9 tiles + 3 rows)
        const int kk_valid = (ORDER == GEMM_ORDER_CHANNEL) ? (min(BK, a.K - kt * BK) + 1) >> 1 : BK / 2;
        read_operands(buf_c, 0, 0);
#pragma unroll
        for (int kk = 0; kk < BK / 2; kk++) {
            const int cur = kk & 1;
            if (kk + 1 < BK / 2)
                read_operands(buf_c, kk + 1, cur ^ 1);
            static_for_slice(kk, [&](auto q) {
                store_slice(set_next, NextBuf{}, q);
                load_slice(set_load, kt + NSET, q);
            });
            if (ORDER != GEMM_ORDER_CHANNEL || kk < kk_valid) {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cur][i], fb[cur][j], acc[i][j], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0); // keep the operand reads one step ahead of their MFMAs
        }
        __syncthreads();
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    // prologue: the first NSET tiles -> sets 0 .. NSET - 1; set 0 -> LDS[0]
    static_for_all([&](auto q) { load_slice(I0{}, kt_begin, q); });
    static_for_all([&](auto q) { load_slice(I1{}, kt_begin + 1, q); });
    if (NSET == 4) {
        static_for_all([&](auto q) { load_slice(I2{}, kt_begin + 2, q); });
        static_for_all([&](auto q) { load_slice(I3{}, kt_begin + 3, q); });
    }
    static_for_all([&](auto q) { store_slice(I0{}, I0{}, q); });
    __syncthreads();
    // step on tile kt (in LDS[kt & 1]): set (kt + 1) % NSET goes to the other LDS buffer, tile kt + NSET is fetched into set kt % NSET
    int kt = kt_begin;
    if (NSET == 2) {
        for (; kt + 1 < kt_end; kt += 2) {
            k_step(I0{}, I1{}, I0{}, kt);
            k_step(I1{}, I0{}, I1{}, kt + 1);
        }
        if (kt < kt_end)
            k_step(I0{}, I1{}, I0{}, kt);
    } else {
        for (; kt + 3 < kt_end; kt += 4) {
            k_step(I0{}, I1{}, I0{}, kt);
            k_step(I1{}, I2{}, I1{}, kt + 1);
            k_step(I0{}, I3{}, I2{}, kt + 2);
            k_step(I1{}, I0{}, I3{}, kt + 3);
        }
        if (kt < kt_end)
            k_step(I0{}, I1{}, I0{}, kt);
        if (kt + 1 < kt_end)
            k_step(I1{}, I2{}, I1{}, kt + 1);
        if (kt + 2 < kt_end)
            k_step(I0{}, I3{}, I2{}, kt + 2);
    }

    gemm_tile_output<T, BM, BN, WM, WN, ACT>(a, acc, &As[0][0][0], m0, n0, g, slice, splitk, image0, wm, wn, h, l32, tid, bias_early);
}

// What a workgroup does with its finished accumulator tile: the split-K partial store, or the
// epilogue (bias, activation, factor) and the NCHW store.  `lds` is LDS that is free after the
// last barrier of the main loop (at least BM floats).  `bias_s`: the bias of the tile's BM rows in LDS (zero past M), staged by the
// kernel when it starts on the tile: requested here, its trip to memory stood between the last matrix instruction and the first store.
template <class T, int BM, int BN, int WM, int WN, int ACT>
__device__ __forceinline__ void gemm_tile_output(const GemmArgs &a, f32x16 (&acc)[BM / WM / 32][BN / WN / 32], float *lds, int m0, int n0,
                                                 int g, int slice, int splitk, uint32_t image0, int wm, int wn, int h, int l32, int tid,
                                                 const float *bias_s)
{
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    // ---- split-K, reduced in place: the slice's accumulators go to the workspace as a register image
    // ([r][thread], write-through); the workgroup that arrives last at the tile's counter adds up all
    // slices in slice order (deterministic), whoever it is, and goes on to the epilogue.  Nobody waits. ----
    if (splitk > 1 && a.sk_cnt != nullptr) {
        static_assert(TM == 1 && TN == 1, "one MFMA block per wavefront");
        constexpr int kThrough = 17; // sc0 | sc1: past the caches in both directions
        constexpr uint32_t image_bytes = BM * BN * 4;
        const __amdgpu_buffer_rsrc_t pr = __builtin_amdgcn_make_buffer_rsrc(a.sk_part, 0, a.sk_part_bytes, 0x00020000);
        const int tile = (g * a.ntiles + n0 / BN) * a.mtiles + m0 / BM;
        const uint32_t base = image0 * image_bytes;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const float v = acc[0][0][r];
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), pr, (uint32_t)tid * 4u,
                                                  base + (uint32_t)slice * image_bytes + (uint32_t)(r * kThreads * 4), kThrough);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): this thread's part has been written through
        __syncthreads();
        int *arrived_s = reinterpret_cast<int *>(lds);
        if (tid == 0)
            *arrived_s = atomicAdd(a.sk_cnt + tile, 1);
        __syncthreads();
        const int arrived = __builtin_amdgcn_readfirstlane(*arrived_s);
        __syncthreads(); // lds is reused by the epilogue
        if (arrived != splitk - 1)
            return;
        if (tid == 0)
            a.sk_cnt[tile] = 0; // left at zero for the next launch (counters that the operator owns are cleared only once)
#pragma unroll
        for (int r = 0; r < 16; r++)
            acc[0][0][r] = 0.0f;
        for (int s0 = 0; s0 < splitk; s0 += 4) { // four slices (64 loads) in flight at a time
            float p[4][16];
#pragma unroll
            for (int ds = 0; ds < 4; ds++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    p[ds][r] = (s0 + ds < splitk) ? __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                          pr, (uint32_t)tid * 4u,
                                                          base + (uint32_t)(s0 + ds) * image_bytes + (uint32_t)(r * kThreads * 4), kThrough))
                                                    : 0.0f;
#pragma unroll
            for (int ds = 0; ds < 4; ds++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    acc[0][0][r] += p[ds][r];
        }
    } else if (splitk > 1) { // raw partial sums in output order, reduced by splitk_reduce_kernel
        if ((a.M & 7) == 0 && a.part_bytes != 0) { // buffer stores with scalar row offsets
            const __amdgpu_buffer_rsrc_t pr = __builtin_amdgcn_make_buffer_rsrc(a.part, 0, a.part_bytes, 0x00020000);
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const int n = n0 + wn * WTN + j * 32 + l32;
                const uint32_t voff =
                    n < a.N ? (uint32_t)((slice * a.Cout + g * a.M + m0 + wm * WTM + 4 * h) * a.N + n) * 4u : kOutOfRange;
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int mrow = i * 32 + 8 * (r >> 2) + (r & 3);
                        const float v = acc[i][j][r]; // a copy: bit_cast of a vector element reads element 0
                        if (m0 + wm * WTM + mrow < a.M)
                            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), pr, voff, (uint32_t)(mrow * a.N) * 4u, 0);
                    }
            }
            return;
        }
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int n = n0 + wn * WTN + j * 32 + l32;
            if (n >= a.N)
                continue;
            float *pb = a.part + ((size_t)slice * a.Cout + (size_t)g * a.M) * a.N + n;
#pragma unroll
            for (int i = 0; i < TM; i++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int m = m0 + wm * WTM + i * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                    if (m < a.M)
                        pb[(size_t)m * a.N] = acc[i][j][r];
                }
            }
        }
        return;
    }

    // ---- epilogue: bias, activation, factor, NCHW store ----
    // Fast path (no factor, M a multiple of 8, y below 2 GiB): the bias of the tile's rows goes
    // through LDS (free after the last barrier) and the stores are buffer stores whose row offset
    // is scalar, instead of a bias load and 64-bit address arithmetic per value.
    const bool pre = a.pre != 0 && a.factor != 0.0f;
    if ((a.factor == 0.0f || (pre && sizeof(T) == 4)) && (a.M & 7) == 0 && a.y_bytes != 0) {
        const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc(a.y, 0, a.y_bytes, 0x00020000);
        const bool clamp = a.act != DLP_ACT_IDENTITY;
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int n = n0 + wn * WTN + j * 32 + l32;
            const int b = (int)fast_div((uint32_t)n, a.ohw_magic, a.ohw_shift);
            const int pix = n - b * a.OHW;
            const uint32_t voff =
                n < a.N ? (uint32_t)(((b * a.Cout + g * a.M + m0 + wm * WTM + 4 * h) * a.OHW + pix) * (int)sizeof(T)) : kOutOfRange;
#pragma unroll
            for (int i = 0; i < TM; i++) {
#pragma unroll
                for (int rq = 0; rq < 4; rq++) {
                    const int mrow = wm * WTM + i * 32 + 8 * rq; // + 4*h + (r & 3); this part is uniform
                    if (m0 + mrow >= a.M)
                        continue;
                    const f32x4 bv = *(const f32x4 *)&bias_s[mrow + 4 * h];
#pragma unroll
                    for (int rr = 0; rr < 4; rr++) {
                        float v = acc[i][j][4 * rq + rr] + bv[rr];
                        const uint32_t soff = (uint32_t)((i * 32 + 8 * rq + rr) * a.OHW * (int)sizeof(T));
                        if (pre)
                            v = fmaf(__builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(yr, voff, soff, 0)), a.factor, v);
                        if (ACT == ACT_CLAMP) {
                            if (clamp) // identity must keep NaNs: no min/max
                                v = clamp_med3(v, a.clamp_lo, a.clamp_hi);
                        } else
                            v = apply_act(v, a.act);
                        if (sizeof(T) == 4)
                            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), yr, voff, soff, 0);
                        else
                            __builtin_amdgcn_raw_buffer_store_b16((short)to_bf16(v).bits, yr, voff, soff, 0);
                    }
                }
            }
        }
        return;
    }
    // accumulator register r of a 32x32 block holds row 8*(r/4) + 4*h + r%4, column l32
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int n = n0 + wn * WTN + j * 32 + l32;
        if (n >= a.N)
            continue;
        const int b = (int)fast_div((uint32_t)n, a.ohw_magic, a.ohw_shift);
        const int pix = n - b * a.OHW;
        T *yb = (T *)a.y + ((size_t)b * a.Cout + (size_t)g * a.M) * a.OHW + pix;
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + wm * WTM + i * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                if (m < a.M) {
                    float v = acc[i][j][r];
                    if (a.bias)
                        v += a.bias[g * a.M + m];
                    if (pre)
                        v = fmaf(to_float(yb[(size_t)m * a.OHW]), a.factor, v);
                    if (ACT == ACT_CLAMP) {
                        if (a.act != DLP_ACT_IDENTITY) // identity must keep NaNs: no min/max
                            v = clamp_med3(v, a.clamp_lo, a.clamp_hi);
                    } else
                        v = apply_act(v, a.act);
                    store_out(yb + (size_t)m * a.OHW, v, pre ? 0.0f : a.factor);
                }
            }
        }
    }
}

// ---- stride-1 "same" convolutions: the input patch of a tile goes through LDS once ----------
// For stride 1, dilation 1 and output size == input size, the pixels that the KH*KW taps of a
// run of 64 output pixels read are one run of 64 + 2*(ph*W + pw) consecutive pixels of each
// input channel plane (one such run per image when the tile crosses an image boundary).  A K
// stage = 16 input channels: its patch [16][PITCH] is loaded once, with coalesced loads and no
// masks, and serves all KH*KW K tiles of the stage.  An MFMA B operand is then a ds_read at
// (lane's patch row + tap shift); padding taps read a row that is always zero.  Every
// address is fixed before the main loop, which is left with MFMAs, LDS reads with immediate
// offsets and the loads of the next stage: no vector-ALU work at all.
// Weights: the same packed tap-major tiles as the gathering kernel (K tile = stage * KH*KW + tap).
template <int N, class F, int... I>
__device__ __forceinline__ void static_for_seq(F &&f, std::integer_sequence<int, I...>)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for_n(F &&f)
{
    static_for_seq<N>(f, std::make_integer_sequence<int, N>{});
}

// STRIDE 2 (3x3, pad 1): the pixels under the taps of 64 consecutive output pixels are still one run of consecutive input pixels
// per image -- from the first output pixel's top-left tap to the last one's bottom-right tap -- only four times as long per
// output (up to 9 input rows of 56 for 64 outputs on 28 columns: rows of 512); a lane's taps sit at 2 * (its pixel) in that run.
// Two such patch buffers would be 64 KB and leave two workgroups per CU, which costs more than the patch saves (measured: no
// faster than the gathering kernel), so the strided instantiation keeps ONE patch buffer (40 KB with the A tiles, three workgroups
// per CU): the next stage's patch waits in registers and is stored in the stage's last K tile, after the barrier behind which
// nobody reads the buffer any more, followed by a second barrier before the next stage's first operands are read.
template <class T, int KH, int KW, int PITCH, int ACT, int STRIDE = 1>
__global__ __launch_bounds__(kThreads) void conv_patch_f32_kernel(GemmArgs a)
{
    constexpr int BM = 64, BN = 64, WM = 2, WN = 2, KHW = KH * KW;
    constexpr int QS = PITCH / 64;  // patch rows per lane
    constexpr int CPW = BK / 4;     // channels of a stage per wavefront
    constexpr int NPL = QS * CPW;   // patch loads per lane and stage
    constexpr int MAXSEG = 3;       // images a tile may touch (H*W >= 32)
    constexpr int ZERO_ROW = PITCH - 1; // never loaded: reads 0 in every channel
    static_assert(PITCH % 64 == 0 && BK == 16, "patch shape");
    constexpr bool SINGLE = STRIDE != 1; // one patch buffer
    constexpr int NPB = SINGLE ? 1 : 2;

    __shared__ __attribute__((aligned(16))) float As[2][BK][BM];
    __shared__ float Ps[NPB][BK][PITCH];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int h = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;

    // ---- stream-K: the K stages of all tiles, in tile order, are dealt evenly to the workgroups ----
    // unit = (tile, stage); workgroup j (XCD-contiguous numbering, as in conv_gemm_f32_kernel) runs
    // units [j*U/G, (j+1)*U/G): the tail of one tile, whole tiles, the head of another.
    int j;
    {
        const int nb = gridDim.x, bid = blockIdx.x;
        const int q = nb >> 3, r = nb & 7;
        const int xcd = bid & 7, slot = bid >> 3;
        j = (xcd < r) ? xcd * (q + 1) + slot : r * (q + 1) + (xcd - r) * q + slot;
    }
    const int ncb = a.nkt / KHW; // stages per tile
    const uint64_t U = (uint64_t)a.sk_units, G = gridDim.x;
    const int u_begin = (int)((uint64_t)j * U / G), u_end = (int)((uint64_t)(j + 1) * U / G);

    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)a.wp, 0, a.wp_bytes, 0x00020000);

    for (int u = u_begin; u < u_end;) {
    int t = (int)fast_div((uint32_t)u, a.ncb_magic, a.ncb_shift); // u / ncb; tile: m tile fastest, then n tile, then group
    const int tile = t;
    const int cb_begin = u - t * ncb;
    const int cb_end = min(ncb, cb_begin + (u_end - u));
    // Which (group, m tile, n tile) the tile-th tile of the stream is -- any bijection is correct; this
    // one is chosen for the L2 of the XCD that runs it.  (1) Each eighth of the stream (one XCD's
    // share) is read transposed, sk_tpw tiles (one workgroup's share) per column: at any time the
    // workgroups of an XCD then work on neighbouring tiles instead of tiles sk_tpw apart, so the halo
    // rows that neighbouring pixel tiles share are fetched once.  (2) Neighbouring tiles are the
    // sk_mb m tiles of one pixel tile, then the next pixel tile: an XCD's share covers few m tiles
    // (little of the weights) and a compact range of pixels.
    {
        const int NT = a.sk_tiles;
        int c = (int)fast_div((uint32_t)t * 8u, a.nt_magic, a.nt_shift); // 8 t / NT (NT < 2^27: y is below 2 GiB)
        int lo = (int)(((int64_t)c * NT) / 8), hi = (int)(((int64_t)(c + 1) * NT) / 8);
        if (t >= hi) {
            c++;
            lo = hi;
            hi = (int)(((int64_t)(c + 1) * NT) / 8);
        }
        const int L = hi - lo, i = t - lo;
        const int q = (int)fast_div((uint32_t)L, a.tpw_magic, a.tpw_shift), r = L - q * a.sk_tpw;
        const int col = (int)fast_div((uint32_t)i, a.tpw_magic, a.tpw_shift), row = i - col * a.sk_tpw;
        // rows 0..r-1 of the ragged L = q*tpw + r layout hold q+1 tiles, the others q; a column index
        // past a short row's end only happens in the last (partial) column, which holds rows < r
        t = lo + row * q + min(row, r) + col;
    }
    const int per_group = a.mtiles * a.ntiles;
    const int g = (int)fast_div((uint32_t)t, a.pg_magic, a.pg_shift);
    t -= g * per_group;
    const int mblk = (int)fast_div((uint32_t)t, a.mbnt_magic, a.mbnt_shift);
    t -= mblk * a.sk_mb * a.ntiles;
    const int nt = (int)fast_div((uint32_t)t, a.mb_magic, a.mb_shift);
    const int mt = mblk * a.sk_mb + (t - nt * a.sk_mb);
    const int m0 = mt * BM, n0 = nt * BN;
    // the bias of the tile's rows, for the epilogue: in LDS long before it is wanted (the barriers of the stages lie between, and the
    // barrier that ends a piece lies between the epilogue of the piece before and this store)
    __shared__ float bias_early[BM];
    if (tid < BM)
        bias_early[tid] = (a.bias && m0 + tid < a.M) ? a.bias[g * a.M + m0 + tid] : 0.0f;

    // ---- the tile's patch: one segment of consecutive plane pixels per image (wavefront-uniform) ----
    const int HW = a.OHW;                            // pixels of an output plane
    const int HWI = STRIDE == 1 ? HW : a.H * a.W;    // ... of an input plane
    const int halo = a.ph * a.W + a.pw;
    const int n_last = min(n0 + BN, a.N) - 1;
    const int b0 = (int)fast_div((uint32_t)n0, a.ohw_magic, a.ohw_shift);
    int seg_row[MAXSEG], seg_a[MAXSEG], seg_len[MAXSEG];
    {
        int row = 0;
#pragma unroll
        for (int s = 0; s < MAXSEG; s++) {
            const int base = (b0 + s) * HW;
            const int first = max(n0, base), last = min(n_last, base + HW - 1);
            int as = 0, len = 0;
            if (first <= last) {
                if (STRIDE == 1) {
                    as = max(0, first - base - halo);
                    len = min(HW, last - base + 1 + halo) - as;
                } else { // from the top-left tap of the first output pixel to the bottom-right tap of the last one
                    const int pf = first - base, pl = last - base;
                    const int oyf = (int)fast_div((uint32_t)pf, a.ow_magic, a.ow_shift), oyl = (int)fast_div((uint32_t)pl, a.ow_magic, a.ow_shift);
                    const int oxf = pf - oyf * a.OW, oxl = pl - oyl * a.OW;
                    as = max(0, (oyf * STRIDE - a.ph) * a.W + oxf * STRIDE - a.pw);
                    len = min(HWI, (oyl * STRIDE - a.ph + KH - 1) * a.W + oxl * STRIDE - a.pw + KW) - as;
                }
            }
            seg_row[s] = row;
            seg_a[s] = as;
            seg_len[s] = len;
            row += len;
        }
    }
    // patch rows lane, lane + 64, ...: byte offset of the pixel in channel 0 of the group (or out of range)
    uint32_t pvoff[QS];
#pragma unroll
    for (int q = 0; q < QS; q++) {
        const int rho = lane + 64 * q;
        uint32_t v = kOutOfRange;
#pragma unroll
        for (int s = 0; s < MAXSEG; s++) {
            const int d = rho - seg_row[s];
            if (d >= 0 && d < seg_len[s])
                v = (uint32_t)((((b0 + s) * a.Cin + g * a.Cin_g) * HWI + seg_a[s] + d) * (int)sizeof(T));
        }
        pvoff[q] = v;
    }
    // this lane's B operand (k = h, column l32 of the wavefront tile) per tap: byte offset in a patch buffer
    uint32_t baddr[KHW];
    {
        const int n = n0 + wn * 32 + l32;
        const bool vn = n < a.N;
        const int b = (int)fast_div((uint32_t)n, a.ohw_magic, a.ohw_shift);
        const int pix = n - b * HW;
        const int oy = (int)fast_div((uint32_t)pix, a.ow_magic, a.ow_shift);
        const int ox = pix - oy * a.OW;
        const int s = b - b0;
        const int row = (STRIDE == 1 ? pix : (oy * a.W + ox) * STRIDE) + (s == 0 ? seg_row[0] - seg_a[0] : s == 1 ? seg_row[1] - seg_a[1] : seg_row[2] - seg_a[2]);
#pragma unroll
        for (int ky = 0; ky < KH; ky++)
#pragma unroll
            for (int kx = 0; kx < KW; kx++) {
                const int yy = oy * STRIDE + ky - a.ph, xx = ox * STRIDE + kx - a.pw;
                const bool ok = vn && yy >= 0 && yy < a.H && xx >= 0 && xx < a.W;
                const int r = ok ? row + (ky - a.ph) * a.W + (kx - a.pw) : ZERO_ROW;
                baddr[ky * KW + kx] = (uint32_t)((h * PITCH + r) * 4);
            }
    }

    const uint32_t a_tile_bytes = BK * BM * 4;
    const uint32_t a_row_base = (uint32_t)((g * a.mtiles + mt) * a.nkt) * a_tile_bytes;

    static_assert((2 * KHW) % 3 == 0, "three A register sets rotate with period 3 inside a pair of stages");
    f32x4 ra[3];      // packed A tiles in flight: tile kt + 3 is requested while tile kt is multiplied
    float preg[NPL];  // patch of the next stage
    float fa[2][BK / 2], fb[2][BK / 2]; // MFMA operands of this K tile and of the next one
    f32x16 acc[1][1];
#pragma unroll
    for (int r = 0; r < 16; r++)
        acc[0][0][r] = 0.0f;

    auto load_a = [&](auto set, int kt) {
        ra[decltype(set)::value] = buf_load4(wr, (uint32_t)(tid * 16), a_row_base + (uint32_t)min(kt, a.nkt - 1) * a_tile_bytes);
    };
    auto store_a = [&](auto set, auto buf_c) {
        *(f32x4 *)&As[decltype(buf_c)::value][tid / (BM / 4)][(tid % (BM / 4)) * 4] = ra[decltype(set)::value];
    };
    auto load_patch = [&](int j, uint32_t stage_soff) { // j = channel-in-wavefront * QS + row slot
        preg[j] = buf_load<T>(xr, pvoff[j % QS], stage_soff + (uint32_t)(j / QS) * a.hw4);
    };
    auto store_patch = [&](auto buf_c, int j) { Ps[SINGLE ? 0 : decltype(buf_c)::value][wave * CPW + j / QS][lane + 64 * (j % QS)] = preg[j]; };
    // operands kk of the K tile (A buffer ABUF, patch buffer PB, tap TAP) into operand set OS
    auto read_operands = [&](auto os_c, auto abuf_c, auto pb_c, auto tap_c, int kk) {
        constexpr int OS = decltype(os_c)::value;
        fa[OS][kk] = As[decltype(abuf_c)::value][2 * kk + h][wm * 32 + l32];
        fb[OS][kk] = *reinterpret_cast<const float *>(reinterpret_cast<const char *>(&Ps[SINGLE ? 0 : decltype(pb_c)::value][0][0]) +
                                                      baddr[decltype(tap_c)::value] + 2 * kk * PITCH * 4);
    };

    // One stage: KHW K tiles on patch buffer P; the patch of stage cb + 1 is requested during
    // the first tile and goes to the other buffer during the last one.  One barrier per K tile,
    // in its middle: before it, the next tile's A (and patch) go to the LDS buffers nobody reads
    // any more; after it, the next tile's operands are read while this tile's MFMAs still run,
    // so a wavefront that is alone on its SIMD does not wait for LDS at the start of a tile.
    auto stage = [&](auto par, int cb) {
        constexpr int P = decltype(par)::value;
        using OtherP = std::integral_constant<int, P ^ 1>;
        const uint32_t next_soff = (uint32_t)(min(cb + 1, ncb - 1) * BK + wave * CPW) * a.hw4;
        static_for_n<KHW>([&](auto tau_c) {
            constexpr int TAU = decltype(tau_c)::value;
            constexpr int IDX = P * KHW + TAU; // K tile counter: modulo 2 for LDS buffers and operand sets, modulo 3 for A registers
            constexpr int BUF = IDX & 1;
            using NextBuf = std::integral_constant<int, BUF ^ 1>;
            using SetNext = std::integral_constant<int, (IDX + 1) % 3>;
            using SetLoad = std::integral_constant<int, IDX % 3>;
            using NextOps = std::integral_constant<int, BUF ^ 1>;
            using NextTap = std::integral_constant<int, (TAU + 1) % KHW>;
            using NextPatch = std::integral_constant<int, (TAU + 1 < KHW) ? P : (P ^ 1)>;
            const int kt = cb * KHW + TAU;
#pragma unroll
            for (int kk = 0; kk < BK / 2; kk++) {
                if (kk == 0)
                    store_a(SetNext{}, NextBuf{});
                if (kk == 1)
                    load_a(SetLoad{}, kt + 3);
#pragma unroll
                for (int j = 0; j < NPL; j++) {
                    if (TAU == 0 && j % (BK / 2) == kk)
                        load_patch(j, next_soff);
                    if (!SINGLE && TAU == KHW - 1 && j / ((NPL + 3) / 4) == kk) // before the barrier
                        store_patch(OtherP{}, j);
                    // one buffer: behind the barrier of the stage's last K tile nobody reads it any more (that tile's operands were
                    // read during the tile before)
                    if (SINGLE && TAU == KHW - 1 && (kk == 4 || kk == 5) && j / (NPL / 2) == kk - 4)
                        store_patch(OtherP{}, j);
                }
                acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[BUF][kk], fb[BUF][kk], acc[0][0], 0, 0, 0);
                if (kk == 3)
                    __syncthreads();
                if (SINGLE && TAU == KHW - 1) {
                    if (kk == 5)
                        __syncthreads(); // the next stage's patch is in place
                    if (kk >= 6) {
#pragma unroll
                        for (int q = 0; q < 4; q++)
                            read_operands(NextOps{}, NextBuf{}, NextPatch{}, NextTap{}, 4 * (kk - 6) + q);
                    }
                } else if (kk >= 4) {
                    read_operands(NextOps{}, NextBuf{}, NextPatch{}, NextTap{}, 2 * (kk - 4));
                    read_operands(NextOps{}, NextBuf{}, NextPatch{}, NextTap{}, 2 * (kk - 4) + 1);
                }
                __builtin_amdgcn_sched_barrier(0); // keep this order: the scheduler would sink the operand reads to their uses
            }
        });
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    {
        static_assert(NPL <= 32, "patch loads and stores are dealt over the steps of a K tile");
        const uint32_t soff0 = (uint32_t)(cb_begin * BK + wave * CPW) * a.hw4;
#pragma unroll
        for (int j = 0; j < NPL; j++)
            load_patch(j, soff0);
        load_a(I0{}, cb_begin * KHW);
        load_a(I1{}, cb_begin * KHW + 1);
        load_a(I2{}, cb_begin * KHW + 2);
#pragma unroll
        for (int j = 0; j < NPL; j++)
            store_patch(I0{}, j);
        store_a(I0{}, I0{});
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK / 2; kk++)
            read_operands(I0{}, I0{}, I0{}, I0{}, kk);
    }
    int cb = cb_begin;
    for (; cb + 1 < cb_end; cb += 2) {
        stage(I0{}, cb);
        stage(I1{}, cb + 1);
    }
    if (cb < cb_end)
        stage(I0{}, cb);

    bool output = true;
    if (cb_begin != 0 || cb_end != ncb) {
        // A piece of a tile: its accumulators go to this workgroup's first or second slot (register
        // image, [r][thread]); the workgroup that arrives last at the tile's counter adds up all the
        // pieces, in workgroup order whoever it is, and writes the tile.  Nobody waits for anybody.
        // Pieces bypass the caches in both directions (write-through stores, uncached loads): a
        // device-wide fence would write back and invalidate a whole L2 per piece.
        constexpr int kThrough = 17; // sc0 | sc1
        const __amdgpu_buffer_rsrc_t pr = __builtin_amdgcn_make_buffer_rsrc(a.sk_part, 0, a.sk_part_bytes, 0x00020000);
        const uint32_t piece_bytes = BM * BN * 4;
        {
            const uint32_t soff = (uint32_t)(2 * j + (u == u_begin ? 0 : 1)) * piece_bytes;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float v = acc[0][0][r];
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), pr, (uint32_t)(r * kThreads + tid) * 4u, soff, kThrough);
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): this thread's piece has been written through
        __syncthreads();
        int *arrived_s = reinterpret_cast<int *>(&As[1][0][0]); // free after the last barrier of the main loop
        if (tid == 0)
            *arrived_s = atomicAdd(a.sk_cnt + tile, 1);
        __syncthreads();
        const int arrived = __builtin_amdgcn_readfirstlane(*arrived_s);
        const uint64_t ut0 = (uint64_t)tile * ncb;
        const int j_first = (int)(((ut0 + 1) * G - 1) / U), j_last = (int)(((ut0 + ncb) * G - 1) / U);
        output = arrived == j_last - j_first;
        if (output) {
            if (tid == 0)
                a.sk_cnt[tile] = 0; // left at zero for the next launch (counters that the operator owns are cleared only once)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[0][0][r] = 0.0f;
            for (int jj = j_first; jj <= j_last; jj++) {
                const int first_tile = (int)((uint64_t)jj * U / G) / ncb; // tile of jj's first piece
                const uint32_t soff = (uint32_t)(2 * jj + (first_tile == tile ? 0 : 1)) * piece_bytes;
#pragma unroll
                for (int r = 0; r < 16; r++)
                    acc[0][0][r] += __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(pr, (uint32_t)(r * kThreads + tid) * 4u, soff, kThrough));
            }
        }
    }
    if (output)
        gemm_tile_output<T, BM, BN, WM, WN, ACT>(a, acc, &As[0][0][0], m0, n0, g, 0, 1, 0u, wm, wn, h, l32, tid, bias_early);
    __syncthreads(); // LDS is reused by the next piece
    u += cb_end - cb_begin;
    }
}

// ---- bfloat16 storage on the bf16 matrix instruction ------------------------------------
// Same implicit GEMM for tensors stored as bf16 whose Cin/groups is a multiple of 32:
// v_mfma_f32_32x32x16_bf16 (fp32 accumulate) is 16 times faster per flop than the fp32
// instruction, so everything is sized for operand delivery instead:
//  * K tile = one filter tap x 32 channels (two MFMA k steps);
//  * an MFMA operand is 8 consecutive k of one row per lane, so LDS holds A as [m][k] and B
//    as [pixel][k] with rows of 32 + 8 bf16 (80 bytes: the 16-byte accesses of 16 consecutive
//    rows fall on distinct banks) and every operand fetch is one ds_read_b128;
//  * the gathered input arrives pixel-per-lane (NCHW keeps pixels contiguous), one 16-bit
//    element per load; a thread owns one pixel and 16 or 32 channels, packs pairs with one
//    VALU op each and stores 16-byte pieces of its pixel's row;
//  * weights are pre-packed as bf16 in [m tile][K tile][m][32] order (16-byte pieces per thread);
//  * 128x128 tiles (wavefront 64x64), or 64x256 when M <= 64.
// The sum over k is accumulated in fp32 exactly as in the fp32 kernel (products of bf16 values
// are exact in fp32), only in a different order.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
// Register sets of tiles in flight (2 or 4).  Measured: 4 sets (two more K steps of load latency
// hidden, 148 instead of 102 VGPRs) are not faster -- the kernel is bound by the vector-memory
// access rate, not by latency -- so 2 sets and three workgroups per CU it is.
#ifndef DLP_BF16_STORE_AUX
#define DLP_BF16_STORE_AUX 2 // 2 = non-temporal: whole-line output runs that this launch does not read again stream past the L2 (64->256 at 56x56, batch 128: 74 -> 54 us)
#endif
#ifndef DLP_BF16_NSET
#define DLP_BF16_NSET 2
#endif
#ifndef DLP_DENSE_NSET
#define DLP_DENSE_NSET 2
#endif
constexpr int BK2 = 32;
constexpr int LDK = BK2 + 8;

// What a workgroup of the bf16 kernels does with its finished accumulator tile: the split-K partial
// store, or the epilogue (bias, activation, factor) and the store to y.  `smem` is the kernel's LDS
// (at least BM * (BN * 2 + 16) bytes), free after the last barrier of the main loop.  `bias_s`: the bias of the tile's BM rows in
// LDS (zero past M), which the kernel stages when it starts -- requested in the epilogue, its trip to memory stood between the
// last matrix instruction and the first store of every tile (36 us of a ResNet-50 pass at batch 128).
template <int BM, int BN, int WM, int WN, int ACT>
__device__ __forceinline__ void bf16_tile_output(const GemmArgs &a, f32x16 (&acc)[BM / WM / 32][BN / WN / 32], unsigned char *smem, int smem_bytes,
                                                 int m0, int n0, int g, int slice, int wm, int wn, int h, int l32, int tid, const float *bias_s)
{
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    if (a.splitk > 1) {
        if ((a.M & 7) == 0 && a.part_bytes != 0) { // buffer stores with scalar row offsets
            const __amdgpu_buffer_rsrc_t pr = __builtin_amdgcn_make_buffer_rsrc(a.part, 0, a.part_bytes, 0x00020000);
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const int n = n0 + wn * WTN + j * 32 + l32;
                const uint32_t voff =
                    n < a.N ? (uint32_t)((slice * a.Cout + g * a.M + m0 + wm * WTM + 4 * h) * a.N + n) * 4u : kOutOfRange;
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int mrow = i * 32 + 8 * (r >> 2) + (r & 3);
                        const float v = acc[i][j][r]; // a copy: bit_cast of a vector element reads element 0
                        if (m0 + wm * WTM + mrow < a.M)
                            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), pr, voff, (uint32_t)(mrow * a.N) * 4u, 0);
                    }
            }
            return;
        }
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int n = n0 + wn * WTN + j * 32 + l32;
            if (n >= a.N)
                continue;
            float *pb = a.part + ((size_t)slice * a.Cout + (size_t)g * a.M) * a.N + n;
#pragma unroll
            for (int i = 0; i < TM; i++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int m = m0 + wm * WTM + i * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                    if (m < a.M)
                        pb[(size_t)m * a.N] = acc[i][j][r];
                }
            }
        }
        return;
    }

    // ---- channels-last output, y[(image, pixel)][channel] (the host checks: no factor or accumulate_first, M a multiple of 8,
    // y 16-byte aligned and below 2 GiB).  The tile goes to LDS as bf16 [n][m]: a lane's four consecutive accumulator rows are four
    // consecutive channels of its pixel, one 8-byte LDS store (pixels 16 bytes more than BM channels apart: the lanes of a
    // store hit different banks), and leaves in 16-byte pieces of 8 channels, BM / 8 consecutive lanes on the contiguous
    // bytes of a pixel. ----
    if (a.y_cl) {
        constexpr int PITCH = BM * 2 + 16;
        const bool pre = a.pre != 0 && a.factor != 0.0f; // the old y joins before the activation: in the second phase
        const bool clamp = a.act != DLP_ACT_IDENTITY && !pre;
        const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc(a.y, 0, a.y_bytes, 0x00020000);
        constexpr int PPR = BM / 8; // pieces of a pixel's row
        static_assert((BN * PPR) % kThreads == 0 && kThreads % PPR == 0, "pieces are dealt to the threads evenly");
        const int piece = tid % PPR, pix_t = tid / PPR;
        const int m = m0 + piece * 8;
        const uint32_t col_off = (uint32_t)(g * a.M + m) * 2u;
        constexpr int STEP = kThreads / PPR;           // pixels between a thread's pieces
        constexpr int PER_THREAD = BN * PPR / kThreads; // pieces per thread
        auto piece_offset = [&](int u) {
            const int n = n0 + pix_t + u * STEP;
            return (n < a.N && m < a.M) ? (uint32_t)n * (uint32_t)a.Cout * 2u + col_off : kOutOfRange;
        };
        // the old values of all the thread's pieces are asked for first: they travel while the tile is rounded and staged
        // (the accumulators are still live here, the operand registers of the main loop are not)
        u32x4 old[PER_THREAD];
        if (pre) {
#pragma unroll
            for (int u = 0; u < PER_THREAD; u++)
                old[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(yr, piece_offset(u), 0, 0));
        }
        __syncthreads(); // every wavefront has read its last operands: LDS takes the tile
#pragma unroll
        for (int j = 0; j < TN; j++) {
            unsigned char *rowp = smem + (wn * WTN + j * 32 + l32) * PITCH + (wm * WTM + 4 * h) * 2;
#pragma unroll
            for (int i = 0; i < TM; i++) {
#pragma unroll
                for (int rq = 0; rq < 4; rq++) {
                    const f32x4 bv = *(const f32x4 *)&bias_s[wm * WTM + i * 32 + 8 * rq + 4 * h];
                    uint32_t bits[4];
#pragma unroll
                    for (int rr = 0; rr < 4; rr++) {
                        float v = acc[i][j][4 * rq + rr] + bv[rr];
                        if (ACT == ACT_CLAMP) {
                            if (clamp)
                                v = clamp_med3(v, a.clamp_lo, a.clamp_hi);
                        } else if (!pre)
                            v = apply_act(v, a.act);
                        bits[rr] = to_bf16(v).bits;
                    }
                    u32x2 o;
                    o[0] = bits[0] | (bits[1] << 16);
                    o[1] = bits[2] | (bits[3] << 16);
                    *(u32x2 *)(rowp + (i * 32 + 8 * rq) * 2) = o;
                }
            }
        }
        __syncthreads();
        // every pixel's run is whole 128-byte lines, and the tensor is too large for the next layer to find it in the last-level cache:
        // streaming stores
        const bool streaming = (a.Cout & 63) == 0 && (BM & 63) == 0 && a.y_bytes >= (96u << 20);
        const unsigned char *src_t = smem + pix_t * PITCH + piece * 16;
#pragma unroll
        for (int u = 0; u < PER_THREAD; u++) {
            u32x4 mine = *(const u32x4 *)(src_t + u * STEP * PITCH);
            if (pre) {
#pragma unroll
                for (int d = 0; d < 4; d++) {
                    float lo = fmaf(__builtin_bit_cast(float, old[u][d] << 16), a.factor, __builtin_bit_cast(float, mine[d] << 16));
                    float hi = fmaf(__builtin_bit_cast(float, old[u][d] & 0xFFFF0000u), a.factor, __builtin_bit_cast(float, mine[d] & 0xFFFF0000u));
                    if (ACT == ACT_CLAMP) {
                        if (a.act != DLP_ACT_IDENTITY) {
                            lo = clamp_med3(lo, a.clamp_lo, a.clamp_hi);
                            hi = clamp_med3(hi, a.clamp_lo, a.clamp_hi);
                        }
                    } else {
                        lo = apply_act(lo, a.act);
                        hi = apply_act(hi, a.act);
                    }
                    mine[d] = (uint32_t)to_bf16(lo).bits | ((uint32_t)to_bf16(hi).bits << 16);
                }
            }
            if (streaming)
                __builtin_amdgcn_raw_buffer_store_b128(mine, yr, piece_offset(u), 0, DLP_BF16_STORE_AUX);
            else
                __builtin_amdgcn_raw_buffer_store_b128(mine, yr, piece_offset(u), 0, 0);
        }
        return;
    }
    // ---- epilogue.  Fast path (no factor, M a multiple of 8, y below 2 GiB): the bias of the
    // tile's rows goes through LDS (free after the last barrier), the result is rounded by the
    // hardware conversion and stored with buffer stores whose row offset is scalar: a handful of
    // VALU operations per value instead of 64-bit address arithmetic and a bias load each. ----
    // Wide stores (a.pxv = 2, 4 or 8 pixels per store; the host sets it when there is no factor, y is
    // 4-byte aligned and below 2 GiB, and pxv divides OH*OW): the tile goes to LDS as bf16 [m][n]
    // (rows padded by 16 bytes: the two half-waves, four rows apart, hit different banks) and is
    // stored to y in runs of pxv pixels per lane, consecutive lanes on consecutive runs of a row --
    // a store instruction costs the same whatever its width, so this is pxv times fewer of them.
    if (a.pxv != 0) {
        constexpr int PITCH = BN * 2 + 16;
        (void)smem_bytes; // the callers check BM * PITCH + BM * 4 <= their LDS
        __syncthreads(); // every wavefront has read its last operands: LDS takes the tile
        const bool pre = a.pre != 0 && a.factor != 0.0f; // the old y joins before the activation: in the second phase
        const bool clamp = a.act != DLP_ACT_IDENTITY && !pre;
#pragma unroll
        for (int j = 0; j < TN; j++) {
            unsigned char *col = smem + (wn * WTN + j * 32 + l32) * 2 + (wm * WTM + 4 * h) * PITCH;
#pragma unroll
            for (int i = 0; i < TM; i++) {
#pragma unroll
                for (int rq = 0; rq < 4; rq++) {
                    const f32x4 bv = *(const f32x4 *)&bias_s[wm * WTM + i * 32 + 8 * rq + 4 * h];
#pragma unroll
                    for (int rr = 0; rr < 4; rr++) {
                        float v = acc[i][j][4 * rq + rr] + bv[rr];
                        if (ACT == ACT_CLAMP) {
                            if (clamp)
                                v = clamp_med3(v, a.clamp_lo, a.clamp_hi);
                        } else if (!pre)
                            v = apply_act(v, a.act);
                        *(uint16_t *)(col + (i * 32 + 8 * rq + rr) * PITCH) = to_bf16(v).bits;
                    }
                }
            }
        }
        __syncthreads();
        const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc(a.y, 0, a.y_bytes, 0x00020000);
        auto store_runs = [&](auto pxv_c) {
            constexpr int PXV = decltype(pxv_c)::value;
            constexpr int RUNS = BN / PXV; // per row
            static_assert((BM * RUNS) % (4 * kThreads) == 0, "runs are dealt to the threads in batches of four");
            static_assert(kThreads % RUNS == 0, "a thread keeps its column of runs: q += kThreads only moves the row");
            // run q = row * RUNS + cp of the staged tile; the image and pixel of a thread's runs are found once
            const int cp = tid % RUNS, row_t = tid / RUNS;
            const int n_run = n0 + cp * PXV;
            const int b_run = (int)fast_div((uint32_t)n_run, a.ohw_magic, a.ohw_shift);
            const uint32_t col_off = (uint32_t)(((b_run * a.Cout + g * a.M + m0) * a.OHW + (n_run - b_run * a.OHW)) * 2);
            const uint32_t row_pitch = (uint32_t)a.OHW * 2u;
            const int rows_ok = n_run < a.N ? a.M - m0 : 0;
            const unsigned char *src_t = smem + row_t * PITCH + cp * (PXV * 2);
            auto run_offset = [&](int q) { // byte offset in y of run q (q = tid + a multiple of kThreads; out of range: nothing is stored)
                const int row = row_t + (q - tid) / RUNS;
                return row < rows_ok ? col_off + (uint32_t)row * row_pitch : kOutOfRange;
            };
            auto run_source = [&](int q) { return src_t + ((q - tid) / RUNS) * PITCH; };
            if (pre) {
                // y = act(staged value + factor * old y): the old runs of four runs are requested together (loads of the stores'
                // width), so that a thread waits for memory twice per tile and not eight times
                for (int q0 = tid; q0 < BM * RUNS; q0 += 4 * kThreads) {
                    uint32_t voff[4], old[4][PXV / 2];
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        voff[u] = run_offset(q0 + u * kThreads);
                        if constexpr (PXV == 8) {
                            const u32x4 o = __builtin_amdgcn_raw_buffer_load_b128(yr, voff[u], 0, 0);
                            old[u][0] = o[0], old[u][1] = o[1], old[u][2] = o[2], old[u][3] = o[3];
                        } else if constexpr (PXV == 4) {
                            const u32x2 o = __builtin_amdgcn_raw_buffer_load_b64(yr, voff[u], 0, 0);
                            old[u][0] = o[0], old[u][1] = o[1];
                        } else
                            old[u][0] = __builtin_amdgcn_raw_buffer_load_b32(yr, voff[u], 0, 0);
                    }
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        const int q = q0 + u * kThreads;
                        const unsigned char *src = run_source(q);
                        uint32_t mine[PXV / 2];
#pragma unroll
                        for (int d = 0; d < PXV / 2; d++) {
                            mine[d] = ((const uint32_t *)src)[d];
                            float lo = fmaf(__builtin_bit_cast(float, old[u][d] << 16), a.factor, __builtin_bit_cast(float, mine[d] << 16));
                            float hi = fmaf(__builtin_bit_cast(float, old[u][d] & 0xFFFF0000u), a.factor, __builtin_bit_cast(float, mine[d] & 0xFFFF0000u));
                            if (ACT == ACT_CLAMP) {
                                if (a.act != DLP_ACT_IDENTITY) {
                                    lo = clamp_med3(lo, a.clamp_lo, a.clamp_hi);
                                    hi = clamp_med3(hi, a.clamp_lo, a.clamp_hi);
                                }
                            } else {
                                lo = apply_act(lo, a.act);
                                hi = apply_act(hi, a.act);
                            }
                            mine[d] = (uint32_t)to_bf16(lo).bits | ((uint32_t)to_bf16(hi).bits << 16);
                        }
                        if constexpr (PXV == 8) {
                            u32x4 o;
                            o[0] = mine[0], o[1] = mine[1], o[2] = mine[2], o[3] = mine[3];
                            __builtin_amdgcn_raw_buffer_store_b128(o, yr, voff[u], 0, DLP_BF16_STORE_AUX);
                        } else if constexpr (PXV == 4) {
                            u32x2 o;
                            o[0] = mine[0], o[1] = mine[1];
                            __builtin_amdgcn_raw_buffer_store_b64(o, yr, voff[u], 0, 0);
                        } else
                            __builtin_amdgcn_raw_buffer_store_b32(mine[0], yr, voff[u], 0, 0);
                    }
                }
                return;
            }
#pragma unroll 4
            for (int q = tid; q < BM * RUNS; q += kThreads) {
                const uint32_t voff = run_offset(q);
                const unsigned char *src = run_source(q);
                if constexpr (PXV == 8)
                    __builtin_amdgcn_raw_buffer_store_b128(*(const u32x4 *)src, yr, voff, 0, DLP_BF16_STORE_AUX);
                else if constexpr (PXV == 4)
                    __builtin_amdgcn_raw_buffer_store_b64(*(const u32x2 *)src, yr, voff, 0, 0);
                else
                    __builtin_amdgcn_raw_buffer_store_b32(*(const uint32_t *)src, yr, voff, 0, 0);
            }
        };
        if (a.pxv == 8)
            store_runs(std::integral_constant<int, 8>{});
        else if (a.pxv == 4)
            store_runs(std::integral_constant<int, 4>{});
        else
            store_runs(std::integral_constant<int, 2>{});
        return;
    }
    if (a.factor == 0.0f && (a.M & 7) == 0 && a.y_bytes != 0) {
        const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc(a.y, 0, a.y_bytes, 0x00020000);
        const bool clamp = a.act != DLP_ACT_IDENTITY;
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int n = n0 + wn * WTN + j * 32 + l32;
            const int b = (int)fast_div((uint32_t)n, a.ohw_magic, a.ohw_shift);
            const int pix = n - b * a.OHW;
            const uint32_t voff = n < a.N ? (uint32_t)(((b * a.Cout + g * a.M + m0 + wm * WTM + 4 * h) * a.OHW + pix) * 2) : kOutOfRange;
#pragma unroll
            for (int i = 0; i < TM; i++) {
#pragma unroll
                for (int rq = 0; rq < 4; rq++) {
                    const int mrow = wm * WTM + i * 32 + 8 * rq; // + 4*h + (r & 3); uniform part
                    if (m0 + mrow >= a.M)
                        continue;
                    const f32x4 bv = *(const f32x4 *)&bias_s[mrow + 4 * h];
#pragma unroll
                    for (int rr = 0; rr < 4; rr++) {
                        float v = acc[i][j][4 * rq + rr] + bv[rr];
                        if (ACT == ACT_CLAMP) {
                            if (clamp)
                                v = clamp_med3(v, a.clamp_lo, a.clamp_hi);
                        } else
                            v = apply_act(v, a.act);
                        __builtin_amdgcn_raw_buffer_store_b16((short)to_bf16(v).bits, yr, voff, (uint32_t)((i * 32 + 8 * rq + rr) * a.OHW * 2), 0);
                    }
                }
            }
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int n = n0 + wn * WTN + j * 32 + l32;
        if (n >= a.N)
            continue;
        const int b = (int)fast_div((uint32_t)n, a.ohw_magic, a.ohw_shift);
        const int pix = n - b * a.OHW;
        bf16_t *yb = (bf16_t *)a.y + ((size_t)b * a.Cout + (size_t)g * a.M) * a.OHW + pix;
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + wm * WTM + i * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                if (m < a.M) {
                    float v = acc[i][j][r];
                    if (a.bias)
                        v += a.bias[g * a.M + m];
                    const bool pre = a.pre != 0 && a.factor != 0.0f;
                    if (pre)
                        v = fmaf(to_float(yb[(size_t)m * a.OHW]), a.factor, v);
                    if (ACT == ACT_CLAMP) {
                        if (a.act != DLP_ACT_IDENTITY)
                            v = clamp_med3(v, a.clamp_lo, a.clamp_hi);
                    } else
                        v = apply_act(v, a.act);
                    store_out(yb + (size_t)m * a.OHW, v, pre ? 0.0f : a.factor);
                }
            }
        }
    }
}

// PXL > 0 selects the dense loader (1x1, stride 1, no padding: a plain GEMM W * X per image):
// a lane loads PXL consecutive pixels of 8 consecutive channels with 8- or 16-byte loads (the
// texture path handles four lanes per clock whatever the width of the load, so a 16-bit load per
// element is an eighth of its rate), transposes the 8 x PXL block in registers (one v_perm per
// dword) and stores each pixel's 8 channels as one 16-byte piece.  The B tile is then kept as
// [8-channel group][pixel][8 channels] with the pixel index XOR-swizzled (pixel ^ (pixel / 8 % 8))
// so that both these stores (pixels PXL apart across lanes) and the operand reads (consecutive
// pixels across lanes) are free of bank conflicts.  64 * 4 / PXL lanes suffice for a tile, so the
// B tiles are dealt to the wavefronts in turn (LW wavefronts per tile).
// SX = 2: the same for 1x1 stride-2 convolutions whose output width is a multiple of PXL: a lane
// loads 2 * PXL consecutive input pixels of an even input row and keeps the even ones.
// XT = 1: a.x is the channels-last copy of the input ([image][pixel][channel], made by stage_channels_last_kernel; a.H, a.W,
// a.sh, a.sw describe that copy): a pixel's 32 channels of a K tile are 64 consecutive bytes, four 16-byte pieces that go to
// LDS as they come, exactly like the weight tile.  Any kernel extent, stride, padding and image size.
template <int BM, int BN, int WM, int WN, int ORDER, int ACT, int NSET, int PXL, int SX = 1, int XT = 0>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu((BM == 128 || PXL == 8 || (PXL == 4 && SX == 1) || XT == 1) ? 3 : 2))) void conv_gemm_bf16_kernel(GemmArgs a)
{
    static_assert(PXL == 0 || ((PXL == 2 || PXL == 4 || PXL == 8) && PXL * SX >= 4 && PXL * SX <= 8 && ORDER == GEMM_ORDER_TAP_BF16),
                  "dense loader variants: loads of 8 or 16 bytes");
    static_assert(XT == 0 || (PXL == 0 && ORDER == GEMM_ORDER_TAP_BF16), "the channels-last loader is a tap-major gather");
    static_assert(WM * WN == 4, "four wavefronts per workgroup");
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    static_assert(TM >= 1 && TN >= 1 && WTM % 32 == 0 && WTN % 32 == 0, "tile shape");
    constexpr int KSPLIT = kThreads / BN;   // channel groups among the B loader threads
    static_assert(KSPLIT >= 1 && BN % 64 == 0 && BK2 % KSPLIT == 0, "B loader shape");
    constexpr int B_LD = BK2 / KSPLIT;      // channels per thread per K tile
    static_assert(B_LD % 8 == 0, "a thread stores whole 16-byte pieces");
    constexpr int A_V4 = BM * BK2 * 2 / 16; // 16-byte pieces of a packed A tile
    static_assert(A_V4 % kThreads == 0, "A loader shape");
    constexpr int A_LD = A_V4 / kThreads;

    constexpr int A_TILE_BYTES = BM * LDK * 2, B_TILE_BYTES = BN * LDK * 2;
    __shared__ __attribute__((aligned(16))) unsigned char smem[2 * A_TILE_BYTES + 2 * B_TILE_BYTES];
    auto As = reinterpret_cast<uint16_t(*)[BM][LDK]>(smem);
    auto Bs = reinterpret_cast<uint16_t(*)[BN][LDK]>(smem + 2 * A_TILE_BYTES);
    unsigned char *const bs_bytes = smem + 2 * A_TILE_BYTES;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int h = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;

    int t; // XCD-aware renumbering, as in the fp32 kernel
    {
        const int nb = gridDim.x, bid = blockIdx.x;
        const int q = nb >> 3, r = nb & 7;
        const int xcd = bid & 7, slot = bid >> 3;
        t = (xcd < r) ? xcd * (q + 1) + slot : r * (q + 1) + (xcd - r) * q + slot;
    }
    const int tm = (int)fast_div((uint32_t)t, a.mt_magic, a.mt_shift);
    const int mt = t - tm * a.mtiles;
    const int tn = (int)fast_div((uint32_t)tm, a.ntl_magic, a.ntl_shift);
    const int nt = tm - tn * a.ntiles;
    const int slice = (int)fast_div((uint32_t)tn, a.gr_magic, a.gr_shift);
    const int g = tn - slice * a.groups;
    const int m0 = mt * BM, n0 = nt * BN;
    const int kt_begin = slice * a.kt_per_slice;
    const int kt_end = min(kt_begin + a.kt_per_slice, a.nkt);
    // the bias of the tile's rows, for the epilogue: in LDS long before it is wanted (the barriers of the main loop lie between)
    __shared__ float bias_early[BM];
    if (tid < BM)
        bias_early[tid] = (a.bias && m0 + tid < a.M) ? a.bias[g * a.M + m0 + tid] : 0.0f;

    const __amdgpu_buffer_rsrc_t xr =
        __builtin_amdgcn_make_buffer_rsrc((void *)((const char *)a.x - a.x_shift), 0, a.x_bytes + a.x_shift, 0x00020000);
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)a.wp, 0, a.wp_bytes, 0x00020000);
    ConstInt *ktab = (ConstInt *)a.ktab;

    // ---- per-thread gather state: one output pixel, B_LD channels of every K tile ----
    const int p = tid % BN;
    const int ks = (KSPLIT == 1) ? 0 : __builtin_amdgcn_readfirstlane(tid / BN);
    uint32_t vbase;
    uint32_t my = 0, mx = 0; // tap-major: my = tap mask; channel-major: row / column masks
    {
        const int n = n0 + p;
        const int b = (int)fast_div((uint32_t)n, a.ohw_magic, a.ohw_shift);
        const int pix = n - b * a.OHW;
        const int oy = (int)fast_div((uint32_t)pix, a.ow_magic, a.ow_shift);
        const int ox = pix - oy * a.OW;
        const int iy0 = oy * a.sh - a.ph;
        const int ix0 = ox * a.sw - a.pw;
        vbase = (uint32_t)((((b * a.Cin + g * a.Cin_g) * a.H + oy * a.sh) * a.W + ox * a.sw) * 2);
        if (n < a.N) {
            uint32_t ry = 0, rx = 0;
            for (int ky = 0; ky < a.KH; ky++) {
                int yy = iy0 + ky * a.dh;
                if (yy >= 0 && yy < a.H)
                    ry |= 1u << ky;
            }
            for (int kx = 0; kx < a.KW; kx++) {
                int xx = ix0 + kx * a.dw;
                if (xx >= 0 && xx < a.W)
                    rx |= 1u << kx;
            }
            if (ORDER == GEMM_ORDER_TAP_BF16) {
                for (int ky = 0; ky < a.KH; ky++)
                    if ((ry >> ky) & 1u)
                        my |= rx << (ky * a.KW);
            } else {
                my = ry;
                mx = rx;
            }
        }
    }

    // channels-last loader: B_PC 16-byte pieces per thread and K tile; piece = (pixel (tid / 4) + 64 j, channels 8 (tid % 4) ..)
    constexpr int B_PC = BN * 4 / kThreads;
    uint32_t xbase[B_PC], xmask[B_PC];
    if constexpr (XT) {
#pragma unroll
        for (int j = 0; j < B_PC; j++) {
            const int n = n0 + (tid >> 2) + j * (kThreads / 4);
            xbase[j] = kOutOfRange;
            xmask[j] = 0;
            if (n < a.N) {
                const int b = (int)fast_div((uint32_t)n, a.ohw_magic, a.ohw_shift);
                const int pix = n - b * a.OHW;
                const int oy = (int)fast_div((uint32_t)pix, a.ow_magic, a.ow_shift);
                const int ox = pix - oy * a.OW;
                const int iy0 = oy * a.sh - a.ph;
                const int ix0 = ox * a.sw - a.pw;
                xbase[j] = (uint32_t)((((b * a.H + oy * a.sh) * a.W + ox * a.sw) * a.Cin + g * a.Cin_g) * 2 + (tid & 3) * 16);
                uint32_t rx = 0;
                for (int kx = 0; kx < a.KW; kx++) {
                    const int xx = ix0 + kx * a.dw;
                    if (xx >= 0 && xx < a.W)
                        rx |= 1u << kx;
                }
                for (int ky = 0; ky < a.KH; ky++) {
                    const int yy = iy0 + ky * a.dh;
                    if (yy >= 0 && yy < a.H)
                        xmask[j] |= rx << (ky * a.KW);
                }
            }
        }
    }

    // A loader: 16-byte pieces of the packed tile, in tile order -- or, for 1x1 convolutions, of the weight
    // matrix itself ([Cout][Cin] has k innermost already: a tile row is 64 bytes of a matrix row, a.wp is w)
    uint32_t a_tile_bytes = BM * BK2 * 2;
    uint32_t a_row_base = (uint32_t)((g * a.mtiles + mt) * a.nkt) * a_tile_bytes;
    uint32_t a_voff[A_LD];
#pragma unroll
    for (int j = 0; j < A_LD; j++)
        a_voff[j] = (uint32_t)(tid + j * kThreads) * 16u;
    if (a.wdirect) {
        a_tile_bytes = BK2 * 2;
        a_row_base = 0;
#pragma unroll
        for (int j = 0; j < A_LD; j++) {
            const int idx = tid + j * kThreads, m = m0 + (idx >> 2);
            a_voff[j] = m < a.M ? (uint32_t)(g * a.M + m) * (uint32_t)a.K * 2u + (uint32_t)(idx & 3) * 16u : kOutOfRange;
        }
    }

    // ---- dense loader state: block = 8 channels x PXL pixels; blocks of a tile = 4 * BN / PXL ----
    constexpr int PXN = PXL ? PXL : 1;
    constexpr int NPQ = BN / PXN;                  // pixel groups of a tile
    constexpr int LW = PXL ? 4 * NPQ / 64 : 4;     // wavefronts that load one B tile
    constexpr int NSETB = NSET * LW / 4 ? NSET * LW / 4 : 1; // a wavefront loads every 4/LW-th tile: that many fewer register sets
    constexpr int DW = PXL ? PXL * SX / 2 : 1;     // dwords per load
    static_assert(LW == 1 || LW == 2 || LW == 4, "loader wavefronts");
    uint32_t dvoff = kOutOfRange; // byte offset of (first channel of the block, first pixel) in x
    uint32_t dslot[PXN];          // LDS byte offsets of the block's pixels inside a B tile
    uint32_t brd[TN];             // LDS byte offset of this lane's operand pixel (channel group h)
    uint32_t rbw[NSETB][8][DW];
    const int my_turn = wave / LW; // tile T is loaded by this wavefront when T % (4 / LW) == my_turn
    if constexpr (PXL > 0) {
        const int blk = (wave % LW) * 64 + lane;
        const int oct = blk / NPQ, pq = blk % NPQ;
        const int n = n0 + pq * PXL; // PXL divides OH*OW (stride 2: OW): the run stays inside one image (one row)
        if (n < a.N) {
            const int b = (int)fast_div((uint32_t)n, a.ohw_magic, a.ohw_shift);
            const int pix = n - b * a.OHW;
            uint32_t in_pix = (uint32_t)pix;
            if (SX == 2) {
                const int oy = (int)fast_div((uint32_t)pix, a.ow_magic, a.ow_shift);
                in_pix = (uint32_t)(oy * 2 * a.W + (pix - oy * a.OW) * 2);
            }
            dvoff = (uint32_t)(b * a.Cin + g * a.Cin_g + oct * 8) * a.hw4 + in_pix * 2u;
        }
#pragma unroll
        for (int q = 0; q < PXN; q++) {
            const int x = pq * PXL + q;
            dslot[q] = (uint32_t)((oct * BN + (x ^ ((x >> 3) & 7))) * 16);
        }
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int x = wn * WTN + j * 32 + l32;
            brd[j] = (uint32_t)((h * BN + (x ^ ((x >> 3) & 7))) * 16);
        }
    }
    auto my_tile = [&](int kt) { return LW == 4 || (kt & (4 / LW - 1)) == my_turn; };
    auto load_b = [&](auto set, int kt) {
        constexpr int S = (decltype(set)::value * LW / 4) % NSETB;
        const uint32_t soff = (uint32_t)(kt * BK2) * a.hw4;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if constexpr (DW == 4) {
                const u32x4 v = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(xr, dvoff, soff + (uint32_t)i * a.hw4, 0));
#pragma unroll
                for (int d = 0; d < DW; d++)
                    rbw[S][i][d] = v[d];
            } else if constexpr (DW == 2) {
                const u32x2 v = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(xr, dvoff, soff + (uint32_t)i * a.hw4, 0));
#pragma unroll
                for (int d = 0; d < DW; d++)
                    rbw[S][i][d] = v[d];
            }
        }
    };
    auto store_b = [&](auto set, auto buf_c) {
        constexpr int S = (decltype(set)::value * LW / 4) % NSETB;
        constexpr int BUF = decltype(buf_c)::value;
#pragma unroll
        for (int q = 0; q < PXN; q++) {
            u32x4 v;
#pragma unroll
            for (int j = 0; j < 4; j++) { // channels 2j (low half) and 2j+1 of pixel q
                if constexpr (SX == 2) // pixel q is the low half of dword q
                    v[j] = __builtin_amdgcn_perm(rbw[S][2 * j + 1][q], rbw[S][2 * j][q], 0x05040100u);
                else
                    v[j] = __builtin_amdgcn_perm(rbw[S][2 * j + 1][q / 2], rbw[S][2 * j][q / 2], (q & 1) ? 0x07060302u : 0x05040100u);
            }
            *(u32x4 *)(bs_bytes + BUF * B_TILE_BYTES + dslot[q]) = v;
        }
    };

    // NSET register sets hold the tiles in flight: at K step i they hold tiles i+1 .. i+NSET; the
    // step stores tile i+1 to LDS and at once reuses that set for the loads of tile i+NSET+1, so a
    // load has NSET K steps to land (one step is only a few hundred matrix cycles here).
    u32x4 ra[NSET][A_LD];
    uint32_t rb[NSET][B_LD]; // one bf16 each, zero extended
    uint32_t vsel[NSET];
    u32x4 rbx[NSET][B_PC];   // channels-last loader: the pieces as they come

    auto load_half = [&](auto set, int kt, auto half_c) {
        constexpr int S = decltype(set)::value;
        constexpr int Q = decltype(half_c)::value;
        // tiles past the end of this workgroup's K range are never multiplied: no loads for them (with two or four K tiles in
        // all, as in the 1x1 layers of 64 or 128 channels, they would be more than half of all loads); a uniform branch
        if (kt >= kt_end)
            return;
        if (Q == 0) {
            const uint32_t a_soff = a_row_base + (uint32_t)kt * a_tile_bytes;
#pragma unroll
            for (int j = 0; j < A_LD; j++)
                ra[S][j] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(wr, a_voff[j], a_soff, 0));
        }
        if constexpr (PXL > 0) {
            if (Q == 1 && my_tile(kt))
                load_b(set, kt);
        } else if constexpr (XT) {
            // table entry of a K tile: {byte offset of (tap, channel block) in the channels-last copy, tap bit, -, -}
            ConstInt *e = ktab + kt * 4;
            const uint32_t xoff = (uint32_t)e[0], tap = (uint32_t)e[1];
            constexpr int PH = B_PC / 2 ? B_PC / 2 : 1;
#pragma unroll
            for (int j = Q * PH; j < (Q + 1) * PH && j < B_PC; j++) {
                const uint32_t m = (uint32_t)__builtin_amdgcn_sbfe((int)xmask[j], tap, 1u);
                rbx[S][j] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(xr, opaque((xbase[j] & m) | (kOutOfRange & ~m)), xoff, 0));
            }
        } else if (ORDER == GEMM_ORDER_TAP_BF16) {
            // table entry of a K tile: {x byte offset of (channel block, tap), tap bit, -, -}
            ConstInt *e = ktab + kt * 4;
            const uint32_t xoff = (uint32_t)e[0], tap = (uint32_t)e[1];
            if (Q == 0) {
                // bit `tap` of the pixel's tap mask, spread over a word, picks the offset (two VALU operations)
                const uint32_t m = (uint32_t)__builtin_amdgcn_sbfe((int)my, tap, 1u);
                vsel[S] = opaque((vbase & m) | (kOutOfRange & ~m));
            }
#pragma unroll
            for (int i = Q * (B_LD / 2); i < (Q + 1) * (B_LD / 2); i++)
                rb[S][i] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(xr, vsel[S], xoff + (uint32_t)(ks * B_LD + i) * a.hw4, 0);
        } else {
            // channel-major (Cin/groups not a multiple of 32, e.g. the 3-channel stem): one table
            // entry per k = {x byte offset of (c, ky, kx), ky | kx << 8}
            ConstInt *e = ktab + (kt * BK2 + ks * B_LD) * 2;
#pragma unroll
            for (int i = Q * (B_LD / 2); i < (Q + 1) * (B_LD / 2); i++) {
                const uint32_t xoff = (uint32_t)e[2 * i], tap = (uint32_t)e[2 * i + 1];
                const bool ok = ((my >> (tap & 0xff)) & (mx >> (tap >> 8)) & 1u) != 0;
                rb[S][i] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(xr, opaque(ok ? vbase : kOutOfRange), xoff, 0);
            }
        }
    };
    // kt = the tile that set S holds
    auto store_half = [&](auto set, auto buf_c, auto half_c, int kt) {
        constexpr int S = decltype(set)::value;
        constexpr int BUF = decltype(buf_c)::value;
        constexpr int Q = decltype(half_c)::value;
        if (kt >= kt_end) // nothing was loaded for it (load_half)
            return;
        if (Q == 0) {
#pragma unroll
            for (int j = 0; j < A_LD; j++) {
                const int idx = tid + j * kThreads; // 16-byte piece of the [BM][32] tile: row idx/4, piece idx%4
                *(u32x4 *)&As[BUF][idx >> 2][(idx & 3) * 8] = ra[S][j];
            }
        }
        if constexpr (PXL > 0) {
            if (Q == 0 && my_tile(kt))
                store_b(set, buf_c);
            return;
        }
        if constexpr (XT) {
            constexpr int PH = B_PC / 2 ? B_PC / 2 : 1;
#pragma unroll
            for (int j = Q * PH; j < (Q + 1) * PH && j < B_PC; j++)
                *(u32x4 *)&Bs[BUF][(tid >> 2) + j * (kThreads / 4)][(tid & 3) * 8] = rbx[S][j];
            return;
        }
#pragma unroll
        for (int q = Q * (B_LD / 16); q < (Q + 1) * (B_LD / 16); q++) {
            u32x4 v;
#pragma unroll
            for (int d = 0; d < 4; d++)
                v[d] = rb[S][8 * q + 2 * d] | (rb[S][8 * q + 2 * d + 1] << 16);
            *(u32x4 *)&Bs[BUF][p][ks * B_LD + 8 * q] = v;
        }
    };
    static_assert(B_LD % 16 == 0, "each half of a K step stores whole pieces");

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[i][j][r] = 0.0f;

    // K step i (compile-time residue mod NSET) on tile kt = kt_begin + i, resident in LDS[i % 2]
    auto k_step = [&](auto step_c, int kt) {
        constexpr int STEP = decltype(step_c)::value;
        constexpr int BUF = STEP & 1;
        using NextBuf = std::integral_constant<int, BUF ^ 1>;
        const std::integral_constant<int, (STEP + 1) % NSET> set{};
        bf16x8 fa[2][TM], fb[2][TN];
#pragma unroll
        for (int s = 0; s < 2; s++) {
#pragma unroll
            for (int i = 0; i < TM; i++)
                fa[s][i] = *(const bf16x8 *)&As[BUF][wm * WTM + i * 32 + l32][s * 16 + h * 8];
#pragma unroll
            for (int j = 0; j < TN; j++) {
                if constexpr (PXL > 0)
                    fb[s][j] = *(const bf16x8 *)(bs_bytes + BUF * B_TILE_BYTES + brd[j] + s * (2 * BN * 16));
                else
                    fb[s][j] = *(const bf16x8 *)&Bs[BUF][wn * WTN + j * 32 + l32][s * 16 + h * 8];
            }
        }
        store_half(set, NextBuf{}, std::integral_constant<int, 0>{}, kt + 1);
        load_half(set, kt + NSET + 1, std::integral_constant<int, 0>{});
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[0][i], fb[0][j], acc[i][j], 0, 0, 0);
        store_half(set, NextBuf{}, std::integral_constant<int, 1>{}, kt + 1);
        load_half(set, kt + NSET + 1, std::integral_constant<int, 1>{});
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[1][i], fb[1][j], acc[i][j], 0, 0, 0);
        __syncthreads();
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    static_assert(NSET == 2 || NSET == 4, "the K loop is unrolled NSET times");
    load_half(I0{}, kt_begin, I0{});
    load_half(I0{}, kt_begin, I1{});
    load_half(I1{}, kt_begin + 1, I0{});
    load_half(I1{}, kt_begin + 1, I1{});
    if constexpr (NSET == 4) {
        load_half(I2{}, kt_begin + 2, I0{});
        load_half(I2{}, kt_begin + 2, I1{});
        load_half(I3{}, kt_begin + 3, I0{});
        load_half(I3{}, kt_begin + 3, I1{});
    }
    store_half(I0{}, I0{}, I0{}, kt_begin);
    store_half(I0{}, I0{}, I1{}, kt_begin);
    load_half(I0{}, kt_begin + NSET, I0{});
    load_half(I0{}, kt_begin + NSET, I1{});
    __syncthreads();
    int kt = kt_begin;
    for (; kt + NSET - 1 < kt_end; kt += NSET) {
        k_step(I0{}, kt);
        k_step(I1{}, kt + 1);
        if constexpr (NSET == 4) {
            k_step(I2{}, kt + 2);
            k_step(I3{}, kt + 3);
        }
    }
    if (kt < kt_end)
        k_step(I0{}, kt);
    if constexpr (NSET == 4) {
        if (kt + 1 < kt_end)
            k_step(I1{}, kt + 1);
        if (kt + 2 < kt_end)
            k_step(I2{}, kt + 2);
    }

    static_assert(BM * (BN * 2 + 16) + BM * 4 <= (int)sizeof(smem), "the staged output tile fits the operand buffers");
    static_assert(BN * (BM * 2 + 16) + BM * 4 <= (int)sizeof(smem), "and so does the channels-last one");
    bf16_tile_output<BM, BN, WM, WN, ACT>(a, acc, smem, (int)sizeof(smem), m0, n0, g, slice, wm, wn, h, l32, tid, bias_early);
}

#ifndef DLP_PATCH_BF16_NA
#define DLP_PATCH_BF16_NA 3
#endif
// ---- stride-1 3x3 "same" convolutions on the bf16 matrix instruction: the input patch goes through LDS once ----
// The bf16 counterpart of conv_patch_f32_kernel.  A K stage = 32 input channels: the pixels that the
// nine taps of the tile's BN output pixels read -- one run of consecutive plane pixels per image the
// tile touches, BN + 2*(W+1) in all -- are loaded once per stage with 8- or 16-byte loads (PXP pixels
// of 8 channels per lane), transposed in registers like the dense loader's blocks, and kept in LDS as
// [8-channel group][patch row][8 channels] (rows in order: the reads of consecutive lanes are then
// consecutive 16-byte pieces whatever the tap's shift, free of bank conflicts; the few stores per
// stage, 8 rows apart across lanes, are not).  The B operand of tap (ky,kx) is a 16-byte LDS read at
// (lane's patch row + (ky-1)*W + (kx-1)); taps that fall into the padding read a row that is always zero.  Compared with gathering every tap from memory with
// 16-bit loads this is 9 * 8 times fewer trips through the texture path, which is what bounds that
// kernel.  Runs start on multiples of PXP pixels of their plane (H*W % PXP == 0), so every load is
// dword aligned.  Weights: the packed tap-major tiles of conv_gemm_bf16_kernel (K tile = stage * 9 + tap), read from memory
// straight into the matrix instruction's registers (a wavefront owns 32 filters and all the pixels of the tile: WM x WN = 4 x 1
// on the 128 x 128 tile, 2 x 2 on 64 x 256), so that the patch is the only thing ever stored to LDS and a stage needs one barrier.
template <int BM, int BN, int WM, int WN, int PITCH, int PXP, int ACT>
__global__ __launch_bounds__(kThreads) void conv_patch_bf16_kernel(GemmArgs a)
{
    constexpr int KHW = 9;
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    static_assert(TM == 1 && WM * WN == 4, "a wavefront owns 32 filters: its share of a weight tile is one operand per half K tile");
    constexpr int P_BUF_BYTES = 4 * PITCH * 16;
    constexpr int MAXSEG = 3;           // images a tile may touch (H*W >= BN / 2 + 1 is checked by the host)
    constexpr int DW = PXP / 2;         // dwords per load
    constexpr int ZERO_ROW = PITCH - 1; // its aligned group of 8 rows is never loaded
    static_assert(PITCH % 8 == 0 && (PXP == 4 || PXP == 8), "patch shape");
    constexpr int NA = DLP_PATCH_BF16_NA; // register sets of weight operands: tile kt + NA is requested when tile kt has been multiplied
    static_assert((2 * KHW) % NA == 0, "the register sets rotate with a period that divides a pair of stages");
    constexpr int OUT_BYTES = (BM * (BN * 2 + 16) > BN * (BM * 2 + 16) ? BM * (BN * 2 + 16) : BN * (BM * 2 + 16)) + BM * 4; // the staged output tile
    constexpr int SMEM_BYTES = 2 * P_BUF_BYTES > OUT_BYTES ? 2 * P_BUF_BYTES : OUT_BYTES;

    __shared__ __attribute__((aligned(16))) unsigned char smem[SMEM_BYTES];
    unsigned char *const ps_bytes = smem;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int h = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;

    int t; // XCD-aware renumbering, as in the other kernels
    {
        const int nb = gridDim.x, bid = blockIdx.x;
        const int q = nb >> 3, r = nb & 7;
        const int xcd = bid & 7, slot = bid >> 3;
        t = (xcd < r) ? xcd * (q + 1) + slot : r * (q + 1) + (xcd - r) * q + slot;
    }
    const int tm = (int)fast_div((uint32_t)t, a.mt_magic, a.mt_shift);
    const int mt = t - tm * a.mtiles;
    const int g = (int)fast_div((uint32_t)tm, a.ntl_magic, a.ntl_shift);
    const int nt = tm - g * a.ntiles;
    const int m0 = mt * BM, n0 = nt * BN;
    const int ncb = a.nkt / KHW; // stages
    // the bias of the tile's rows, for the epilogue: in LDS long before it is wanted (the barriers of the main loop lie between)
    __shared__ float bias_early[BM];
    if (tid < BM)
        bias_early[tid] = (a.bias && m0 + tid < a.M) ? a.bias[g * a.M + m0 + tid] : 0.0f;

    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)a.wp, 0, a.wp_bytes, 0x00020000);

    // ---- the tile's patch: one segment of consecutive plane pixels per image, PXP-aligned at both ends ----
    const int HW = a.OHW;
    const int halo = a.W + 1;
    const int n_last = min(n0 + BN, a.N) - 1;
    const int b0 = (int)fast_div((uint32_t)n0, a.ohw_magic, a.ohw_shift);
    int seg_row[MAXSEG], seg_a[MAXSEG], seg_len[MAXSEG];
    {
        int row = 0;
#pragma unroll
        for (int s = 0; s < MAXSEG; s++) {
            const int base = (b0 + s) * HW;
            const int first = max(n0, base), last = min(n_last, base + HW - 1);
            int as = 0, len = 0;
            if (first <= last) {
                as = max(0, first - base - halo) & ~(PXP - 1);
                len = ((min(HW, last - base + 1 + halo) + PXP - 1) & ~(PXP - 1)) - as;
            }
            seg_row[s] = row;
            seg_a[s] = as;
            seg_len[s] = len;
            row += len;
        }
    }
    // loader: this lane's block = 8 channels (group oct) x patch rows [rho0, rho0 + PXP)
    const int nbr = a.pp_nbr; // row blocks of the largest patch of this launch
    const bool loader = tid < 4 * nbr;
    const int oct = tid / nbr, rho0 = (tid - oct * nbr) * PXP;
    uint32_t pvoff = kOutOfRange;
    uint32_t dslot[PXP];
    if (loader) {
#pragma unroll
        for (int s = 0; s < MAXSEG; s++) {
            const int d = rho0 - seg_row[s];
            if (d >= 0 && d < seg_len[s])
                pvoff = (uint32_t)((b0 + s) * a.Cin + g * a.Cin_g + oct * 8) * a.hw4 + (uint32_t)(seg_a[s] + d) * 2u;
        }
    }
#pragma unroll
    for (int q = 0; q < PXP; q++)
        dslot[q] = (uint32_t)(((oct & 3) * PITCH + rho0 + q) * 16);
    // this lane's B operands (channel group h of a k step, pixel l32 of block j) per tap: byte offset in a patch buffer
    uint32_t baddr[TN][KHW];
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int n = n0 + wn * WTN + j * 32 + l32;
        const bool vn = n < a.N;
        const int b = (int)fast_div((uint32_t)n, a.ohw_magic, a.ohw_shift);
        const int pix = n - b * HW;
        const int oy = (int)fast_div((uint32_t)pix, a.ow_magic, a.ow_shift);
        const int ox = pix - oy * a.OW;
        const int s = b - b0;
        const int row = pix + (s == 0 ? seg_row[0] - seg_a[0] : s == 1 ? seg_row[1] - seg_a[1] : seg_row[2] - seg_a[2]);
#pragma unroll
        for (int ky = 0; ky < 3; ky++)
#pragma unroll
            for (int kx = 0; kx < 3; kx++) {
                const int yy = oy + ky - 1, xx = ox + kx - 1;
                const bool ok = vn && yy >= 0 && yy < a.H && xx >= 0 && xx < a.W;
                const int r = ok ? row + (ky - 1) * a.W + (kx - 1) : ZERO_ROW;
                baddr[j][ky * 3 + kx] = (uint32_t)((h * PITCH + r) * 16);
            }
    }
    if (tid < 8) { // the zero row of both buffers, all four channel groups
        const u32x4 z = {0u, 0u, 0u, 0u};
        *(u32x4 *)(ps_bytes + (tid >> 2) * P_BUF_BYTES + ((tid & 3) * PITCH + ZERO_ROW) * 16) = z;
    }

    // The weights never touch LDS: a wavefront's operand of a half K tile -- filter wm * 32 + l32, sixteen bytes of its row of the
    // packed tile [BM][32] -- comes from memory (the last-level caches: every workgroup reads the same tiles) straight into
    // the register the matrix instruction reads.  LDS stores run at a quarter of the rate of LDS loads on this chip (measured:
    // 67 against 200 bytes per clock and compute unit), and a weight tile written per K tile was as much LDS time as all
    // the operand reads of that K tile together.
    const uint32_t a_tile_bytes = BM * BK2 * 2;
    const uint32_t a_row_base = (uint32_t)((g * a.mtiles + mt) * a.nkt) * a_tile_bytes;
    const uint32_t a_voff = (uint32_t)((wm * 32 + l32) * (BK2 * 2) + h * 16);
    bf16x8 fa[NA][2]; // weight operands in flight: [register set][half of the K tile]
    uint32_t rbw[8][DW];
    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[i][j][r] = 0.0f;

    auto load_a = [&](auto set, int kt) {
        constexpr int S = decltype(set)::value;
        const uint32_t a_soff = a_row_base + (uint32_t)min(kt, a.nkt - 1) * a_tile_bytes;
#pragma unroll
        for (int s = 0; s < 2; s++)
            fa[S][s] = __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(wr, a_voff + (uint32_t)s * 32u, a_soff, 0));
    };
    auto load_patch = [&](int cb) {
        if (!loader)
            return;
        const uint32_t soff = (uint32_t)(cb * BK2) * a.hw4;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if constexpr (PXP == 8) {
                const u32x4 v = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(xr, pvoff, soff + (uint32_t)i * a.hw4, 0));
#pragma unroll
                for (int d = 0; d < DW; d++)
                    rbw[i][d] = v[d];
            } else {
                const u32x2 v = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(xr, pvoff, soff + (uint32_t)i * a.hw4, 0));
#pragma unroll
                for (int d = 0; d < DW; d++)
                    rbw[i][d] = v[d];
            }
        }
    };
    auto store_patch = [&](auto buf_c) {
        constexpr int PB = decltype(buf_c)::value;
        if (!loader)
            return;
#pragma unroll
        for (int q = 0; q < PXP; q++) {
            u32x4 v;
#pragma unroll
            for (int j = 0; j < 4; j++) // channels 2j (low half) and 2j+1 of patch row rho0 + q
                v[j] = __builtin_amdgcn_perm(rbw[2 * j + 1][q / 2], rbw[2 * j][q / 2], (q & 1) ? 0x07060302u : 0x05040100u);
            *(u32x4 *)(ps_bytes + PB * P_BUF_BYTES + dslot[q]) = v;
        }
    };

    // B operands of half a K tile (patch buffer PB, tap TAP, half S)
    bf16x8 fb[2][TN];
    auto read_operands = [&](auto pb_c, auto tap_c, auto s_c) {
        constexpr int S = decltype(s_c)::value;
#pragma unroll
        for (int j = 0; j < TN; j++)
            fb[S][j] = *(const bf16x8 *)(ps_bytes + decltype(pb_c)::value * P_BUF_BYTES + baddr[j][decltype(tap_c)::value] + S * (2 * PITCH * 16));
    };

    // One stage: nine K tiles (taps) on patch buffer P.  The operands of each half of a K tile are read from LDS while the
    // matrix instructions of the half before run; the weight operands of tile kt + NA are requested as soon as those of tile kt
    // have been used.  The patch of the next stage is requested during the first tap and goes to the other buffer during the
    // last one: the only LDS stores of a stage, and the only barrier (between them and the first reads of the next stage).
    auto stage = [&](auto par, int cb) {
        constexpr int P = decltype(par)::value;
        using OtherP = std::integral_constant<int, P ^ 1>;
        const bool has_next = cb + 1 < ncb;
        static_for_n<KHW>([&](auto tau_c) {
            constexpr int TAU = decltype(tau_c)::value;
            constexpr int IDX = P * KHW + TAU; // K tile counter modulo 2 * KHW
            using Set = std::integral_constant<int, IDX % NA>;
            using NextTap = std::integral_constant<int, (TAU + 1) % KHW>;
            using NextPatch = std::integral_constant<int, (TAU + 1 < KHW) ? P : (P ^ 1)>;
            const int kt = cb * KHW + TAU;
            if (TAU == KHW - 1 && has_next)
                store_patch(OtherP{});
#pragma unroll
            for (int j = 0; j < TN; j++)
                acc[0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[Set::value][0], fb[0][j], acc[0][j], 0, 0, 0);
            if (TAU == KHW - 1)
                __syncthreads();
            read_operands(NextPatch{}, NextTap{}, std::integral_constant<int, 0>{});
            if (TAU == 0 && has_next)
                load_patch(cb + 1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < TN; j++)
                acc[0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[Set::value][1], fb[1][j], acc[0][j], 0, 0, 0);
            read_operands(NextPatch{}, NextTap{}, std::integral_constant<int, 1>{});
            load_a(Set{}, kt + NA);
            __builtin_amdgcn_sched_barrier(0); // keep this order: the scheduler would sink the operand reads to their uses
        });
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    load_patch(0);
    static_for_n<NA>([&](auto set) { load_a(set, decltype(set)::value); });
    store_patch(I0{});
    __syncthreads();
    read_operands(I0{}, I0{}, I0{});
    read_operands(I0{}, I0{}, I1{});
    int cb = 0;
    for (; cb + 1 < ncb; cb += 2) {
        stage(I0{}, cb);
        stage(I1{}, cb + 1);
    }
    if (cb < ncb)
        stage(I0{}, cb);
    __syncthreads(); // the operand reads issued after the last barrier are done before LDS is reused

    bf16_tile_output<BM, BN, WM, WN, ACT>(a, acc, smem, (int)sizeof(smem), m0, n0, g, 0, wm, wn, h, l32, tid, bias_early);
}

// Channels-last copy of a bf16 input for conv_gemm_bf16_kernel<..., XT = 1>: xt[b][py][px][c] = x[b][c][py * sy][px * sx]
// (sy, sx > 1 only for a 1x1 convolution, whose stride then lives in the copy).  One workgroup transposes 64 channels of an
// image through LDS and writes 16-byte pieces (8 channels of a pixel; 8 lanes = the 128 bytes of a pixel's 64 channels).
//  MODE 0: 64 pixels per workgroup, read one element at a time (any size and alignment, strided copies);
//  MODE 1: the whole image (at most 256 pixels): 64 channels x P pixels are one contiguous run, read in 16-byte pieces;
//  MODE 2: 64 pixels per workgroup, P a multiple of 8: 16-byte pieces of 8 pixels.
// MODE 1 and 2 need x 16-byte aligned; all modes need xt 16-byte aligned and C a multiple of 8.
struct StageArgs {
    const uint16_t *x;
    uint16_t *xt;
    int C, H, W, PH, PW, sy, sx; // the copy is PH x PW pixels
    uint32_t pw_magic, pw_shift;
};
constexpr int kStageFlatPixels = 256;
template <int MODE>
__global__ __launch_bounds__(256) void stage_channels_last_kernel(StageArgs a)
{
    constexpr int PITCH = 66; // 16-bit elements per LDS row (MODE 0, 2): 33 dwords, so that the 8 x 8 reads of a piece spread over the banks
    __shared__ __attribute__((aligned(16))) uint16_t tile[MODE == 1 ? 64 * kStageFlatPixels : 64 * PITCH];
    const int P = a.PH * a.PW;
    const int p0 = MODE == 1 ? 0 : (int)blockIdx.x * 64, c0 = (int)blockIdx.y * 64, b = (int)blockIdx.z;
    const int tid = (int)threadIdx.x;
    const int pitch = MODE == 1 ? P : PITCH;
    const int nch = min(64, a.C - c0);
    if constexpr (MODE == 0) {
        const int lane = tid & 63, row = tid >> 6;
        const int p = p0 + lane;
        int src = p;
        if (a.sy != 1 || a.sx != 1) {
            const int py = (int)fast_div((uint32_t)p, a.pw_magic, a.pw_shift);
            src = py * a.sy * a.W + (p - py * a.PW) * a.sx;
        }
        const uint16_t *xp = a.x + ((size_t)b * a.C + c0) * ((size_t)a.H * a.W) + src;
#pragma unroll 4
        for (int c = row; c < 64; c += 4)
            if (p < P && c < nch)
                tile[c * PITCH + lane] = xp[(size_t)c * ((size_t)a.H * a.W)];
    } else if constexpr (MODE == 1) {
        const u32x4 *xp = reinterpret_cast<const u32x4 *>(a.x + ((size_t)b * a.C + c0) * (size_t)P);
        const int pieces = nch * P / 8; // nch is a multiple of 8
        for (int q = tid; q < pieces; q += 256)
            reinterpret_cast<u32x4 *>(tile)[q] = xp[q];
    } else {
#pragma unroll
        for (int r = 0; r < 2; r++) {
            const int q = tid + 256 * r, c = q >> 3, pg = q & 7;
            if (c < nch && p0 + 8 * pg < P) {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(a.x + ((size_t)b * a.C + c0 + c) * (size_t)P + p0 + 8 * pg);
#pragma unroll
                for (int d = 0; d < 4; d++)
                    *reinterpret_cast<uint32_t *>(&tile[c * PITCH + 8 * pg + 2 * d]) = v[d];
            }
        }
    }
    __syncthreads();
    const int npx = MODE == 1 ? P : min(64, P - p0);
    for (int q = tid; q < npx * 8; q += 256) {
        const int oct = q & 7, p = q >> 3;
        if (oct * 8 < nch) {
            u32x4 v;
#pragma unroll
            for (int d = 0; d < 4; d++)
                v[d] = (uint32_t)tile[(oct * 8 + 2 * d) * pitch + p] | ((uint32_t)tile[(oct * 8 + 2 * d + 1) * pitch + p] << 16);
            *reinterpret_cast<u32x4 *>(a.xt + ((size_t)b * P + p0 + p) * a.C + c0 + oct * 8) = v;
        }
    }
}

// Sums the split-K slices in slice order (deterministic) and applies the epilogue.
// One grid row (blockIdx.y) per output channel, four consecutive pixels per thread:
// 16-byte loads of the partial sums, no 64-bit index arithmetic.
template <class T, int ACT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(GemmArgs a)
{
    const int row = blockIdx.y;
    const int n4 = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (n4 >= a.N)
        return;
    const size_t total = (size_t)a.Cout * a.N;
    const float *pp = a.part + (size_t)row * a.N + n4;
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    const bool vec = ((a.N & 3) == 0); // then n4 + 3 < N and every slice row is 16-byte aligned
    for (int s = 0; s < a.splitk; s++) {
        if (vec) {
            const f32x4 t = *(const f32x4 *)(pp + (size_t)s * total);
            v[0] += t[0];
            v[1] += t[1];
            v[2] += t[2];
            v[3] += t[3];
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (n4 + i < a.N)
                    v[i] += pp[(size_t)s * total + i];
        }
    }
    const float bv = a.bias ? a.bias[row] : 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int n = n4 + i;
        if (n >= a.N)
            break;
        float r = v[i] + bv;
        const int b = (int)fast_div((uint32_t)n, a.ohw_magic, a.ohw_shift);
        const int pix = n - b * a.OHW;
        T *yp = (T *)a.y + ((size_t)b * a.Cout + row) * a.OHW + pix;
        const bool pre = a.pre != 0 && a.factor != 0.0f;
        if (pre)
            r = fmaf(to_float(*yp), a.factor, r);
        if (ACT == ACT_CLAMP) {
            if (a.act != DLP_ACT_IDENTITY)
                r = clamp_med3(r, a.clamp_lo, a.clamp_hi);
        } else
            r = apply_act(r, a.act);
        store_out(yp, r, pre ? 0.0f : a.factor);
    }
}

// The same for a channels-last bf16 y: a thread sums eight consecutive channels of PX consecutive pixels (consecutive threads on
// consecutive pixels: the partial sums are read in whole lines, 4 * PX bytes a load) and writes each pixel's eight channels as one
// 16-byte piece.  Cout a multiple of 8; PX = 4 needs N in fours and 16-byte aligned partial sums.
template <int ACT, int PX>
__global__ __launch_bounds__(256) void splitk_reduce_cl_kernel(GemmArgs a)
{
    typedef float vec_t __attribute__((ext_vector_type(PX)));
    // PX = 4: eight neighbouring lanes take eight channel groups of the same four pixels, the next eight lanes the next four pixels:
    // loads of a (slice, channel) and stores of a pixel both come in whole 128-byte lines (with a lane per pixel the stores of a
    // wavefront were 64 pieces of 16 bytes in 64 different lines)
    const int c0 = PX == 1 ? (int)blockIdx.y * 8 : ((int)blockIdx.y * 8 + ((int)threadIdx.x & 7)) * 8;
    const int n = PX == 1 ? (int)(blockIdx.x * blockDim.x + threadIdx.x) : ((int)blockIdx.x * 32 + ((int)threadIdx.x >> 3)) * PX;
    if (n >= a.N || c0 >= a.Cout)
        return;
    const size_t total = (size_t)a.Cout * a.N;
    const float *pp = a.part + (size_t)c0 * a.N + n;
    // the old y first, then the slices: eight loads on their way per wait (the sums keep the order slice 0, 1, 2 ...)
    u32x4 *yp = (u32x4 *)((uint16_t *)a.y + (size_t)n * a.Cout + c0);
    const size_t ystep = (size_t)a.Cout / 8; // 16-byte pieces between pixels
    const bool pre = a.pre != 0 && a.factor != 0.0f;
    u32x4 old[PX];
    if (pre) {
#pragma unroll
        for (int q = 0; q < PX; q++)
            old[q] = yp[q * ystep];
    }
    vec_t v[8];
#pragma unroll
    for (int i = 0; i < 8; i++)
        v[i] = a.bias ? a.bias[c0 + i] : 0.0f;
    for (int s = 0; s < a.splitk; s++) {
        vec_t t[8];
#pragma unroll
        for (int i = 0; i < 8; i++)
            t[i] = *(const vec_t *)(pp + (size_t)s * total + (size_t)i * a.N);
#pragma unroll
        for (int i = 0; i < 8; i++)
            v[i] += t[i];
    }
#pragma unroll
    for (int q = 0; q < PX; q++) {
        u32x4 out;
#pragma unroll
        for (int d = 0; d < 4; d++) {
            float lo = v[2 * d][q], hi = v[2 * d + 1][q];
            if (pre) {
                lo = fmaf(__builtin_bit_cast(float, old[q][d] << 16), a.factor, lo);
                hi = fmaf(__builtin_bit_cast(float, old[q][d] & 0xFFFF0000u), a.factor, hi);
            }
            if (ACT == ACT_CLAMP) {
                if (a.act != DLP_ACT_IDENTITY) {
                    lo = clamp_med3(lo, a.clamp_lo, a.clamp_hi);
                    hi = clamp_med3(hi, a.clamp_lo, a.clamp_hi);
                }
            } else {
                lo = apply_act(lo, a.act);
                hi = apply_act(hi, a.act);
            }
            out[d] = (uint32_t)to_bf16(lo).bits | ((uint32_t)to_bf16(hi).bits << 16);
        }
        yp[q * ystep] = out;
    }
}

// Weights [Cout][Cin/groups][KH][KW] -> packed[group][m tile][K tile][k][m in tile], zero padded.
template <class T>
__global__ __launch_bounds__(256) void pack_weights_kernel(GemmPlan p, int groups, int cin_g, int khw, const T *__restrict__ w,
                                                           float *__restrict__ out, int *__restrict__ zero, int nzero)
{
    // side job: clear the tile counters of the stream launch that follows on the stream
    for (int i = (int)(blockIdx.x * 256 + threadIdx.x); i < nzero; i += (int)gridDim.x * 256)
        zero[i] = 0;
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long total = (long long)groups * p.mtiles * p.nkt * BK * p.BM;
    if (idx >= total)
        return;
    const int mi = (int)(idx % p.BM);
    long long r = idx / p.BM;
    const int k = (int)(r % BK);
    r /= BK;
    const int kt = (int)(r % p.nkt);
    r /= p.nkt;
    const int mt = (int)(r % p.mtiles);
    const int g = (int)(r / p.mtiles);
    const int m = mt * p.BM + mi;
    int col; // column of the [M][K] weight matrix of this group
    if (p.order == GEMM_ORDER_TAP) {
        const int cb = kt / khw, tap = kt - cb * khw;
        col = (cb * BK + k) * khw + tap;
    } else {
        col = kt * BK + k;
    }
    float v = 0.0f;
    if (m < p.M && col < p.K)
        v = to_float(w[((size_t)g * p.M + m) * p.K + col]);
    out[idx] = v;
}

// bf16 matrix-instruction path: packed[group][m tile][K tile][m in tile][32 channels of one tap], bf16
__global__ __launch_bounds__(256) void pack_weights_bf16_kernel(GemmPlan p, int groups, int cin_g, int khw, const bf16_t *__restrict__ w,
                                                                bf16_t *__restrict__ out, int *__restrict__ zero, int nzero)
{
    for (int i = (int)(blockIdx.x * 256 + threadIdx.x); i < nzero; i += (int)gridDim.x * 256)
        zero[i] = 0; // as in pack_weights_kernel
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long total = (long long)groups * p.mtiles * p.nkt * p.BM * BK2;
    if (idx >= total)
        return;
    const int k = (int)(idx % BK2);
    long long r = idx / BK2;
    const int mi = (int)(r % p.BM);
    r /= p.BM;
    const int kt = (int)(r % p.nkt);
    r /= p.nkt;
    const int mt = (int)(r % p.mtiles);
    const int g = (int)(r / p.mtiles);
    const int m = mt * p.BM + mi;
    int col;
    if (p.order == GEMM_ORDER_TAP_BF16) {
        const int cb = kt / khw, tap = kt - cb * khw;
        col = (cb * BK2 + k) * khw + tap;
    } else {
        col = kt * BK2 + k;
    }
    bf16_t v;
    v.bits = 0;
    if (m < p.M && col < p.K)
        v = w[((size_t)g * p.M + m) * p.K + col];
    out[idx] = v;
}

// Tap-major K orders: the same packed layouts as the two kernels above, written through an LDS
// transpose.  One workgroup takes 16 filters x one block of KB channels: that is 16 runs of
// KB*khw consecutive source elements (read coalesced), which it scatters into the khw K tiles
// of the channel block, 16 consecutive filters ([k][m] tiles) or KB consecutive channels
// ([m][k] tiles) at a time.  Dynamic LDS: 16 * (KB*khw + 1) elements of TI.
template <class TI, class TO, int KB, bool M_MAJOR>
__global__ __launch_bounds__(256) void pack_weights_tap_kernel(GemmPlan p, int ncb, int khw, const TI *__restrict__ w,
                                                               TO *__restrict__ out, int *__restrict__ zero, int nzero)
{
    // side job: clear the tile counters of the stream-K launch that follows on the stream
    for (int i = (int)(blockIdx.x * 256 + threadIdx.x); i < nzero; i += (int)gridDim.x * 256)
        zero[i] = 0;
    extern __shared__ __align__(16) unsigned char pack_smem[];
    TI *lds = reinterpret_cast<TI *>(pack_smem);
    const int run = KB * khw, ld = run + 1;
    const int mchunks = p.BM / 16;
    int bid = (int)blockIdx.x;
    const int mc = bid % mchunks;
    bid /= mchunks;
    const int cb = bid % ncb;
    bid /= ncb;
    const int mt = bid % p.mtiles;
    const int g = bid / p.mtiles;
    const int m_base = mt * p.BM + mc * 16;
    const int col0 = cb * run;
    const int total = 16 * run;
    // each wavefront reads four filter rows, 16 bytes per lane, all four loads in flight at once
    // (the source rows start on 16-byte boundaries: K is a multiple of KB and the host checks w)
    constexpr int VEC = 16 / (int)sizeof(TI);
    struct alignas(16) Vec {
        TI e[VEC];
    };
    const int wv = (int)threadIdx.x >> 6;
    for (int j = ((int)threadIdx.x & 63) * VEC; j < run; j += 64 * VEC) {
        Vec v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int m = m_base + wv + 4 * q;
            v[q] = Vec();
            if (m < p.M)
                v[q] = *reinterpret_cast<const Vec *>(w + ((size_t)g * p.M + m) * p.K + col0 + j);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                lds[(wv + 4 * q) * ld + j + e] = v[q].e[e];
    }
    __syncthreads();
    TO *tile0 = out + ((size_t)(g * p.mtiles + mt) * p.nkt + (size_t)cb * khw) * (KB * p.BM);
#pragma unroll 4
    for (int idx = (int)threadIdx.x; idx < total; idx += 256) {
        int r, k;
        if (M_MAJOR) {
            k = idx % KB;
            r = (idx / KB) % 16;
        } else {
            r = idx % 16;
            k = (idx / 16) % KB;
        }
        const int tap = idx / (16 * KB);
        const TI v = lds[r * ld + k * khw + tap];
        TO *dst = tile0 + (size_t)tap * (KB * p.BM) + (M_MAJOR ? (mc * 16 + r) * KB + k : k * p.BM + mc * 16 + r);
        if constexpr (sizeof(TO) == sizeof(TI))
            *dst = v;
        else
            *dst = to_float(v);
    }
}

bool bf16_mfma_order(int order) { return order == GEMM_ORDER_TAP_BF16 || order == GEMM_ORDER_CHANNEL_BF16; }

// Split-K factor for a launch of `tiles` output tiles over `nkt` K tiles.
// The 64x64 tile runs up to 8 workgroups per CU; measured on the ResNet shapes the
// kernel needs on the order of 1200 workgroups in flight to keep the matrix pipes of
// 256 CUs busy, and a split only pays when every slice still has a long K loop
// (the partial sums cost one extra pass over the output per slice).
#ifndef DLP_SPLITK_MIN_KT
#define DLP_SPLITK_MIN_KT 24
#endif
int choose_splitk(long long tiles, int nkt, int order)
{
    if (bf16_mfma_order(order)) {
        // large tiles, two workgroups per CU: about 512 fill the chip; K tiles are 32 deep
        if (tiles >= 400)
            return 1;
        long long s = (512 + tiles / 2) / tiles;
        const long long max_by_k = nkt / 8;
        if (s > max_by_k)
            s = max_by_k;
        if (s > 16)
            s = 16;
        return s < 1 ? 1 : (int)s;
    }
    if (tiles >= 1000)
        return 1;
    long long s = (1200 + tiles / 2) / tiles; // round(1200 / tiles)
    const long long max_by_k = nkt / DLP_SPLITK_MIN_KT;
    if (s > max_by_k)
        s = max_by_k;
    if (s > 16)
        s = 16;
    return s < 1 ? 1 : (int)s;
}

bool generic_act(int activation) { return activation == DLP_ACT_TANH || activation == DLP_ACT_SIGMOID; }

// Workspace of a split launch.  fp32-instruction kernels reduce in place: one counter per tile (256-byte
// rounded) | one BM x BN accumulator image per tile and slice.  bf16-instruction kernels: partial sums
// in output order, [slice][Cout][N], for splitk_reduce_kernel.
size_t split_counter_bytes(long long tiles) { return (size_t)((tiles * sizeof(int) + 255) / 256 * 256); }
size_t split_workspace_bytes(const GemmPlan &p, const GemmArgs &a, int groups, int s)
{
    if (s <= 1)
        return 0;
    if (bf16_mfma_order(p.order))
        return (size_t)s * a.Cout * a.N * sizeof(float);
    const long long tiles = (long long)a.mtiles * a.ntiles * groups;
    return split_counter_bytes(tiles) + (size_t)tiles * s * p.BM * p.BN * sizeof(float);
}

int device_cu_count();

// counters | accumulator images of a launch planned by plan_split (fp32-instruction kernels)
size_t split_total_bytes(const GemmPlan &p, const GemmArgs &a, int groups)
{
    if (bf16_mfma_order(p.order))
        return split_workspace_bytes(p, a, groups, a.splitk);
    if (a.splitk <= 1 && a.tail_tiles == 0)
        return 0;
    const long long tiles = (long long)a.mtiles * a.ntiles * groups;
    const long long images = (a.splitk > 1 ? (tiles - a.tail_tiles) * a.splitk : 0) + (long long)a.tail_tiles * a.tail_splitk;
    return split_counter_bytes(tiles) + (size_t)images * p.BM * p.BN * sizeof(float);
}

// Multipliers for the kernels' decode of a workgroup number into (row tile, pixel tile, group, K slice).
void set_tile_magics(GemmArgs &a, int groups)
{
    const long long tiles_main = (long long)a.mtiles * a.ntiles * groups - a.tail_tiles;
    make_magic((uint32_t)std::max(a.mtiles, 1), a.mt_magic, a.mt_shift);
    make_magic((uint32_t)std::max(a.ntiles, 1), a.ntl_magic, a.ntl_shift);
    make_magic((uint32_t)std::max(groups, 1), a.gr_magic, a.gr_shift);
    make_magic((uint32_t)std::max<long long>(tiles_main, 1), a.tm_magic, a.tm_shift);
    make_magic((uint32_t)std::max(a.tail_tiles, 1), a.tt_magic, a.tt_shift);
}

void plan_split(const GemmPlan &p, GemmArgs &a, int groups, bool have_ws, size_t ws_bytes)
{
    a.mtiles = p.mtiles;
    a.ntiles = (a.N + p.BN - 1) / p.BN;
    const long long tiles = (long long)a.mtiles * a.ntiles * groups;
    int s = choose_splitk(tiles, a.nkt, p.order);
    if (s > 1 && (!have_ws || ws_bytes < split_workspace_bytes(p, a, groups, s)))
        s = 1; // no (or too small a) workspace: run unsplit
    a.kt_per_slice = ((a.nkt + s - 1) / s + 1) / 2 * 2;              // even: LDS buffer parity is static
    a.splitk = (a.nkt + a.kt_per_slice - 1) / a.kt_per_slice; // every slice starts inside the K range
    a.tail_tiles = 0;
    a.tail_splitk = 1;
    a.tail_kt = a.kt_per_slice;
    // The workgroups of one launch are all resident at once (up to eight per CU) or nearly so, and a CU is done when
    // its workgroups are: with 6.1 workgroups per CU some CUs carry 7 and the others idle for 1/7 of the time.  The
    // tiles of the last, partial round of workgroups are therefore cut into finer K slices, about one per CU, and
    // launched last: every CU then carries the same number of whole workgroups plus one small piece.
    // (measured on the ResNet-18 shapes at batch 64: 3x3 stride-2 layers, 36 to 144 K tiles, 2 to 6 % faster; 1x1 layers of
    // 4 to 16 K tiles up to 16 % slower, as the pieces' trip through the workspace then costs more than the idle time)
    if (!bf16_mfma_order(p.order) && have_ws && tiles * a.splitk < 0x7fffffffLL && a.nkt >= DLP_SPLITK_MIN_KT) {
        const int cus = device_cu_count();
        const long long wgs = tiles * a.splitk, full = wgs / cus * cus;
        if (full > 0 && full < wgs) {
            const long long tail = tiles - full / a.splitk;
            // the tail's K tiles per CU, even; no finer than sixteen slices per tile: the workgroup that arrives last reads the others'
            // pieces back four at a time, and a tail of two tiles of a small launch is not worth a 64-way reduction
            // (1x1 2048->512 at 7x7, batch 16: 46 -> 26 us)
            const long long kt2 = std::max<long long>(((tail * a.nkt + cus - 1) / cus + 1) / 2 * 2, ((a.nkt + 15) / 16 + 1) / 2 * 2);
            const long long s2 = (a.nkt + kt2 - 1) / kt2;
            if (kt2 < a.kt_per_slice && s2 <= 64 && tail * s2 < 0x7fffffffLL - wgs) {
                a.tail_tiles = (int)tail;
                a.tail_kt = (int)kt2;
                a.tail_splitk = (int)s2;
                if (ws_bytes < split_total_bytes(p, a, groups)) {
                    a.tail_tiles = 0;
                    a.tail_splitk = 1;
                    a.tail_kt = a.kt_per_slice;
                }
            }
        }
    }
    a.main_wgs = (int)((tiles - a.tail_tiles) * a.splitk);
    set_tile_magics(a, groups);
}

template <class T, int BM, int BN, int WM, int WN, int ORDER, int MASK, int ACT>
int launch_inst(const ConvGeom &g, GemmArgs &a, hipStream_t stream, int nset = 2)
{
    long long blocks = (long long)a.mtiles * a.ntiles * g.groups * a.splitk;
    if (blocks > 0x7fffffffLL)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "convolution too large for a single launch");
    blocks = (long long)a.main_wgs + (long long)a.tail_tiles * a.tail_splitk;
    {
        TimingScope ts("conv_gemm", stream);
        if constexpr (ORDER == GEMM_ORDER_TAP && ACT == ACT_CLAMP && std::is_same<T, float>::value) {
            if (nset == 4)
                DLP_LAUNCH_TIMED(ts, (conv_gemm_f32_kernel<T, BM, BN, WM, WN, ORDER, MASK, ACT, 4>), dim3((unsigned)blocks), dim3(kThreads), 0, stream, a);
            else
                DLP_LAUNCH_TIMED(ts, (conv_gemm_f32_kernel<T, BM, BN, WM, WN, ORDER, MASK, ACT>), dim3((unsigned)blocks), dim3(kThreads), 0, stream, a);
        } else
            DLP_LAUNCH_TIMED(ts, (conv_gemm_f32_kernel<T, BM, BN, WM, WN, ORDER, MASK, ACT>), dim3((unsigned)blocks), dim3(kThreads), 0, stream, a);
    }
    if (a.splitk > 1 && a.sk_cnt == nullptr) {
        TimingScope ts("splitk_reduce", stream);
        if (a.Cout > 65535)
            return fail(DLP_ERR_NOT_IMPLEMENTED, "split-K reduction: more than 65535 output channels");
        hipLaunchKernelGGL((splitk_reduce_kernel<T, ACT>), dim3((unsigned)((a.N + 1023) / 1024), (unsigned)a.Cout), dim3(256), 0, stream, a);
    }
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

typedef void (*Bf16Kernel)(GemmArgs);
template <int BM, int BN, int WM, int WN>
Bf16Kernel bf16_kernel_of_tile(int order, int pxl, int sx, bool xt)
{
    if (order == GEMM_ORDER_TAP_BF16 && sx == 2 && pxl == 4)
        return conv_gemm_bf16_kernel<BM, BN, WM, WN, GEMM_ORDER_TAP_BF16, ACT_CLAMP, DLP_DENSE_NSET, 4, 2>;
    if (order == GEMM_ORDER_TAP_BF16 && pxl == 8)
        return conv_gemm_bf16_kernel<BM, BN, WM, WN, GEMM_ORDER_TAP_BF16, ACT_CLAMP, DLP_DENSE_NSET, 8>;
    if (order == GEMM_ORDER_TAP_BF16 && pxl == 4)
        return conv_gemm_bf16_kernel<BM, BN, WM, WN, GEMM_ORDER_TAP_BF16, ACT_CLAMP, DLP_DENSE_NSET, 4>;
    if (order == GEMM_ORDER_TAP_BF16 && xt)
        return conv_gemm_bf16_kernel<BM, BN, WM, WN, GEMM_ORDER_TAP_BF16, ACT_CLAMP, DLP_BF16_NSET, 0, 1, 1>;
    if (order == GEMM_ORDER_TAP_BF16)
        return conv_gemm_bf16_kernel<BM, BN, WM, WN, GEMM_ORDER_TAP_BF16, ACT_CLAMP, DLP_BF16_NSET, 0>;
    return conv_gemm_bf16_kernel<BM, BN, WM, WN, GEMM_ORDER_CHANNEL_BF16, ACT_CLAMP, 2, 0>;
}
Bf16Kernel bf16_kernel(int tile, int order, int pxl, int sx, bool xt)
{
    return tile == 2 ? bf16_kernel_of_tile<128, 128, 2, 2>(order, pxl, sx, xt) : bf16_kernel_of_tile<64, 256, 1, 4>(order, pxl, sx, xt);
}

// Largest number of patch rows any pixel tile of conv_patch_bf16_kernel needs (same arithmetic as the kernel).
int bf16_patch_rows(const ConvGeom &g, int BN, int pxp)
{
    const long long N = (long long)g.B * g.OH * g.OW;
    const int HW = g.OH * g.OW, halo = g.W + 1;
    const long long ntiles = (N + BN - 1) / BN;
    int most = 0;
    // the offset of a tile inside its image repeats after HW / gcd(BN, HW) tiles; the last tile may be short
    long long period = HW;
    for (long long x = BN, y = HW; y != 0;) {
        const long long r = x % y;
        x = y;
        y = r;
        period = HW / x;
    }
    for (long long i = 0; i < std::min(ntiles, period + 1); i++) {
        const long long nt = i < period ? i : ntiles - 1;
        const long long n0 = nt * BN, n_last = std::min(n0 + BN, N) - 1;
        const long long b0 = n0 / HW;
        int rows = 0;
        for (int s = 0; s < 3; s++) {
            const long long base = (b0 + s) * HW;
            const long long first = std::max(n0, base), last = std::min(n_last, base + HW - 1);
            if (first <= last) {
                const int as = (int)std::max<long long>(0, first - base - halo) & ~(pxp - 1);
                rows += (((int)std::min<long long>(HW, last - base + 1 + halo) + pxp - 1) & ~(pxp - 1)) - as;
            }
        }
        most = std::max(most, rows);
    }
    return most;
}

int launch_patch_bf16(const ConvGeom &g, const GemmPlan &p, GemmArgs &a, hipStream_t stream)
{
    a.mtiles = p.mtiles;
    a.ntiles = (a.N + p.BN - 1) / p.BN;
    a.splitk = 1;
    a.kt_per_slice = a.nkt;
    a.part = nullptr;
    a.part_bytes = 0;
    a.pp_nbr = p.pp_nbr;
    a.tail_tiles = 0;
    set_tile_magics(a, g.groups);
    const long long blocks = (long long)a.mtiles * a.ntiles * g.groups;
    if (blocks > 0x7fffffffLL)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "convolution too large for a single launch");
    TimingScope ts("conv_gemm", stream);
    const dim3 grid((unsigned)blocks), block(kThreads);
    if (p.tile == 2 && p.patch_bf16 == 8)
        DLP_LAUNCH_TIMED(ts, (conv_patch_bf16_kernel<128, 128, 4, 1, kPatchPitchBf16_128, 8, ACT_CLAMP>), grid, block, 0, stream, a);
    else if (p.tile == 2)
        DLP_LAUNCH_TIMED(ts, (conv_patch_bf16_kernel<128, 128, 4, 1, kPatchPitchBf16_128, 4, ACT_CLAMP>), grid, block, 0, stream, a);
    else if (p.patch_bf16 == 8)
        DLP_LAUNCH_TIMED(ts, (conv_patch_bf16_kernel<64, 256, 2, 2, kPatchPitchBf16_256, 8, ACT_CLAMP>), grid, block, 0, stream, a);
    else
        DLP_LAUNCH_TIMED(ts, (conv_patch_bf16_kernel<64, 256, 2, 2, kPatchPitchBf16_256, 4, ACT_CLAMP>), grid, block, 0, stream, a);
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

// The channels-last copy that the XT kernels read: geometry, and size in bytes (256-byte rounded).
struct XtGeom {
    int H, W, sy, sx; // pixels of the copy; strides of the copy (1x1 convolutions without padding fold theirs into it)
};
XtGeom xt_geom(const ConvGeom &g)
{
    if (g.x_channels_last) // the input itself, as it lies
        return {g.H, g.W, 1, 1};
    if (g.KH == 1 && g.KW == 1 && g.ph == 0 && g.pw == 0)
        return {g.OH, g.OW, g.sh, g.sw};
    return {g.H, g.W, 1, 1};
}
size_t xt_bytes(const ConvGeom &g, int batch)
{
    if (g.x_channels_last) // no copy
        return 0;
    const XtGeom t = xt_geom(g);
    return ((size_t)batch * t.H * t.W * g.Cin * sizeof(bf16_t) + 255) / 256 * 256;
}

int launch_bf16_mfma(const ConvGeom &g, const GemmPlan &p, int pxl, GemmArgs &a, hipStream_t stream, void *xt)
{
    long long blocks = (long long)a.mtiles * a.ntiles * g.groups * a.splitk;
    if (blocks > 0x7fffffffLL)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "convolution too large for a single launch");
    if (xt != nullptr) {
        const XtGeom t = xt_geom(g);
        if (!g.x_channels_last) {
        StageArgs sa;
        sa.x = (const uint16_t *)a.x;
        sa.xt = (uint16_t *)xt;
        sa.C = g.Cin; sa.H = g.H; sa.W = g.W; sa.PH = t.H; sa.PW = t.W; sa.sy = t.sy; sa.sx = t.sx;
        make_magic((uint32_t)t.W, sa.pw_magic, sa.pw_shift);
        if (g.B > 65535 || (g.Cin + 63) / 64 > 65535)
            return fail(DLP_ERR_NOT_IMPLEMENTED, "channels-last staging: more than 65535 images or channel blocks");
        {
            TimingScope ts("stage_input", stream);
            const int P = t.H * t.W;
            const bool whole = t.sy == 1 && t.sx == 1 && ((uintptr_t)a.x & 15) == 0;
            const dim3 grid64((unsigned)((P + 63) / 64), (unsigned)((g.Cin + 63) / 64), (unsigned)g.B);
            if (whole && P <= kStageFlatPixels)
                DLP_LAUNCH_TIMED(ts, stage_channels_last_kernel<1>, dim3(1, grid64.y, grid64.z), dim3(256), 0, stream, sa);
            else if (whole && P % 8 == 0)
                DLP_LAUNCH_TIMED(ts, stage_channels_last_kernel<2>, grid64, dim3(256), 0, stream, sa);
            else
                DLP_LAUNCH_TIMED(ts, stage_channels_last_kernel<0>, grid64, dim3(256), 0, stream, sa);
        }
        }
        // the convolution the matrix kernel now sees: the copy as input, strides that the copy has taken over set to 1
        a.x = xt;
        a.x_bytes = (uint32_t)((size_t)g.B * t.H * t.W * g.Cin * sizeof(bf16_t));
        a.H = t.H;
        a.W = t.W;
        a.sh = g.sh / t.sy;
        a.sw = g.sw / t.sx;
        a.x_shift = (uint32_t)(((size_t)g.ph * t.W + g.pw) * g.Cin * sizeof(bf16_t));
        a.ktab += (p.nkt + 2) * BK2; // the second table of conv_gemm_fill_ktab
    }
    {
        TimingScope ts("conv_gemm", stream);
        const Bf16Kernel kernel = bf16_kernel(p.tile, p.order, pxl, p.dense_sx, xt != nullptr);
        DLP_LAUNCH_TIMED(ts, kernel, dim3((unsigned)blocks), dim3(kThreads), 0, stream, a);
    }
    if (a.splitk > 1) {
        TimingScope ts("splitk_reduce", stream);
        if (a.Cout > 65535)
            return fail(DLP_ERR_NOT_IMPLEMENTED, "split-K reduction: more than 65535 output channels");
        // the form with four pixels per thread only where it still gives every CU a workgroup: on the small launches of small batches
        // (ResNet-50 at batch 16: 56 workgroups instead of 256) it took 75 us more per pass than the plain one
        if (a.y_cl && (a.N & 3) == 0 && ((uintptr_t)a.part & 15) == 0 && (long long)((a.N + 127) / 128) * ((a.Cout + 63) / 64) >= dlp_cu_count())
            hipLaunchKernelGGL((splitk_reduce_cl_kernel<ACT_CLAMP, 4>), dim3((unsigned)((a.N + 127) / 128), (unsigned)((a.Cout + 63) / 64)), dim3(256), 0, stream, a);
        else if (a.y_cl)
            hipLaunchKernelGGL((splitk_reduce_cl_kernel<ACT_CLAMP, 1>), dim3((unsigned)((a.N + 255) / 256), (unsigned)(a.Cout / 8)), dim3(256), 0, stream, a);
        else
            hipLaunchKernelGGL((splitk_reduce_kernel<bf16_t, ACT_CLAMP>), dim3((unsigned)((a.N + 1023) / 1024), (unsigned)a.Cout), dim3(256), 0, stream, a);
    }
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

// Stream-K launch shape of the LDS-patch kernel: three workgroups per CU (measured best of 1..4:
// one wavefront per SIMD already keeps its matrix pipe ~90 % busy, the others cover barriers and
// the prologue), every one with the same number of (tile, stage) units, but no fewer than 4
// stages per workgroup.
constexpr int kPatchWgsPerCu = 3;
constexpr int kPatchWgsPerCuStrided = 3;
constexpr int kPatchPitchStrided = 512;
// Longest patch (input pixels of all the images a tile touches) of a 64-pixel tile of a stride-2 3x3 pad-1 convolution: the
// kernel's own segment arithmetic, run over every position a tile can have inside a plane.
static int strided_patch_rows(const ConvGeom &g)
{
    const int ohw = g.OH * g.OW, hwi = g.H * g.W;
    if (ohw > (1 << 16))
        return 1 << 30;
    int worst = 0;
    for (int nt = 0; nt < ohw; nt++) { // n0 = 64 nt takes every residue modulo the plane that a tile start can have
        const long long n0 = 64ll * nt, n_last = n0 + 63;
        const long long b0 = n0 / ohw;
        int total = 0;
        for (int s = 0; s < 3; s++) {
            const long long base = (b0 + s) * ohw;
            const long long first = std::max(n0, base), last = std::min(n_last, base + ohw - 1);
            if (first > last)
                continue;
            const int pf = (int)(first - base), pl = (int)(last - base);
            const int oyf = pf / g.OW, oxf = pf % g.OW, oyl = pl / g.OW, oxl = pl % g.OW;
            const int as = std::max(0, (oyf * 2 - 1) * g.W + oxf * 2 - 1);
            total += std::min(hwi, (oyl * 2 - 1 + 2) * g.W + oxl * 2 - 1 + 3) - as;
        }
        worst = std::max(worst, total);
    }
    return worst;
}
int device_cu_count() { return dlp_cu_count(); }
struct PatchShape {
    long long tiles, units;
    int grid;
    size_t cnt_bytes, ws_bytes; // tile counters | two 64x64 fp32 pieces per workgroup
};
PatchShape patch_shape(const ConvGeom &g, const GemmPlan &p, long long N)
{
    PatchShape ps;
    ps.tiles = (long long)p.mtiles * ((N + 63) / 64) * g.groups;
    ps.units = ps.tiles * (p.nkt / (g.KH * g.KW));
    long long grid = ps.units / 4;
    const long long slots = (long long)device_cu_count() * (g.sh == 1 ? kPatchWgsPerCu : kPatchWgsPerCuStrided);
    grid = grid < 1 ? 1 : grid > slots ? slots : grid;
    ps.grid = (int)grid;
    ps.cnt_bytes = (size_t)((ps.tiles * sizeof(int) + 255) / 256 * 256);
    ps.ws_bytes = ps.cnt_bytes + (size_t)ps.grid * 2 * 64 * 64 * sizeof(float);
    return ps;
}

int launch_patch(const ConvGeom &g, const GemmPlan &p, GemmArgs &a, hipStream_t stream, void *part_ws, size_t part_bytes, int *own_counters)
{
    a.mtiles = p.mtiles;
    a.ntiles = (a.N + p.BN - 1) / p.BN;
    a.splitk = 1;
    a.kt_per_slice = a.nkt;
    a.part = nullptr;
    a.part_bytes = 0;
    const PatchShape ps = patch_shape(g, p, a.N);
    if (ps.units > 0x7fffffffLL)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "convolution too large for a single launch");
    a.sk_units = (int)ps.units;
    int grid = ps.grid;
    // same test as in conv_gemm_pack_weights, which clears the counters
    if (part_ws != nullptr && part_bytes >= patch_shape(g, p, (long long)g.B * g.OH * g.OW).ws_bytes && part_bytes >= ps.ws_bytes) {
        a.sk_cnt = own_counters ? own_counters : (int *)part_ws; // zeroed by conv_gemm_pack_weights, which is handed the same workspace
        a.sk_part = (float *)((char *)part_ws + ps.cnt_bytes);
        a.sk_part_bytes = (uint32_t)(ps.ws_bytes - ps.cnt_bytes);
    } else { // no room for pieces: one whole tile per workgroup
        a.sk_cnt = nullptr;
        a.sk_part = nullptr;
        a.sk_part_bytes = 0;
        grid = (int)ps.tiles;
    }
    // tile order (see the kernel): tiles per workgroup, and how many m tiles run side by side --
    // the divisor of mtiles for which one XCD's share of the tiles touches the fewest bytes
    // (mb m tiles of weights + its pixel tiles of input)
    a.sk_tpw = (int)std::max<long long>(1, (ps.tiles + grid / 2) / grid);
    {
        const double a_bytes = 64.0 * a.K * 4, x_bytes = 64.0 * a.Cin_g * 4, share = (double)ps.tiles / 8;
        double best = 0;
        a.sk_mb = 1;
        for (int mb = 1; mb <= p.mtiles; mb++) {
            if (p.mtiles % mb)
                continue;
            const double cost = mb * a_bytes + share / mb * x_bytes;
            if (mb == 1 || cost < best) {
                best = cost;
                a.sk_mb = mb;
            }
        }
    }
    make_magic((uint32_t)(a.nkt / 9), a.ncb_magic, a.ncb_shift);
    a.sk_tiles = (int)ps.tiles;
    make_magic((uint32_t)ps.tiles, a.nt_magic, a.nt_shift);
    make_magic((uint32_t)a.sk_tpw, a.tpw_magic, a.tpw_shift);
    make_magic((uint32_t)(a.mtiles * a.ntiles), a.pg_magic, a.pg_shift);
    make_magic((uint32_t)(a.sk_mb * a.ntiles), a.mbnt_magic, a.mbnt_shift);
    make_magic((uint32_t)a.sk_mb, a.mb_magic, a.mb_shift);
    TimingScope ts("conv_gemm", stream);
    if (g.sh == 2) { // the shortest rows that hold the longest patch: fewer (empty) loads and LDS stores per stage
        const int rows = strided_patch_rows(g);
        if (rows < 320)
            DLP_LAUNCH_TIMED(ts, (conv_patch_f32_kernel<float, 3, 3, 320, ACT_CLAMP, 2>), dim3((unsigned)grid), dim3(kThreads), 0, stream, a);
        else if (rows < 384)
            DLP_LAUNCH_TIMED(ts, (conv_patch_f32_kernel<float, 3, 3, 384, ACT_CLAMP, 2>), dim3((unsigned)grid), dim3(kThreads), 0, stream, a);
        else if (rows < 448)
            DLP_LAUNCH_TIMED(ts, (conv_patch_f32_kernel<float, 3, 3, 448, ACT_CLAMP, 2>), dim3((unsigned)grid), dim3(kThreads), 0, stream, a);
        else
            DLP_LAUNCH_TIMED(ts, (conv_patch_f32_kernel<float, 3, 3, kPatchPitchStrided, ACT_CLAMP, 2>), dim3((unsigned)grid), dim3(kThreads), 0, stream, a);
    } else
        DLP_LAUNCH_TIMED(ts, (conv_patch_f32_kernel<float, 3, 3, kPatchPitch, ACT_CLAMP>), dim3((unsigned)grid), dim3(kThreads), 0, stream, a);
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

template <class T, int BM, int BN, int WM, int WN>
int launch_tile(const ConvGeom &g, const GemmPlan &p, GemmArgs &a, int act, hipStream_t stream)
{
    if (act == ACT_GENERIC)
        return launch_inst<T, BM, BN, WM, WN, GEMM_ORDER_CHANNEL, GEMM_MASK_ROWCOL, ACT_GENERIC>(g, a, stream);
    if (p.order == GEMM_ORDER_TAP) {
        // At most about one workgroup per CU: nothing else covers a workgroup's waits, so it keeps four K tiles in flight
        // instead of two (measured alone on cold tensors, batch 64: 1x1 192->64 at 14x14 10.5 -> 9.3 us, 384->64 16.0 -> 13.4,
        // 960->160 at 7x7 21.6 -> 20.3; launches with more workgroups per CU lose 3 to 10 % with four).
        const long long wgs = (long long)a.main_wgs + (long long)a.tail_tiles * a.tail_splitk;
        const int nset = (wgs * 5 <= (long long)device_cu_count() * 6 && a.kt_per_slice >= 8) ? 4 : 2;
        return launch_inst<T, BM, BN, WM, WN, GEMM_ORDER_TAP, GEMM_MASK_TAPS, ACT_CLAMP>(g, a, stream, nset);
    }
    if (p.mask == GEMM_MASK_TAPS)
        return launch_inst<T, BM, BN, WM, WN, GEMM_ORDER_CHANNEL, GEMM_MASK_TAPS, ACT_CLAMP>(g, a, stream);
    return launch_inst<T, BM, BN, WM, WN, GEMM_ORDER_CHANNEL, GEMM_MASK_ROWCOL, ACT_CLAMP>(g, a, stream);
}

// Workgroup tiles.  Small tiles win on this chip: fp32 MFMA is slow enough (64 cycles
// per 32x32x2 block) that one 32x32 block per wavefront already hides the LDS traffic,
// and 8 resident workgroups per CU hide everything else.
struct TileShape {
    int id, BM, BN;
};
constexpr TileShape kTiles[] = {{0, 64, 64}, {1, 32, 128}, {2, 128, 128}, {3, 64, 256}}; // 2, 3: bf16 matrix-instruction path

int tile_choice(int M) { return M > 32 ? 0 : 1; }

template <class F>
int with_tile(int choice, F &&f)
{
    using std::integral_constant;
    if (choice == 1)
        return f(integral_constant<int, 32>{}, integral_constant<int, 128>{}, integral_constant<int, 1>{}, integral_constant<int, 4>{});
    return f(integral_constant<int, 64>{}, integral_constant<int, 64>{}, integral_constant<int, 2>{}, integral_constant<int, 2>{});
}

} // namespace

GemmPlan conv_gemm_plan(const ConvGeom &g, int activation)
{
    GemmPlan p;
    p.wdirect = 0;
    p.stem = conv_stem_supported(g) ? 1 : 0;
    p.dense_pxl = 0;
    p.dense_sx = 1;
    p.patch_bf16 = 0;
    p.pp_nbr = 0;
    p.xt = 0;
    p.pointwise = conv_pointwise_supported(g, activation) ? 1 : 0;
    const int cin_g = g.Cin / g.groups;
    p.M = g.Cout / g.groups;
    p.K = cin_g * g.KH * g.KW;
    p.nkt = (p.K + BK - 1) / BK; // the tap-major order has the same count: K is a multiple of 16 there
    const bool small_kernel = g.KH * g.KW <= 31; // one mask bit per tap, bit 31 kept free for the never-valid spare tiles
    if (generic_act(activation)) { // the rare activations share one instantiation per tile
        p.order = GEMM_ORDER_CHANNEL;
        p.mask = GEMM_MASK_ROWCOL;
    } else {
        p.order = (small_kernel && cin_g % BK == 0) ? GEMM_ORDER_TAP : GEMM_ORDER_CHANNEL;
        p.mask = small_kernel ? GEMM_MASK_TAPS : GEMM_MASK_ROWCOL;
    }
    p.tile = tile_choice(p.M);
    // 1x1 convolutions whose last tile of 64 filters would be at most half full take tiles of 32 filters (x 128 pixels): no matrix
    // instruction is spent on rows that do not exist (batch 64, cold: 384->96 at 14x14 21.5 -> 18.6 us, 960->160 at 7x7 21.9 -> 19.1)
    if (g.KH == 1 && g.KW == 1 && p.M > 32 && (p.M % 64) != 0 && (p.M % 64) <= 32)
        p.tile = 1;
    // 1x1 convolutions in the tap-major order: a K tile is 16 consecutive input channels of the filter rows, which the
    // kernel reads from the weight tensor in place (when it is 16-byte aligned): nothing is packed
    p.wdirect = g.dtype == DLP_FLOAT && p.order == GEMM_ORDER_TAP && g.KH == 1 && g.KW == 1;
    // stride-1 3x3 "same" convolutions whose 64-pixel patch fits the LDS rows (W <= 62): LDS-patch kernel
    p.patch = g.dtype == DLP_FLOAT && p.order == GEMM_ORDER_TAP && p.tile == 0 && g.KH == 3 && g.KW == 3 && g.sh == 1 && g.sw == 1 &&
              g.dh == 1 && g.dw == 1 && g.ph == 1 && g.pw == 1 && g.H * g.W >= 32 && 64 + 2 * (g.W + 1) < kPatchPitch;
    // ... and stride-2 ones (3x3, pad 1) whose longest patch fits rows of 512, from 128 input channels on.  Measured alone on cold
    // tensors at batch 64, patch / gathering kernel with the packing launch: 128->256 at 28x28 77 / 89-94 us, 256->512 at 14x14 76 / 81-83,
    // 64->128 at 56x56 92-96 / 88-91: with four stages per tile the set-up of the long patch is not paid back.
    // (DLP_NO_STRIDED_PATCH in the environment keeps every strided layer on the gathering kernel, for measurements.)
    static const bool no_strided_patch = getenv("DLP_NO_STRIDED_PATCH") != nullptr;
    if (!no_strided_patch && g.dtype == DLP_FLOAT && p.order == GEMM_ORDER_TAP && p.tile == 0 && g.KH == 3 && g.KW == 3 && g.sh == 2 && g.sw == 2 &&
        g.dh == 1 && g.dw == 1 && g.ph == 1 && g.pw == 1 && g.OH * g.OW >= 32 && cin_g >= 128 && strided_patch_rows(g) < kPatchPitchStrided)
        p.patch = 1;
    if (g.dtype == DLP_BFLOAT16 && !generic_act(activation)) { // bf16 matrix instruction
        const bool tap_major = small_kernel && cin_g % BK2 == 0;
        p.order = tap_major ? GEMM_ORDER_TAP_BF16 : GEMM_ORDER_CHANNEL_BF16;
        p.mask = tap_major ? GEMM_MASK_TAPS : GEMM_MASK_ROWCOL;
        p.nkt = (p.K + BK2 - 1) / BK2;
        p.tile = p.M > 64 ? 2 : 3;
        p.wdirect = tap_major && g.KH == 1 && g.KW == 1; // [Cout][Cin] is read in place (when w is 16-byte aligned)
        if (tap_major && g.KH == 1 && g.KW == 1 && g.sh == 1 && g.sw == 1 && g.ph == 0 && g.pw == 0 && (g.H * g.W) % 4 == 0)
            p.dense_pxl = (g.H * g.W) % 8 == 0 ? 8 : 4;
        // 1x1 stride 2 on even-sized images: runs of 4 (2) output pixels of a row = 8 (4) consecutive input pixels
        if (tap_major && g.KH == 1 && g.KW == 1 && g.sh == 2 && g.sw == 2 && g.ph == 0 && g.pw == 0 && g.W % 2 == 0 && g.H % 2 == 0) {
            // (runs of 2 output pixels exist as a kernel variant, but the channels-last staging below is faster there:
            // 80 against 88 us on 512->1024 at 28x28, batch 128)
            const int pxl = g.OW % 4 == 0 ? 4 : 0;
            if (pxl) {
                p.dense_pxl = pxl;
                p.dense_sx = 2;
            }
        }
        // stride-1 3x3 "same" convolutions whose largest patch fits the LDS rows and one block per lane: LDS-patch kernel
        if (tap_major && g.KH == 3 && g.KW == 3 && g.sh == 1 && g.sw == 1 && g.dh == 1 && g.dw == 1 && g.ph == 1 && g.pw == 1 &&
            (g.H * g.W) % 4 == 0 && g.B > 0) {
            const int pxp = (g.H * g.W) % 8 == 0 ? 8 : 4;
            const int BN = p.tile == 2 ? 128 : 256, pitch = p.tile == 2 ? kPatchPitchBf16_128 : kPatchPitchBf16_256;
            const int rows = bf16_patch_rows(g, BN, pxp), nbr = (rows + pxp - 1) / pxp;
            if ((BN - 2) / (g.H * g.W) + 2 <= 3 && nbr * pxp <= pitch - 8 && 4 * nbr <= kThreads) {
                p.patch_bf16 = pxp;
                p.pp_nbr = nbr;
            }
        }
        if (g.x_channels_last) { // (conv_gemm_layouts_supported has checked tap_major) the channels-last loader, on x as it lies
            p.dense_pxl = 0;
            p.dense_sx = 1;
            p.patch_bf16 = 0;
        }
        // everything else in the tap-major order (strided and dilated kernels, odd image sizes): channels-last staging
        p.xt = tap_major && p.dense_pxl == 0 && p.patch_bf16 == 0 && g.Cin <= 65535 * 64 &&
               (size_t)g.H * g.W * g.Cin * sizeof(bf16_t) < kOutOfRange / 2;
    }
    p.BM = 64;
    p.BN = 64;
    for (const TileShape &ts : kTiles)
        if (ts.id == p.tile) {
            p.BM = ts.BM;
            p.BN = ts.BN;
        }
    p.mtiles = (p.M + p.BM - 1) / p.BM;
    p.wpack_bytes = (size_t)g.groups * p.mtiles * p.nkt * BK * p.BM * sizeof(float);
    if (bf16_mfma_order(p.order))
        p.wpack_bytes = (size_t)g.groups * p.mtiles * p.nkt * BK2 * p.BM * sizeof(bf16_t);
    p.wpack_bytes = (p.wpack_bytes + 255) / 256 * 256;
    return p;
}

size_t conv_gemm_ktab_entries(const ConvGeom &g)
{
    // one 8-byte entry per k (the tap-major order uses two entries per K tile); two spare
    // tiles of never-valid entries are what the software pipeline fetches past the end
    const int K = (g.Cin / g.groups) * g.KH * g.KW;
    return (size_t)((K + BK2 - 1) / BK2 + 2) * BK2; // whole K tiles of the widest kernel (32)
}

void conv_gemm_fill_ktab(const ConvGeom &g, int activation, KTabEntry *tab_entries)
{
    int32_t *tab = (int32_t *)tab_entries;
    const size_t words = conv_gemm_ktab_entries(g) * 2;
    for (size_t i = 0; i < words; i++)
        tab[i] = 0; // spare entries: offsets 0, never-valid tap (tap 31 / row-col code 31 below)
    const GemmPlan p = conv_gemm_plan(g, activation);
    const int cin_g = g.Cin / g.groups;
    const int esize = (int)dtype_size(g.dtype); // gather offsets are bytes of the storage type
    if (p.order == GEMM_ORDER_TAP || p.order == GEMM_ORDER_TAP_BF16) {
        const int cblock = p.order == GEMM_ORDER_TAP ? BK : BK2; // channels per K tile
        int t = 0;
        for (int cb = 0; cb < cin_g / cblock; cb++)
            for (int ky = 0; ky < g.KH; ky++)
                for (int kx = 0; kx < g.KW; kx++, t++) {
                    tab[4 * t + 0] = ((cb * cblock * g.H + ky * g.dh) * g.W + kx * g.dw) * esize;
                    tab[4 * t + 1] = ky * g.KW + kx; // tap number = its bit in the per-pixel tap mask
                }
        for (; (size_t)(4 * t + 1) < words; t++)
            tab[4 * t + 1] = 31; // bit 31 of a tap mask is never set (at most 31 taps use this order)
        if (p.xt) {
            // second table, (nkt + 2) * 32 words in (the first uses 4 * (nkt + 2) of them): the same K tiles as byte offsets into
            // the channels-last copy of the input
            const XtGeom xg = xt_geom(g);
            int32_t *tab2 = tab + (p.nkt + 2) * BK2;
            t = 0;
            for (int cb = 0; cb < cin_g / cblock; cb++)
                for (int ky = 0; ky < g.KH; ky++)
                    for (int kx = 0; kx < g.KW; kx++, t++) {
                        tab2[4 * t + 0] = ((ky * g.dh * xg.W + kx * g.dw) * g.Cin + cb * cblock) * esize;
                        tab2[4 * t + 1] = ky * g.KW + kx;
                    }
        }
        return;
    }
    size_t k = 0;
    for (int c = 0; c < cin_g; c++)
        for (int ky = 0; ky < g.KH; ky++)
            for (int kx = 0; kx < g.KW; kx++, k++) {
                tab[2 * k + 0] = ((c * g.H + ky * g.dh) * g.W + kx * g.dw) * esize;
                tab[2 * k + 1] = (p.mask == GEMM_MASK_ROWCOL) ? (ky | (kx << 8)) : (int32_t)(1u << (ky * g.KW + kx));
            }
    if (p.mask == GEMM_MASK_ROWCOL)
        for (; 2 * k + 1 < words; k++)
            tab[2 * k + 1] = 31 | (31 << 8); // bit 31 of the row / column masks is never set
}

size_t conv_gemm_workspace_bytes(const ConvGeom &g, int activation)
{
    // the batch of the shape given at create is a hint: without one (0) the workspace is sized for a single image, so that
    // it always holds the packed weights, which every batch needs
    const int B = std::max(g.B, 1);
    const GemmPlan p = conv_gemm_plan(g, activation);
    if (p.patch)
        return p.wpack_bytes + patch_shape(g, p, (long long)B * g.OH * g.OW).ws_bytes;
    GemmArgs a;
    a.N = B * g.OH * g.OW;
    a.Cout = g.Cout;
    a.nkt = p.nkt;
    plan_split(p, a, g.groups, true, (size_t)-1);
    return p.wpack_bytes + split_total_bytes(p, a, g.groups) + (p.xt ? xt_bytes(g, B) : 0);
}

namespace {
__global__ __launch_bounds__(256) void clear_counters_kernel(int *p, int n)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n)
        p[i] = 0;
}
} // namespace

int conv_gemm_pack_weights(const ConvGeom &g, const GemmPlan &p, const void *w, void *wpacked, hipStream_t stream, void *part_ws,
                           size_t part_bytes, int mode, bool counters_owned)
{
    if (p.wdirect && ((uintptr_t)w & 15) == 0) { // conv_gemm_launch reads w in place: only the counters are left to do
        // (a buffer packed ahead of time is filled all the same: a later call may come with a weight pointer that cannot be read in place)
        if (bf16_mfma_order(p.order) && mode != GEMM_PACK_ONLY)
            return DLP_OK;
        // fp32: weights packed once ahead of time are still the faster operand (one 16-byte LDS store per thread and
        // K tile instead of four); reading in place only saves the packing launch of a call that would pack every time
        if (mode != GEMM_PACK_ONLY)
            mode = GEMM_CLEAR_ONLY;
    }
    if (p.stem)
        return DLP_OK; // conv_stem_f32_kernel reads w in place and keeps no counters
    int *zero = nullptr; // tile counters of the stream-K launch that follows
    int nzero = 0;
    if (mode != GEMM_PACK_ONLY && p.patch && part_ws != nullptr) {
        const PatchShape ps = patch_shape(g, p, (long long)g.B * g.OH * g.OW);
        if (part_bytes >= ps.ws_bytes && ps.tiles <= 0x7fffffffLL) {
            zero = (int *)part_ws;
            nzero = (int)ps.tiles;
        }
    }
    if (mode != GEMM_PACK_ONLY && !p.patch && !bf16_mfma_order(p.order) && part_ws != nullptr) { // counters of the in-place split-K reduction
        GemmArgs a;
        a.N = g.B * g.OH * g.OW;
        a.Cout = g.Cout;
        a.nkt = p.nkt;
        plan_split(p, a, g.groups, true, part_bytes);
        if (a.splitk > 1 || a.tail_tiles > 0) {
            zero = (int *)part_ws;
            nzero = (int)((long long)a.mtiles * a.ntiles * g.groups);
        }
    }
    if (counters_owned) { // the kernels leave the operator's own counters at zero
        zero = nullptr;
        nzero = 0;
    }
    if (mode == GEMM_CLEAR_ONLY) { // the weights were packed earlier: only the counters of the coming launch
        if (zero != nullptr) {
            TimingScope ts("clear_counters", stream);
            hipLaunchKernelGGL(clear_counters_kernel, dim3((unsigned)((nzero + 255) / 256)), dim3(256), 0, stream, zero, nzero);
            DLP_HIP_TRY(hipGetLastError());
        }
        return DLP_OK;
    }
    const long long total = (long long)g.groups * p.mtiles * p.nkt * (bf16_mfma_order(p.order) ? BK2 : BK) * p.BM;
    if (total >= 0x7fffffffLL * 256)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "weight tensor too large");
    TimingScope ts("pack_weights", stream);
    const int khw = g.KH * g.KW;
    if ((p.order == GEMM_ORDER_TAP || p.order == GEMM_ORDER_TAP_BF16) && ((uintptr_t)w & 15) == 0) {
        const int ncb = p.nkt / khw;
        const dim3 grid((unsigned)((long long)g.groups * p.mtiles * ncb * (p.BM / 16)));
        if (p.order == GEMM_ORDER_TAP_BF16)
            hipLaunchKernelGGL((pack_weights_tap_kernel<bf16_t, bf16_t, BK2, true>), grid, dim3(256),
                               16 * (BK2 * khw + 1) * sizeof(bf16_t), stream, p, ncb, khw, (const bf16_t *)w, (bf16_t *)wpacked, zero, nzero);
        else if (g.dtype == DLP_BFLOAT16)
            hipLaunchKernelGGL((pack_weights_tap_kernel<bf16_t, float, BK, false>), grid, dim3(256),
                               16 * (BK * khw + 1) * sizeof(bf16_t), stream, p, ncb, khw, (const bf16_t *)w, (float *)wpacked, zero, nzero);
        else
            hipLaunchKernelGGL((pack_weights_tap_kernel<float, float, BK, false>), grid, dim3(256),
                               16 * (BK * khw + 1) * sizeof(float), stream, p, ncb, khw, (const float *)w, (float *)wpacked, zero, nzero);
    } else if (bf16_mfma_order(p.order))
        hipLaunchKernelGGL(pack_weights_bf16_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, p, g.groups,
                           g.Cin / g.groups, g.KH * g.KW, (const bf16_t *)w, (bf16_t *)wpacked, zero, nzero);
    else if (g.dtype == DLP_BFLOAT16)
        hipLaunchKernelGGL(pack_weights_kernel<bf16_t>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, p, g.groups,
                           g.Cin / g.groups, g.KH * g.KW, (const bf16_t *)w, (float *)wpacked, zero, nzero);
    else
        hipLaunchKernelGGL(pack_weights_kernel<float>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, p, g.groups,
                           g.Cin / g.groups, g.KH * g.KW, (const float *)w, (float *)wpacked, zero, nzero);
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

// Channels-last x and / or y: served by the bf16 matrix-instruction kernels only (x: the channels-last loader, i.e. input
// channels per group in multiples of 32 and a kernel extent the tap masks hold; y: output channels per group in eights).
static bool layouts_supported(const ConvGeom &g, const GemmPlan &p);
bool conv_gemm_layouts_supported(const ConvGeom &g, int activation)
{
    if (!g.x_channels_last && !g.y_channels_last)
        return true;
    return layouts_supported(g, conv_gemm_plan(g, activation));
}
static bool layouts_supported(const ConvGeom &g, const GemmPlan &p)
{
    if (!g.x_channels_last && !g.y_channels_last)
        return true;
    if (!bf16_mfma_order(p.order) || p.stem || p.pointwise || p.patch)
        return false;
    if (g.x_channels_last && !p.xt)
        return false;
    if (g.y_channels_last && (p.M & 7) != 0)
        return false;
    return true;
}

size_t conv_gemm_counter_count(const ConvGeom &g, const GemmPlan &p)
{
    if (g.B <= 0 || bf16_mfma_order(p.order) || p.stem)
        return 0;
    const long long N = (long long)g.B * g.OH * g.OW;
    return (size_t)((long long)p.mtiles * ((N + p.BN - 1) / p.BN) * g.groups);
}

int conv_gemm_launch(const ConvGeom &g, const GemmPlan &p, const KTabEntry *dev_ktab, const void *x, const void *wpacked,
                     void *y, const Epilogue &ep, hipStream_t stream, int n_valid, void *part_ws, size_t part_bytes, const void *w,
                     int *own_counters)
{
    if (g.dtype != DLP_FLOAT && g.dtype != DLP_BFLOAT16)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "implicit-GEMM convolution: float_data and bfloat16_data are implemented");
    const size_t esize = dtype_size(g.dtype);
    DLP_REQUIRE(g.KH <= 31 && g.KW <= 31, "kernel extent above 31 is not supported by the gather masks");
    const size_t x_elems = (size_t)g.B * g.Cin * g.H * g.W;
    const size_t y_elems = (size_t)g.B * g.Cout * g.OH * g.OW;
    const size_t x_shift = ((size_t)g.ph * g.W + g.pw) * esize;
    if (x_elems * esize + x_shift >= kOutOfRange || p.wpack_bytes >= kOutOfRange || y_elems >= 0x7fffffffULL)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "tensors of 2 GiB or more are not supported by the 32-bit buffer addressing");
    if (g.B == 0)
        return DLP_OK;
    if (!layouts_supported(g, p))
        return fail(DLP_ERR_NOT_IMPLEMENTED, "channels-last tensors: served by the bf16 matrix-instruction kernels only (input channels per group in "
                                             "multiples of 32 for x, output channels per group in eights for y)");
    if (p.stem) {
        if (w == nullptr || n_valid >= 0)
            return fail(DLP_ERR_NOT_IMPLEMENTED, "stem convolution: needs the weight tensor and the whole batch");
        return conv_stem_launch(g, x, w, y, ep, stream, g.pool_ph, g.pool_pw);
    }
    if (g.pool_ph > 0)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "max pooling inside the convolution: the bf16 stem kernel only");
    // few output channels, 1x1: X streams from memory straight into the matrix instructions (needs the filter as it lies in memory)
    if (p.pointwise && w != nullptr && n_valid < 0 && (((uintptr_t)x | (uintptr_t)w | (uintptr_t)y) & 15) == 0 && ep.activation != DLP_ACT_TANH &&
        ep.activation != DLP_ACT_SIGMOID)
        return conv_pointwise_launch(g, x, w, y, ep, stream);

    GemmArgs a;
    a.x = x;
    a.wp = (const float *)wpacked;
    a.bias = ep.bias;
    a.y = y;
    a.ktab = (const int32_t *)dev_ktab;
    a.M = p.M;
    a.K = p.K;
    a.nkt = p.nkt;
    a.N = g.B * g.OH * g.OW;
    if (n_valid >= 0 && n_valid < a.N)
        a.N = n_valid;
    if (a.N == 0)
        return DLP_OK;
    a.Cout = g.Cout;
    a.groups = g.groups;
    a.part = (float *)part_ws;
    a.Cin = g.Cin;
    a.Cin_g = g.Cin / g.groups;
    a.H = g.H;
    a.W = g.W;
    a.OW = g.OW;
    a.OHW = g.OH * g.OW;
    a.sh = g.sh; a.sw = g.sw; a.ph = g.ph; a.pw = g.pw; a.dh = g.dh; a.dw = g.dw;
    a.KH = g.KH; a.KW = g.KW;
    a.x_bytes = (uint32_t)(x_elems * esize);
    a.wp_bytes = (uint32_t)p.wpack_bytes;
    a.wdirect = 0;
    if (p.wdirect && w != nullptr && ((uintptr_t)w & 15) == 0) { // same test as in conv_gemm_pack_weights
        a.wdirect = 1;
        a.wp = (const float *)w;
        a.wp_bytes = (uint32_t)((size_t)g.Cout * p.K * esize);
    }
    a.y_bytes = y_elems * esize < kOutOfRange ? (uint32_t)(y_elems * esize) : 0;
    a.x_shift = (uint32_t)x_shift;
    a.hw4 = (uint32_t)(g.H * g.W * esize);
    make_magic((uint32_t)a.OHW, a.ohw_magic, a.ohw_shift);
    make_magic((uint32_t)a.OW, a.ow_magic, a.ow_shift);
    a.factor = ep.factor;
    a.pre = ep.accumulate_first;
    a.act = ep.activation;
    a.clamp_lo = -__builtin_huge_valf();
    a.clamp_hi = __builtin_huge_valf();
    if (ep.activation == DLP_ACT_RELU || ep.activation == DLP_ACT_RELU6)
        a.clamp_lo = 0.0f;
    if (ep.activation == DLP_ACT_RELU6)
        a.clamp_hi = 6.0f;
    const int act = generic_act(ep.activation) ? ACT_GENERIC : ACT_CLAMP;
    if (p.patch)
        return launch_patch(g, p, a, stream, part_ws, part_bytes, own_counters);
    // workspace behind the packed weights, bf16 kernels: channels-last copy of the input | split-K partial sums
    void *xt = nullptr;
    if (g.x_channels_last) {
        if (!p.xt || n_valid >= 0 || ((uintptr_t)x & 15) != 0 || x_elems * esize + ((size_t)g.ph * g.W + g.pw) * g.Cin * esize >= kOutOfRange)
            return fail(DLP_ERR_NOT_IMPLEMENTED, "channels-last input: needs the bf16 matrix-instruction kernel, a 16-byte aligned x below 2 GiB and the whole batch");
        xt = const_cast<void *>(x);
    } else if (p.xt && part_ws != nullptr && part_bytes >= xt_bytes(g, g.B) && ((uintptr_t)part_ws & 15) == 0 && n_valid < 0 &&
        xt_bytes(g, g.B) + ((size_t)g.ph * g.W + g.pw) * g.Cin * esize < kOutOfRange) {
        xt = part_ws;
        part_ws = (char *)part_ws + xt_bytes(g, g.B);
        part_bytes -= xt_bytes(g, g.B);
        a.part = (float *)part_ws;
    }
    plan_split(p, a, g.groups, part_ws != nullptr, part_bytes);
    a.sk_cnt = nullptr;
    a.part_bytes = 0;
    if ((a.splitk > 1 || a.tail_tiles > 0) && !bf16_mfma_order(p.order)) {
        // reduced in place; the counters were cleared by conv_gemm_pack_weights (same workspace, a batch at least as large)
        const long long tiles = (long long)a.mtiles * a.ntiles * g.groups;
        const size_t images = split_total_bytes(p, a, g.groups) - split_counter_bytes(tiles);
        if (images >= kOutOfRange)
            return fail(DLP_ERR_NOT_IMPLEMENTED, "split-K workspace of 2 GiB or more");
        a.sk_cnt = own_counters ? own_counters : (int *)part_ws;
        a.sk_part = (float *)((char *)part_ws + split_counter_bytes(tiles));
        a.sk_part_bytes = (uint32_t)images;
    } else if (a.splitk > 1) {
        const size_t used = (size_t)a.splitk * a.Cout * a.N * sizeof(float);
        a.part_bytes = used < kOutOfRange ? (uint32_t)used : 0;
    }

    a.pxv = 0;
    a.y_cl = 0;
    if (g.y_channels_last) {
        if (!bf16_mfma_order(p.order) || (p.M & 7) != 0 || a.y_bytes == 0 || ((uintptr_t)y & 15) != 0 || !(ep.factor == 0.0f || ep.accumulate_first))
            return fail(DLP_ERR_NOT_IMPLEMENTED, "channels-last output: needs the bf16 matrix-instruction kernel, output channels per group in eights, a 16-byte "
                                                 "aligned y below 2 GiB, and factor 0 or accumulate_before_activation");
        a.y_cl = 1;
    }
    if (bf16_mfma_order(p.order)) {
        // wide output stores: runs of 8, 4 or 2 pixels that stay inside one image, dword aligned
        if ((ep.factor == 0.0f || ep.accumulate_first) && a.y_bytes != 0 && ((uintptr_t)y & 3) == 0 && a.splitk == 1 && !a.y_cl)
            a.pxv = a.OHW % 8 == 0 ? 8 : a.OHW % 4 == 0 ? 4 : a.OHW % 2 == 0 ? 2 : 0;
        // dense loader (1x1, stride 1, no padding): runs of 8 or 4 input pixels, dword aligned
        if (p.patch_bf16 && ((uintptr_t)x & 3) == 0)
            return launch_patch_bf16(g, p, a, stream);
        const int pxl = ((uintptr_t)x & 3) == 0 ? p.dense_pxl : 0;
        return launch_bf16_mfma(g, p, pxl, a, stream, xt);
    }
    return with_tile(p.tile, [&](auto bm, auto bn, auto wm, auto wn) {
        if (g.dtype == DLP_BFLOAT16)
            return launch_tile<bf16_t, decltype(bm)::value, decltype(bn)::value, decltype(wm)::value, decltype(wn)::value>(g, p, a, act, stream);
        return launch_tile<float, decltype(bm)::value, decltype(bn)::value, decltype(wm)::value, decltype(wn)::value>(g, p, a, act, stream);
    });
}

} // namespace dlp
