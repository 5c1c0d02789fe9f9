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
//    pipe of its SIMD (measured: MFMA time and VALU time add up), so the gather is
//    built to need almost no VALU work in the main loop:
//      - every global load is a buffer load whose address is
//        resource base + per-thread VGPR offset (loop invariant) + SGPR offset (per k),
//        the SGPR part coming from a small table read through the scalar unit;
//      - padding and tile tails are handled by swapping the VGPR offset for an
//        out-of-range one, which the buffer load returns as 0.0 (no branches);
//      - K is walked tap-major whenever Cin/groups is a multiple of 16: one K tile =
//        one filter tap x 16 input channels, so the in-image test is one bit test
//        per K tile instead of one per element.  The sum over K is order-free, the
//        weights are fetched in the matching order (stride KH*KW, L2 resident).
//        Other shapes (e.g. the 3-channel stem) use a per-element table.
//  * software pipeline of distance two: tile kt+2 is in flight from memory to
//    registers while tile kt+1 moves registers -> LDS and tile kt feeds the MFMAs.
//  * layers with too few output tiles for 256 CUs split K over several
//    workgroups; partial sums go through the workspace and are reduced in a
//    fixed order by a second kernel (deterministic).
#include "dlp_internal.hpp"

#include <cstdlib>
#include <type_traits>
#include <vector>

namespace dlp {

typedef float f32x16 __attribute__((ext_vector_type(16)));

namespace {

constexpr int kThreads = 256;
constexpr int BK = 16;
constexpr uint32_t kOutOfRange = 0x80000000u; // >= num_records of every buffer we accept

// K ordering / gather table flavour
enum { ORDER_CHANNEL = 0, ORDER_TAP = 1 };
// In-image test: one bit per tap (KH*KW <= 32) or separate row / column masks
enum { MASK_TAPS = 1, MASK_ROWCOL = 2 };
// Epilogue flavour: clamp covers identity / relu / relu6 with two constants
enum { ACT_CLAMP = 0, ACT_GENERIC = 1 };

struct GemmArgs {
    const float *x;
    const float *w;
    const float *bias;
    float *y;
    const int32_t *ktab;
    int M, N, K, nkt;
    int mtiles, ntiles;
    int splitk, kt_per_slice; // K tiles are dealt to `splitk` slices of kt_per_slice (even) tiles
    float *part;              // split-K partial sums [slice][Cout][N]
    int Cin, Cin_g, H, W, Cout, OW, OHW, groups;
    int sh, sw, ph, pw, dh, dw, KH, KW;
    uint32_t x_bytes, w_bytes;
    uint32_t x_shift; // bytes by which the X resource base is moved back (padding offset)
    uint32_t hw4;     // H*W*4: byte stride between input channels
    uint32_t ohw_magic, ohw_shift, ow_magic, ow_shift;
    float factor;
    int act;
    float clamp_lo, clamp_hi;
};

typedef __attribute__((address_space(4))) const int32_t ConstInt;

// q = n / d for 0 <= n < 2^31 with host-made (magic, shift)
__device__ __forceinline__ uint32_t fast_div(uint32_t n, uint32_t magic, uint32_t shift)
{
    return (__umulhi(n, magic) + n) >> shift;
}

__device__ __forceinline__ float buf_load(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
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

template <int BM, int BN, int WM, int WN, int ORDER, int MASK, int ACT>
__global__ __launch_bounds__(kThreads) void conv_gemm_f32_kernel(GemmArgs a)
{
    static_assert(BK == 16, "the slice helpers assume 8 MFMA steps per K tile");
    static_assert(WM * WN == 4, "four wavefronts per workgroup");
    constexpr int WTM = BM / WM, WTN = BN / WN; // wavefront tile
    constexpr int TM = WTM / 32, TN = WTN / 32; // MFMA blocks per wavefront
    static_assert(TM >= 1 && TN >= 1 && WTM % 32 == 0 && WTN % 32 == 0, "tile shape");
    constexpr int LDA = BM + 2; // stride = 2 (mod 32): transposed A stores hit 32 distinct banks
    constexpr int LDB = BN;
    constexpr int KSPLIT = kThreads / BN;    // k slices among the B loader threads
    static_assert(KSPLIT >= 1 && BN % 64 == 0 && BK % KSPLIT == 0, "B loader shape");
    constexpr int B_LD = BK / KSPLIT;        // gathered elements per thread per K step (contiguous k)
    constexpr int A_LD = BM * BK / kThreads; // weight elements per thread per K step
    static_assert(A_LD >= 1, "weight loader shape");

    __shared__ float As[2][BK][LDA];
    __shared__ float Bs[2][BK][LDB];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int h = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;

    // tile decode: m tile fastest, then n tile, then group, then K slice
    int t = blockIdx.x;
    const int mt = t % a.mtiles;
    t /= a.mtiles;
    const int nt = t % a.ntiles;
    t /= a.ntiles;
    const int g = t % a.groups;
    const int slice = t / a.groups;
    const int m0 = mt * BM, n0 = nt * BN;
    const int kt_begin = slice * a.kt_per_slice;
    const int kt_end = min(kt_begin + a.kt_per_slice, a.nkt);

    // The X resource starts one padding offset before the tensor, so that the
    // per-pixel window origin is a non-negative offset; taps that the masks let
    // through never address below the tensor.
    const __amdgpu_buffer_rsrc_t xr =
        __builtin_amdgcn_make_buffer_rsrc((void *)((const char *)a.x - a.x_shift), 0, a.x_bytes + a.x_shift, 0x00020000);
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, a.w_bytes, 0x00020000);
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
        vbase = (uint32_t)((((b * a.Cin + g * a.Cin_g) * a.H + oy * a.sh) * a.W + ox * a.sw) * 4);
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
            if (MASK == MASK_TAPS) {
                for (int ky = 0; ky < a.KH; ky++)
                    if ((ry >> ky) & 1u)
                        my |= rx << (ky * a.KW);
            } else {
                my = ry;
                mx = rx;
            }
        }
    }

    // ---- per-thread weight loader state: row (m) part of the address ----
    const int ak = tid & 15;
    const int am = tid >> 4;
    uint32_t a_voff[A_LD];
#pragma unroll
    for (int j = 0; j < A_LD; j++) {
        const int m = m0 + am + 16 * j;
        uint32_t off;
        if (ORDER == ORDER_TAP)
            off = (uint32_t)((((g * a.M + m) * a.Cin_g + ak) * (a.KH * a.KW)) * 4);
        else
            off = (uint32_t)(((g * a.M + m) * a.K + ak) * 4);
        a_voff[j] = (m < a.M) ? off : kOutOfRange;
    }

    // Two register sets for staged tiles: tile kt+2 is being fetched from memory
    // into one set while tile kt+1 moves from the other set into LDS and tile kt
    // (already in LDS) feeds the matrix cores.  A global load therefore has a whole
    // K step to land before anything waits on it.
    float ra[2][A_LD], rb[2][B_LD];
    uint32_t vsel[2] = {kOutOfRange, kOutOfRange}; // ORDER_TAP: this tile's (masked) pixel offset
    uint32_t akm[2] = {0, 0};                      // ORDER_CHANNEL: K-tail mask of the weight loads

    // one slice of the loads of tile kt into register set S: called once per MFMA
    // group so that vector-memory issue is spread under the MFMAs
    auto load_slice = [&](auto set, int kt, auto slice_q) {
        constexpr int S = decltype(set)::value;
        constexpr int Q = decltype(slice_q)::value;
        if (ORDER == ORDER_TAP) {
            // table entry of a K tile: {x byte offset of (channel block, tap), tap bit, weight byte offset, -}
            ConstInt *e = ktab + kt * 4;
            const uint32_t xoff = (uint32_t)e[0], tapbit = (uint32_t)e[1], woff = (uint32_t)e[2];
            if (Q == 0)
                vsel[S] = opaque((my & tapbit) ? vbase : kOutOfRange);
#pragma unroll
            for (int j = 0; j < A_LD; j++)
                if (j % (BK / 2) == Q)
                    ra[S][j] = buf_load(wr, a_voff[j], woff);
#pragma unroll
            for (int i = 0; i < B_LD; i++)
                if (i % (BK / 2) == Q)
                    rb[S][i] = buf_load(xr, vsel[S], xoff + (uint32_t)(ks * B_LD + i) * a.hw4);
        } else {
            const int k0 = kt * BK;
            if (Q == 0) // rows past K (tail of the last tile, tiles fetched past the end) read nothing
                akm[S] = (k0 + ak < a.K) ? 0u : kOutOfRange;
            const uint32_t k0c = (uint32_t)min(k0, (a.nkt - 1) * BK) * 4u; // SGPR part stays inside the tensor
#pragma unroll
            for (int j = 0; j < A_LD; j++)
                if (j % (BK / 2) == Q)
                    ra[S][j] = buf_load(wr, opaque(a_voff[j] | akm[S]), k0c);
            // table entry of a k: {x byte offset of (c,ky,kx), tap bit or ky|kx<<8}
            ConstInt *e = ktab + (k0 + ks * B_LD) * 2;
#pragma unroll
            for (int i = 0; i < B_LD; i++) {
                if (i % (BK / 2) != Q)
                    continue;
                const uint32_t xoff = (uint32_t)e[2 * i], tap = (uint32_t)e[2 * i + 1];
                bool ok;
                if (MASK == MASK_TAPS)
                    ok = (my & tap) != 0;
                else
                    ok = ((my >> (tap & 0xff)) & (mx >> (tap >> 8)) & 1u) != 0;
                rb[S][i] = buf_load(xr, opaque(ok ? vbase : kOutOfRange), xoff);
            }
        }
    };
    auto store_slice = [&](auto set, auto buf_c, auto slice_q) {
        constexpr int S = decltype(set)::value;
        constexpr int BUF = decltype(buf_c)::value;
        constexpr int Q = decltype(slice_q)::value;
#pragma unroll
        for (int j = 0; j < A_LD; j++)
            if (j % (BK / 2) == Q)
                As[BUF][ak][am + 16 * j] = ra[S][j];
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
        read_operands(buf_c, 0, 0);
#pragma unroll
        for (int kk = 0; kk < BK / 2; kk++) {
            const int cur = kk & 1;
            if (kk + 1 < BK / 2)
                read_operands(buf_c, kk + 1, cur ^ 1);
            static_for_slice(kk, [&](auto q) {
                store_slice(set_next, NextBuf{}, q);
                load_slice(set_load, kt + 2, q);
            });
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cur][i], fb[cur][j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    // prologue: first tile -> set 0 -> LDS[0]; second tile -> set 1
    static_for_all([&](auto q) { load_slice(I0{}, kt_begin, q); });
    static_for_all([&](auto q) { load_slice(I1{}, kt_begin + 1, q); });
    static_for_all([&](auto q) { store_slice(I0{}, I0{}, q); });
    __syncthreads();
    // tiles fetched past kt_end are never multiplied: the table has two spare entries
    int kt = kt_begin;
    for (; kt + 1 < kt_end; kt += 2) {
        k_step(I0{}, I1{}, I0{}, kt);
        k_step(I1{}, I0{}, I1{}, kt + 1);
    }
    if (kt < kt_end)
        k_step(I0{}, I1{}, I0{}, kt);

    // ---- split-K: raw partial sums to the workspace, reduced by a second kernel ----
    if (a.splitk > 1) {
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
    // accumulator register r of a 32x32 block holds row 8*(r/4) + 4*h + r%4, column l32
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int n = n0 + wn * WTN + j * 32 + l32;
        if (n >= a.N)
            continue;
        const int b = (int)fast_div((uint32_t)n, a.ohw_magic, a.ohw_shift);
        const int pix = n - b * a.OHW;
        float *yb = a.y + ((size_t)b * a.Cout + (size_t)g * a.M) * a.OHW + pix;
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + wm * WTM + i * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                if (m < a.M) {
                    float v = acc[i][j][r];
                    if (a.bias)
                        v += a.bias[g * a.M + m];
                    if (ACT == ACT_CLAMP) {
                        if (a.act != DLP_ACT_IDENTITY) // identity must keep NaNs: no min/max
                            v = fminf(fmaxf(v, a.clamp_lo), a.clamp_hi);
                    } else
                        v = apply_act(v, a.act);
                    store_out(yb + (size_t)m * a.OHW, v, a.factor);
                }
            }
        }
    }
}

// Sums the split-K slices in slice order (deterministic) and applies the epilogue.
template <int ACT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(GemmArgs a)
{
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; // row * N + n
    const long long total = (long long)a.Cout * a.N;
    if (idx >= total)
        return;
    const int row = (int)(idx / a.N);
    const int n = (int)(idx - (long long)row * a.N);
    float v = 0.0f;
    for (int s = 0; s < a.splitk; s++)
        v += a.part[(size_t)s * total + idx];
    if (a.bias)
        v += a.bias[row];
    if (ACT == ACT_CLAMP) {
        if (a.act != DLP_ACT_IDENTITY)
            v = fminf(fmaxf(v, a.clamp_lo), a.clamp_hi);
    } else
        v = apply_act(v, a.act);
    const int b = n / a.OHW;
    const int pix = n - b * a.OHW;
    store_out(a.y + ((size_t)b * a.Cout + row) * a.OHW + pix, v, a.factor);
}

// Split-K factor for a launch of `tiles` output tiles over `nkt` K tiles.
// Workgroups of one launch are co-resident, so the time is set by the busiest CU:
// pick the factor that fills whole rounds of the 256 CUs best, keeping at least
// 8 K tiles per slice; 1 = no split.
int choose_splitk(long long tiles, int nkt)
{
    const int kCUs = 256;
    if (tiles >= 2 * kCUs || nkt < 16)
        return 1;
    int best = 1;
    double best_eff = (double)tiles / (double)(((tiles + kCUs - 1) / kCUs) * kCUs);
    for (int s = 2; s <= 8; s++) {
        if (nkt / s < 8)
            break;
        const long long blocks = tiles * s;
        const double eff = (double)blocks / (double)(((blocks + kCUs - 1) / kCUs) * kCUs);
        if (eff > best_eff + 0.05) {
            best_eff = eff;
            best = s;
        }
    }
    return best;
}

bool generic_act(int activation) { return activation == DLP_ACT_TANH || activation == DLP_ACT_SIGMOID; }

// K ordering and mask flavour of a geometry (the gather table is built to match).
void gather_mode(const ConvGeom &g, int activation, int &order, int &mask)
{
    const int cin_g = g.Cin / g.groups;
    if (generic_act(activation)) { // the rare activations share one instantiation per tile
        order = ORDER_CHANNEL;
        mask = MASK_ROWCOL;
        return;
    }
    const bool small_kernel = g.KH * g.KW <= 32;
    order = (small_kernel && cin_g % BK == 0) ? ORDER_TAP : ORDER_CHANNEL;
    mask = small_kernel ? MASK_TAPS : MASK_ROWCOL;
}

int k_tiles(const ConvGeom &g)
{
    const int K = (g.Cin / g.groups) * g.KH * g.KW; // tap-major order has the same count: K is a multiple of 16 there
    return (K + BK - 1) / BK;
}

template <int BM, int BN>
void plan_split(GemmArgs &a, int groups, size_t ws_bytes)
{
    a.mtiles = (a.M + BM - 1) / BM;
    a.ntiles = (a.N + BN - 1) / BN;
    int s = choose_splitk((long long)a.mtiles * a.ntiles * groups, a.nkt);
    if (s > 1 && (a.part == nullptr || ws_bytes < (size_t)s * a.Cout * a.N * sizeof(float)))
        s = 1; // no (or too small a) workspace: run unsplit
    a.kt_per_slice = ((a.nkt + s - 1) / s + 1) / 2 * 2;              // even: LDS buffer parity is static
    a.splitk = (a.nkt + a.kt_per_slice - 1) / a.kt_per_slice; // every slice starts inside the K range
}

template <int BM, int BN, int WM, int WN, int ORDER, int MASK, int ACT>
int launch_inst(const ConvGeom &g, GemmArgs &a, hipStream_t stream)
{
    long long blocks = (long long)a.mtiles * a.ntiles * g.groups * a.splitk;
    if (blocks > 0x7fffffffLL)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "convolution too large for a single launch");
    hipLaunchKernelGGL((conv_gemm_f32_kernel<BM, BN, WM, WN, ORDER, MASK, ACT>), dim3((unsigned)blocks), dim3(kThreads), 0, stream, a);
    if (a.splitk > 1) {
        const long long total = (long long)a.Cout * a.N;
        hipLaunchKernelGGL((splitk_reduce_kernel<ACT>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, a);
    }
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

template <int BM, int BN, int WM, int WN>
int launch_tile(const ConvGeom &g, GemmArgs &a, int order, int mask, int act, size_t ws_bytes, hipStream_t stream)
{
    plan_split<BM, BN>(a, g.groups, ws_bytes);
    if (act == ACT_GENERIC)
        return launch_inst<BM, BN, WM, WN, ORDER_CHANNEL, MASK_ROWCOL, ACT_GENERIC>(g, a, stream);
    if (order == ORDER_TAP)
        return launch_inst<BM, BN, WM, WN, ORDER_TAP, MASK_TAPS, ACT_CLAMP>(g, a, stream);
    if (mask == MASK_TAPS)
        return launch_inst<BM, BN, WM, WN, ORDER_CHANNEL, MASK_TAPS, ACT_CLAMP>(g, a, stream);
    return launch_inst<BM, BN, WM, WN, ORDER_CHANNEL, MASK_ROWCOL, ACT_CLAMP>(g, a, stream);
}

void make_magic(uint32_t d, uint32_t &magic, uint32_t &shift)
{
    // q = (umulhi(n, magic) + n) >> shift  ==  n / d   for 0 <= n < 2^31
    shift = 0;
    while ((1ull << shift) < d)
        shift++;
    magic = (uint32_t)(((1ull << 32) * ((1ull << shift) - d)) / d + 1);
}

// tile shape by rows per group; the experiment knob is for tuning runs only
int tile_choice(int M)
{
    if (const char *e = getenv("DLP_TILE_EXPERIMENT")) {
        int v = atoi(e);
        if (v > 0)
            return v;
    }
    if (M > 64)
        return 6;
    if (M > 32)
        return 5;
    return 8;
}

} // namespace

size_t conv_gemm_ktab_entries(const ConvGeom &g)
{
    // one 8-byte entry per k (ORDER_TAP uses two entries per K tile); two spare tiles of
    // never-valid entries are what the software pipeline fetches past the end
    return (size_t)(k_tiles(g) + 2) * BK;
}

void conv_gemm_fill_ktab(const ConvGeom &g, int activation, KTabEntry *tab_entries)
{
    int32_t *tab = (int32_t *)tab_entries;
    const size_t words = conv_gemm_ktab_entries(g) * 2;
    for (size_t i = 0; i < words; i++)
        tab[i] = 0; // spare entries: no tap bit (row/col code 31 below), offsets 0
    int order, mask;
    gather_mode(g, activation, order, mask);
    const int cin_g = g.Cin / g.groups;
    const int khw = g.KH * g.KW;
    if (order == ORDER_TAP) {
        int t = 0;
        for (int cb = 0; cb < cin_g / BK; cb++)
            for (int ky = 0; ky < g.KH; ky++)
                for (int kx = 0; kx < g.KW; kx++, t++) {
                    tab[4 * t + 0] = ((cb * BK * g.H + ky * g.dh) * g.W + kx * g.dw) * 4;
                    tab[4 * t + 1] = (int32_t)(1u << (ky * g.KW + kx));
                    tab[4 * t + 2] = (cb * BK * khw + ky * g.KW + kx) * 4;
                }
        return;
    }
    size_t k = 0;
    for (int c = 0; c < cin_g; c++)
        for (int ky = 0; ky < g.KH; ky++)
            for (int kx = 0; kx < g.KW; kx++, k++) {
                tab[2 * k + 0] = ((c * g.H + ky * g.dh) * g.W + kx * g.dw) * 4;
                tab[2 * k + 1] = (mask == MASK_ROWCOL) ? (ky | (kx << 8)) : (int32_t)(1u << (ky * g.KW + kx));
            }
    if (mask == MASK_ROWCOL)
        for (; 2 * k + 1 < words; k++)
            tab[2 * k + 1] = 31 | (31 << 8); // bit 31 of the row / column masks is never set
}

static void fill_dims(const ConvGeom &g, GemmArgs &a, int n_valid)
{
    a.M = g.Cout / g.groups;
    a.N = g.B * g.OH * g.OW;
    if (n_valid >= 0 && n_valid < a.N)
        a.N = n_valid;
    a.K = (g.Cin / g.groups) * g.KH * g.KW;
    a.nkt = k_tiles(g);
    a.Cout = g.Cout;
    a.groups = g.groups;
}

template <class F>
static auto with_tile(int choice, F &&f)
{
    switch (choice) {
    case 1: return f(std::integral_constant<int, 64>{}, std::integral_constant<int, 128>{}, std::integral_constant<int, 1>{}, std::integral_constant<int, 4>{});
    case 2: return f(std::integral_constant<int, 64>{}, std::integral_constant<int, 128>{}, std::integral_constant<int, 2>{}, std::integral_constant<int, 2>{});
    case 3: return f(std::integral_constant<int, 128>{}, std::integral_constant<int, 64>{}, std::integral_constant<int, 2>{}, std::integral_constant<int, 2>{});
    case 5: return f(std::integral_constant<int, 64>{}, std::integral_constant<int, 256>{}, std::integral_constant<int, 1>{}, std::integral_constant<int, 4>{});
    case 7: return f(std::integral_constant<int, 64>{}, std::integral_constant<int, 64>{}, std::integral_constant<int, 2>{}, std::integral_constant<int, 2>{});
    case 8: return f(std::integral_constant<int, 32>{}, std::integral_constant<int, 256>{}, std::integral_constant<int, 1>{}, std::integral_constant<int, 4>{});
    case 9: return f(std::integral_constant<int, 128>{}, std::integral_constant<int, 64>{}, std::integral_constant<int, 4>{}, std::integral_constant<int, 1>{});
    default: return f(std::integral_constant<int, 128>{}, std::integral_constant<int, 128>{}, std::integral_constant<int, 2>{}, std::integral_constant<int, 2>{});
    }
}

// Workspace the split-K path wants for this geometry (0 when it would not split).
size_t conv_gemm_workspace_bytes(const ConvGeom &g)
{
    if (g.B <= 0)
        return 0;
    GemmArgs a;
    fill_dims(g, a, -1);
    a.part = (float *)16; // any non-null value: ask for the unconstrained plan
    with_tile(tile_choice(a.M), [&](auto bm, auto bn, auto, auto) {
        plan_split<decltype(bm)::value, decltype(bn)::value>(a, g.groups, (size_t)-1);
        return 0;
    });
    return a.splitk > 1 ? (size_t)a.splitk * a.Cout * a.N * sizeof(float) : 0;
}

int conv_gemm_launch(const ConvGeom &g, const KTabEntry *dev_ktab, const void *x, const void *w,
                     void *y, const Epilogue &ep, hipStream_t stream, int n_valid, void *ws, size_t ws_bytes)
{
    if (g.dtype != DLP_FLOAT)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "implicit-GEMM convolution: only float_data is implemented");
    DLP_REQUIRE(g.KH <= 31 && g.KW <= 31, "kernel extent above 31 is not supported by the gather masks");
    const size_t x_elems = (size_t)g.B * g.Cin * g.H * g.W;
    const size_t w_elems = (size_t)g.Cout * (g.Cin / g.groups) * g.KH * g.KW;
    const size_t y_elems = (size_t)g.B * g.Cout * g.OH * g.OW;
    const size_t x_shift = ((size_t)g.ph * g.W + g.pw) * 4;
    if (x_elems * 4 + x_shift >= kOutOfRange || w_elems * 4 >= kOutOfRange || y_elems >= 0x7fffffffULL)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "tensors of 2 GiB or more are not supported by the 32-bit buffer addressing");
    if (g.B == 0)
        return DLP_OK;

    GemmArgs a;
    a.x = (const float *)x;
    a.w = (const float *)w;
    a.bias = ep.bias;
    a.y = (float *)y;
    a.ktab = (const int32_t *)dev_ktab;
    fill_dims(g, a, n_valid);
    if (a.N == 0)
        return DLP_OK;
    a.part = (float *)ws;
    a.Cin = g.Cin;
    a.Cin_g = g.Cin / g.groups;
    a.H = g.H;
    a.W = g.W;
    a.OW = g.OW;
    a.OHW = g.OH * g.OW;
    a.sh = g.sh; a.sw = g.sw; a.ph = g.ph; a.pw = g.pw; a.dh = g.dh; a.dw = g.dw;
    a.KH = g.KH; a.KW = g.KW;
    a.x_bytes = (uint32_t)(x_elems * 4);
    a.w_bytes = (uint32_t)(w_elems * 4);
    a.x_shift = (uint32_t)x_shift;
    a.hw4 = (uint32_t)(g.H * g.W * 4);
    make_magic((uint32_t)a.OHW, a.ohw_magic, a.ohw_shift);
    make_magic((uint32_t)a.OW, a.ow_magic, a.ow_shift);
    a.factor = ep.factor;
    a.act = ep.activation;
    a.clamp_lo = -__builtin_huge_valf();
    a.clamp_hi = __builtin_huge_valf();
    if (ep.activation == DLP_ACT_RELU || ep.activation == DLP_ACT_RELU6)
        a.clamp_lo = 0.0f;
    if (ep.activation == DLP_ACT_RELU6)
        a.clamp_hi = 6.0f;
    const int act = generic_act(ep.activation) ? ACT_GENERIC : ACT_CLAMP;
    int order, mask;
    gather_mode(g, ep.activation, order, mask); // same rule the gather table was built with

    return with_tile(tile_choice(a.M), [&](auto bm, auto bn, auto wm, auto wn) {
        return launch_tile<decltype(bm)::value, decltype(bn)::value, decltype(wm)::value, decltype(wn)::value>(g, a, order, mask, act,
                                                                                                                    ws_bytes, stream);
    });
}

} // namespace dlp
