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
//  * all addressing of the gather is hoisted: per pixel a base offset and a bit
//    mask of the window taps that fall inside the image, per k a table entry
//    (offset, tap bit) read through the scalar unit.  Out-of-window taps and tile
//    tails are redirected to an out-of-range buffer offset, which the buffer
//    load returns as 0.0 -- the main loop has no divergent control flow.
//  * global loads of tile kt+1 are issued before the MFMAs of tile kt
//    (register-staged double buffering, one barrier per K step).
#include "dlp_internal.hpp"

#include <type_traits>

namespace dlp {

typedef float f32x16 __attribute__((ext_vector_type(16)));

namespace {

constexpr int kThreads = 256;
constexpr int BK = 16;
constexpr uint32_t kOutOfRange = 0x80000000u; // >= num_records of every buffer we accept

// How the validity of a gathered tap is decided:
//  MASK_NONE : every tap of every pixel is inside the image (pad 0 fits) -- only tile tails are masked
//  MASK_TAPS : KH*KW <= 32, one bit per tap in a single per-pixel word
//  MASK_ROWCOL: any kernel up to 31x31, separate row and column masks
enum { MASK_NONE = 0, MASK_TAPS = 1, MASK_ROWCOL = 2 };
// Epilogue flavour: clamp covers identity / relu / relu6 with two constants, no branches
enum { ACT_CLAMP = 0, ACT_GENERIC = 1 };

struct GemmArgs {
    const float *x;
    const float *w;
    const float *bias;
    float *y;
    const KTabEntry *ktab;
    int M, N, K, nkt;
    int mtiles, ntiles;
    int splitk, kt_per_slice; // K tiles are dealt to `splitk` slices of kt_per_slice (even) tiles
    float *part;              // split-K partial sums [slice][Cout][N]
    int Cin, Cin_g, H, W, Cout, OW, OHW, groups;
    int sh, sw, ph, pw, dh, dw, KH, KW;
    uint32_t x_bytes, w_bytes;
    float factor;
    int act;
    float clamp_lo, clamp_hi;
};

typedef __attribute__((address_space(4))) KTabEntry KTabConst;

__device__ __forceinline__ float buf_load(__amdgpu_buffer_rsrc_t r, uint32_t byte_off)
{
    // keep the offset a single opaque value: the select that produced it must stay a
    // v_cndmask, not become two loads under divergent branches
    asm("" : "+v"(byte_off));
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, byte_off, 0, 0));
}

// call f(integral_constant<int, kk>) for the compile-time value matching the runtime-unrolled kk
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

template <int BM, int BN, int WM, int WN, int MASK, int ACT>
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

    __shared__ float As[2][BK][LDA];
    __shared__ float Bs[2][BK][LDB];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int h = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;

    // tile decode: m tile fastest, then n tile, then group
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

    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, a.w_bytes, 0x00020000);

    // ---- per-thread gather state (one output pixel per thread) ----
    const int p = tid % BN;
    const int ks = (KSPLIT == 1) ? 0 : __builtin_amdgcn_readfirstlane(tid / BN);
    int base;
    uint32_t my = 0, mx = 0; // MASK_TAPS: my = tap mask; MASK_ROWCOL: row / column masks
    {
        const int n = n0 + p;
        const bool vn = n < a.N;
        const int b = n / a.OHW;
        const int pix = n - b * a.OHW;
        const int oy = pix / a.OW;
        const int ox = pix - oy * a.OW;
        const int iy0 = oy * a.sh - a.ph;
        const int ix0 = ox * a.sw - a.pw;
        base = ((b * a.Cin + g * a.Cin_g) * a.H + iy0) * a.W + ix0;
        if (MASK == MASK_NONE) {
            // (base + offset)*4 lands in [2^31, 2^32) for every table offset: out of range
            if (!vn)
                base = 0x20000000;
        } else if (vn) {
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

    // ---- per-thread weight loader state ----
    const int ak = tid & 15;
    const int am = tid >> 4;
    uint32_t a_off[A_LD];
#pragma unroll
    for (int j = 0; j < A_LD; j++) {
        int m = m0 + am + 16 * j;
        a_off[j] = (m < a.M) ? (uint32_t)(((g * a.M + m) * a.K + ak) * 4) : kOutOfRange;
    }

    // Two register sets for staged tiles: tile kt+2 is being fetched from memory
    // into one set while tile kt+1 moves from the other set into LDS and tile kt
    // (already in LDS) feeds the matrix cores.  A global load therefore has a whole
    // K step to land before anything waits on it.
    float ra[2][A_LD], rb[2][B_LD];

    // one slice of the loads of tile kt into register set S: called once per MFMA
    // group so that address arithmetic and vector-memory issue hide under MFMAs
    auto load_slice = [&](auto set, int kt, auto slice) {
        constexpr int S = decltype(set)::value;
        constexpr int Q = decltype(slice)::value;
        const int k0 = kt * BK;
        const uint32_t kmask = (k0 + ak < a.K) ? 0u : kOutOfRange;
#pragma unroll
        for (int j = 0; j < A_LD; j++)
            if (j % (BK / 2) == Q)
                ra[S][j] = buf_load(wr, (a_off[j] + (uint32_t)(k0 * 4)) | kmask);
        // the table is read-only for the whole launch and the index is wavefront-uniform:
        // constant address space makes these scalar loads (s_load), off the vector path
        const KTabConst *tab = (const KTabConst *)(a.ktab) + k0 + ks * B_LD;
#pragma unroll
        for (int i = 0; i < B_LD; i++) {
            if (i % (BK / 2) != Q)
                continue;
            const KTabEntry e = {tab[i].offset, tab[i].tap};
            uint32_t off = (uint32_t)((base + e.offset) * 4);
            if (MASK == MASK_TAPS) {
                off = (my & (uint32_t)e.tap) ? off : kOutOfRange;
            } else if (MASK == MASK_ROWCOL) {
                const int ky = e.tap & 0xff, kx = e.tap >> 8;
                off = ((my >> ky) & (mx >> kx) & 1u) ? off : kOutOfRange;
            }
            rb[S][i] = buf_load(xr, off);
        }
    };
    auto store_slice = [&](auto set, int buf, auto slice) {
        constexpr int S = decltype(set)::value;
        constexpr int Q = decltype(slice)::value;
#pragma unroll
        for (int j = 0; j < A_LD; j++)
            if (j % (BK / 2) == Q)
                As[buf][ak][am + 16 * j] = ra[S][j];
#pragma unroll
        for (int i = 0; i < B_LD; i++)
            if (i % (BK / 2) == Q)
                Bs[buf][ks * B_LD + i][p] = rb[S][i];
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
    auto read_operands = [&](int buf, int kk, int slot) {
        const int k = 2 * kk + h;
#pragma unroll
        for (int i = 0; i < TM; i++)
            fa[slot][i] = As[buf][k][wm * WTM + i * 32 + l32];
#pragma unroll
        for (int j = 0; j < TN; j++)
            fb[slot][j] = Bs[buf][k][wn * WTN + j * 32 + l32];
    };

    // One K step: MFMAs of tile kt (in LDS[buf]); register set SN (tile kt+1) goes to
    // LDS[buf^1]; tile kt+2 is fetched into register set SL.  Operands of step kk+1
    // are read from LDS before the MFMAs of step kk are issued.
    auto k_step = [&](auto set_next, auto set_load, int kt) {
        const int buf = kt & 1;
        read_operands(buf, 0, 0);
#pragma unroll
        for (int kk = 0; kk < BK / 2; kk++) {
            const int cur = kk & 1;
            if (kk + 1 < BK / 2)
                read_operands(buf, kk + 1, cur ^ 1);
            static_for_slice(kk, [&](auto q) {
                store_slice(set_next, buf ^ 1, q);
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
    static_for_all([&](auto q) { store_slice(I0{}, 0, q); });
    __syncthreads();
    // tile counts are even (the host rounds up; tiles past K load zeros through the masks)
    for (int kt = kt_begin; kt < kt_end; kt += 2) {
        k_step(I1{}, I0{}, kt);
        k_step(I0{}, I1{}, kt + 1);
    }

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
        const int b = n / a.OHW;
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

// Split-K factor for a launch of `tiles` output tiles over `nkt` (even) K tiles.
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

template <int BM, int BN>
void plan_split(GemmArgs &a, int groups, size_t ws_bytes)
{
    a.mtiles = (a.M + BM - 1) / BM;
    a.ntiles = (a.N + BN - 1) / BN;
    int s = choose_splitk((long long)a.mtiles * a.ntiles * groups, a.nkt);
    if (s > 1 && (a.part == nullptr || ws_bytes < (size_t)s * a.Cout * a.N * sizeof(float)))
        s = 1; // no (or too small a) workspace: run unsplit
    a.splitk = s;
    a.kt_per_slice = ((a.nkt + s - 1) / s + 1) / 2 * 2;
}

template <int BM, int BN, int WM, int WN, int MASK, int ACT>
int launch_inst(const ConvGeom &g, GemmArgs &a, hipStream_t stream)
{
    long long blocks = (long long)a.mtiles * a.ntiles * g.groups * a.splitk;
    if (blocks > 0x7fffffffLL)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "convolution too large for a single launch");
    hipLaunchKernelGGL((conv_gemm_f32_kernel<BM, BN, WM, WN, MASK, ACT>), dim3((unsigned)blocks), dim3(kThreads), 0, stream, a);
    if (a.splitk > 1) {
        const long long total = (long long)a.Cout * a.N;
        hipLaunchKernelGGL((splitk_reduce_kernel<ACT>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, a);
    }
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

template <int BM, int BN, int WM, int WN>
int launch_tile(const ConvGeom &g, GemmArgs &a, int mask, int act, size_t ws_bytes, hipStream_t stream)
{
    plan_split<BM, BN>(a, g.groups, ws_bytes);
    if (act == ACT_CLAMP) {
        if (mask == MASK_NONE)
            return launch_inst<BM, BN, WM, WN, MASK_NONE, ACT_CLAMP>(g, a, stream);
        if (mask == MASK_TAPS)
            return launch_inst<BM, BN, WM, WN, MASK_TAPS, ACT_CLAMP>(g, a, stream);
        return launch_inst<BM, BN, WM, WN, MASK_ROWCOL, ACT_CLAMP>(g, a, stream);
    }
    // tanh / sigmoid: rare, one generic instantiation per tile
    return launch_inst<BM, BN, WM, WN, MASK_ROWCOL, ACT_GENERIC>(g, a, stream);
}

bool generic_act(int activation) { return activation == DLP_ACT_TANH || activation == DLP_ACT_SIGMOID; }

int mask_mode(const ConvGeom &g, int activation)
{
    if (generic_act(activation))
        return MASK_ROWCOL; // the rare activations share one instantiation per tile
    // no tap can fall outside the image (no padding, last window fits) and no K tail
    const bool fits_h = g.ph == 0 && (g.OH - 1) * g.sh + (g.KH - 1) * g.dh < g.H;
    const bool fits_w = g.pw == 0 && (g.OW - 1) * g.sw + (g.KW - 1) * g.dw < g.W;
    const int K = (g.Cin / g.groups) * g.KH * g.KW;
    if (fits_h && fits_w && K % BK == 0)
        return MASK_NONE;
    if (g.KH * g.KW <= 32)
        return MASK_TAPS;
    return MASK_ROWCOL;
}

} // namespace

size_t conv_gemm_ktab_entries(const ConvGeom &g)
{
    // K tiles rounded up to an even count, plus two tiles of never-valid entries that
    // the software pipeline prefetches past the end
    size_t K = (size_t)(g.Cin / g.groups) * g.KH * g.KW;
    size_t tiles = (K + BK - 1) / BK;
    tiles = (tiles + 1) / 2 * 2 + 2;
    return tiles * BK;
}

void conv_gemm_fill_ktab(const ConvGeom &g, int activation, KTabEntry *tab)
{
    const int cin_g = g.Cin / g.groups;
    const size_t Kp = conv_gemm_ktab_entries(g);
    const int mode = mask_mode(g, activation);
    size_t k = 0;
    for (int c = 0; c < cin_g; c++)
        for (int ky = 0; ky < g.KH; ky++)
            for (int kx = 0; kx < g.KW; kx++, k++) {
                tab[k].offset = (c * g.H + ky * g.dh) * g.W + kx * g.dw;
                tab[k].tap = (mode == MASK_ROWCOL) ? (ky | (kx << 8)) : (int32_t)(1u << ((ky * g.KW + kx) & 31));
            }
    for (; k < Kp; k++) {
        // padding rows of the last K tile: never valid (MASK_NONE has no K tail)
        tab[k].offset = 0;
        tab[k].tap = (mode == MASK_ROWCOL) ? (31 | (31 << 8)) : 0;
    }
}

// Workspace the split-K path wants for this geometry (0 when it would not split).
size_t conv_gemm_workspace_bytes(const ConvGeom &g)
{
    if (g.B <= 0)
        return 0;
    GemmArgs a;
    a.M = g.Cout / g.groups;
    a.N = g.B * g.OH * g.OW;
    a.Cout = g.Cout;
    a.nkt = (((g.Cin / g.groups) * g.KH * g.KW + BK - 1) / BK + 1) / 2 * 2;
    a.part = (float *)16; // any non-null value: ask for the unconstrained plan
    if (a.M > 64)
        plan_split<128, 128>(a, g.groups, (size_t)-1);
    else if (a.M > 32)
        plan_split<64, 256>(a, g.groups, (size_t)-1);
    else
        plan_split<32, 256>(a, g.groups, (size_t)-1);
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
    if (x_elems * 4 >= 0x20000000ULL * 4 || w_elems * 4 >= kOutOfRange || y_elems >= 0x7fffffffULL)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "tensors of 2 GiB or more are not supported by the 32-bit buffer addressing");
    if (g.B == 0)
        return DLP_OK;

    GemmArgs a;
    a.x = (const float *)x;
    a.w = (const float *)w;
    a.bias = ep.bias;
    a.y = (float *)y;
    a.ktab = dev_ktab;
    a.M = g.Cout / g.groups;
    a.N = g.B * g.OH * g.OW;
    if (n_valid >= 0 && n_valid < a.N)
        a.N = n_valid;
    if (a.N == 0)
        return DLP_OK;
    a.K = (g.Cin / g.groups) * g.KH * g.KW;
    a.nkt = ((a.K + BK - 1) / BK + 1) / 2 * 2;
    a.Cin = g.Cin;
    a.Cin_g = g.Cin / g.groups;
    a.H = g.H;
    a.W = g.W;
    a.Cout = g.Cout;
    a.groups = g.groups;
    a.part = (float *)ws;
    a.OW = g.OW;
    a.OHW = g.OH * g.OW;
    a.sh = g.sh; a.sw = g.sw; a.ph = g.ph; a.pw = g.pw; a.dh = g.dh; a.dw = g.dw;
    a.KH = g.KH; a.KW = g.KW;
    a.x_bytes = (uint32_t)(x_elems * 4);
    a.w_bytes = (uint32_t)(w_elems * 4);
    a.factor = ep.factor;
    a.act = ep.activation;
    a.clamp_lo = -__builtin_huge_valf();
    a.clamp_hi = __builtin_huge_valf();
    if (ep.activation == DLP_ACT_RELU || ep.activation == DLP_ACT_RELU6)
        a.clamp_lo = 0.0f;
    if (ep.activation == DLP_ACT_RELU6)
        a.clamp_hi = 6.0f;
    const int act = generic_act(ep.activation) ? ACT_GENERIC : ACT_CLAMP;
    const int mask = mask_mode(g, ep.activation); // same rule the gather table was built with

    if (a.M > 64)
        return launch_tile<128, 128, 2, 2>(g, a, mask, act, ws_bytes, stream);
    if (a.M > 32)
        return launch_tile<64, 256, 1, 4>(g, a, mask, act, ws_bytes, stream);
    return launch_tile<32, 256, 1, 4>(g, a, mask, act, ws_bytes, stream);
}

} // namespace dlp
