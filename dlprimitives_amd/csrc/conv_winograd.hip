// Winograd F(2x2,3x3) convolution forward for gfx950.
//
// Replaces the reference's Conv2DForwardWinograd / winograd_fwd.cl
// (src/core/conv.cpp:223-297, src/kernels/winograd_fwd.cl): 3x3, stride 1,
// pad 1, dilation 1, groups 1, with the reference's transform matrices
//   G   = [[1,0,0],[1/2,1/2,1/2],[1/2,-1/2,1/2],[0,0,1]]      (:103-135)
//   B^T = [[1,0,-1,0],[0,1,1,0],[0,-1,1,0],[0,1,0,-1]]        (:35-69)
//   A^T = [[1,1,1,0],[0,1,-1,-1]]                             (:138-158)
// and the same order of additions inside each transform.  Odd H/W are handled
// by masked loads and stores as in the reference (:294-311,417-435).
//
// Two kernels per call, like the reference (filter transform, then one fused kernel):
//   wino_filter_kernel : U[e][c][n] = (G k G^T)[e], zero padded to the tile sizes, in the workspace
//     (stored so that the four k pairs of a chunk are 16 contiguous bytes per (k half, n))
//   wino_fused_kernel  : per workgroup 32 output channels x 32 tiles x all 16 transform
//     elements e.  The 16 element-wise products are 16 independent GEMMs
//       M_e[n][t] = sum_c U_e[c][n] * V_e[c][t]
//     on the fp32 matrix cores: wavefront w owns e = 4w..4w+3, one 32x32 accumulator block
//     each.  Per K chunk of 8 input channels, each of the 256 threads loads the 4x4 input
//     patch of one (channel, tile), transforms it (B^T d B, 32 additions) and writes the 16
//     values to LDS in [e][c][t] order, where the MFMA B operand is a conflict-free ds_read;
//     the A operand (U) is read straight from the L2-resident workspace into registers in MFMA
//     layout (lanes along n: 128-byte runs).  V and M never touch HBM.
//     Patch loads are buffer loads whose per-thread offsets (with the padding / tail masks
//     baked in as out-of-range offsets, which read as 0) are loop invariant; the channel
//     chunk advances through the scalar offset, so the loop needs no address arithmetic.
//     Loads run one chunk ahead of the transform and two ahead of the MFMAs (LDS is double
//     buffered, one barrier per chunk).
//     Epilogue: accumulators go through LDS (two passes of 16 channels), each thread
//     gathers the 16 e of one (n, tile), applies A^T m A, bias, activation, factor and
//     stores the 2x2 outputs; consecutive lanes hold consecutive tiles of a row.
#include "dlp_internal.hpp"

#include <cstdlib>
#include <type_traits>

namespace dlp {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t kOutOfRange = 0x80000000u; // >= num_records of every buffer accepted here
constexpr int KC = 8;                          // input channels per K chunk
constexpr int TT = 32;                         // tiles per workgroup
constexpr int NT = 32;                         // output channels per workgroup
constexpr int kThreads = 256;

struct WinoArgs {
    const void *x;
    void *y;
    const float *U;
    const float *bias;
    int C, N, H, W;
    int tw, tpi, T; // tiles per row, per image, in this launch
    int Cpad, Npad, nchunks, nblocks;
    uint32_t tpi_magic, tpi_shift, tw_magic, tw_shift;
    uint32_t x_bytes, u_bytes;
    int th;                  // tile rows per image
    int stage_stride;        // staged variant: floats per channel of the staging buffer
    uint32_t ss_magic, ss_shift;
    float factor;
    int pre; // the old value of y is added before the activation
    int act;
};

template <class T>
__device__ __forceinline__ float ld_elem(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff);
template <>
__device__ __forceinline__ float ld_elem<float>(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}
template <>
__device__ __forceinline__ float ld_elem<bf16_t>(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff)
{
    return __builtin_bit_cast(float, (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, 0) << 16);
}

// U[e][c][n] = (G k G^T)[e], src/kernels/winograd_fwd.cl:103-135; zero for padded c, n.
template <class T>
__global__ __launch_bounds__(256) void wino_filter_kernel(int N, int C, int Npad, int Cpad, const T *__restrict__ w, float *__restrict__ U)
{
    const int idx = blockIdx.x * blockDim.x + threadIdx.x; // c * Npad + n over the padded domain
    if (idx >= Npad * Cpad)
        return;
    const int c = idx / Npad, n = idx - c * Npad;
    float u[16];
#pragma unroll
    for (int e = 0; e < 16; e++)
        u[e] = 0.0f;
    if (n < N && c < C) {
        const T *kp = w + ((size_t)n * C + c) * 9;
        float k[9];
#pragma unroll
        for (int i = 0; i < 9; i++)
            k[i] = to_float(kp[i]);
        float gk[3][4];
#pragma unroll
        for (int j = 0; j < 3; j++) {
            gk[j][0] = k[j];
            gk[j][1] = 0.5f * (k[j] + k[3 + j] + k[6 + j]);
            gk[j][2] = 0.5f * (k[j] - k[3 + j] + k[6 + j]);
            gk[j][3] = k[6 + j];
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            u[4 * i + 0] = gk[0][i];
            u[4 * i + 1] = 0.5f * (gk[0][i] + gk[1][i] + gk[2][i]);
            u[4 * i + 2] = 0.5f * (gk[0][i] - gk[1][i] + gk[2][i]);
            u[4 * i + 3] = gk[2][i];
        }
    }
    // [e][chunk of 8 channels][c & 1][n][(c % 8) / 2]: a lane of the fused kernel reads the four
    // k pairs of a chunk with one 16-byte load
    const size_t estride = (size_t)Cpad * Npad;
    const size_t in_e = ((size_t)((c / 8) * 2 + (c & 1)) * Npad + n) * 4 + (c % 8) / 2;
#pragma unroll
    for (int e = 0; e < 16; e++)
        U[(size_t)e * estride + in_e] = u[e];
}

// keep a selected offset one opaque value, so that the select stays a v_cndmask
__device__ __forceinline__ uint32_t opaque(uint32_t v)
{
    asm("" : "+v"(v));
    return v;
}

// NLOAD == 0: every thread gathers its 4x4 patch straight from global memory (any shape).
// NLOAD > 0 : the input rows that the 32 tiles of the workgroup touch are first copied to LDS
//             with coalesced loads (NLOAD elements per thread and chunk, each input element
//             once) and the patches are gathered from there; used when those rows fit.
// NOB: blocks of 32 output channels per workgroup.  The input transform of a (channel, tile) is the same work whatever the number of
// output channels it is multiplied into, and it shares issue cycles with the matrix pipe: with two blocks every transformed value
// feeds twice the matrix instructions (8 per wavefront and element pair instead of 4), at 128 accumulator registers per lane.
template <class T, bool TAIL, int NLOAD, int NOB = 1>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void wino_fused_kernel(WinoArgs a)
{
    constexpr int NTW = NT * NOB; // output channels per workgroup
    // main loop: V[buffer][e][c in chunk][tile]; epilogue: M[e][n in pass][tile]
    __shared__ float lds[2 * 16 * KC * TT];
    static_assert(2 * 16 * KC * TT == 16 * (NT / 2) * TT, "the epilogue reuses the V buffers");
    constexpr bool STAGED = NLOAD > 0;
    constexpr int RAW = STAGED ? NLOAD * kThreads : 1; // floats of one staging buffer (+ one zero word)
    __shared__ float raw[STAGED ? 2 * (RAW + 4) : 1];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int h = lane >> 5;

    // Workgroup ids are dealt round-robin to the 8 XCDs; renumber so that each XCD walks a
    // contiguous range: the channel blocks of one tile block (same input patches) share an L2.
    int id;
    {
        const int nb = gridDim.x, bid = blockIdx.x;
        const int q = nb >> 3, r = nb & 7;
        const int xcd = bid & 7, slot = bid >> 3;
        id = (xcd < r) ? xcd * (q + 1) + slot : r * (q + 1) + (xcd - r) * q + slot;
    }
    const int n0 = (id % a.nblocks) * NTW;
    const int t0 = (id / a.nblocks) * TT;

    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t ur = __builtin_amdgcn_make_buffer_rsrc((void *)a.U, 0, a.u_bytes, 0x00020000);

    // ---- the (channel, tile) this thread transforms; the same tile is its output column ----
    const int cl = tid >> 5; // channel inside a chunk; a wavefront holds 2 channels x 32 tiles
    const int tl = tid & 31;
    const int t = t0 + tl;
    const bool tile_ok = t < a.T;
    const int b = (int)fast_div((uint32_t)t, a.tpi_magic, a.tpi_shift);
    const int rc = t - b * a.tpi;
    const int ty = (int)fast_div((uint32_t)rc, a.tw_magic, a.tw_shift);
    const int tx = rc - ty * a.tw;
    const int x_last = (a.C - 1) / KC;     // last chunk that exists in x
    const uint32_t chunk_bytes = (uint32_t)(KC * a.H * a.W) * (uint32_t)sizeof(T);
    const int last = a.nchunks - 1;        // last chunk of U (zero padded)

    // Direct variant: voff[k] = byte offset of patch element k in x (or out of range).
    // Staged variant: voff[k] = byte offset of patch element k inside a staging buffer (or of
    // its zero word); goff[i] = byte offset in x of the i-th element this thread copies.
    uint32_t voff[16];
    uint32_t goff[STAGED ? NLOAD : 1];
    int gch[STAGED ? NLOAD : 1]; // channel inside the chunk of that element (tail test)
    if (!STAGED) {
        const int row = 2 * ty - 1, col = 2 * tx - 1;
        const int base = (b * a.C + cl) * a.H * a.W;
#pragma unroll
        for (int dr = 0; dr < 4; dr++)
#pragma unroll
            for (int dc = 0; dc < 4; dc++) {
                const int yy = row + dr, xx = col + dc;
                const bool ok = tile_ok && yy >= 0 && yy < a.H && xx >= 0 && xx < a.W;
                voff[4 * dr + dc] = ok ? (uint32_t)(base + yy * a.W + xx) * (uint32_t)sizeof(T) : kOutOfRange;
            }
    } else {
        // The 32 tiles cover at most four images (checked on the host); per image the rows
        // they touch are one contiguous run of each channel plane.  Runs are laid out back to
        // back in the staging buffer, stage_stride floats per channel.
        const int tlast = min(t0 + TT, a.T) - 1;
        const int b0 = (int)fast_div((uint32_t)t0, a.tpi_magic, a.tpi_shift);
        const int b1 = (int)fast_div((uint32_t)tlast, a.tpi_magic, a.tpi_shift);
        const int ty0 = (int)fast_div((uint32_t)(t0 - b0 * a.tpi), a.tw_magic, a.tw_shift);
        const int ty1 = (int)fast_div((uint32_t)(tlast - b1 * a.tpi), a.tw_magic, a.tw_shift);
        int seg_r0[4], seg_start[4], seg_len[4];
        int total = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int bi = b0 + k;
            const int tya = (k == 0) ? ty0 : 0;
            const int tyb = (bi == b1) ? ty1 : a.th - 1;
            const int r0 = max(2 * tya - 1, 0), r1 = min(2 * tyb + 2, a.H - 1);
            seg_r0[k] = r0;
            seg_start[k] = total;
            seg_len[k] = (bi <= b1) ? (r1 - r0 + 1) * a.W : 0;
            total += seg_len[k];
        }
        // patch element -> staging offset
        {
            const int k = b - b0;
            int r0 = seg_r0[0], st = seg_start[0];
#pragma unroll
            for (int q = 1; q < 4; q++)
                if (k == q) {
                    r0 = seg_r0[q];
                    st = seg_start[q];
                }
            const int row = 2 * ty - 1, col = 2 * tx - 1;
            const int base = cl * a.stage_stride + st;
#pragma unroll
            for (int dr = 0; dr < 4; dr++)
#pragma unroll
                for (int dc = 0; dc < 4; dc++) {
                    const int yy = row + dr, xx = col + dc;
                    const bool ok = tile_ok && yy >= 0 && yy < a.H && xx >= 0 && xx < a.W;
                    voff[4 * dr + dc] = (uint32_t)(ok ? base + (yy - r0) * a.W + xx : RAW) * 4u;
                }
        }
        // copied element -> x offset
#pragma unroll
        for (int i = 0; i < NLOAD; i++) {
            const int f = tid + i * kThreads;
            const int ch = (int)fast_div((uint32_t)f, a.ss_magic, a.ss_shift);
            const int pos = f - ch * a.stage_stride;
            int k = -1;
#pragma unroll
            for (int q = 0; q < 4; q++)
                if (pos >= seg_start[q] && pos < seg_start[q] + seg_len[q])
                    k = q;
            int r0 = 0, st = 0;
#pragma unroll
            for (int q = 0; q < 4; q++)
                if (k == q) {
                    r0 = seg_r0[q];
                    st = seg_start[q];
                }
            const bool ok = k >= 0 && ch < KC;
            goff[i] = ok ? (uint32_t)((((b0 + k) * a.C + ch) * a.H + r0) * a.W + (pos - st)) * (uint32_t)sizeof(T) : kOutOfRange;
            gch[i] = ch;
        }
        if (tid < 8)
            raw[(tid >> 2) * (RAW + 4) + RAW + (tid & 3)] = 0.0f; // the zero words of both buffers
    }

    // ---- direct variant: patches in flight; set k % 2 holds chunk k, loaded two chunks ahead ----
    float P[2][16];
    auto load_patch = [&](auto set, int chunk) {
        constexpr int S = decltype(set)::value;
        const int ch = min(chunk, x_last); // later chunks meet zero filter values or are never multiplied
        const uint32_t soff = (uint32_t)ch * chunk_bytes;
        if (TAIL) {
            // C is not a multiple of the chunk: channels past C read as 0 (one compare + selects
            // per chunk; the select stays one opaque value so that it is not turned into branches)
            const bool c_ok = ch * KC + cl < a.C;
#pragma unroll
            for (int k = 0; k < 16; k++)
                P[S][k] = ld_elem<T>(xr, opaque(c_ok ? voff[k] : kOutOfRange), soff);
        } else {
#pragma unroll
            for (int k = 0; k < 16; k++)
                P[S][k] = ld_elem<T>(xr, voff[k], soff);
        }
    };
    // ---- staged variant: rows of chunk k travel global -> G -> raw[k % 2] -> P[k % 2] ----
    float G[STAGED ? NLOAD : 1];
    auto load_rows_to = [&](float *dst, int chunk) {
        const int ch = min(chunk, x_last);
        const uint32_t soff = (uint32_t)ch * chunk_bytes;
#pragma unroll
        for (int i = 0; i < NLOAD; i++) {
            if (TAIL)
                dst[i] = ld_elem<T>(xr, opaque(ch * KC + gch[i] < a.C ? goff[i] : kOutOfRange), soff);
            else
                dst[i] = ld_elem<T>(xr, goff[i], soff);
        }
    };
    auto store_rows_from = [&](auto buf_c, const float *src) {
        constexpr int BUF = decltype(buf_c)::value;
#pragma unroll
        for (int i = 0; i < NLOAD; i++)
            raw[BUF * (RAW + 4) + tid + i * kThreads] = src[i];
    };
    auto load_rows = [&](int chunk) { load_rows_to(G, chunk); };
    auto store_rows = [&](auto buf_c) { store_rows_from(buf_c, G); };
    auto gather_patch = [&](auto buf_c) {
        constexpr int BUF = decltype(buf_c)::value;
        const char *basep = (const char *)(raw + BUF * (RAW + 4));
#pragma unroll
        for (int k = 0; k < 16; k++)
            P[BUF][k] = *(const float *)(basep + voff[k]);
    };
    // V = B^T d B of the patch in P -> LDS[buf][e][cl][tl], src/kernels/winograd_fwd.cl:35-69
    auto transform_patch = [&](auto buf_c) { // chunk parity == LDS buffer == patch register set
        constexpr int BUF = decltype(buf_c)::value;
        float bt[4][4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            bt[0][j] = P[BUF][0 + j] - P[BUF][8 + j];
            bt[1][j] = P[BUF][4 + j] + P[BUF][8 + j];
            bt[2][j] = P[BUF][8 + j] - P[BUF][4 + j];
            bt[3][j] = P[BUF][4 + j] - P[BUF][12 + j];
        }
        float *dst = lds + BUF * (16 * KC * TT) + cl * TT + tl;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            dst[(4 * i + 0) * (KC * TT)] = bt[i][0] - bt[i][2];
            dst[(4 * i + 1) * (KC * TT)] = bt[i][1] + bt[i][2];
            dst[(4 * i + 2) * (KC * TT)] = bt[i][2] - bt[i][1];
            dst[(4 * i + 3) * (KC * TT)] = bt[i][1] - bt[i][3];
        }
    };

    // ---- A operand: U[e][chunk][k half][n][k pair]: one 16-byte load per lane = the operands
    //      of the four k pairs of a chunk; lane = (k half h, channel l32), e = 4*wave + ei ----
    const uint32_t u_voff = (uint32_t)(h * a.Npad + l32) * 16u;
    f32x4 A[2][4][NOB];
    auto load_u = [&](auto set, int chunk) {
        constexpr int S = decltype(set)::value;
        const int ch = min(chunk, last);
#pragma unroll
        for (int ei = 0; ei < 4; ei++) {
            const uint32_t soff = (uint32_t)((((4 * wave + ei) * a.nchunks + ch) * 2) * a.Npad + n0) * 16u;
#pragma unroll
            for (int ob = 0; ob < NOB; ob++)
                A[S][ei][ob] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(ur, u_voff, soff + (uint32_t)(ob * NT * 16), 0));
        }
    };

    f32x16 acc[4][NOB];
#pragma unroll
    for (int ei = 0; ei < 4; ei++)
#pragma unroll
        for (int ob = 0; ob < NOB; ob++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[ei][ob][r] = 0.0f;

    // bias of the four output channels this thread finishes in the epilogue (fetched now, so
    // that the epilogue does not wait on memory)
    float bias_v[4 * NOB];
#pragma unroll
    for (int i = 0; i < 4 * NOB; i++) {
        const int n = n0 + (i >> 1) * (NT / 2) + (tid >> 5) + 8 * (i & 1);
        bias_v[i] = (a.bias && n < a.N) ? a.bias[n] : 0.0f;
    }

    // One chunk.  Direct: U of chunk+1 -> the other register set; patch of chunk+1 -> LDS[BUF^1],
    // its registers then take the patch of chunk+3; chunk (LDS[BUF], U set BUF) -> matrix cores.
    // Staged: additionally rows of chunk+2 move registers -> raw[BUF] (free since the patches of
    // this chunk were gathered one step ago) and rows of chunk+3 are requested from memory.
    auto k_step = [&](auto buf_c, int chunk) {
        constexpr int BUF = decltype(buf_c)::value;
        using Next = std::integral_constant<int, BUF ^ 1>;
        load_u(Next{}, chunk + 1);
        if (STAGED) {
            store_rows(buf_c);
            load_rows(chunk + 3);
            gather_patch(Next{});
        }
        float Bv[4][KC / 2];
        const float *src = lds + BUF * (16 * KC * TT) + lane;
#pragma unroll
        for (int ei = 0; ei < 4; ei++)
#pragma unroll
            for (int j = 0; j < KC / 2; j++)
                Bv[ei][j] = src[((4 * wave + ei) * KC + 2 * j) * TT];
        transform_patch(Next{});
        if (!STAGED)
            load_patch(Next{}, chunk + 3);
#pragma unroll
        for (int j = 0; j < KC / 2; j++)
#pragma unroll
            for (int ei = 0; ei < 4; ei++)
#pragma unroll
                for (int ob = 0; ob < NOB; ob++)
                    acc[ei][ob] = __builtin_amdgcn_mfma_f32_32x32x2f32(A[BUF][ei][ob][j], Bv[ei][j], acc[ei][ob], 0, 0, 0);
        __syncthreads();
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    if (STAGED) {
        float G1[STAGED ? NLOAD : 1]; // second set, prologue only: chunks 0 and 1 are requested together
        load_rows(0);
        load_rows_to(G1, 1);
        load_u(I0{}, 0);
        store_rows(I0{});
        load_rows(2);
        store_rows_from(I1{}, G1);
        __syncthreads();
        gather_patch(I0{});
        transform_patch(I0{});
    } else {
        load_patch(I0{}, 0);
        load_patch(I1{}, 1);
        load_u(I0{}, 0);
        transform_patch(I0{});
        load_patch(I0{}, 2);
    }
    __syncthreads();
    // the chunk count is even (U is zero padded to it): no remainder step, so the accumulators
    // keep one register home through the loop
    for (int chunk = 0; chunk < a.nchunks; chunk += 2) {
        k_step(I0{}, chunk);
        k_step(I1{}, chunk + 1);
    }

    // ---- epilogue: y tile = A^T m A, bias, activation, factor (winograd_fwd.cl:138-158,406-436) ----
    // accumulator register r of a 32x32 block holds row (channel) 8*(r/4) + 4*h + r%4, column (tile) l32
    T *const ybase = (T *)a.y;
#pragma unroll
    for (int pass = 0; pass < 2 * NOB; pass++) { // 16 output channels per pass
#pragma unroll
        for (int ei = 0; ei < 4; ei++)
#pragma unroll
            for (int r8 = 0; r8 < 8; r8++) {
                const int nl = 8 * (r8 >> 2) + 4 * h + (r8 & 3); // channel inside the pass, 0..15
                lds[((4 * wave + ei) * (NT / 2) + nl) * TT + l32] = acc[ei][pass >> 1][8 * (pass & 1) + r8];
            }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < 2; q++) {
            const int nl = (tid >> 5) + 8 * q;
            const int n = n0 + pass * (NT / 2) + nl;
            float m[16];
#pragma unroll
            for (int e = 0; e < 16; e++)
                m[e] = lds[(e * (NT / 2) + nl) * TT + tl];
            if (n < a.N && tile_ok) {
                float at[2][4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    at[0][j] = m[j] + m[4 + j] + m[8 + j];
                    at[1][j] = m[4 + j] - m[8 + j] - m[12 + j];
                }
                float o[4];
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    o[2 * i + 0] = at[i][0] + at[i][1] + at[i][2];
                    o[2 * i + 1] = at[i][1] - at[i][2] - at[i][3];
                }
                const float bv = bias_v[2 * pass + q];
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; i++)
                    v[i] = o[i] + bv;
                const int row = 2 * ty, col = 2 * tx;
                T *yp = ybase + (((size_t)b * a.N + n) * a.H + row) * a.W + col;
                const bool r1 = row + 1 < a.H, c1 = col + 1 < a.W; // odd H / W: the last tile is cut
                const bool pre = a.pre != 0 && a.factor != 0.0f;
                if (pre) {
                    v[0] = fmaf(to_float(yp[0]), a.factor, v[0]);
                    if (c1)
                        v[1] = fmaf(to_float(yp[1]), a.factor, v[1]);
                    if (r1) {
                        v[2] = fmaf(to_float(yp[a.W]), a.factor, v[2]);
                        if (c1)
                            v[3] = fmaf(to_float(yp[a.W + 1]), a.factor, v[3]);
                    }
                }
                if (a.act != DLP_ACT_IDENTITY) { // one uniform branch for the four values
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        v[i] = apply_act(v[i], a.act);
                }
                if (a.factor != 0.0f && !pre) {
                    store_out(yp, v[0], a.factor);
                    if (c1)
                        store_out(yp + 1, v[1], a.factor);
                    if (r1) {
                        store_out(yp + a.W, v[2], a.factor);
                        if (c1)
                            store_out(yp + a.W + 1, v[3], a.factor);
                    }
                } else {
                    store_plain(yp, v[0]);
                    if (c1)
                        store_plain(yp + 1, v[1]);
                    if (r1) {
                        store_plain(yp + a.W, v[2]);
                        if (c1)
                            store_plain(yp + a.W + 1, v[3]);
                    }
                }
            }
        }
        if (pass + 1 < 2 * NOB)
            __syncthreads();
    }
}

template <class T>
int launch_typed(const ConvGeom &g, const WinoPlan &plan, const void *x, const void *w, void *y, void *ws, const Epilogue &ep,
                 hipStream_t stream, int mode)
{
    float *U = (float *)ws;
    if (mode != WINO_RUN_ONLY) {
        TimingScope ts("winograd_filter", stream);
        const int total = plan.Npad * plan.Cpad;
        hipLaunchKernelGGL(wino_filter_kernel<T>, dim3((total + 255) / 256), dim3(256), 0, stream, g.Cout, g.Cin, plan.Npad, plan.Cpad,
                           (const T *)w, U);
    }
    if (mode == WINO_FILTER_ONLY) {
        DLP_HIP_TRY(hipGetLastError());
        return DLP_OK;
    }
    WinoArgs a;
    a.U = U;
    a.bias = ep.bias;
    a.C = g.Cin;
    a.N = g.Cout;
    a.H = g.H;
    a.W = g.W;
    a.tw = (g.W + 1) / 2;
    a.tpi = ((g.H + 1) / 2) * a.tw;
    a.Cpad = plan.Cpad;
    a.Npad = plan.Npad;
    a.nchunks = plan.Cpad / KC;
    const int nob = winograd_blocks_per_workgroup(g, plan);
    a.nblocks = plan.Npad / (NT * nob);
    make_magic((uint32_t)a.tpi, a.tpi_magic, a.tpi_shift);
    make_magic((uint32_t)a.tw, a.tw_magic, a.tw_shift);
    a.u_bytes = (uint32_t)(16u * (size_t)plan.Cpad * plan.Npad * sizeof(float));
    a.th = (g.H + 1) / 2;
    a.stage_stride = plan.stage_stride;
    a.ss_magic = a.ss_shift = 0;
    if (plan.stage_stride > 0)
        make_magic((uint32_t)plan.stage_stride, a.ss_magic, a.ss_shift);
    a.factor = ep.factor;
    a.pre = ep.accumulate_first;
    a.act = ep.activation;
    const size_t x_img = (size_t)g.Cin * g.H * g.W, y_img = (size_t)g.Cout * g.H * g.W;
    for (int b0 = 0; b0 < g.B; b0 += plan.chunk_imgs) {
        const int nb = (g.B - b0 < plan.chunk_imgs) ? g.B - b0 : plan.chunk_imgs;
        a.x = (const T *)x + (size_t)b0 * x_img;
        a.y = (T *)y + (size_t)b0 * y_img;
        a.T = nb * a.tpi;
        a.x_bytes = (uint32_t)((size_t)nb * x_img * sizeof(T));
        const unsigned grid = (unsigned)(((a.T + TT - 1) / TT) * a.nblocks);
        TimingScope ts("winograd_fused", stream);
        const bool tail = (g.Cin % KC) != 0;
#define DLP_WINO_LAUNCH(NL)                                                                                          \
    do {                                                                                                             \
        if (tail && nob == 2)                                                                                        \
            DLP_LAUNCH_TIMED(ts, (wino_fused_kernel<T, true, NL, 2>), dim3(grid), dim3(kThreads), 0, stream, a);     \
        else if (tail)                                                                                               \
            DLP_LAUNCH_TIMED(ts, (wino_fused_kernel<T, true, NL, 1>), dim3(grid), dim3(kThreads), 0, stream, a);     \
        else if (nob == 2)                                                                                           \
            DLP_LAUNCH_TIMED(ts, (wino_fused_kernel<T, false, NL, 2>), dim3(grid), dim3(kThreads), 0, stream, a);    \
        else                                                                                                         \
            DLP_LAUNCH_TIMED(ts, (wino_fused_kernel<T, false, NL, 1>), dim3(grid), dim3(kThreads), 0, stream, a);    \
    } while (0)
        if (plan.stage_loads == 8)
            DLP_WINO_LAUNCH(8);
        else if (plan.stage_loads == 16)
            DLP_WINO_LAUNCH(16);
        else
            DLP_WINO_LAUNCH(0);
#undef DLP_WINO_LAUNCH
    }
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

} // namespace

// Blocks of 32 output channels per workgroup: two halve the input transforms per flop but also the number of workgroups, so
// only where that still leaves one and a half workgroups per compute unit (measured on the ResNet-18 shapes at batch 16 / 32 / 64:
// 392 workgroups of two blocks beat 784 of one by 11-13 %, 196-256 of two lose 6-40 % to twice as many of one).
// DLP_WINO_NOB=1 / 2 in the environment pins the choice, for measurements.
int winograd_blocks_per_workgroup(const ConvGeom &g, const WinoPlan &plan)
{
    if (plan.Npad % (2 * NT) != 0)
        return 1;
    static const int pin = getenv("DLP_WINO_NOB") != nullptr ? atoi(getenv("DLP_WINO_NOB")) : 0;
    if (pin == 1 || pin == 2)
        return pin;
    return winograd_workgroups(g, plan, 2) * 2 >= 3ll * dlp_cu_count() ? 2 : 1;
}

// Workgroups of the fused kernel for a batch that fits one launch, with nob blocks of 32 output channels each
long long winograd_workgroups(const ConvGeom &g, const WinoPlan &plan, int nob)
{
    const long long tiles = (long long)g.B * ((g.H + 1) / 2) * ((g.W + 1) / 2);
    return (tiles + TT - 1) / TT * (plan.Npad / (NT * nob));
}

bool winograd_supported(const ConvGeom &g)
{
    // one image (input and output) must stay below 2^30 bytes: byte offsets are 32-bit
    const size_t img = (size_t)(g.Cin > g.Cout ? g.Cin : g.Cout) * g.H * g.W * sizeof(float);
    return (g.dtype == DLP_FLOAT || g.dtype == DLP_BFLOAT16) && g.KH == 3 && g.KW == 3 && g.ph == 1 && g.pw == 1 && g.dh == 1 &&
           g.dw == 1 && g.sh == 1 && g.sw == 1 && g.groups == 1 && img < ((size_t)1 << 30) &&
           (size_t)g.Cin * g.Cout <= ((size_t)1 << 24); // the transformed filter stays below 2^31 bytes
}

WinoPlan winograd_plan(const ConvGeom &g)
{
    WinoPlan p;
    p.Cpad = (g.Cin + 2 * KC - 1) / (2 * KC) * (2 * KC); // an even number of K chunks
    p.Npad = (g.Cout + NT - 1) / NT * NT;
    // images per launch: input bytes, and tile count, of a launch stay below 2^30
    const size_t img = (size_t)(g.Cin > g.Cout ? g.Cin : g.Cout) * g.H * g.W * sizeof(float);
    size_t imgs = ((size_t)1 << 30) / (img ? img : 1);
    if (imgs < 1)
        imgs = 1;
    if (imgs > 65536)
        imgs = 65536;
    p.chunk_imgs = (int)imgs;
    p.ws_bytes = sizeof(float) * 16 * (size_t)p.Cpad * p.Npad;

    // Staging: over all alignments of a block of TT consecutive tiles, the input rows touched
    // per channel (one contiguous run per image) and the number of images.
    const int tw = (g.W + 1) / 2, th = (g.H + 1) / 2, tpi = tw * th;
    int max_rows = 0, max_segs = 0;
    for (int k = 0; k < tpi; k++) {
        int pos = (int)(((long long)k * TT) % tpi), rem = TT, rows = 0, segs = 0;
        while (rem > 0) {
            const int n = rem < tpi - pos ? rem : tpi - pos;
            const int tya = pos / tw, tyb = (pos + n - 1) / tw;
            const int r0 = 2 * tya - 1 > 0 ? 2 * tya - 1 : 0, r1 = 2 * tyb + 2 < g.H - 1 ? 2 * tyb + 2 : g.H - 1;
            rows += r1 - r0 + 1;
            segs++;
            rem -= n;
            pos = 0;
        }
        max_rows = rows > max_rows ? rows : max_rows;
        max_segs = segs > max_segs ? segs : max_segs;
    }
    p.stage_stride = 0;
    p.stage_loads = 0;
    const int stride = (max_rows * g.W + 3) / 4 * 4;
    if (max_segs <= 4 && KC * stride <= 16 * kThreads) {
        p.stage_stride = stride;
        p.stage_loads = KC * stride <= 8 * kThreads ? 8 : 16;
    }
    return p;
}

int winograd_launch(const ConvGeom &g, const WinoPlan &plan, const void *x, const void *w, void *y, void *ws, size_t ws_bytes,
                    const Epilogue &ep, hipStream_t stream, int mode)
{
    DLP_REQUIRE(winograd_supported(g), "geometry is not Winograd compatible");
    DLP_REQUIRE(ws != nullptr && ws_bytes >= plan.ws_bytes, "workspace smaller than workspace()");
    if (g.B == 0 && mode != WINO_FILTER_ONLY)
        return DLP_OK;
    if (g.dtype == DLP_BFLOAT16)
        return launch_typed<bf16_t>(g, plan, x, w, y, ws, ep, stream, mode);
    return launch_typed<float>(g, plan, x, w, y, ws, ep, stream, mode);
}

} // namespace dlp
