// InnerProduct forward on the matrix cores.
//
// Replaces the reference's IPForwardImpl / StandardSGEMM path
// (src/core/ip.cpp:15-50, src/gemm.cpp:240-345):
//   y[B x Out] = act(x[B x In] * w[Out x In]^T + bias[Out])
//
// Two kernels: ip_stream_kernel (further down; rows on 16-byte boundaries: the weights go through LDS in runs of 1 KB per row)
// and ip_direct_kernel (every other alignment), which share the operand layout and the way K slices are reduced.
//
// Both operands are stored with the reduction index innermost, which is exactly what a matrix
// instruction wants in a lane: ip_direct_kernel loads them straight from memory into operand
// registers -- no LDS, no repacking of the weights, no barriers.
//  * A wavefront owns 32 outputs x up to 128 batch rows (NB blocks of 32) over one slice of K.
//    A lane (row = lane % 32, half = lane / 32) loads 16 bytes of its weight row and of its NB
//    batch rows per step: 4 consecutive k in fp32 (half h takes k = 8t + 4h .. +3; the four
//    v_mfma_f32_32x32x2_f32 of the step pair element e of half 0 with element e of half 1 --
//    the sum over k is order free as long as both operands use the same pairing), or the 8
//    consecutive k of one v_mfma_f32_32x32x16_bf16 operand for bf16 tensors.
//  * The layer is bound by reading w once from HBM, so K is split over enough wavefronts to have
//    the whole chip loading; the slices of a tile leave their partial sums in an op-owned buffer
//    (write-through) and the wavefront that arrives last at the tile's counter adds them up in
//    slice order (deterministic), applies bias and activation, writes y and resets the counter.
//    Nobody waits for anybody.
// The reduction over k is accumulated in fp32 in a different order than the reference's sgemm.
//
// Shapes the direct kernel does not take (bf16 rows that are not dword aligned) run as a 1x1
// convolution over 1x1 images through the implicit-GEMM kernel:
//   x[b][c] sits at element b*In + c = NCHW [B, In, 1, 1],  y[b][o] at b*Out + o = NCHW [B, Out, 1, 1].
#include "dlp_internal.hpp"

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <type_traits>

namespace dlp {

typedef float ip_f32x16 __attribute__((ext_vector_type(16)));
typedef float ip_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t ip_u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 ip_bf16x8 __attribute__((ext_vector_type(8)));

namespace {

constexpr uint32_t kIpOutOfRange = 0x80000000u;

struct IpArgs {
    const void *x, *w;
    const float *bias;
    void *y;
    float *part; // [tile][slice][NB*16][64] partial sums (register images)
    int *cnt;    // slices arrived, per tile; zero between launches
    int B, In, Out;
    int S;                // K slices
    int ngroups, gps;     // groups of KG k in all, per slice
    int mblocks, nchunks; // tiles = mblocks * nchunks; a chunk = NB * 32 batch rows
    int act;
    uint32_t x_bytes, w_bytes, part_bytes;
};

// 16 bytes of a row: elements [k0, k0 + 16 / sizeof(T)), k0 = group offset (scalar, through soff) + the
// lane's half (in row_off).  With `tail` set (In is not a multiple of the group), a piece that reaches
// past the end of the row is read dword by dword and only up to the row's end: what follows belongs to
// the next row, or lies outside the tensor.  (bf16 rows have an even length: a dword is all in or all out.)
// WIDE: rows start on 16-byte boundaries, a whole piece is one 16-byte load (which wants that alignment).
template <class T, bool WIDE>
__device__ __forceinline__ ip_u32x4 load_piece(__amdgpu_buffer_rsrc_t r, uint32_t row_off, uint32_t soff, int k0, int In, bool tail)
{
    constexpr int E = 16 / (int)sizeof(T);
    constexpr int EPD = 4 / (int)sizeof(T); // elements per dword
    if (!WIDE || (tail && k0 + E > In)) {
        ip_u32x4 v;
#pragma unroll
        for (int d = 0; d < 4; d++)
            v[d] = (k0 + d * EPD < In) ? (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(r, row_off + 4u * (uint32_t)d, soff, 0) : 0u;
        return v;
    }
    return __builtin_bit_cast(ip_u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, row_off, soff, 0));
}

// What the wavefront that owns a tile's K slice does with its accumulators: with several slices, the partial sums go to the
// scratch buffer (write-through) and the wavefront that arrives last at the tile's counter adds all slices in slice order; then
// bias, activation and the store of y.
template <class T, int NB>
__device__ __forceinline__ void ip_finish(const IpArgs &a, ip_f32x16 (&acc)[NB], int tile, int slice, int m0, int n0, int lane, int l32, int h)
{
    if (a.S > 1) {
        constexpr int kThrough = 17; // sc0 | sc1: past the caches in both directions
        constexpr uint32_t image_bytes = NB * 16 * 64 * 4;
        const __amdgpu_buffer_rsrc_t pr = __builtin_amdgcn_make_buffer_rsrc(a.part, 0, a.part_bytes, 0x00020000);
        const uint32_t base = (uint32_t)(tile * a.S) * image_bytes;
#pragma unroll
        for (int j = 0; j < NB; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float v = acc[j][r];
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), pr, (uint32_t)lane * 4u,
                                                      base + (uint32_t)slice * image_bytes + (uint32_t)((j * 16 + r) * 256), kThrough);
            }
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): the partial sums have been written through
        int arrived = 0;
        if (lane == 0)
            arrived = atomicAdd(a.cnt + tile, 1);
        arrived = __builtin_amdgcn_readfirstlane(arrived);
        if (arrived != a.S - 1)
            return;
        if (lane == 0)
            atomicExch(a.cnt + tile, 0); // ready for the next launch on the stream
#pragma unroll
        for (int j = 0; j < NB; j++) {
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[j][r] = 0.0f;
            // four slices (64 loads) in flight at a time: these loads come from memory, not from a cache
            for (int s0 = 0; s0 < a.S; s0 += 4) {
                float p[4][16];
#pragma unroll
                for (int ds = 0; ds < 4; ds++)
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        p[ds][r] = (s0 + ds < a.S) ? __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                         pr, (uint32_t)lane * 4u,
                                                         base + (uint32_t)(s0 + ds) * image_bytes + (uint32_t)((j * 16 + r) * 256), kThrough))
                                                   : 0.0f;
#pragma unroll
                for (int ds = 0; ds < 4; ds++) // slice order
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        acc[j][r] += p[ds][r];
            }
        }
    }

    // epilogue: accumulator register r of a block holds output m0 + 8*(r/4) + 4*h + r%4 of batch row n0 + 32*j + l32
#pragma unroll
    for (int j = 0; j < NB; j++) {
        const int n = n0 + j * 32 + l32;
        if (n >= a.B)
            continue;
        T *yrow = (T *)a.y + (size_t)n * a.Out;
#pragma unroll
        for (int rq = 0; rq < 4; rq++) {
            const int mq = m0 + 8 * rq + 4 * h; // four consecutive outputs
            float v[4];
#pragma unroll
            for (int rr = 0; rr < 4; rr++) {
                v[rr] = acc[j][4 * rq + rr];
                if (a.bias && mq + rr < a.Out)
                    v[rr] += a.bias[mq + rr];
                v[rr] = apply_act(v[rr], a.act);
            }
            if (sizeof(T) == 4 && (a.Out & 3) == 0 && ((uintptr_t)a.y & 15) == 0) {
                if (mq < a.Out)
                    *(ip_f32x4 *)((float *)yrow + mq) = ip_f32x4{v[0], v[1], v[2], v[3]};
            } else {
#pragma unroll
                for (int rr = 0; rr < 4; rr++)
                    if (mq + rr < a.Out)
                        store_plain(yrow + mq + rr, v[rr]);
            }
        }
    }
}

template <class T, int NB, bool WIDE>
__global__ __launch_bounds__(256) void ip_direct_kernel(IpArgs a)
{
    constexpr int KG = 32 / (int)sizeof(T); // k per step: 8 (fp32: four MFMAs) or 16 (bf16: one)
    constexpr int KH = KG / 2;              // k per lane and step
    const int lane = threadIdx.x & 63;
    const int l32 = lane & 31, h = lane >> 5;
    const int gw = (int)blockIdx.x * 4 + (int)(threadIdx.x >> 6); // wavefront = work item; no LDS, no barriers
    const int items = a.mblocks * a.nchunks * a.S;
    if (gw >= items)
        return;
    const int nc = gw % a.nchunks;
    const int slice = (gw / a.nchunks) % a.S;
    const int mb = gw / (a.nchunks * a.S);
    const int tile = mb * a.nchunks + nc;
    const int m0 = mb * 32, n0 = nc * (NB * 32);

    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, a.w_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
    // rows past the end are clamped to the last one (valid memory); their results are never stored
    // (byte offsets of the lane's row + its half of a group; the group goes through the scalar offset)
    const uint32_t half_off = (uint32_t)(h * KH * (int)sizeof(T));
    const uint32_t a_off = (uint32_t)min(m0 + l32, a.Out - 1) * (uint32_t)a.In * (uint32_t)sizeof(T) + half_off;
    uint32_t b_off[NB];
#pragma unroll
    for (int j = 0; j < NB; j++)
        b_off[j] = (uint32_t)min(n0 + j * 32 + l32, a.B - 1) * (uint32_t)a.In * (uint32_t)sizeof(T) + half_off;
    const bool tail = a.In % KG != 0;

    ip_f32x16 acc[NB];
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
        for (int r = 0; r < 16; r++)
            acc[j][r] = 0.0f;

    const int g_begin = slice * a.gps, g_end = min(g_begin + a.gps, a.ngroups);
    auto load_group = [&](int g, ip_u32x4 &fa, ip_u32x4 (&fb)[NB]) {
        const int k0 = g * KG + h * KH;
        const uint32_t soff = (uint32_t)(g * KG * (int)sizeof(T));
        fa = load_piece<T, WIDE>(wr, a_off, soff, k0, a.In, tail);
#pragma unroll
        for (int j = 0; j < NB; j++)
            fb[j] = load_piece<T, WIDE>(xr, b_off[j], soff, k0, a.In, tail);
    };
    auto multiply = [&](const ip_u32x4 &fa, const ip_u32x4 (&fb)[NB]) {
        if constexpr (sizeof(T) == 4) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const uint32_t ae = fa[e]; // copies: bit_cast applied to a vector element reads element 0
#pragma unroll
                for (int j = 0; j < NB; j++) {
                    const uint32_t be = fb[j][e];
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, ae), __builtin_bit_cast(float, be), acc[j], 0, 0, 0);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < NB; j++)
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(ip_bf16x8, fa), __builtin_bit_cast(ip_bf16x8, fb[j]), acc[j], 0, 0, 0);
        }
    };
    // four groups (a 128-byte line of every row) in flight per wavefront
    constexpr int DEPTH = 4;
    ip_u32x4 fa[DEPTH], fb[DEPTH][NB];
#pragma unroll
    for (int d = 0; d < DEPTH; d++)
        if (g_begin + d < g_end)
            load_group(g_begin + d, fa[d], fb[d]);
    for (int g = g_begin; g < g_end; g += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            if (g + d < g_end) {
                multiply(fa[d], fb[d]);
                if (g + d + DEPTH < g_end)
                    load_group(g + d + DEPTH, fa[d], fb[d]);
            }
        }
    }

    ip_finish<T, NB>(a, acc, tile, slice, m0, n0, lane, l32, h);
}

// ---- large weight matrices at small batch: w streamed through LDS in runs of 1 KB per row ----
// The direct kernel above reads 32 bytes of each of 32 rows per load instruction: with rows tens of kilobytes apart that is
// 32768 concurrent streams of 128 bytes for the memory system, and a 411 MB matrix arrives at 2.7 TB/s.  Here a workgroup owns
// 32 outputs x 32 batch rows over one K slice and walks it in chunks of 1 KB per row: every wavefront load is 1 KB of ONE row
// (what a copy kernel issues), the chunk of the next step travels into registers while this one is multiplied, the tiles go
// to LDS as they lie in memory ([row][1 KB + 16]: the 16-byte operand reads of 16 lanes cover 256 consecutive bytes, no bank
// conflicts), and the four wavefronts each take a quarter of the chunk's k with the same operand layout as the direct kernel
// (a lane's 16 bytes: four k of four fp32 matrix instructions, or the eight k of one bf16 instruction).  The wavefronts'
// accumulators are added in wavefront order through LDS; wavefront 0 then finishes the slice like the direct kernel does.
constexpr int kIpRowBytes = 1024;            // bytes of a row per chunk
constexpr int kIpLdsRow = kIpRowBytes + 16;  // LDS bytes per row
// LDS of an instance: the tile of w and XR (+ 1 row of zeros when XR < 32) rows of x.  32 rows of x: 65 KB, two workgroups per
// compute unit; 16 rows (batches of at most 16): 50 KB, three.
constexpr int ip_stream_lds_bytes(int xr) { return (32 + xr + (xr < 32 ? 1 : 0)) * kIpLdsRow; }

template <class T, int XR>
__global__ __launch_bounds__(256) void ip_stream_kernel(IpArgs a)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char ip_lds[]; // ip_stream_lds_bytes(XR), asked for at launch
    unsigned char *Ws = ip_lds, *Xs = ip_lds + 32 * kIpLdsRow;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, h = lane >> 5;
    const int wg = (int)blockIdx.x;
    const int nc = wg % a.nchunks;
    const int slice = (wg / a.nchunks) % a.S;
    const int mb = wg / (a.nchunks * a.S);
    const int tile = mb * a.nchunks + nc;
    const int m0 = mb * 32, n0 = nc * 32;

    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, a.w_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
    const uint32_t row_bytes = (uint32_t)a.In * (uint32_t)sizeof(T); // a multiple of 16
    // piece i of this thread: row wave + 4 i of the tile, bytes [16 lane, 16 lane + 16) of the chunk.  Rows of w past the end are
    // clamped to the last one (valid memory; their results are never stored), batch rows past the end read as zeros.
    uint32_t w_off[8], x_off[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int r = wave + 4 * i;
        w_off[i] = (uint32_t)min(m0 + r, a.Out - 1) * row_bytes + (uint32_t)lane * 16u;
        x_off[i] = n0 + r < a.B ? (uint32_t)(n0 + r) * row_bytes + (uint32_t)lane * 16u : kIpOutOfRange;
    }
    constexpr int XP = XR / 4; // pieces of x per thread
    ip_u32x4 rw[8], rx[XP];
    auto load_chunk = [&](int c) {
        const uint32_t soff = (uint32_t)c * (uint32_t)kIpRowBytes;
        const bool inside = soff + (uint32_t)lane * 16u < row_bytes; // the last chunk of a row may be short: what follows is the next row
#pragma unroll
        for (int i = 0; i < 8; i++) {
            rw[i] = __builtin_bit_cast(ip_u32x4, __builtin_amdgcn_raw_buffer_load_b128(wr, inside ? w_off[i] : kIpOutOfRange, soff, 0));
            if (i < XP)
                rx[i] = __builtin_bit_cast(ip_u32x4, __builtin_amdgcn_raw_buffer_load_b128(xr, inside ? x_off[i] : kIpOutOfRange, soff, 0));
        }
    };
    // batch rows past XR do not exist: their lanes read a row of zeros
    const int x_row = l32 < XR ? l32 : XR;
    if (XR < 32) {
        for (int i = tid; i < kIpLdsRow / 16; i += 256)
            *(ip_u32x4 *)(Xs + XR * kIpLdsRow + i * 16) = ip_u32x4{0u, 0u, 0u, 0u};
    }

    ip_f32x16 acc[1];
#pragma unroll
    for (int r = 0; r < 16; r++)
        acc[0][r] = 0.0f;

    const int c_begin = slice * a.gps, c_end = min(c_begin + a.gps, a.ngroups); // chunks of this slice
    if (c_begin < c_end)
        load_chunk(c_begin);
    for (int c = c_begin; c < c_end; c++) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            *(ip_u32x4 *)(Ws + (wave + 4 * i) * kIpLdsRow + lane * 16) = rw[i];
            if (i < XP)
                *(ip_u32x4 *)(Xs + (wave + 4 * i) * kIpLdsRow + lane * 16) = rx[i];
        }
        __syncthreads();
        if (c + 1 < c_end)
            load_chunk(c + 1);
        // this wavefront's quarter of the chunk: eight steps of 32 bytes per row
#pragma unroll
        for (int g = 0; g < 8; g++) {
            const int koff = wave * 256 + g * 32 + h * 16;
            const ip_u32x4 fa = *(const ip_u32x4 *)(Ws + l32 * kIpLdsRow + koff);
            const ip_u32x4 fb = *(const ip_u32x4 *)(Xs + x_row * kIpLdsRow + koff);
            if constexpr (sizeof(T) == 4) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const uint32_t ae = fa[e], be = fb[e]; // copies: bit_cast applied to a vector element reads element 0
                    acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, ae), __builtin_bit_cast(float, be), acc[0], 0, 0, 0);
                }
            } else {
                acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(ip_bf16x8, fa), __builtin_bit_cast(ip_bf16x8, fb), acc[0], 0, 0, 0);
            }
        }
        __syncthreads(); // the tiles are overwritten by the next chunk
    }

    // the four quarters, added in wavefront order by wavefront 0 (register images [wavefront][r][lane] in LDS)
    float *red = reinterpret_cast<float *>(Ws);
    if (wave != 0) {
#pragma unroll
        for (int r = 0; r < 16; r++)
            red[((wave - 1) * 16 + r) * 64 + lane] = acc[0][r];
    }
    __syncthreads();
    if (wave != 0)
        return;
#pragma unroll
    for (int q = 0; q < 3; q++)
#pragma unroll
        for (int r = 0; r < 16; r++)
            acc[0][r] += red[(q * 16 + r) * 64 + lane];
    ip_finish<T, 1>(a, acc, tile, slice, m0, n0, lane, l32, h);
}

} // namespace

size_t ip_direct_scratch_bytes(int batch, int inputs, int outputs, int dtype, IpPlan *plan)
{
    IpPlan p;
    const int kg = dtype == DLP_FLOAT ? 8 : 16;
    // One block of 32 batch rows per wavefront: the wavefronts of a workgroup are the batch chunks of one
    // (output block, K slice), so they share its weights through the L1 and the work spreads over 4x the
    // SIMDs (the fp32 matrix instruction is slow: 64 clocks per 32x32x2 block).
    p.nb = 1;
    p.mblocks = (outputs + 31) / 32;
    p.nchunks = (batch + p.nb * 32 - 1) / (p.nb * 32);
    p.ngroups = (inputs + kg - 1) / kg;
    // K slices: about one wavefront per SIMD (1024), slices of at least 8 steps, at most 16 slices, and
    // partial sums (4 KB per tile and slice, written and read once) that stay below half the bytes of w.
    // Measured on 25088 -> 4096 at batch 16 (411 MB of weights): 155 us = 2.7 TB/s this way; 4096
    // wavefronts with eight groups in flight each: 195 us.
    const long long tiles = (long long)p.mblocks * p.nchunks;
    const long long w_bytes = (long long)outputs * inputs * (dtype == DLP_FLOAT ? 4 : 2);
    long long s = (1024 + tiles - 1) / tiles;
    s = std::min<long long>(s, p.ngroups / 8);
    s = std::min<long long>(s, w_bytes / (8192 * tiles));
    s = std::max<long long>(1, std::min<long long>(s, 16));
    p.gps = (int)((p.ngroups + s - 1) / s);
    p.S = (p.ngroups + p.gps - 1) / p.gps;
    p.cnt_bytes = (size_t)((tiles * sizeof(int) + 255) / 256 * 256);
    p.part_bytes = p.S > 1 ? (size_t)tiles * p.S * p.nb * 16 * 64 * sizeof(float) : 0;
    if (plan)
        *plan = p;
    return p.cnt_bytes + p.part_bytes;
}

bool ip_direct_supported(int inputs, int dtype, const void *x, const void *w)
{
    if (dtype == DLP_FLOAT)
        return true; // rows are dword aligned
    return dtype == DLP_BFLOAT16 && inputs % 2 == 0 && (((uintptr_t)x | (uintptr_t)w) & 3) == 0;
}

int ip_direct_launch(int batch, int inputs, int outputs, int dtype, const void *x, const void *w, void *y, const Epilogue &ep, int *counters,
                     float *partials, hipStream_t stream)
{
    IpPlan p;
    ip_direct_scratch_bytes(batch, inputs, outputs, dtype, &p);
    const size_t esize = dtype_size(dtype);
    const size_t x_bytes = (size_t)batch * inputs * esize, w_bytes = (size_t)outputs * inputs * esize;
    if (x_bytes >= kIpOutOfRange || w_bytes >= kIpOutOfRange || p.part_bytes >= kIpOutOfRange)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "tensors of 2 GiB or more are not supported by the 32-bit buffer addressing");
    IpArgs a;
    a.x = x;
    a.w = w;
    a.bias = ep.bias;
    a.y = y;
    a.cnt = counters;
    a.part = partials;
    a.B = batch;
    a.In = inputs;
    a.Out = outputs;
    a.S = p.S;
    a.ngroups = p.ngroups;
    a.gps = p.gps;
    a.mblocks = p.mblocks;
    a.nchunks = p.nchunks;
    a.act = ep.activation;
    a.x_bytes = (uint32_t)x_bytes;
    a.w_bytes = (uint32_t)w_bytes;
    a.part_bytes = (uint32_t)p.part_bytes;
    const long long items = (long long)p.mblocks * p.nchunks * p.S;
    if (items > 0x7fffffffLL)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "inner product too large for a single launch");
    const dim3 grid((unsigned)((items + 3) / 4)), block(256);
    TimingScope ts("ip_direct", stream);
    // 16-byte loads when every row of x and w starts on a 16-byte boundary, dword loads otherwise
    const bool wide = (inputs * esize) % 16 == 0 && (((uintptr_t)x | (uintptr_t)w) & 15) == 0;
    auto launch = [&](auto kernel) { DLP_LAUNCH_TIMED(ts, kernel, grid, block, 0, stream, a); };
    auto pick = [&](auto type_tag, auto nb_c) {
        using T = decltype(type_tag);
        constexpr int NBV = decltype(nb_c)::value;
        if (wide)
            launch(ip_direct_kernel<T, NBV, true>);
        else
            launch(ip_direct_kernel<T, NBV, false>);
    };
    auto pick_nb = [&](auto type_tag) {
        if (p.nb == 1)
            pick(type_tag, std::integral_constant<int, 1>{});
        else if (p.nb == 2)
            pick(type_tag, std::integral_constant<int, 2>{});
        else
            pick(type_tag, std::integral_constant<int, 4>{});
    };
    if (dtype == DLP_BFLOAT16)
        pick_nb(bf16_t{});
    else
        pick_nb(float{});
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

// The streaming kernel: wherever the rows of w and of x start on 16-byte boundaries.  Measured against the direct kernel on cold
// weights, fp32 (bf16): 25088 -> 4096 at batch 16 162 -> 93 us = 4.4 TB/s (83 -> 49), 9216 -> 4096 68 -> 43 (39 -> 23),
// 4096 -> 1000 32 -> 15 (27 -> 11), 2048 -> 1000 at batch 128 26 -> 16 (22 -> 11), 1280 -> 1000 at batch 16 26 -> 12 (18 -> 8),
// 25088 -> 4096 at batch 128 563 -> 318 (263 -> 135).
bool ip_stream_supported(int batch, int inputs, int outputs, int dtype, const void *x, const void *w)
{
    static const char *pin = getenv("DLP_IP_KERNEL"); // "direct" / "stream": one kernel wherever it can run, for measurements
    if (pin && pin[0] == 'd')
        return false;
    if (dtype != DLP_FLOAT && dtype != DLP_BFLOAT16)
        return false;
    const size_t esize = dtype_size(dtype);
    if (batch < 1 || ((size_t)inputs * esize) % 16 != 0 || (((uintptr_t)x | (uintptr_t)w) & 15) != 0)
        return false;
    (void)outputs;
    return true;
}

size_t ip_stream_scratch_bytes(int batch, int inputs, int outputs, int dtype, IpPlan *plan)
{
    IpPlan p;
    const int kc = kIpRowBytes / (int)dtype_size(dtype); // k per chunk
    p.nb = 1;
    p.mblocks = (outputs + 31) / 32;
    p.nchunks = (batch + 31) / 32;
    p.ngroups = (inputs + kc - 1) / kc; // chunks of a row
    // K slices: as many workgroups as fit the compute units at once (three each with the 16-row tile of x, else two), slices of at
    // least two chunks, at most 16 slices, and never more than 1024 tiles x slices once K is cut (4 MiB of partial sums, what the
    // entry point that allocates nothing holds)
    const long long tiles = (long long)p.mblocks * p.nchunks;
    long long s = ((batch <= 16 ? 3ll : 2ll) * dlp_cu_count() + tiles - 1) / tiles;
    s = std::min<long long>(s, std::max<long long>(1, 1024 / tiles));
    s = std::min<long long>(s, p.ngroups / 2);
    s = std::max<long long>(1, std::min<long long>(s, 16));
    p.gps = (int)((p.ngroups + s - 1) / s);
    p.S = (p.ngroups + p.gps - 1) / p.gps;
    p.cnt_bytes = (size_t)((tiles * sizeof(int) + 255) / 256 * 256);
    p.part_bytes = p.S > 1 ? (size_t)tiles * p.S * 16 * 64 * sizeof(float) : 0;
    if (plan)
        *plan = p;
    return p.cnt_bytes + p.part_bytes;
}

// An instance that needs more than 64 KB of LDS has to ask for it, once per device.  Done when an operator is created (best
// effort: there may be no device yet) so that a first enqueue inside a stream capture has nothing left to set up; the launch
// checks again.
template <class T, int XR>
static int ip_stream_instance(const IpArgs *a, dim3 grid, hipStream_t stream, TimingScope *ts)
{
    constexpr int lds = ip_stream_lds_bytes(XR);
    if (lds > 65536) {
        static std::atomic<bool> asked[64];
        int dev = 0;
        DLP_HIP_TRY(hipGetDevice(&dev));
        if (dev < 0 || dev >= 64 || !asked[dev].load()) {
            DLP_HIP_TRY(hipFuncSetAttribute((const void *)ip_stream_kernel<T, XR>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
            if (dev >= 0 && dev < 64)
                asked[dev].store(true);
        }
    }
    if (a == nullptr) // set-up only
        return DLP_OK;
    DLP_LAUNCH_TIMED((*ts), (ip_stream_kernel<T, XR>), grid, dim3(256), lds, stream, *a);
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}
template <class T>
static int ip_stream_dispatch(bool small_batch, const IpArgs *a, dim3 grid, hipStream_t stream, TimingScope *ts)
{
    return small_batch ? ip_stream_instance<T, 16>(a, grid, stream, ts) : ip_stream_instance<T, 32>(a, grid, stream, ts);
}
void ip_stream_prepare(int dtype)
{
    if (dtype != DLP_FLOAT && dtype != DLP_BFLOAT16)
        return;
    for (int small = 0; small < 2; small++)
        (void)(dtype == DLP_BFLOAT16 ? ip_stream_dispatch<bf16_t>(small != 0, nullptr, dim3(1), nullptr, nullptr)
                                     : ip_stream_dispatch<float>(small != 0, nullptr, dim3(1), nullptr, nullptr));
    (void)hipGetLastError(); // no device, no harm: the launch asks again
}

int ip_stream_launch(int batch, int inputs, int outputs, int dtype, const void *x, const void *w, void *y, const Epilogue &ep, int *counters,
                     float *partials, hipStream_t stream)
{
    IpPlan p;
    ip_stream_scratch_bytes(batch, inputs, outputs, dtype, &p);
    const size_t esize = dtype_size(dtype);
    const size_t x_bytes = (size_t)batch * inputs * esize, w_bytes = (size_t)outputs * inputs * esize;
    if (x_bytes >= kIpOutOfRange || w_bytes >= kIpOutOfRange || p.part_bytes >= kIpOutOfRange)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "tensors of 2 GiB or more are not supported by the 32-bit buffer addressing");
    IpArgs a;
    a.x = x;
    a.w = w;
    a.bias = ep.bias;
    a.y = y;
    a.cnt = counters;
    a.part = partials;
    a.B = batch;
    a.In = inputs;
    a.Out = outputs;
    a.S = p.S;
    a.ngroups = p.ngroups;
    a.gps = p.gps;
    a.mblocks = p.mblocks;
    a.nchunks = p.nchunks;
    a.act = ep.activation;
    a.x_bytes = (uint32_t)x_bytes;
    a.w_bytes = (uint32_t)w_bytes;
    a.part_bytes = (uint32_t)p.part_bytes;
    const long long wgs = (long long)p.mblocks * p.nchunks * p.S;
    if (wgs > 0x7fffffffLL)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "inner product too large for a single launch");
    const dim3 grid((unsigned)wgs);
    TimingScope ts("ip_direct", stream);
    // batches of at most 16 rows keep 16 rows of x in LDS: three workgroups per compute unit instead of two
    return dtype == DLP_BFLOAT16 ? ip_stream_dispatch<bf16_t>(batch <= 16, &a, grid, stream, &ts)
                                 : ip_stream_dispatch<float>(batch <= 16, &a, grid, stream, &ts);
}

ConvGeom ip_gemm_geom(int batch, int inputs, int outputs, int dtype)
{
    ConvGeom g;
    g.B = batch;
    g.Cin = inputs;
    g.H = 1;
    g.W = 1;
    g.Cout = outputs;
    g.OH = 1;
    g.OW = 1;
    g.KH = g.KW = 1;
    g.sh = g.sw = 1;
    g.ph = g.pw = 0;
    g.dh = g.dw = 1;
    g.groups = 1;
    g.dtype = dtype;
    return g;
}

} // namespace dlp
