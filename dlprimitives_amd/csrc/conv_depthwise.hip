// Depthwise (groups == channels) convolution forward for gfx950.
//
// Replaces the reference's Conv2DForwardDepthwiseSeparable / `conv` kernel
// (src/core/conv.cpp:436-510, src/kernels/depthwise_separable_conv.cl:20-105),
// which covers stride 1 only, and adds stride 2 (the reference falls back to a
// grouped GEMM with M = 1 there, src/core/conv.cpp:725-727).
//
// The op is HBM-bound (about 2 flop per byte), so no matrix cores: every kernel here reads
// each input element from memory once and writes each output once.  What decides the speed
// is how early the loads of a launch are on their way and how the requests of one wavefront
// look to the memory system, not the arithmetic (replacing the 9 multiply-adds by one changes
// no timing).  Three 3x3 kernels, chosen per shape by depthwise_launch:
//   * depthwise3x3_reg_kernel   fp32, planes of 28 x 28 and larger: a lane owns IV input columns x 7 output rows, loads
//                               its 9 (15 at stride 2) input rows straight into registers, all requested before the first
//                               is used, and gets the column left and right of its own from the neighbouring lanes
//                               (DPP wavefront shifts): no LDS, no barrier, 32 independent wavefronts per CU.
//   * depthwise3x3_plane_kernel small planes (and bf16): runs of whole planes through LDS, contiguous 16-byte loads and
//                               streaming 16-byte stores.
//   * depthwise3x3_kernel       everything else (unaligned tensors, odd widths at stride 2, planes wider than the others take).
// Accumulation order is the reference's everywhere:
// sum = bias; sum = fma(k[dr][dc], x, sum) for dr, dc ascending.
//
// Other odd kernel sizes use a plain direct kernel.
#include "dlp_internal.hpp"

#include <algorithm>
#include <cstdlib>
#include <type_traits>

namespace dlp {
namespace {

constexpr int kStripRows = 7; // divides the usual 56/28/14/7 feature maps

struct DwArgs {
    const void *x; // storage type T (float or bf16_t); arithmetic is fp32
    const void *w;
    const float *bias;
    void *y;
    int planes; // B*C
    int C, H, W, OH, OW;
    int nstrips;          // ceil(OH / kStripRows)
    long long total_cols; // planes * nstrips * OW
    float factor;
    int act;
};

// STRIDE 1: halo lanes 0 and 63 (62 outputs per wavefront)
// STRIDE 2: halo lane 0 only (63 outputs per wavefront)
template <class T, int STRIDE>
__global__ __launch_bounds__(256) void depthwise3x3_kernel(DwArgs a)
{
    constexpr int OUT_PER_WAVE = (STRIDE == 1) ? 62 : 63;
    constexpr int NIN = (kStripRows - 1) * STRIDE + 3; // input rows of a strip
    const int lane = threadIdx.x & 63;
    const long long wave = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const long long f = wave * OUT_PER_WAVE + lane - 1; // flat (plane, strip, ox) index
    const bool in_range = f >= 0 && f < a.total_cols;
    const long long ps = in_range ? f / a.OW : 0;
    const int ox = in_range ? (int)(f - ps * a.OW) : 0;
    const int plane = (int)(ps / a.nstrips);
    const int strip = (int)(ps - (long long)plane * a.nstrips);
    const bool is_out = in_range && lane >= 1 && (STRIDE == 2 || lane <= 62);
    const int c = plane % a.C;
    const int oy0 = strip * kStripRows;

    float k[9];
#pragma unroll
    for (int i = 0; i < 9; i++)
        k[i] = to_float(((const T *)a.w)[c * 9 + i]);
    const float bias = a.bias ? a.bias[c] : 0.0f;

    const T *xp = (const T *)a.x + (size_t)plane * a.H * a.W;
    T *yp = (T *)a.y + (size_t)plane * a.OH * a.OW + ox;

    // columns owned by this lane
    const int x0 = ox * STRIDE;
    const bool v1 = in_range && (STRIDE == 2) && (x0 + 1 < a.W);
    const bool has_left = ox > 0;                           // column x0-1 exists in this plane
    const bool has_right = (STRIDE == 1) && (ox + 1 < a.W); // column x0+1 (stride 1 only)

    // issue every load of the strip before anything consumes one
    float c0[NIN], c1[NIN];
    const int iy0 = oy0 * STRIDE - 1;
#pragma unroll
    for (int r = 0; r < NIN; r++) {
        const int yy = iy0 + r;
        const bool vy = in_range && yy >= 0 && yy < a.H;
        const T *p = xp + (size_t)(vy ? yy : 0) * a.W + x0;
        c0[r] = vy ? to_float(p[0]) : 0.0f;
        c1[r] = 0.0f;
        if (STRIDE == 2)
            c1[r] = (vy && v1) ? to_float(p[1]) : 0.0f;
    }
    // window columns (x0-1, x0, x0+1) of every row
    float left[NIN], right[NIN];
#pragma unroll
    for (int r = 0; r < NIN; r++) {
        if (STRIDE == 1) {
            const float l = __shfl_up(c0[r], 1);
            const float rr = __shfl_down(c0[r], 1);
            left[r] = has_left ? l : 0.0f;
            right[r] = has_right ? rr : 0.0f;
        } else {
            const float l = __shfl_up(c1[r], 1); // previous lane's odd column = 2*ox - 1
            left[r] = has_left ? l : 0.0f;
            right[r] = c1[r];
        }
    }
#pragma unroll
    for (int j = 0; j < kStripRows; j++) {
        const int oy = oy0 + j;
        float sum = bias;
#pragma unroll
        for (int dr = 0; dr < 3; dr++) {
            const int r = j * STRIDE + dr;
            sum = fmaf(k[3 * dr + 0], left[r], sum);
            sum = fmaf(k[3 * dr + 1], c0[r], sum);
            sum = fmaf(k[3 * dr + 2], right[r], sum);
        }
        if (is_out && oy < a.OH)
            store_out(yp + (size_t)oy * a.OW, apply_act(sum, a.act), a.factor);
    }
}

// ---- 3x3, strips in registers --------------------------------------------------------------------
// A lane owns IV neighbouring input columns (IV / STRIDE output columns) of a strip of kRegRows output rows of one plane; the
// ncg = W / IV lanes of a strip sit side by side in a wavefront, which holds spw = 64 / ncg strips (strips are numbered plane by
// plane, top to bottom, so a wavefront and a workgroup cover one contiguous piece of x and of y).  Every input row of the strip
// is requested before the first is used (buffer loads: rows above and below the plane and idle lanes are sent out of range and
// arrive as zeros, so nothing branches), the filter arrives as three 12-byte loads.  The column to the left of a lane's own is the
// last column of the lane before it, the column to the right (stride 1) the first of the lane after it: one DPP wavefront
// shift each, replaced by zero at the ends of a row.  HBM traffic is |x| + |y| (the rows two strips share come out of the
// caches).  Stores are write-back unless a wavefront's share of an output row is a whole run of 128 bytes or more (NT).
constexpr int kRegRows = 7;
constexpr uint32_t kDwOutOfRange = 0x80000000u; // >= num_records of every buffer the kernel is given

struct DwRegArgs {
    const float *x, *w;
    const float *bias;
    float *y;
    uint32_t x_bytes, y_bytes;
    int C, H, W, OH, OW;
    int ncg, nrb, spw, nstrips; // lanes per strip, strips per plane, strips per wavefront, strips in all
    uint32_t ncg_magic, ncg_shift, nrb_magic, nrb_shift, c_magic, c_shift;
    float factor;
    int act;
    float clamp_lo, clamp_hi;
};

typedef float dw_f32x4 __attribute__((ext_vector_type(4)));
typedef float dw_f32x3 __attribute__((ext_vector_type(3)));
typedef float dw_f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int dw_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int dw_u32x2 __attribute__((ext_vector_type(2)));

template <int N>
__device__ __forceinline__ void dw_load(float *d, __amdgpu_buffer_rsrc_t r, uint32_t v, uint32_t s)
{
    if constexpr (N == 4) {
        const dw_f32x4 t = __builtin_bit_cast(dw_f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, v, s, 0));
        d[0] = t.x, d[1] = t.y, d[2] = t.z, d[3] = t.w;
    } else if constexpr (N == 2) {
        const dw_f32x2 t = __builtin_bit_cast(dw_f32x2, __builtin_amdgcn_raw_buffer_load_b64(r, v, s, 0));
        d[0] = t.x, d[1] = t.y;
    } else
        d[0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, v, s, 0));
}
template <int N, int AUX>
__device__ __forceinline__ void dw_store(const float *d, __amdgpu_buffer_rsrc_t r, uint32_t v, uint32_t s)
{
    if constexpr (N == 4) {
        const dw_f32x4 t = {d[0], d[1], d[2], d[3]};
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(dw_u32x4, t), r, v, s, AUX);
    } else if constexpr (N == 2) {
        const dw_f32x2 t = {d[0], d[1]};
        __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(dw_u32x2, t), r, v, s, AUX);
    } else
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, d[0]), r, v, s, AUX);
}
// lane i receives the value of lane i - 1 / i + 1 (lane 0 / 63: zero)
__device__ __forceinline__ float dw_from_prev_lane(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x138 /* wave_shr:1 */, 0xf, 0xf, false));
}
__device__ __forceinline__ float dw_from_next_lane(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x130 /* wave_shl:1 */, 0xf, 0xf, false));
}

// ACT: 0 identity, 1 one clamp (ReLU / ReLU6), 2 tanh / sigmoid.  OLDY: y = factor * y + value.  NT: streaming stores.
template <int STRIDE, int IV, int ACT, bool OLDY, bool NT>
__global__ __launch_bounds__(256) void depthwise3x3_reg_kernel(DwRegArgs a)
{
    constexpr int R = kRegRows;
    constexpr int OV = IV / STRIDE;
    constexpr int NIN = (R - 1) * STRIDE + 3;
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int sl = (int)fast_div((uint32_t)lane, a.ncg_magic, a.ncg_shift);
    const int cg = lane - sl * a.ncg;
    const int strip = wave * a.spw + sl;
    const bool active = sl < a.spw && strip < a.nstrips;
    const int plane = (int)fast_div((uint32_t)strip, a.nrb_magic, a.nrb_shift);
    const int rb = strip - plane * a.nrb;
    const int c = plane - (int)fast_div((uint32_t)plane, a.c_magic, a.c_shift) * a.C;
    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc((void *)a.y, 0, a.y_bytes, 0x00020000);
    // row pitches as scalars: the offset of row r is then an SGPR operand of its load, not vector arithmetic
    const uint32_t w4 = (uint32_t)__builtin_amdgcn_readfirstlane(a.W * 4), ow4 = (uint32_t)__builtin_amdgcn_readfirstlane(a.OW * 4);

    // input rows iy0 - 1 .. iy0 + NIN - 2; row r of the strip exists when 1 <= r <= rows_in (r = 0: when the strip is not the plane's first)
    const int iy0 = rb * (R * STRIDE);
    const uint32_t xbase = active ? (uint32_t)((plane * a.H + iy0) * a.W + cg * IV) * 4u : kDwOutOfRange;
    const int rows_in = a.H - iy0;
    float v[NIN][IV];
    dw_load<IV>(v[0], xr, rb > 0 ? xbase - w4 : kDwOutOfRange, 0);
#pragma unroll
    for (int r = 1; r < NIN; r++)
        dw_load<IV>(v[r], xr, (r <= rows_in) ? xbase : kDwOutOfRange, (uint32_t)(r - 1) * w4);
    float k[9];
    {
        const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, (uint32_t)a.C * 36u, 0x00020000);
        const uint32_t wv = active ? (uint32_t)c * 36u : kDwOutOfRange;
#pragma unroll
        for (int dr = 0; dr < 3; dr++) {
            const dw_f32x3 t = __builtin_bit_cast(dw_f32x3, __builtin_amdgcn_raw_buffer_load_b96(wr, wv, dr * 12, 0));
            k[3 * dr] = t.x, k[3 * dr + 1] = t.y, k[3 * dr + 2] = t.z;
        }
    }
    // no bias: a buffer of no records, every load of it gives 0
    const __amdgpu_buffer_rsrc_t br = __builtin_amdgcn_make_buffer_rsrc((void *)a.bias, 0, a.bias ? (uint32_t)a.C * 4u : 0u, 0x00020000);
    const float bias = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(br, active ? (uint32_t)c * 4u : kDwOutOfRange, 0, 0));

    const bool has_left = cg > 0;
    const bool has_right = cg + 1 < a.ncg;
    const int oy0 = rb * R;
    const int rows_out = a.OH - oy0;
    const uint32_t ybase = active ? (uint32_t)((plane * a.OH + oy0) * a.OW + cg * OV) * 4u : kDwOutOfRange;
    float old[OLDY ? R : 1][OV];
    if (OLDY) {
#pragma unroll
        for (int j = 0; j < R; j++)
            dw_load<OV>(old[OLDY ? j : 0], yr, (j < rows_out) ? ybase : kDwOutOfRange, (uint32_t)j * ow4);
    }
    float left[3], right[3]; // the columns beside the lane's own, of the three rows of the window
    auto edge = [&](int r) {
        const float l = dw_from_prev_lane(v[r][IV - 1]);
        left[r % 3] = has_left ? l : 0.0f;
        if (STRIDE == 1) {
            const float rr = dw_from_next_lane(v[r][0]);
            right[r % 3] = has_right ? rr : 0.0f;
        }
    };
    // input column j = -1 .. IV of row r
    auto col = [&](int r, int j) -> float { return j < 0 ? left[r % 3] : (j >= IV ? right[r % 3] : v[r][j]); };
    edge(0);
    if (STRIDE == 1)
        edge(1);
#pragma unroll
    for (int j = 0; j < R; j++) {
        if (STRIDE == 1)
            edge(j + 2);
        else {
            edge(2 * j + 1);
            edge(2 * j + 2);
        }
        float out[OV];
#pragma unroll
        for (int o = 0; o < OV; o++) {
            float sum = bias;
#pragma unroll
            for (int dr = 0; dr < 3; dr++)
#pragma unroll
                for (int dc = 0; dc < 3; dc++)
                    sum = fmaf(k[3 * dr + dc], col(j * STRIDE + dr, o * STRIDE + dc - 1), sum);
            if (ACT == 1)
                sum = clamp_med3(sum, a.clamp_lo, a.clamp_hi);
            else if (ACT == 2)
                sum = apply_act(sum, a.act);
            if (OLDY)
                sum = fmaf(old[OLDY ? j : 0][o], a.factor, sum);
            out[o] = sum;
        }
        dw_store<OV, NT ? 2 : 0>(out, yr, (j < rows_out) ? ybase : kDwOutOfRange, (uint32_t)j * ow4);
    }
}

// Input columns per lane of the register kernel for this geometry, 0: not taken.
static int reg_columns(const ConvGeom &g, const void *x, const void *y)
{
    if (g.KH != 3 || g.KW != 3 || g.dtype != DLP_FLOAT)
        return 0;
    const long long xb = (long long)g.B * g.Cin * g.H * g.W * 4, yb = (long long)g.B * g.Cin * g.OH * g.OW * 4;
    if (xb >= 0x7fffffffLL || yb >= 0x7fffffffLL || (long long)g.B * g.Cin * ((g.OH + kRegRows - 1) / kRegRows) >= 0x7fffffffLL / 64)
        return 0;
    const uintptr_t ax = (uintptr_t)x, ay = (uintptr_t)y;
    if (g.sh == 1) {
        if (g.W <= 64 && ((ax | ay) & 3) == 0)
            return 1;
        if (g.W % 2 == 0 && g.W <= 128 && ((ax | ay) & 7) == 0)
            return 2;
        if (g.W % 4 == 0 && g.W <= 256 && ((ax | ay) & 15) == 0)
            return 4;
        return 0;
    }
    if (g.W % 2 == 0 && g.W <= 128 && (ax & 7) == 0 && (ay & 3) == 0)
        return 2;
    if (g.W % 4 == 0 && g.W <= 256 && (ax & 15) == 0 && (ay & 7) == 0)
        return 4;
    return 0;
}

// ---- 3x3, whole planes through LDS ------------------------------------------------------------------
// In NCHW the planes of a depthwise convolution are independent and lie one after another in memory, so a run of
// P whole planes is one contiguous piece of x and produces one contiguous piece of y.  A workgroup takes such a
// run of at most 16 KB: it copies it to LDS with 16-byte loads, all in flight at once (every byte of x is read
// exactly once: no halo rows, whatever the plane size), computes from LDS into a second LDS buffer and writes that
// with 16-byte stores.  The filter and bias of the run's channels travel to LDS next to the input.
// The layer is bound by memory, but only if the arithmetic stays out of the way: 9 multiply-adds per output are a
// seventh of the chip's vector rate at 5 TB/s, so every other instruction per output counts.  A lane therefore takes
// a tile of R rows x kPlaneSeg columns of outputs and slides a three-row window down it: 9 (stride 1) input values
// read from LDS per output row of 7, edge handling decided once per tile (padding is read from a block of zeros
// behind the run by choosing the address, so the reads carry no condition), one v_med3 for ReLU / ReLU6.
// R is chosen by the host so that the tiles of a run are about one per thread.
// Accumulation order is the reference's: sum = bias; sum = fma(k[dr][dc], x, sum) for dr, dc ascending.
constexpr int kPlaneSeg = 7;          // output columns of a tile (divides the 56 / 28 / 14 / 7 wide feature maps)
constexpr int kPlaneThreads = 256;
constexpr int kPlaneMaxPieces = 4;    // 16-byte pieces per thread: a run is at most 16 KB
constexpr int kPlaneMaxBytes = kPlaneMaxPieces * kPlaneThreads * 16;
constexpr int kPlaneMaxP = 64;        // planes of a run
constexpr int kPlaneWStride = 11;     // floats per plane in the LDS filter table (9 weights, bias; odd: no bank conflicts)

struct DwPlaneArgs {
    const void *x, *w;
    const float *bias;
    void *y;
    int planes, C, H, W, OH, OW;
    int P;      // planes per run
    int nseg;   // tiles per row of tiles
    int R, nrt; // output rows per tile, rows of tiles per plane
    uint32_t tpp_magic, tpp_shift, nseg_magic, nseg_shift; // divisions by (nrt * nseg) and by nseg
    float factor;
    int act;
    float clamp_lo, clamp_hi;
};

// GENERIC_ACT: tanh / sigmoid; otherwise identity, ReLU or ReLU6 as one clamp (a per-output switch on the activation turns into
// scalar branches around every output, which cost more than the arithmetic)
template <class T, int STRIDE, bool FULL, int NLD, bool GENERIC_ACT>
__global__ __launch_bounds__(kPlaneThreads) void depthwise3x3_plane_kernel(DwPlaneArgs a)
{
    constexpr int kPlanePieces = NLD;
    constexpr int kRunBytes = NLD * kPlaneThreads * 16;
    constexpr int EPP = 16 / (int)sizeof(T);           // elements per 16-byte piece
    constexpr int NIN = (kPlaneSeg - 1) * STRIDE + 3;  // input columns of a tile
    constexpr int NZ = 16;                              // zeros behind the run: what a padding row or column reads
    static_assert(NIN <= NZ, "tile shape");
    __shared__ __attribute__((aligned(16))) unsigned char lds_raw[kRunBytes + NZ * sizeof(T)]; // the run | zeros
    __shared__ __attribute__((aligned(16))) unsigned char lds_out_raw[kRunBytes];              // the run's output
    __shared__ float lds_w[kPlaneMaxP * kPlaneWStride];
    T *lds = reinterpret_cast<T *>(lds_raw);
    T *lds_out = reinterpret_cast<T *>(lds_out_raw);
    T *zeros = reinterpret_cast<T *>(lds_raw + kRunBytes);
    const int tid = threadIdx.x;
    const int HW = a.H * a.W, OHW = a.OH * a.OW;
    const int plane0 = (int)blockIdx.x * a.P;
    const int np = min(a.P, a.planes - plane0); // planes of this run
    const int n_in = np * HW, n_out = np * OHW;
    const T *xg = (const T *)a.x + (size_t)plane0 * HW;
    T *yg = (T *)a.y + (size_t)plane0 * OHW;

    // ---- the run's input, filter and bias: global -> registers (every load issued before anything waits) -> LDS ----
    uint4 piece[kPlanePieces];
#pragma unroll
    for (int q = 0; q < kPlanePieces; q++) {
        const int e0 = (tid + kPlaneThreads * q) * EPP;
        piece[q] = make_uint4(0, 0, 0, 0);
        if (e0 + EPP <= n_in)
            piece[q] = *reinterpret_cast<const uint4 *>(xg + e0);
        else if (e0 < n_in) { // the last piece of the tensor may be cut short
            T tmp[EPP];
#pragma unroll
            for (int e = 0; e < EPP; e++)
                tmp[e] = (e0 + e < n_in) ? xg[e0 + e] : T();
            piece[q] = *reinterpret_cast<const uint4 *>(tmp);
        }
    }
    float wreg[3]; // 9 weights and the bias of every plane of the run: np * 10 <= 640 values
    int w_pl[3], w_j[3];
    {
        const int c0 = plane0 % a.C;
#pragma unroll
        for (int q = 0; q < 3; q++) {
            const int i = tid + kPlaneThreads * q;
            w_pl[q] = i / 10;
            w_j[q] = i - w_pl[q] * 10;
            wreg[q] = 0.0f;
            if (w_pl[q] < np) {
                int c = c0 + w_pl[q];
                c = c >= a.C ? c % a.C : c;
                wreg[q] = w_j[q] < 9 ? to_float(((const T *)a.w)[c * 9 + w_j[q]]) : (a.bias ? a.bias[c] : 0.0f);
            }
        }
    }
    if (tid < NZ)
        zeros[tid] = T();
#pragma unroll
    for (int q = 0; q < kPlanePieces; q++)
        if ((tid + kPlaneThreads * q) * EPP < n_in)
            *reinterpret_cast<uint4 *>(lds_raw + (tid + kPlaneThreads * q) * 16) = piece[q];
#pragma unroll
    for (int q = 0; q < 3; q++)
        if (w_pl[q] < np)
            lds_w[w_pl[q] * kPlaneWStride + w_j[q]] = wreg[q];
    __syncthreads();

    // ---- tiles of R x kPlaneSeg outputs: numbered (plane, row of tiles, tile in the row) ----
    const int tpp = a.nrt * a.nseg;
    const int tiles = np * tpp;
    for (int tile = tid; tile < tiles; tile += kPlaneThreads) {
        const int pl = (int)fast_div((uint32_t)tile, a.tpp_magic, a.tpp_shift);
        const int rem = tile - pl * tpp;
        const int ty = (int)fast_div((uint32_t)rem, a.nseg_magic, a.nseg_shift);
        const int ox0 = (rem - ty * a.nseg) * kPlaneSeg;
        const int oy0 = ty * a.R;
        const int rows = min(a.R, a.OH - oy0);
        const int out_n = min(kPlaneSeg, a.OW - ox0);
        T *pout = lds_out + pl * OHW + oy0 * a.OW + ox0;
        const float *kw = lds_w + pl * kPlaneWStride;
        float k[9];
#pragma unroll
        for (int i = 0; i < 9; i++)
            k[i] = kw[i];
        const float bias = kw[9];
        const T *pin = lds + pl * HW;
        const int ix0 = ox0 * STRIDE - 1;
        const bool left_ok = ix0 >= 0, right_ok = ix0 + NIN - 1 < a.W;
        const bool clamp = a.act != DLP_ACT_IDENTITY;
        float v[3][NIN]; // the window: input rows of the current output row
        auto load_row = [&](auto slot_c, int iy) {
            constexpr int SL = decltype(slot_c)::value;
            const bool vy = iy >= 0 && iy < a.H;
            if (FULL) {
                // every tile is whole (OW is a multiple of kPlaneSeg): only the first and the last column of the window can
                // fall outside the image; a padding row reads zeros[j], a padding column zeros[0]
                const T *row = vy ? pin + iy * a.W + ix0 : zeros;
                const T *first = left_ok ? row : zeros, *last = right_ok ? row + (NIN - 1) : zeros;
                v[SL][0] = to_float(*first);
#pragma unroll
                for (int j = 1; j < NIN - 1; j++)
                    v[SL][j] = to_float(row[j]);
                v[SL][NIN - 1] = to_float(*last);
            } else {
                const T *row = pin + (vy ? iy : 0) * a.W;
#pragma unroll
                for (int j = 0; j < NIN; j++) {
                    const int ix = ix0 + j;
                    v[SL][j] = (vy && ix >= 0 && ix < a.W) ? to_float(row[ix]) : 0.0f;
                }
            }
        };
        auto compute_row = [&](auto s0_c, auto s1_c, auto s2_c, int r) { // output row r of the tile from window slots s0, s1, s2
            constexpr int S0 = decltype(s0_c)::value, S1 = decltype(s1_c)::value, S2 = decltype(s2_c)::value;
#pragma unroll
            for (int o = 0; o < kPlaneSeg; o++) {
                float sum = bias;
#pragma unroll
                for (int dc = 0; dc < 3; dc++)
                    sum = fmaf(k[dc], v[S0][o * STRIDE + dc], sum);
#pragma unroll
                for (int dc = 0; dc < 3; dc++)
                    sum = fmaf(k[3 + dc], v[S1][o * STRIDE + dc], sum);
#pragma unroll
                for (int dc = 0; dc < 3; dc++)
                    sum = fmaf(k[6 + dc], v[S2][o * STRIDE + dc], sum);
                if (GENERIC_ACT)
                    sum = apply_act(sum, a.act);
                else {
                    const float clamped = clamp_med3(sum, a.clamp_lo, a.clamp_hi);
                    sum = clamp ? clamped : sum; // identity keeps NaNs: no clamp
                }
                if (FULL || o < out_n)
                    store_plain(pout + r * a.OW + o, sum);
            }
        };
        using I0 = std::integral_constant<int, 0>;
        using I1 = std::integral_constant<int, 1>;
        using I2 = std::integral_constant<int, 2>;
        const int iy0 = oy0 * STRIDE - 1;
        if (STRIDE == 1) { // the window moves down one row per output row: one new row each, slots rotate
            load_row(I0{}, iy0);
            load_row(I1{}, iy0 + 1);
            for (int r = 0; r < rows; r += 3) {
                load_row(I2{}, iy0 + r + 2);
                compute_row(I0{}, I1{}, I2{}, r);
                if (r + 1 < rows) {
                    load_row(I0{}, iy0 + r + 3);
                    compute_row(I1{}, I2{}, I0{}, r + 1);
                }
                if (r + 2 < rows) {
                    load_row(I1{}, iy0 + r + 4);
                    compute_row(I2{}, I0{}, I1{}, r + 2);
                }
            }
        } else { // two rows per output row: the last row of one window is the first of the next
            load_row(I0{}, iy0);
            for (int r = 0; r < rows; r += 2) {
                load_row(I1{}, iy0 + 2 * r + 1);
                load_row(I2{}, iy0 + 2 * r + 2);
                compute_row(I0{}, I1{}, I2{}, r);
                if (r + 1 < rows) {
                    load_row(I0{}, iy0 + 2 * r + 3);
                    load_row(I1{}, iy0 + 2 * r + 4);
                    compute_row(I2{}, I0{}, I1{}, r + 1);
                }
                // an even number of rows later the first window slot holds the shared row again
            }
        }
    }
    __syncthreads();

    // ---- the run's output: LDS -> global, 16 bytes per store ----
#pragma unroll
    for (int q = 0; q < kPlanePieces; q++) {
        const int e0 = (tid + kPlaneThreads * q) * EPP;
        if (e0 >= n_out)
            continue;
        const uint4 r = *reinterpret_cast<const uint4 *>(lds_out_raw + (tid + kPlaneThreads * q) * 16);
        if (e0 + EPP <= n_out && a.factor == 0.0f) {
            // streaming store: the run leaves in whole cache lines and is not read again by this launch
            __builtin_nontemporal_store(dw_u32x4{r.x, r.y, r.z, r.w}, reinterpret_cast<dw_u32x4 *>(yg + e0));
        } else { // y = factor * y + value (reference: depthwise_separable_conv.cl:96-101), and the cut last piece
            T tmp[EPP];
            *reinterpret_cast<uint4 *>(tmp) = r;
#pragma unroll
            for (int e = 0; e < EPP; e++)
                if (e0 + e < n_out)
                    store_out(yg + e0 + e, to_float(tmp[e]), a.factor);
        }
    }
}

// Planes per run for this geometry (0: the plane kernel does not take it): as many as fit 16 KB of input and 64 planes,
// and such that every run starts on a 16-byte boundary in x and in y.
static int plane_run(const ConvGeom &g, bool always = false)
{
    if (g.KH != 3 || g.KW != 3)
        return 0;
    const long long es = (long long)dtype_size(g.dtype);
    const long long in_bytes = (long long)g.H * g.W * es, out_bytes = (long long)g.OH * g.OW * es;
    if (in_bytes > kPlaneMaxBytes)
        return 0;
    // Measured on the MobileNet shapes at batch 64 (fp32, back-to-back launches on tensors that start cold): the plane kernel against the
    // strip kernel 47.7 / 51.9 us (C144 at 56 x 56), 19.0 / 21.8, 13.3 / 15.7, 9.0 / 11.5 us at stride 1; 36.3 / 32.9, 13.8 / 15.3,
    // 10.1 / 10.0, 7.6 / 7.7 us at stride 2: with large planes at stride 2 a run holds few tiles (112 for 256 threads) and the strip kernel wins.
    // With bf16 tensors the plane kernel wins throughout (its loads and stores stay 16 bytes wide).
    if (g.dtype == DLP_FLOAT && g.sh == 2 && in_bytes > 8192 && !always)
        return 0;
    const long long pmax = std::min<long long>(kPlaneMaxP, kPlaneMaxBytes / in_bytes);
    auto gcd = [](long long x, long long y) {
        while (y) {
            const long long r = x % y;
            x = y;
            y = r;
        }
        return x;
    };
    const long long s_in = 16 / gcd(16, in_bytes), s_out = 16 / gcd(16, out_bytes);
    const long long step = s_in / gcd(s_in, s_out) * s_out;
    return (int)(pmax / step * step);
}

// Any odd kernel size, stride 1 or 2, pad = K/2: one output per thread.
template <class T>
__global__ __launch_bounds__(256) void depthwise_direct_kernel(DwArgs a, int K, int stride)
{
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long total = (long long)a.planes * a.OH * a.OW;
    if (idx >= total)
        return;
    const int ox = (int)(idx % a.OW);
    const long long t = idx / a.OW;
    const int oy = (int)(t % a.OH);
    const int plane = (int)(t / a.OH);
    const int c = plane % a.C;
    const int pad = K / 2;
    const T *xp = (const T *)a.x + (size_t)plane * a.H * a.W;
    const T *kp = (const T *)a.w + (size_t)c * K * K;
    float sum = a.bias ? a.bias[c] : 0.0f;
    for (int dr = 0; dr < K; dr++) {
        const int yy = oy * stride - pad + dr;
        for (int dc = 0; dc < K; dc++) {
            const int xx = ox * stride - pad + dc;
            const float v = (yy >= 0 && yy < a.H && xx >= 0 && xx < a.W) ? to_float(xp[(size_t)yy * a.W + xx]) : 0.0f;
            sum = fmaf(to_float(kp[dr * K + dc]), v, sum);
        }
    }
    store_out((T *)a.y + idx, apply_act(sum, a.act), a.factor);
}

} // namespace

bool depthwise_supported(const ConvGeom &g)
{
    return (g.dtype == DLP_FLOAT || g.dtype == DLP_BFLOAT16) && g.groups == g.Cin && g.Cout == g.Cin && g.Cin > 1 && g.KH == g.KW && g.KH % 2 == 1 &&
           g.ph == g.KH / 2 && g.pw == g.KW / 2 && g.dh == 1 && g.dw == 1 && g.sh == g.sw && (g.sh == 1 || g.sh == 2);
}

int depthwise_launch(const ConvGeom &g, const void *x, const void *w, void *y, const Epilogue &ep, hipStream_t stream)
{
    DLP_REQUIRE(depthwise_supported(g), "geometry is not depthwise separable");
    if (g.B == 0)
        return DLP_OK;
    DwArgs a;
    a.x = x;
    a.w = w;
    a.bias = ep.bias;
    a.y = y;
    const bool bf16 = g.dtype == DLP_BFLOAT16;
    a.planes = g.B * g.Cin;
    a.C = g.Cin;
    a.H = g.H;
    a.W = g.W;
    a.OH = g.OH;
    a.OW = g.OW;
    a.nstrips = (g.OH + kStripRows - 1) / kStripRows;
    a.total_cols = (long long)a.planes * a.nstrips * g.OW;
    a.factor = ep.factor;
    a.act = ep.activation;
    TimingScope ts("sep_conv", stream);
    // DLP_DEPTHWISE_KERNEL = reg | plane | strip pins the 3x3 kernel where it applies (measurements); unset: by shape
    static const char *pin = getenv("DLP_DEPTHWISE_KERNEL");
    const bool pin_reg = pin && pin[0] == 'r', pin_plane = pin && pin[0] == 'p', pin_strip = pin && pin[0] == 's';
    // Measured at batch 64 on cold tensors, register kernel / plane kernel (stride 1; stride 2): 56 x 56 40.0 / 48.2 us (26.3 / 32.8 with
    // the strip kernel), 28 x 28 16.5 / 17.8 (10.9 / 13.1), 14 x 14 12.0 / 11.5 (8.1 / 9.1), 7 x 7 10.7 / 6.9: planes of 14 x 14 and
    // smaller at stride 1 and 7 x 7 at stride 2 are too short a run per lane for direct loads and go through LDS.
    const int iv = (pin_plane || pin_strip) ? 0 : reg_columns(g, x, y);
    const bool small_plane = g.sh == 1 ? g.H * g.W < 400 : g.H * g.W < 100;
    if (iv > 0 && (pin_reg || !small_plane)) {
        DwRegArgs ra;
        ra.x = (const float *)x;
        ra.w = (const float *)w;
        ra.bias = ep.bias;
        ra.y = (float *)y;
        ra.x_bytes = (uint32_t)((size_t)a.planes * g.H * g.W * 4);
        ra.y_bytes = (uint32_t)((size_t)a.planes * g.OH * g.OW * 4);
        ra.C = g.Cin;
        ra.H = g.H;
        ra.W = g.W;
        ra.OH = g.OH;
        ra.OW = g.OW;
        ra.ncg = g.W / iv;
        ra.nrb = (g.OH + kRegRows - 1) / kRegRows;
        ra.spw = 64 / ra.ncg;
        ra.nstrips = a.planes * ra.nrb;
        make_magic((uint32_t)ra.ncg, ra.ncg_magic, ra.ncg_shift);
        make_magic((uint32_t)ra.nrb, ra.nrb_magic, ra.nrb_shift);
        make_magic((uint32_t)ra.C, ra.c_magic, ra.c_shift);
        ra.factor = ep.factor;
        ra.act = ep.activation;
        ra.clamp_lo = 0.0f;
        ra.clamp_hi = ep.activation == DLP_ACT_RELU6 ? 6.0f : __builtin_huge_valf();
        const int waves = (ra.nstrips + ra.spw - 1) / ra.spw;
        const dim3 grid((unsigned)((waves + 3) / 4)), block(256);
        const int act = (ep.activation == DLP_ACT_TANH || ep.activation == DLP_ACT_SIGMOID) ? 2 : (ep.activation == DLP_ACT_IDENTITY ? 0 : 1);
        const bool oldy = ep.factor != 0.0f;
        // streaming stores pay when a wavefront's piece of an output row is whole cache lines (one column per lane, rows of 48 floats up)
        const bool nt = !oldy && iv == 1 && g.sh == 1 && g.OW >= 48;
        auto launch = [&](auto stride_c, auto iv_c) {
            constexpr int S = decltype(stride_c)::value, IV = decltype(iv_c)::value;
            if (oldy) {
                if (act == 0)
                    DLP_LAUNCH_TIMED(ts, (depthwise3x3_reg_kernel<S, IV, 0, true, false>), grid, block, 0, stream, ra);
                else if (act == 1)
                    DLP_LAUNCH_TIMED(ts, (depthwise3x3_reg_kernel<S, IV, 1, true, false>), grid, block, 0, stream, ra);
                else
                    DLP_LAUNCH_TIMED(ts, (depthwise3x3_reg_kernel<S, IV, 2, true, false>), grid, block, 0, stream, ra);
            } else if (act == 2)
                DLP_LAUNCH_TIMED(ts, (depthwise3x3_reg_kernel<S, IV, 2, false, false>), grid, block, 0, stream, ra);
            else if (act == 0)
                DLP_LAUNCH_TIMED(ts, (depthwise3x3_reg_kernel<S, IV, 0, false, false>), grid, block, 0, stream, ra);
            else if (nt && S == 1 && IV == 1)
                DLP_LAUNCH_TIMED(ts, (depthwise3x3_reg_kernel<S, IV, 1, false, (S == 1 && IV == 1)>), grid, block, 0, stream, ra);
            else
                DLP_LAUNCH_TIMED(ts, (depthwise3x3_reg_kernel<S, IV, 1, false, false>), grid, block, 0, stream, ra);
        };
        using I1 = std::integral_constant<int, 1>;
        using I2 = std::integral_constant<int, 2>;
        using I4 = std::integral_constant<int, 4>;
        if (g.sh == 1 && iv == 1)
            launch(I1{}, I1{});
        else if (g.sh == 1 && iv == 2)
            launch(I1{}, I2{});
        else if (g.sh == 1)
            launch(I1{}, I4{});
        else if (iv == 2)
            launch(I2{}, I2{});
        else
            launch(I2{}, I4{});
        DLP_HIP_TRY(hipGetLastError());
        return DLP_OK;
    }
    const int run = pin_strip ? 0 : plane_run(g, pin_plane);
    if (run > 0 && (((uintptr_t)x | (uintptr_t)y) & 15) == 0) {
        DwPlaneArgs pa;
        pa.x = x;
        pa.w = w;
        pa.bias = ep.bias;
        pa.y = y;
        pa.planes = a.planes;
        pa.C = g.Cin;
        pa.H = g.H;
        pa.W = g.W;
        pa.OH = g.OH;
        pa.OW = g.OW;
        pa.P = run;
        pa.nseg = (g.OW + kPlaneSeg - 1) / kPlaneSeg;
        // rows per tile: about one tile per thread (up to 7 rows: the window slides, so a taller tile reads fewer input rows per output)
        pa.R = (int)std::min<long long>(7, std::max<long long>(1, ((long long)run * pa.nseg * g.OH + kPlaneThreads - 1) / kPlaneThreads));
        pa.nrt = (g.OH + pa.R - 1) / pa.R;
        make_magic((uint32_t)(pa.nrt * pa.nseg), pa.tpp_magic, pa.tpp_shift);
        make_magic((uint32_t)pa.nseg, pa.nseg_magic, pa.nseg_shift);
        pa.factor = ep.factor;
        pa.act = ep.activation;
        pa.clamp_lo = 0.0f;
        pa.clamp_hi = ep.activation == DLP_ACT_RELU6 ? 6.0f : __builtin_huge_valf();
        const dim3 grid((unsigned)(((long long)a.planes + run - 1) / run)), block(kPlaneThreads);
        const bool full = g.OW % kPlaneSeg == 0;
        const bool generic = ep.activation == DLP_ACT_TANH || ep.activation == DLP_ACT_SIGMOID;
        auto launch = [&](auto type_tag, auto stride_c) {
            using T = decltype(type_tag);
            constexpr int S = decltype(stride_c)::value;
            const long long run_bytes = (long long)run * g.H * g.W * (long long)dtype_size(g.dtype);
            auto with_nld = [&](auto nld_c) {
                constexpr int N = decltype(nld_c)::value;
                if (generic)
                    DLP_LAUNCH_TIMED(ts, (depthwise3x3_plane_kernel<T, S, false, N, true>), grid, block, 0, stream, pa);
                else if (full)
                    DLP_LAUNCH_TIMED(ts, (depthwise3x3_plane_kernel<T, S, true, N, false>), grid, block, 0, stream, pa);
                else
                    DLP_LAUNCH_TIMED(ts, (depthwise3x3_plane_kernel<T, S, false, N, false>), grid, block, 0, stream, pa);
            };
            if (run_bytes <= 4096)
                with_nld(std::integral_constant<int, 1>{});
            else if (run_bytes <= 8192)
                with_nld(std::integral_constant<int, 2>{});
            else
                with_nld(std::integral_constant<int, 4>{});
        };
        if (!bf16 && g.sh == 1)
            launch(float{}, std::integral_constant<int, 1>{});
        else if (!bf16)
            launch(float{}, std::integral_constant<int, 2>{});
        else if (g.sh == 1)
            launch(bf16_t{}, std::integral_constant<int, 1>{});
        else
            launch(bf16_t{}, std::integral_constant<int, 2>{});
        DLP_HIP_TRY(hipGetLastError());
        return DLP_OK;
    }
    if (g.KH == 3) {
        const int per_wave = g.sh == 1 ? 62 : 63;
        const long long waves = (a.total_cols + per_wave - 1) / per_wave;
        const long long blocks = (waves + 3) / 4;
        if (blocks > 0x7fffffffLL)
            return fail(DLP_ERR_NOT_IMPLEMENTED, "depthwise convolution too large for a single launch");
        if (g.sh == 1 && !bf16)
            DLP_LAUNCH_TIMED(ts, (depthwise3x3_kernel<float, 1>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
        else if (g.sh == 1)
            DLP_LAUNCH_TIMED(ts, (depthwise3x3_kernel<bf16_t, 1>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
        else if (!bf16)
            DLP_LAUNCH_TIMED(ts, (depthwise3x3_kernel<float, 2>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
        else
            DLP_LAUNCH_TIMED(ts, (depthwise3x3_kernel<bf16_t, 2>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
    } else {
        const long long total = (long long)a.planes * g.OH * g.OW;
        const long long blocks = (total + 255) / 256;
        if (blocks > 0x7fffffffLL)
            return fail(DLP_ERR_NOT_IMPLEMENTED, "depthwise convolution too large for a single launch");
        if (bf16)
            DLP_LAUNCH_TIMED(ts, depthwise_direct_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, a, g.KH, g.sh);
        else
            DLP_LAUNCH_TIMED(ts, depthwise_direct_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, stream, a, g.KH, g.sh);
    }
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

} // namespace dlp
