// Operators of a network that sit away from the convolutions: Interpolation (nearest, nearest-exact, bilinear),
// Reduction over any subset of the dimensions (sum, sum of squares, sum of magnitudes, mean), and the forward
// pass of the three losses (MSELoss, NLLLoss, SoftmaxWithLoss).  All of them are bound by memory traffic:
// the kernels read every input element once, with the lanes of a wave on neighbouring addresses, and keep sums in fp32.
#include "dlp_internal.hpp"

#include <algorithm>
#include <cmath>
#include <cstring>

namespace dlp {
namespace {

// ---- Interpolation ----------------------------------------------------------------------------------------------

struct InterpArgs {
    int src_h, src_w, tgt_h, tgt_w;
    float scale_y, scale_x; // source steps per target step
    float offset;           // nearest: 0, nearest-exact: 0.5
    int align_corners;
    uint32_t th_magic, th_shift; // division by tgt_h
    int strips;                  // bilinear: strips of kInterpStripRows output rows per plane
    uint32_t st_magic, st_shift; // division by strips
    long long total_strips;      // planes * strips
    int col_bits;                // a block covers 2^col_bits columns and 256 >> col_bits rows
    long long rows;              // planes * tgt_h
};

// position of a nearest source sample: int((p + offset) * scale), clamped (src/kernels/interpolate_2d.cl:11-15)
__device__ __forceinline__ int nearest_pos(int p, float scale, int limit, float offset)
{
    const int s = (int)__fmul_rn(__fadd_rn((float)p, offset), scale);
    return min(s, limit - 1);
}
// position of a bilinear sample on the source axis (src/kernels/interpolate_2d.cl:104-109)
__device__ __forceinline__ float linear_pos(int p, float scale, int align_corners)
{
    if (align_corners)
        return __fmul_rn((float)p, scale);
    return fmaxf(__fsub_rn(__fmul_rn(scale, __fadd_rn((float)p, 0.5f)), 0.5f), 0.0f);
}

// sixteen bytes of T
template <class T>
struct Pack {
    static constexpr int N = 16 / sizeof(T);
    T v[N];
};
template <class T>
__device__ __forceinline__ Pack<T> load_pack(const T *p)
{
    Pack<T> r;
    __builtin_memcpy(&r, __builtin_assume_aligned(p, 16), 16);
    return r;
}
template <class T>
__device__ __forceinline__ void store_pack(T *p, const Pack<T> &v)
{
    __builtin_memcpy(__builtin_assume_aligned(p, 16), &v, 16);
}

// Nearest: one lane per VEC neighbouring outputs of a row (VEC > 1: one 16-byte store); a block covers a patch of 2^col_bits lanes by
// 256 >> col_bits rows, rows counted through all planes, so narrow images still fill the lanes.  The stores of a wave are contiguous
// runs of output rows; the loads go to the few input rows the patch maps to and are served by the caches.
template <class T, int VEC>
__global__ __launch_bounds__(256) void interpolate_nearest_kernel(InterpArgs a, const T *__restrict__ x, T *__restrict__ y)
{
    const int tid = threadIdx.x;
    const int cols = 1 << a.col_bits;
    const int c_first = (blockIdx.y * cols + (tid & (cols - 1))) * VEC;
    const long long row = (long long)blockIdx.x * (256 >> a.col_bits) + (tid >> a.col_bits);
    if (c_first >= a.tgt_w || row >= a.rows)
        return;
    const uint32_t plane = fast_div((uint32_t)row, a.th_magic, a.th_shift);
    const int r = (int)((uint32_t)row - plane * (uint32_t)a.tgt_h);
    const T *src = x + ((size_t)plane * a.src_h + nearest_pos(r, a.scale_y, a.src_h, a.offset)) * a.src_w;
    T out[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++)
        out[e] = src[nearest_pos(c_first + e, a.scale_x, a.src_w, a.offset)];
    T *dst = y + (size_t)row * a.tgt_w + c_first;
    if (VEC > 1)
        __builtin_memcpy(__builtin_assume_aligned(dst, 16), out, sizeof(out));
    else
        dst[0] = out[0];
}

// Bilinear: a lane owns one output column of a strip of kInterpStripRows output rows of one plane.  The column's two source columns
// and weights are fixed; going down the strip the lane keeps the horizontally blended values of the two source rows and loads a
// source row only when the strip moves onto it (going up by 2, five source rows serve eight output rows: 10 loads instead of 32).
// Order of the arithmetic: horizontal blend of each source row, then the vertical blend of the two results -- the reference's kernel
// adds four taps each weighted by a product (src/kernels/interpolate_2d.cl:111-140), so results agree to rounding, not bit for bit.
constexpr int kInterpStripRows = 8;
template <class T>
__global__ __launch_bounds__(256) void interpolate_bilinear_kernel(InterpArgs a, const T *__restrict__ x, T *__restrict__ y)
{
    const int tid = threadIdx.x;
    const int cols = 1 << a.col_bits;
    const int c = blockIdx.y * cols + (tid & (cols - 1));
    const long long strip = (long long)blockIdx.x * (256 >> a.col_bits) + (tid >> a.col_bits);
    if (c >= a.tgt_w || strip >= a.total_strips)
        return;
    const uint32_t plane = fast_div((uint32_t)strip, a.st_magic, a.st_shift);
    const int r_begin = (int)((uint32_t)strip - plane * (uint32_t)a.strips) * kInterpStripRows;
    const int r_end = min(r_begin + kInterpStripRows, a.tgt_h);
    const T *xp = x + (size_t)plane * a.src_h * a.src_w;
    T *yp = y + ((size_t)plane * a.tgt_h + r_begin) * a.tgt_w + c;
    const float cf = linear_pos(c, a.scale_x, a.align_corners);
    const int c0 = (int)cf;
    const int c1 = c0 + (c0 < a.src_w - 1 ? 1 : 0);
    const float wc1 = cf - (float)c0, wc0 = 1.0f - wc1;
    int have0 = -1, have1 = -1; // the source rows whose blends are in h0 / h1
    float h0 = 0.0f, h1 = 0.0f;
    for (int r = r_begin; r < r_end; r++, yp += a.tgt_w) {
        const float rf = linear_pos(r, a.scale_y, a.align_corners);
        const int r0 = (int)rf;
        const int r1 = r0 + (r0 < a.src_h - 1 ? 1 : 0);
        const float wr1 = rf - (float)r0, wr0 = 1.0f - wr1;
        if (r0 != have0) {
            if (r0 == have1)
                h0 = h1;
            else {
                const T *row = xp + (size_t)r0 * a.src_w;
                h0 = wc0 * to_float(row[c0]) + wc1 * to_float(row[c1]);
            }
            have0 = r0;
        }
        if (r1 != have1) {
            if (r1 == r0)
                h1 = h0;
            else {
                const T *row = xp + (size_t)r1 * a.src_w;
                h1 = wc0 * to_float(row[c0]) + wc1 * to_float(row[c1]);
            }
            have1 = r1;
        }
        store_plain(yp, wr0 * h0 + wr1 * h1);
    }
}

// ---- Reduction --------------------------------------------------------------------------------------------------

enum { kReduceSqDiff = 4 }; // internal: sum of (x - x2)^2, the body of MSELoss

// The tensor as runs of neighbouring dimensions that are all kept or all reduced, outermost first; unused runs have extent 1.
struct ReduceArgs {
    uint32_t kdim[3], rdim[3];      // extents of the kept / reduced runs
    long long kstride[3], rstride[3]; // element strides of the runs in x
    uint32_t r1_magic, r1_shift, r2_magic, r2_shift; // divisions by rdim[1], rdim[2]
    uint32_t k1_magic, k1_shift, k2_magic, k2_shift; // divisions by kdim[1], kdim[2]
    uint32_t R;                     // reduced elements per output
    uint32_t outputs;
    uint32_t splits, chunk;         // a reduction is cut into `splits` pieces of `chunk` elements (the last one shorter)
    int method;
    float coeff;
};

// what one element adds to the sum (selects, no branches: the loads of later iterations may move above it)
__device__ __forceinline__ float reduce_term(int method, float v)
{
    const float sq = v * v, mag = fabsf(v);
    return method == DLP_REDUCE_SUMSQ || method == kReduceSqDiff ? sq : (method == DLP_REDUCE_ABSSUM ? mag : v);
}
__device__ __forceinline__ size_t kept_offset(const ReduceArgs &a, uint32_t o)
{
    const uint32_t q2 = fast_div(o, a.k2_magic, a.k2_shift);
    const uint32_t i2 = o - q2 * a.kdim[2];
    const uint32_t i0 = fast_div(q2, a.k1_magic, a.k1_shift);
    const uint32_t i1 = q2 - i0 * a.kdim[1];
    return (size_t)(i0 * a.kstride[0] + i1 * a.kstride[1] + i2 * a.kstride[2]);
}
__device__ __forceinline__ size_t reduced_offset(const ReduceArgs &a, uint32_t j)
{
    const uint32_t q2 = fast_div(j, a.r2_magic, a.r2_shift);
    const uint32_t j2 = j - q2 * a.rdim[2];
    const uint32_t j0 = fast_div(q2, a.r1_magic, a.r1_shift);
    const uint32_t j1 = q2 - j0 * a.rdim[1];
    return (size_t)(j0 * a.rstride[0] + j1 * a.rstride[1] + j2 * a.rstride[2]);
}

__device__ __forceinline__ float wave_sum(float v)
{
    for (int off = 32; off > 0; off >>= 1)
        v += __shfl_xor(v, off);
    return v;
}

template <class T>
__device__ __forceinline__ void reduce_emit(const ReduceArgs &a, uint32_t o, uint32_t piece, float sum, T *y, float *partial)
{
    if (a.splits > 1)
        partial[(size_t)piece * a.outputs + o] = sum; // piece-major: neighbouring outputs next to each other
    else
        store_plain(y + o, sum * a.coeff);
}

// The innermost dimension is reduced: one group of LANES lanes per (output, piece) walks the reduced elements in memory order.
// ONE_RUN: the reduced elements of an output are contiguous, no index arithmetic.  TWO: the elements are x - x2.  WIDE: the innermost reduced run is a whole
// number of 16-byte packs and everything starts on a 16-byte address, so a lane loads a pack at a time.
template <class T, int LANES, bool ONE_RUN, bool WIDE, bool TWO>
__global__ __launch_bounds__(256) void reduce_inner_kernel(ReduceArgs a, const T *__restrict__ x, const T *__restrict__ x2, T *__restrict__ y,
                                                            float *__restrict__ partial)
{
    constexpr int VEC = WIDE ? 16 / sizeof(T) : 1;
    constexpr int GROUPS = 256 / LANES;
    __shared__ float sums[4];
    const uint32_t unit = blockIdx.x * GROUPS + threadIdx.x / LANES; // (output, piece)
    const int lane = threadIdx.x % LANES;
    const bool live = unit < a.outputs * a.splits; // whole groups of lanes are live or not: the shuffles below stay inside a group
    float sum = 0.0f;
    uint32_t o = 0, piece = 0;
    if (live) {
        o = unit / a.splits;
        piece = unit - o * a.splits;
        const uint32_t j_begin = piece * a.chunk, j_end = min(a.R, j_begin + a.chunk);
        const size_t base = kept_offset(a, o);
#pragma unroll 4
        for (uint32_t j = j_begin + lane * VEC; j < j_end; j += LANES * VEC) {
            const size_t off = base + (ONE_RUN ? (size_t)j : reduced_offset(a, j));
            if (WIDE) {
                const Pack<T> v = load_pack(x + off);
                Pack<T> w;
                if (TWO)
                    w = load_pack(x2 + off);
#pragma unroll
                for (int e = 0; e < VEC; e++)
                    sum += reduce_term(a.method, TWO ? to_float(v.v[e]) - to_float(w.v[e]) : to_float(v.v[e]));
            } else
                sum += reduce_term(a.method, TWO ? to_float(x[off]) - to_float(x2[off]) : to_float(x[off]));
        }
    }
    if (LANES <= 64) {
        for (int off = LANES / 2; off > 0; off >>= 1)
            sum += __shfl_xor(sum, off);
        if (live && lane == 0)
            reduce_emit(a, o, piece, sum, y, partial);
    } else { // one group is the whole block
        sum = wave_sum(sum);
        if (threadIdx.x % 64 == 0)
            sums[threadIdx.x / 64] = sum;
        __syncthreads();
        if (live && threadIdx.x == 0)
            reduce_emit(a, o, piece, sums[0] + sums[1] + sums[2] + sums[3], y, partial);
    }
}

// The innermost dimension is kept: a lane owns VEC neighbouring outputs (VEC > 1: a 16-byte pack; the innermost kept run is a whole
// number of packs then), a wave 64 * VEC of them, so for every reduced index a wave reads one contiguous stretch; the four waves of a
// block take every fourth reduced index and add up through LDS.
template <class T, int VEC>
__global__ __launch_bounds__(256) void reduce_outer_kernel(ReduceArgs a, const T *__restrict__ x, T *__restrict__ y, float *__restrict__ partial)
{
    __shared__ float sums[4][VEC][64];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const uint32_t o = (blockIdx.x * 64 + lane) * VEC;
    const uint32_t piece = blockIdx.y;
    const bool live = o < a.outputs;
    float sum[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++)
        sum[e] = 0.0f;
    if (live) {
        const uint32_t j_begin = piece * a.chunk, j_end = min(a.R, j_begin + a.chunk);
        const size_t base = kept_offset(a, o);
#pragma unroll 4
        for (uint32_t j = j_begin + wave; j < j_end; j += 4) {
            const size_t off = base + reduced_offset(a, j);
            if (VEC > 1) {
                const Pack<T> v = load_pack(x + off);
#pragma unroll
                for (int e = 0; e < VEC; e++)
                    sum[e] += reduce_term(a.method, to_float(v.v[e]));
            } else
                sum[0] += reduce_term(a.method, to_float(x[off]));
        }
    }
#pragma unroll
    for (int e = 0; e < VEC; e++)
        sums[wave][e][lane] = sum[e];
    __syncthreads();
    if (live && wave == 0) {
#pragma unroll
        for (int e = 0; e < VEC; e++)
            reduce_emit(a, o + e, piece, sums[0][e][lane] + sums[1][e][lane] + sums[2][e][lane] + sums[3][e][lane], y, partial);
    }
}

// adds up the pieces of every output (partial[piece][output]) in a fixed order: LANES lanes per output, a lane takes every
// LANES-th piece, four loads in flight.  LANES 1: a thread per output, for a handful of pieces of many outputs (neighbouring
// threads read neighbouring values); 64: a wave per output; 256: the block, for hundreds of pieces of a few outputs.
template <class T, int LANES>
__global__ __launch_bounds__(256) void reduce_finish_kernel(uint32_t outputs, uint32_t splits, float coeff, const float *__restrict__ partial,
                                                             T *__restrict__ y)
{
    __shared__ float sums[4];
    const uint32_t o = blockIdx.x * (256 / LANES) + threadIdx.x / LANES;
    const uint32_t lane = threadIdx.x % LANES;
    const bool live = o < outputs; // LANES > 1: the same for all lanes of a wave, and of the block when LANES is 256
    float sum = 0.0f;
    if (live) {
        const float *p = partial + o;
        const size_t step = (size_t)outputs * LANES;
        uint32_t s = lane;
        for (; s + 3 * LANES < splits; s += 4 * LANES) {
            const float *q = p + (size_t)s * outputs;
            sum += (q[0] + q[step]) + (q[2 * step] + q[3 * step]);
        }
        for (; s < splits; s += LANES)
            sum += p[(size_t)s * outputs];
    }
    if (LANES == 1) {
        if (live)
            store_plain(y + o, sum * coeff);
        return;
    }
    sum = wave_sum(sum);
    if (LANES == 64) {
        if (live && lane == 0)
            store_plain(y + o, sum * coeff);
    } else {
        if (threadIdx.x % 64 == 0)
            sums[threadIdx.x / 64] = sum;
        __syncthreads();
        if (live && threadIdx.x == 0)
            store_plain(y + o, (sums[0] + sums[1] + sums[2] + sums[3]) * coeff);
    }
}

// ---- losses -----------------------------------------------------------------------------------------------------

template <class T>
__global__ __launch_bounds__(256) void sqdiff_kernel(size_t n, const T *__restrict__ a, const T *__restrict__ b, T *__restrict__ y)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const float d = to_float(a[i]) - to_float(b[i]);
        store_plain(y + i, d * d);
    }
}

template <class L>
__device__ __forceinline__ long long label_of(const L *labels, int b)
{
    return (long long)labels[b];
}

// y[b] = -x[b][label[b]] (0 for a label outside the classes), or their sum times scale in y[0]; one block
template <class T, class L>
__global__ __launch_bounds__(256) void nll_loss_kernel(int batch, int classes, int reduce, float scale, const T *__restrict__ x,
                                                        const L *__restrict__ labels, T *__restrict__ y)
{
    __shared__ float sums[4];
    float sum = 0.0f;
    for (int b = threadIdx.x; b < batch; b += 256) {
        const long long index = label_of(labels, b);
        float v = 0.0f;
        if (index >= 0 && index < classes)
            v = -to_float(x[(size_t)b * classes + index]);
        if (reduce)
            sum += v;
        else
            store_plain(y + b, v * scale);
    }
    if (!reduce)
        return;
    sum = wave_sum(sum);
    if (threadIdx.x % 64 == 0)
        sums[threadIdx.x / 64] = sum;
    __syncthreads();
    if (threadIdx.x == 0)
        store_plain(y, (sums[0] + sums[1] + sums[2] + sums[3]) * scale);
}

// running maximum m and sum s of exp(v - m) over the values seen so far, one more value taken in
__device__ __forceinline__ void softmax_step(float &m, float &s, float v)
{
    if (v > m) {
        s = s * expf(m - v) + 1.0f;
        m = v;
    } else
        s += expf(v - m);
}

// loss of every row: -(x[label] - max - log(sum of exp(x - max))), 0 for a label outside the classes; one wave per row, one pass
// over it: every lane keeps the maximum of its share and the sum relative to that maximum, the lanes are merged at the end.
// WIDE: rows are whole numbers of 16-byte packs on 16-byte addresses.
template <class T, class L, bool WIDE>
__global__ __launch_bounds__(256) void softmax_loss_rows_kernel(int batch, int classes, const T *__restrict__ x, const L *__restrict__ labels,
                                                                 float *__restrict__ row_loss)
{
    constexpr int VEC = WIDE ? 16 / sizeof(T) : 1;
    const int b = blockIdx.x * 4 + threadIdx.x / 64;
    const int lane = threadIdx.x % 64;
    if (b >= batch)
        return;
    const T *row = x + (size_t)b * classes;
    float m = -INFINITY, s = 0.0f;
#pragma unroll 2
    for (int c = lane * VEC; c < classes; c += 64 * VEC) {
        if (WIDE) {
            const Pack<T> v = load_pack(row + c);
            float top = to_float(v.v[0]);
#pragma unroll
            for (int e = 1; e < VEC; e++)
                top = fmaxf(top, to_float(v.v[e]));
            if (top > m) { // one rescale per pack
                s *= expf(m - top);
                m = top;
            }
#pragma unroll
            for (int e = 0; e < VEC; e++)
                s += expf(to_float(v.v[e]) - m);
        } else
            softmax_step(m, s, to_float(row[c]));
    }
    float top = m;
    for (int off = 32; off > 0; off >>= 1)
        top = fmaxf(top, __shfl_xor(top, off));
    s = m == -INFINITY ? 0.0f : s * expf(m - top); // a lane that saw nothing adds nothing
    s = wave_sum(s);
    if (lane == 0) {
        const long long index = label_of(labels, b);
        row_loss[b] = index >= 0 && index < classes ? -(to_float(row[index]) - top - logf(s)) : 0.0f;
    }
}

// y[0] = scale * sum of n floats, stored as T; one block
template <class T>
__global__ __launch_bounds__(256) void reduce_rows_kernel(int n, float scale, const float *__restrict__ v, T *__restrict__ y)
{
    __shared__ float sums[4];
    float sum = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256)
        sum += v[i];
    sum = wave_sum(sum);
    if (threadIdx.x % 64 == 0)
        sums[threadIdx.x / 64] = sum;
    __syncthreads();
    if (threadIdx.x == 0)
        store_plain(y, (sums[0] + sums[1] + sums[2] + sums[3]) * scale);
}

} // namespace

// x viewed as kept / reduced runs; fails when the tensor needs more than three runs of either kind
static int plan_reduce(int rank, const int *shape, const int *reduce, ReduceArgs &a, bool &inner_reduced)
{
    uint32_t dims[8];
    long long strides[8];
    int kinds[8];
    int nd = 0;
    long long stride = 1;
    for (int j = rank - 1; j >= 0; j--) { // innermost first
        const int d = shape[j];
        if (d != 1) {
            const int kind = reduce[j] ? 1 : 0;
            if (nd > 0 && kinds[nd - 1] == kind)
                dims[nd - 1] *= (uint32_t)d;
            else {
                dims[nd] = (uint32_t)d;
                strides[nd] = stride;
                kinds[nd] = kind;
                nd++;
            }
        }
        stride *= d;
    }
    for (int i = 0; i < 3; i++) {
        a.kdim[i] = a.rdim[i] = 1;
        a.kstride[i] = a.rstride[i] = 0;
    }
    int nk = 0, nr = 0;
    for (int i = 0; i < nd; i++) { // innermost first: fill the slots from the back
        if (kinds[i]) {
            if (nr == 3)
                return fail(DLP_ERR_NOT_IMPLEMENTED, "reduction: more than three separate groups of reduced dimensions");
            a.rdim[2 - nr] = dims[i];
            a.rstride[2 - nr] = strides[i];
            nr++;
        } else {
            if (nk == 3)
                return fail(DLP_ERR_NOT_IMPLEMENTED, "reduction: more than three separate groups of kept dimensions");
            a.kdim[2 - nk] = dims[i];
            a.kstride[2 - nk] = strides[i];
            nk++;
        }
    }
    inner_reduced = nd == 0 || kinds[0] == 1;
    make_magic(a.rdim[1], a.r1_magic, a.r1_shift);
    make_magic(a.rdim[2], a.r2_magic, a.r2_shift);
    make_magic(a.kdim[1], a.k1_magic, a.k1_shift);
    make_magic(a.kdim[2], a.k2_magic, a.k2_shift);
    return DLP_OK;
}

// How a reduction is cut: enough pieces to give every compute unit eight blocks.  Innermost dimension reduced: a block per piece,
// pieces of at least 8192 elements.  Innermost dimension kept: a block per 64 * outer_vec outputs and piece, at least 64 reduced
// indices per piece (16 per wave).
static void plan_splits(ReduceArgs &a, bool inner_reduced, int outer_vec)
{
    const long long want_blocks = 8ll * dlp_cu_count();
    long long splits = 1;
    if (inner_reduced) {
        if ((long long)a.outputs < want_blocks)
            splits = std::min<long long>((want_blocks + a.outputs - 1) / a.outputs, a.R / 8192);
    } else {
        const long long blocks = ((long long)a.outputs + 64 * outer_vec - 1) / (64 * outer_vec);
        if (blocks < want_blocks)
            splits = std::min<long long>((want_blocks + blocks - 1) / blocks, a.R / 64);
    }
    splits = std::max<long long>(1, std::min<long long>(splits, 1024));
    uint32_t chunk = (uint32_t)((a.R + splits - 1) / splits);
    chunk = (chunk + 63) / 64 * 64; // keeps the pieces of a contiguous run on 16-byte addresses
    a.chunk = chunk;
    a.splits = (uint32_t)((a.R + chunk - 1) / chunk);
    if (a.splits <= 1) {
        a.splits = 1;
        a.chunk = a.R;
    }
}

struct ReduceCall {
    ReduceArgs a;
    bool inner_reduced;
    size_t workspace;
};

static int prepare_reduce(int dtype, int method, float coeff, int rank, const int *shape, const int *reduce, ReduceCall &c, size_t &total)
{
    if (dtype != DLP_FLOAT && dtype != DLP_BFLOAT16)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "reduction: float_data and bfloat16_data are implemented");
    DLP_REQUIRE(rank >= 1 && rank <= 8 && shape != nullptr && reduce != nullptr, "rank 1 to 8, the shape and the reduced dimensions are needed");
    size_t outputs = 1, R = 1;
    for (int j = 0; j < rank; j++) {
        DLP_REQUIRE(shape[j] >= 0, "negative extent");
        if (reduce[j])
            R *= (size_t)shape[j];
        else
            outputs *= (size_t)shape[j];
    }
    total = outputs * R;
    DLP_REQUIRE(outputs < (1ull << 31) && R < (1ull << 31), "reduction: fewer than 2^31 outputs and reduced elements per output");
    c.a.R = (uint32_t)R;
    c.a.outputs = (uint32_t)outputs;
    c.workspace = 0;
    if (total == 0) // an extent of 0: nothing to plan (and no divisors to prepare)
        return DLP_OK;
    int st = plan_reduce(rank, shape, reduce, c.a, c.inner_reduced);
    if (st != DLP_OK)
        return st;
    c.a.R = (uint32_t)R;
    c.a.outputs = (uint32_t)outputs;
    c.a.method = method;
    c.a.coeff = coeff;
    const int pack = int(16 / dtype_size(dtype));
    plan_splits(c.a, c.inner_reduced, c.a.kdim[2] % pack == 0 ? pack : 1);
    c.workspace = c.a.splits > 1 ? (size_t)c.a.outputs * c.a.splits * sizeof(float) : 0;
    return DLP_OK;
}

template <class T>
static int launch_reduce(const ReduceCall &c, const void *x, const void *x2, void *y, void *workspace, hipStream_t st)
{
    const ReduceArgs &a = c.a;
    float *partial = (float *)workspace;
    const T *xp = (const T *)x, *xp2 = (const T *)x2;
    T *yp = (T *)y;
    constexpr int PACK = 16 / sizeof(T);
    const bool aligned = (uintptr_t)x % 16 == 0 && (uintptr_t)x2 % 16 == 0;
    TimingScope ts("reduction", st);
    if (c.inner_reduced) {
        const bool one_run = a.rdim[0] == 1 && a.rdim[1] == 1;
        DLP_REQUIRE(x2 == nullptr || one_run, "a difference of two tensors is reduced as a whole");
        // 16-byte loads: the innermost reduced run and the pieces are whole packs (every other stride is a multiple of that run)
        const bool wide = aligned && a.rdim[2] % PACK == 0 && a.chunk % PACK == 0;
        const uint32_t units = a.outputs * a.splits;
        const uint32_t steps = std::min(a.R, a.chunk) / (wide ? PACK : 1); // loads per (output, piece)
        // lanes per (output, piece): the whole block for long runs, a wave, or a quarter of one for short ones
        const int lanes = steps >= 1024 ? 256 : (steps > 64 ? 64 : 16);
        const unsigned blocks = (unsigned)((units + (256 / lanes) - 1) / (256 / lanes));
#define DLP_REDUCE_INNER2(L, ONE, WIDE, TWO) \
    hipLaunchKernelGGL((reduce_inner_kernel<T, L, ONE, WIDE, TWO>), dim3(blocks), dim3(256), 0, st, a, xp, xp2, yp, partial)
#define DLP_REDUCE_INNER(L)                           \
    do {                                              \
        if (xp2 != nullptr && wide)                   \
            DLP_REDUCE_INNER2(L, true, true, true);   \
        else if (xp2 != nullptr)                      \
            DLP_REDUCE_INNER2(L, true, false, true);  \
        else if (one_run && wide)                     \
            DLP_REDUCE_INNER2(L, true, true, false);  \
        else if (one_run)                             \
            DLP_REDUCE_INNER2(L, true, false, false); \
        else if (wide)                                \
            DLP_REDUCE_INNER2(L, false, true, false); \
        else                                          \
            DLP_REDUCE_INNER2(L, false, false, false);\
    } while (0)
        if (lanes == 256)
            DLP_REDUCE_INNER(256);
        else if (lanes == 64)
            DLP_REDUCE_INNER(64);
        else
            DLP_REDUCE_INNER(16);
#undef DLP_REDUCE_INNER
#undef DLP_REDUCE_INNER2
    } else {
        DLP_REQUIRE(a.splits <= 65535 && x2 == nullptr, "reduction: too many pieces, or a difference along an outer dimension");
        if (aligned && a.kdim[2] % PACK == 0)
            hipLaunchKernelGGL((reduce_outer_kernel<T, PACK>), dim3((a.outputs + 64 * PACK - 1) / (64 * PACK), a.splits), dim3(256), 0, st, a, xp, yp, partial);
        else
            hipLaunchKernelGGL((reduce_outer_kernel<T, 1>), dim3((a.outputs + 63) / 64, a.splits), dim3(256), 0, st, a, xp, yp, partial);
    }
    DLP_HIP_TRY(hipGetLastError());
    if (a.splits > 1) {
        if (a.splits >= 256)
            hipLaunchKernelGGL((reduce_finish_kernel<T, 256>), dim3(a.outputs), dim3(256), 0, st, a.outputs, a.splits, a.coeff, partial, yp);
        else if (a.splits > 8)
            hipLaunchKernelGGL((reduce_finish_kernel<T, 64>), dim3((a.outputs + 3) / 4), dim3(256), 0, st, a.outputs, a.splits, a.coeff, partial, yp);
        else
            hipLaunchKernelGGL((reduce_finish_kernel<T, 1>), dim3((a.outputs + 255) / 256), dim3(256), 0, st, a.outputs, a.splits, a.coeff, partial, yp);
        DLP_HIP_TRY(hipGetLastError());
    }
    return DLP_OK;
}

static int run_reduce(int dtype, const ReduceCall &c, const void *x, const void *x2, void *y, void *workspace, size_t workspace_bytes,
                      void *stream)
{
    DLP_REQUIRE(x != nullptr && y != nullptr, "null tensor pointer");
    DLP_REQUIRE(c.workspace == 0 || (workspace != nullptr && workspace_bytes >= c.workspace), "the workspace is smaller than the size the workspace query gives");
    if (dtype == DLP_BFLOAT16)
        return launch_reduce<bf16_t>(c, x, x2, y, workspace, (hipStream_t)stream);
    return launch_reduce<float>(c, x, x2, y, workspace, (hipStream_t)stream);
}

} // namespace dlp

using namespace dlp;

extern "C" {

int dlp_interpolate2d_fwd_enqueue(int dtype, int method, int align_corners, double scale_y, double scale_x, int planes, int src_h, int src_w,
                                  int tgt_h, int tgt_w, const void *x, void *y, void *stream)
{
    if (dtype != DLP_FLOAT && dtype != DLP_BFLOAT16)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "interpolation: float_data and bfloat16_data are implemented");
    DLP_REQUIRE(method >= DLP_INTERPOLATE_NEAREST && method <= DLP_INTERPOLATE_BILINEAR, "unknown interpolation method");
    DLP_REQUIRE(method == DLP_INTERPOLATE_BILINEAR || !align_corners, "align_corners goes with bilinear only");
    DLP_REQUIRE(planes >= 0 && src_h > 0 && src_w > 0 && tgt_h > 0 && tgt_w > 0, "shape");
    DLP_REQUIRE((scale_y <= 0) == (scale_x <= 0), "both scales or neither");
    if (method == DLP_INTERPOLATE_BILINEAR && align_corners) {
        scale_y = tgt_h > 1 ? double(src_h - 1) / (tgt_h - 1) : 0.0;
        scale_x = tgt_w > 1 ? double(src_w - 1) / (tgt_w - 1) : 0.0;
    } else if (scale_y <= 0) {
        scale_y = double(src_h) / tgt_h;
        scale_x = double(src_w) / tgt_w;
    } else {
        DLP_REQUIRE(tgt_h == int(src_h * scale_y) && tgt_w == int(src_w * scale_x), "the output size is int(input size * scale)");
        scale_y = 1.0 / scale_y;
        scale_x = 1.0 / scale_x;
    }
    if (planes == 0)
        return DLP_OK;
    DLP_REQUIRE(x != nullptr && y != nullptr, "null tensor pointer");
    InterpArgs a;
    a.src_h = src_h;
    a.src_w = src_w;
    a.tgt_h = tgt_h;
    a.tgt_w = tgt_w;
    a.scale_y = float(scale_y);
    a.scale_x = float(scale_x);
    a.offset = method == DLP_INTERPOLATE_NEAREST_EXACT ? 0.5f : 0.0f;
    a.align_corners = align_corners ? 1 : 0;
    a.rows = (long long)planes * tgt_h;
    DLP_REQUIRE(a.rows < (1ll << 31), "interpolation: fewer than 2^31 output rows");
    make_magic((uint32_t)tgt_h, a.th_magic, a.th_shift);
    const int pack = int(16 / dtype_size(dtype));
    // outputs per lane.  nearest: a pack (one 16-byte store) where the rows allow it.  bilinear: one column; the time goes to the
    // loads, which a lane with several columns only spreads over more cache lines (measured: no gain going up, 2.4 times slower
    // going down), so its lanes go down a strip of rows instead and keep what they loaded
    const int vec = method != DLP_INTERPOLATE_BILINEAR && tgt_w % pack == 0 && (uintptr_t)y % 16 == 0 ? pack : 1;
    const int lanes_w = tgt_w / vec;
    a.col_bits = 0;
    while ((1 << a.col_bits) < lanes_w && a.col_bits < 8)
        a.col_bits++;
    const int cols = 1 << a.col_bits, rows_per_block = 256 >> a.col_bits;
    const long long row_blocks = (a.rows + rows_per_block - 1) / rows_per_block;
    const dim3 grid((unsigned)row_blocks, (unsigned)((lanes_w + cols - 1) / cols)), block(256);
    DLP_REQUIRE(grid.y <= 65535, "interpolation: the output is too wide");
    a.strips = (tgt_h + kInterpStripRows - 1) / kInterpStripRows;
    a.total_strips = (long long)planes * a.strips;
    make_magic((uint32_t)a.strips, a.st_magic, a.st_shift);
    const dim3 strip_grid((unsigned)((a.total_strips + rows_per_block - 1) / rows_per_block), grid.y);
    hipStream_t st = (hipStream_t)stream;
    TimingScope ts("interpolation", st);
    const bool bilinear = method == DLP_INTERPOLATE_BILINEAR;
#define DLP_INTERP(T, V)                                                                                              \
    do {                                                                                                              \
        if (bilinear)                                                                                                 \
            hipLaunchKernelGGL(interpolate_bilinear_kernel<T>, strip_grid, block, 0, st, a, (const T *)x, (T *)y);    \
        else                                                                                                          \
            hipLaunchKernelGGL((interpolate_nearest_kernel<T, V>), grid, block, 0, st, a, (const T *)x, (T *)y);        \
    } while (0)
    if (dtype == DLP_BFLOAT16) {
        if (vec > 1)
            DLP_INTERP(bf16_t, 8);
        else
            DLP_INTERP(bf16_t, 1);
    } else {
        if (vec > 1)
            DLP_INTERP(float, 4);
        else
            DLP_INTERP(float, 1);
    }
#undef DLP_INTERP
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

static int reduce_coeff(int method, float output_scale, const ReduceCall &c, float &coeff)
{
    DLP_REQUIRE(method >= DLP_REDUCE_SUM && method <= DLP_REDUCE_MEAN, "unknown reduction method");
    // mean: output_scale * outputs / elements, as Reduction::get_coeff (src/ops/reduction.cpp:323-329)
    coeff = method == DLP_REDUCE_MEAN ? output_scale * float(c.a.outputs) / float((size_t)c.a.outputs * c.a.R) : output_scale;
    return DLP_OK;
}

int dlp_reduce_fwd_workspace(int dtype, int method, int rank, const int *shape, const int *reduce, size_t *bytes)
{
    DLP_REQUIRE(bytes != nullptr, "null result pointer");
    DLP_REQUIRE(method >= DLP_REDUCE_SUM && method <= DLP_REDUCE_MEAN, "unknown reduction method");
    ReduceCall c;
    size_t total = 0;
    int st = prepare_reduce(dtype, method, 1.0f, rank, shape, reduce, c, total);
    if (st != DLP_OK)
        return st;
    *bytes = total == 0 ? 0 : c.workspace;
    return DLP_OK;
}

int dlp_reduce_fwd_enqueue(int dtype, int method, float output_scale, int rank, const int *shape, const int *reduce, const void *x, void *y,
                           void *workspace, size_t workspace_bytes, void *stream)
{
    DLP_REQUIRE(method >= DLP_REDUCE_SUM && method <= DLP_REDUCE_MEAN, "unknown reduction method");
    ReduceCall c;
    size_t total = 0;
    int st = prepare_reduce(dtype, method, 1.0f, rank, shape, reduce, c, total);
    if (st != DLP_OK)
        return st;
    if (c.a.outputs == 0)
        return DLP_OK;
    DLP_REQUIRE(total > 0, "reduction over no elements");
    st = reduce_coeff(method, output_scale, c, c.a.coeff);
    if (st != DLP_OK)
        return st;
    return run_reduce(dtype, c, x, nullptr, y, workspace, workspace_bytes, stream);
}

int dlp_mse_loss_fwd_workspace(int dtype, int reduce, size_t n, size_t *bytes)
{
    DLP_REQUIRE(bytes != nullptr, "null result pointer");
    DLP_REQUIRE(reduce >= DLP_LOSS_REDUCE_NONE && reduce <= DLP_LOSS_REDUCE_MEAN, "unknown loss reduction");
    *bytes = 0;
    if (reduce == DLP_LOSS_REDUCE_NONE || n == 0)
        return DLP_OK;
    DLP_REQUIRE(n < (1ull << 31), "loss over fewer than 2^31 elements");
    const int shape[1] = {(int)n}, dims[1] = {1};
    ReduceCall c;
    size_t total = 0;
    int st = prepare_reduce(dtype, kReduceSqDiff, 1.0f, 1, shape, dims, c, total);
    if (st != DLP_OK)
        return st;
    *bytes = c.workspace;
    return DLP_OK;
}

int dlp_mse_loss_fwd_enqueue(int dtype, int reduce, size_t n, const void *a, const void *b, void *y, void *workspace, size_t workspace_bytes,
                             void *stream)
{
    if (dtype != DLP_FLOAT && dtype != DLP_BFLOAT16)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "MSE loss: float_data and bfloat16_data are implemented");
    DLP_REQUIRE(reduce >= DLP_LOSS_REDUCE_NONE && reduce <= DLP_LOSS_REDUCE_MEAN, "unknown loss reduction");
    DLP_REQUIRE(n > 0 || reduce == DLP_LOSS_REDUCE_NONE, "loss over no elements");
    if (n == 0)
        return DLP_OK;
    DLP_REQUIRE(a != nullptr && b != nullptr && y != nullptr, "null tensor pointer");
    hipStream_t st = (hipStream_t)stream;
    if (reduce == DLP_LOSS_REDUCE_NONE) {
        const unsigned blocks = (unsigned)std::min<size_t>((n + 255) / 256, 256 * 32);
        TimingScope ts("mse_loss", st);
        if (dtype == DLP_BFLOAT16)
            hipLaunchKernelGGL(sqdiff_kernel<bf16_t>, dim3(blocks), dim3(256), 0, st, n, (const bf16_t *)a, (const bf16_t *)b, (bf16_t *)y);
        else
            hipLaunchKernelGGL(sqdiff_kernel<float>, dim3(blocks), dim3(256), 0, st, n, (const float *)a, (const float *)b, (float *)y);
        DLP_HIP_TRY(hipGetLastError());
        return DLP_OK;
    }
    DLP_REQUIRE(n < (1ull << 31), "loss over fewer than 2^31 elements");
    const int shape[1] = {(int)n}, dims[1] = {1};
    ReduceCall c;
    size_t total = 0;
    int rc = prepare_reduce(dtype, kReduceSqDiff, reduce == DLP_LOSS_REDUCE_MEAN ? 1.0f / float(n) : 1.0f, 1, shape, dims, c, total);
    if (rc != DLP_OK)
        return rc;
    return run_reduce(dtype, c, a, b, y, workspace, workspace_bytes, stream);
}

int dlp_nll_loss_fwd_enqueue(int dtype, int label_dtype, int reduce, int batch, int classes, const void *x, const void *labels, void *y,
                             void *stream)
{
    if (dtype != DLP_FLOAT && dtype != DLP_BFLOAT16)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "NLL loss: float_data and bfloat16_data are implemented");
    if (label_dtype != DLP_FLOAT && label_dtype != DLP_INT32)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "NLLLoss label must be either int or float");
    DLP_REQUIRE(reduce >= DLP_LOSS_REDUCE_NONE && reduce <= DLP_LOSS_REDUCE_MEAN, "unknown loss reduction");
    DLP_REQUIRE(batch > 0 && classes > 0, "shape");
    DLP_REQUIRE(x != nullptr && labels != nullptr && y != nullptr, "null tensor pointer");
    const float scale = reduce == DLP_LOSS_REDUCE_MEAN ? 1.0f / float(batch) : 1.0f;
    const int red = reduce != DLP_LOSS_REDUCE_NONE;
    hipStream_t st = (hipStream_t)stream;
    TimingScope ts("nll_loss", st);
    if (dtype == DLP_BFLOAT16) {
        if (label_dtype == DLP_INT32)
            hipLaunchKernelGGL((nll_loss_kernel<bf16_t, int>), dim3(1), dim3(256), 0, st, batch, classes, red, scale, (const bf16_t *)x, (const int *)labels, (bf16_t *)y);
        else
            hipLaunchKernelGGL((nll_loss_kernel<bf16_t, float>), dim3(1), dim3(256), 0, st, batch, classes, red, scale, (const bf16_t *)x, (const float *)labels, (bf16_t *)y);
    } else {
        if (label_dtype == DLP_INT32)
            hipLaunchKernelGGL((nll_loss_kernel<float, int>), dim3(1), dim3(256), 0, st, batch, classes, red, scale, (const float *)x, (const int *)labels, (float *)y);
        else
            hipLaunchKernelGGL((nll_loss_kernel<float, float>), dim3(1), dim3(256), 0, st, batch, classes, red, scale, (const float *)x, (const float *)labels, (float *)y);
    }
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

int dlp_softmax_loss_fwd_workspace(int batch, size_t *bytes)
{
    DLP_REQUIRE(bytes != nullptr && batch >= 0, "null result pointer or negative batch");
    *bytes = (size_t)batch * sizeof(float);
    return DLP_OK;
}

int dlp_softmax_loss_fwd_enqueue(int dtype, int label_dtype, int batch, int classes, const void *x, const void *labels, void *y,
                                 void *workspace, size_t workspace_bytes, void *stream)
{
    if (dtype != DLP_FLOAT && dtype != DLP_BFLOAT16)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "softmax loss: float_data and bfloat16_data are implemented");
    if (label_dtype != DLP_FLOAT && label_dtype != DLP_INT32)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "the labels of SoftmaxWithLoss must be either int or float");
    DLP_REQUIRE(batch > 0 && classes > 0, "shape");
    DLP_REQUIRE(x != nullptr && labels != nullptr && y != nullptr, "null tensor pointer");
    DLP_REQUIRE(workspace != nullptr && workspace_bytes >= (size_t)batch * sizeof(float), "the workspace holds one float per row");
    hipStream_t st = (hipStream_t)stream;
    float *rows = (float *)workspace;
    const dim3 grid((unsigned)((batch + 3) / 4)), block(256);
    {
        TimingScope ts("softmax_loss", st);
        const bool wide = (uintptr_t)x % 16 == 0 && classes % int(16 / dtype_size(dtype)) == 0;
#define DLP_SOFTMAX_LOSS(T, L)                                                                                                                 \
    do {                                                                                                                                       \
        if (wide)                                                                                                                              \
            hipLaunchKernelGGL((softmax_loss_rows_kernel<T, L, true>), grid, block, 0, st, batch, classes, (const T *)x, (const L *)labels, rows); \
        else                                                                                                                                   \
            hipLaunchKernelGGL((softmax_loss_rows_kernel<T, L, false>), grid, block, 0, st, batch, classes, (const T *)x, (const L *)labels, rows); \
    } while (0)
        if (dtype == DLP_BFLOAT16) {
            if (label_dtype == DLP_INT32)
                DLP_SOFTMAX_LOSS(bf16_t, int);
            else
                DLP_SOFTMAX_LOSS(bf16_t, float);
        } else {
            if (label_dtype == DLP_INT32)
                DLP_SOFTMAX_LOSS(float, int);
            else
                DLP_SOFTMAX_LOSS(float, float);
        }
#undef DLP_SOFTMAX_LOSS
        DLP_HIP_TRY(hipGetLastError());
    }
    // the mean over the rows: one block adds up the fp32 row losses in a fixed order and stores the result as `dtype`
    TimingScope ts("softmax_loss", st);
    if (dtype == DLP_BFLOAT16)
        hipLaunchKernelGGL((reduce_rows_kernel<bf16_t>), dim3(1), dim3(256), 0, st, batch, 1.0f / float(batch), (const float *)rows, (bf16_t *)y);
    else
        hipLaunchKernelGGL((reduce_rows_kernel<float>), dim3(1), dim3(256), 0, st, batch, 1.0f / float(batch), (const float *)rows, (float *)y);
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

} // extern "C"
