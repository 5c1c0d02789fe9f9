// Glue operators of the ResNet / MobileNet graphs around the convolution path:
// 2-D pooling, global pooling and element-wise combination of two tensors.
// All three are HBM-bound streaming kernels (no LDS tiling, no matrix cores).
//
// They replace, for forward inference only:
//   core::Pooling2DForward (include/dlprim/core/pool.hpp:29-70, src/core/pool.cpp) with the
//     arithmetic of Pooling2D::forward_cpu (src/ops/pooling.cpp:281-328, functors :116-145),
//   the global pooling variants (GlobalPooling::forward_cpu, src/ops/pooling.cpp:427-452),
//   Elementwise::forward for equal shapes (src/ops/elementwise.cpp:517-559).
#include "dlp_internal.hpp"

#include <new>

namespace dlp {
namespace {

struct PoolArgs {
    const void *x; // storage type T
    void *y;
    int planes, H, W, OH, OW;
    int kh, kw, ph, pw, sh, sw;
    int mode; // 0 max, 1 avg
    int count_include_pad;
};

// one output element per thread; consecutive threads on consecutive output columns
template <class T>
__global__ __launch_bounds__(256) void pool2d_kernel(PoolArgs a)
{
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long total = (long long)a.planes * a.OH * a.OW;
    if (idx >= total)
        return;
    const int oc = (int)(idx % a.OW);
    const long long t = idx / a.OW;
    const int orow = (int)(t % a.OH);
    const long long plane = t / a.OH;
    const T *src = (const T *)a.x + plane * a.H * a.W;
    int row0 = orow * a.sh - a.ph, col0 = oc * a.sw - a.pw;
    int row1 = row0 + a.kh, col1 = col0 + a.kw;
    const int dr_pad = min(row1, a.H + a.ph) - max(-a.ph, row0);
    const int dc_pad = min(col1, a.W + a.pw) - max(-a.pw, col0);
    row0 = max(row0, 0);
    col0 = max(col0, 0);
    row1 = min(row1, a.H);
    col1 = min(col1, a.W);
    float val = a.mode == 0 ? -3.402823466e+38f : 0.0f;
    for (int r = row0; r < row1; r++)
        for (int c = col0; c < col1; c++) {
            const float v = to_float(src[(size_t)r * a.W + c]);
            val = a.mode == 0 ? fmaxf(val, v) : val + v;
        }
    if (a.mode != 0) {
        const int dr = row1 - row0, dc = col1 - col0;
        if (dr == a.kh && dc == a.kw)
            val = val * (1.0f / (a.kh * a.kw));
        else if (a.count_include_pad)
            val = val / (float)(dr_pad * dc_pad);
        else
            val = val * (1.0f / (dr * dc));
    }
    store_plain((T *)a.y + idx, val);
}

// Max pooling 3x3, stride 2, padding 1 (the ResNet stem): lanes own output columns of a strip of
// kMaxStrip output rows, as in the stride-2 depthwise kernel.  A lane loads the two input columns it
// owns (2*ox, 2*ox + 1: one 8- or 4-byte load when the row is aligned for it) of every input row of
// the strip before it consumes any, takes column 2*ox - 1 from the lane to its left (lane 0 of a
// wavefront is a halo lane that stores nothing; adjacent wavefronts overlap by it), and reuses the
// row shared by consecutive output rows from registers: every input element is read once (plus
// one halo row per strip) instead of 2.25 times.  Padding is ignored by max, as in the reference.
constexpr int kMaxStrip = 7;

template <class T>
__global__ __launch_bounds__(256) void maxpool3x3s2p1_kernel(PoolArgs a, int nstrips, long long total_cols, int pairs)
{
    constexpr int NIN = 2 * kMaxStrip + 1;
    constexpr float kLowest = -3.402823466e+38f;
    const int lane = threadIdx.x & 63;
    const long long wave = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const long long f = wave * 63 + lane - 1; // flat (plane, strip, ox) index
    const bool in_range = f >= 0 && f < total_cols;
    const long long ps = in_range ? f / a.OW : 0;
    const int ox = in_range ? (int)(f - ps * a.OW) : 0;
    const long long plane = ps / nstrips;
    const int strip = (int)(ps - plane * nstrips);
    const int oy0 = strip * kMaxStrip;
    const T *xp = (const T *)a.x + plane * a.H * a.W;
    const int x0 = 2 * ox;
    const bool v0 = in_range && x0 < a.W, v1 = in_range && x0 + 1 < a.W;
    const bool has_left = ox > 0;

    float c0[NIN], c1[NIN];
    const int iy0 = 2 * oy0 - 1;
#pragma unroll
    for (int r = 0; r < NIN; r++) {
        const int yy = iy0 + r;
        const bool vy = yy >= 0 && yy < a.H;
        const T *p = xp + (size_t)(vy ? yy : 0) * a.W + x0;
        c0[r] = kLowest;
        c1[r] = kLowest;
        if (pairs) { // even W, aligned base: both columns exist and sit in one aligned pair
            if (vy && v0) {
                if constexpr (sizeof(T) == 4) {
                    const float2 v = *(const float2 *)p;
                    c0[r] = v.x;
                    c1[r] = v.y;
                } else {
                    const uint32_t v = *(const uint32_t *)p;
                    c0[r] = __builtin_bit_cast(float, v << 16);
                    c1[r] = __builtin_bit_cast(float, v & 0xffff0000u);
                }
            }
        } else {
            if (vy && v0)
                c0[r] = to_float(p[0]);
            if (vy && v1)
                c1[r] = to_float(p[1]);
        }
    }
    float m[NIN]; // maximum over the row's three window columns
#pragma unroll
    for (int r = 0; r < NIN; r++) {
        const float l = __shfl_up(c1[r], 1); // the left lane's odd column = 2*ox - 1
        m[r] = fmaxf(fmaxf(has_left ? l : kLowest, c0[r]), c1[r]);
    }
    if (!in_range || lane == 0)
        return;
    T *yp = (T *)a.y + plane * a.OH * a.OW + ox;
#pragma unroll
    for (int j = 0; j < kMaxStrip; j++) {
        const int oy = oy0 + j;
        if (oy < a.OH)
            store_plain(yp + (size_t)oy * a.OW, fmaxf(fmaxf(m[2 * j], m[2 * j + 1]), m[2 * j + 2]));
    }
}

// The same pooling for rows of whole groups of eight input columns (W % 8 == 0, OW == W / 2, 16-byte aligned tensors): a lane owns
// FOUR output columns, loads their eight input columns of a row with one 16-byte load (two for float) and stores four results at
// once -- a quarter of the memory instructions per byte, which is what bounds the kernel above on 2-byte elements (the texture
// path takes four lanes per clock whatever the width of the access).
template <class T>
__global__ __launch_bounds__(256) void maxpool3x3s2p1_wide_kernel(PoolArgs a, int nstrips, long long total_groups, int groups_per_row)
{
    constexpr int NIN = 2 * kMaxStrip + 1;
    constexpr float kLowest = -3.402823466e+38f;
    typedef uint32_t pool_u32x4 __attribute__((ext_vector_type(4)));
    typedef uint32_t pool_u32x2 __attribute__((ext_vector_type(2)));
    typedef float pool_f32x4 __attribute__((ext_vector_type(4)));
    const int lane = threadIdx.x & 63;
    const long long wave = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const long long f = wave * 63 + lane - 1; // flat (plane, strip, group of four output columns) index
    const bool in_range = f >= 0 && f < total_groups;
    const long long ps = in_range ? f / groups_per_row : 0;
    const int gx = in_range ? (int)(f - ps * groups_per_row) : 0;
    const long long plane = ps / nstrips;
    const int strip = (int)(ps - plane * nstrips);
    const int oy0 = strip * kMaxStrip;
    const T *xp = (const T *)a.x + plane * a.H * a.W + 8 * gx;
    const bool has_left = gx > 0;

    float m[NIN][4]; // maxima over the three window columns of the four outputs, per input row
    const int iy0 = 2 * oy0 - 1;
#pragma unroll
    for (int r = 0; r < NIN; r++) {
        const int yy = iy0 + r;
        const bool vy = in_range && yy >= 0 && yy < a.H;
        const T *p = xp + (size_t)(vy ? yy : 0) * a.W;
        float c[8];
#pragma unroll
        for (int e = 0; e < 8; e++)
            c[e] = kLowest;
        if (vy) {
            if constexpr (sizeof(T) == 4) {
                const pool_f32x4 v0 = *(const pool_f32x4 *)p, v1 = *(const pool_f32x4 *)(p + 4);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    c[e] = v0[e];
                    c[4 + e] = v1[e];
                }
            } else {
                const pool_u32x4 v = *(const pool_u32x4 *)p;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    c[2 * e] = __builtin_bit_cast(float, v[e] << 16);
                    c[2 * e + 1] = __builtin_bit_cast(float, v[e] & 0xffff0000u);
                }
            }
        }
        const float l = __shfl_up(c[7], 1); // the left lane's last column = 8 * gx - 1
        m[r][0] = fmaxf(fmaxf(has_left ? l : kLowest, c[0]), c[1]);
        m[r][1] = fmaxf(fmaxf(c[1], c[2]), c[3]);
        m[r][2] = fmaxf(fmaxf(c[3], c[4]), c[5]);
        m[r][3] = fmaxf(fmaxf(c[5], c[6]), c[7]);
    }
    if (!in_range || lane == 0)
        return;
    T *yp = (T *)a.y + plane * a.OH * a.OW + 4 * gx;
#pragma unroll
    for (int j = 0; j < kMaxStrip; j++) {
        const int oy = oy0 + j;
        if (oy >= a.OH)
            continue;
        float o[4];
#pragma unroll
        for (int q = 0; q < 4; q++)
            o[q] = fmaxf(fmaxf(m[2 * j][q], m[2 * j + 1][q]), m[2 * j + 2][q]);
        if constexpr (sizeof(T) == 4) {
            pool_f32x4 v;
            v[0] = o[0], v[1] = o[1], v[2] = o[2], v[3] = o[3];
            *(pool_f32x4 *)(yp + (size_t)oy * a.OW) = v;
        } else {
            // the values are bf16 already (maxima of stored values): the upper halves are the results
            pool_u32x2 v;
            v[0] = (__builtin_bit_cast(uint32_t, o[0]) >> 16) | (__builtin_bit_cast(uint32_t, o[1]) & 0xffff0000u);
            v[1] = (__builtin_bit_cast(uint32_t, o[2]) >> 16) | (__builtin_bit_cast(uint32_t, o[3]) & 0xffff0000u);
            *(pool_u32x2 *)(yp + (size_t)oy * a.OW) = v;
        }
    }
}

// LPP lanes per plane (64: one wavefront per plane; 16: four planes per wavefront, for the 7x7 and
// smaller planes at the end of a network): lanes stride over the plane, then a shuffle reduction.
// The average is accumulated per lane in ascending index order and combined pairwise,
// so it differs from the reference's single running sum only by fp32 rounding.
template <class T, int LPP>
__global__ __launch_bounds__(256) void global_pool_kernel(const T *__restrict__ x, T *__restrict__ y, long long planes, int plane_size,
                                                          int mode)
{
    constexpr int PPB = 256 / LPP; // planes per workgroup
    const int sub = threadIdx.x % LPP;
    const long long plane = (long long)blockIdx.x * PPB + threadIdx.x / LPP;
    const bool ok = plane < planes;
    const T *src = x + (ok ? plane : 0) * plane_size;
    float v = mode == 0 ? -3.402823466e+38f : 0.0f;
    if (ok)
        for (int i = sub; i < plane_size; i += LPP) {
            const float t = to_float(src[i]);
            v = mode == 0 ? fmaxf(v, t) : v + t;
        }
#pragma unroll
    for (int off = LPP / 2; off >= 1; off >>= 1) {
        const float o = __shfl_down(v, off, LPP);
        v = mode == 0 ? fmaxf(v, o) : v + o;
    }
    if (ok && sub == 0)
        store_plain(y + plane, mode == 0 ? v : v * (1.0f / plane_size));
}

// Global pooling of a channels-last x ([image][pixel][channel]): one thread per image and VEC consecutive channels, consecutive
// threads on consecutive channels (every load of a wavefront is one run of a pixel's channels, VEC elements a lane, eight pixels'
// loads in flight), a single running sum per channel in pixel order as in the reference (src/kernels/global_pooling.cl accumulates
// the same way per plane).  With one channel per thread the 25.7 MB of ResNet-50's last tensor at batch 128 took 17 us.
template <class T, int VEC>
__global__ __launch_bounds__(256) void global_pool_cl_kernel(const T *__restrict__ x, T *__restrict__ y, int batch, int channels, int plane_size,
                                                             int mode)
{
    struct alignas(sizeof(T) * VEC) Pack {
        T e[VEC];
    };
    const int cgroups = channels / VEC;
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i >= (long long)batch * cgroups)
        return;
    const int b = (int)(i / cgroups), c = (int)(i - (long long)b * cgroups) * VEC;
    const T *src = x + (size_t)b * plane_size * channels + c;
    float v[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++)
        v[e] = mode == 0 ? -3.402823466e+38f : 0.0f;
#pragma unroll 8
    for (int p = 0; p < plane_size; p++) {
        const Pack t = *reinterpret_cast<const Pack *>(src + (size_t)p * channels);
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            const float f = to_float(t.e[e]);
            v[e] = mode == 0 ? fmaxf(v[e], f) : v[e] + f;
        }
    }
#pragma unroll
    for (int e = 0; e < VEC; e++)
        store_plain(y + (size_t)b * channels + c + e, mode == 0 ? v[e] : v[e] * (1.0f / plane_size));
}

__device__ __forceinline__ float eltwise_one(float x0, float x1, int op, float c1, float c2, int act)
{
    float r;
    if (op == 0)
        r = x0 * c1 + x1 * c2;
    else if (op == 1)
        r = x0 * x1 * (c1 * c2);
    else
        r = fmaxf(x0 * c1, x1 * c2);
    return apply_act(r, act);
}

// Measured inside whole networks (ResNet-50 at batch 64, fp32: the 16 sums 0.75 -> 0.65 ms): one 16-byte pack per thread in a grid
// as large as the tensor (a capped grid walks the tensor with a power-of-two stride, which keeps a workgroup on the same memory
// channels) and non-temporal accesses on both sides (bit 0: loads, bit 1: stores).
#ifndef ELT_NT
#define ELT_NT 3
#endif
#ifndef ELT_ONESHOT
#define ELT_ONESHOT 1
#endif
// 16 bytes per thread and step (4 floats or 8 bf16) over the 16-byte aligned body [0, n16 * VEC);
// the last n - n16 * VEC elements are done one by one by the first threads.
template <class T>
__global__ __launch_bounds__(256) void eltwise_kernel(size_t n, int op, float c1, float c2, int act, const T *__restrict__ a,
                                                      const T *__restrict__ b, T *__restrict__ c)
{
    constexpr int VEC = 16 / (int)sizeof(T);
    struct alignas(16) Pack {
        T v[VEC];
    };
    const size_t n16 = n / VEC;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    typedef unsigned int elt_u32x4 __attribute__((ext_vector_type(4)));
    for (size_t k = i; k < n16; k += stride) {
        Pack pa, pb;
        if (ELT_NT & 1) {
            *(elt_u32x4 *)&pa = __builtin_nontemporal_load((const elt_u32x4 *)a + k);
            *(elt_u32x4 *)&pb = __builtin_nontemporal_load((const elt_u32x4 *)b + k);
        } else {
            pa = ((const Pack *)a)[k];
            pb = ((const Pack *)b)[k];
        }
        Pack pc;
#pragma unroll
        for (int e = 0; e < VEC; e++)
            store_plain(&pc.v[e], eltwise_one(to_float(pa.v[e]), to_float(pb.v[e]), op, c1, c2, act));
        if (ELT_NT & 2)
            __builtin_nontemporal_store(*(const elt_u32x4 *)&pc, (elt_u32x4 *)c + k);
        else
            ((Pack *)c)[k] = pc;
    }
    for (size_t k = n16 * VEC + i; k < n; k += stride)
        store_plain(c + k, eltwise_one(to_float(a[k]), to_float(b[k]), op, c1, c2, act));
}

// any alignment: one element per thread and step
template <class T>
__global__ __launch_bounds__(256) void eltwise_scalar_kernel(size_t n, int op, float c1, float c2, int act, const T *__restrict__ a,
                                                             const T *__restrict__ b, T *__restrict__ c)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride)
        store_plain(c + i, eltwise_one(to_float(a[i]), to_float(b[i]), op, c1, c2, act));
}

// Broadcasting operands: the output index is taken apart into at most four (collapsed) dimensions, whose strides in a and b are
// 0 where that operand has extent 1.  The innermost dimension runs along consecutive threads.
struct BcastArgs {
    unsigned dims[4];          // output extents, dims[3] innermost; unused leading ones are 1
    long long sa[4], sb[4];    // element strides of a and b
};
template <class T>
__global__ __launch_bounds__(256) void eltwise_bcast_kernel(size_t n, BcastArgs g, int op, float c1, float c2, int act, const T *__restrict__ a,
                                                            const T *__restrict__ b, T *__restrict__ c)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        size_t r = i;
        long long oa = 0, ob = 0;
#pragma unroll
        for (int d = 3; d >= 0; d--) {
            const size_t q = r / g.dims[d], k = r - q * g.dims[d];
            oa += (long long)k * g.sa[d];
            ob += (long long)k * g.sb[d];
            r = q;
        }
        store_plain(c + i, eltwise_one(to_float(a[oa]), to_float(b[ob]), op, c1, c2, act));
    }
}

} // namespace

// y = act(x): 16 bytes per thread and step over the aligned body, the tail one by one.
template <class T>
__global__ __launch_bounds__(256) void activation_kernel(size_t n, int act, const T *__restrict__ x, T *__restrict__ y, int vec_ok)
{
    constexpr int VEC = 16 / (int)sizeof(T);
    struct alignas(16) Pack {
        T v[VEC];
    };
    const size_t n16 = vec_ok ? n / VEC : 0;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t k = i; k < n16; k += stride) {
        const Pack px = ((const Pack *)x)[k];
        Pack py;
#pragma unroll
        for (int e = 0; e < VEC; e++)
            store_plain(&py.v[e], apply_act(to_float(px.v[e]), act));
        ((Pack *)y)[k] = py;
    }
    for (size_t k = n16 * VEC + i; k < n; k += stride)
        store_plain(y + k, apply_act(to_float(x[k]), act));
}

// The parameterised pointwise operators (src/ops/pointwise.cpp:90-95,120-126,154-158): 0 Threshold y = x > p0 ? 1 : 0,
// 1 Abs y = |x|, 2 Hardtanh y = max(p0, min(p1, x)).
__device__ __forceinline__ float pointwise_one(float v, int op, float p0, float p1)
{
    switch (op) {
    case 0: return v > p0 ? 1.0f : 0.0f;
    case 1: return fabsf(v);
    default: return fmaxf(p0, fminf(p1, v));
    }
}
template <class T>
__global__ __launch_bounds__(256) void pointwise_kernel(size_t n, int op, float p0, float p1, const T *__restrict__ x, T *__restrict__ y, int vec_ok)
{
    constexpr int VEC = 16 / (int)sizeof(T);
    struct alignas(16) Pack {
        T v[VEC];
    };
    const size_t n16 = vec_ok ? n / VEC : 0;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t k = i; k < n16; k += stride) {
        const Pack px = ((const Pack *)x)[k];
        Pack py;
#pragma unroll
        for (int e = 0; e < VEC; e++)
            store_plain(&py.v[e], pointwise_one(to_float(px.v[e]), op, p0, p1));
        ((Pack *)y)[k] = py;
    }
    for (size_t k = n16 * VEC + i; k < n; k += stride)
        store_plain(y + k, pointwise_one(to_float(x[k]), op, p0, p1));
}

// y[b][c][i] = act(x[b][c][i] * scale[c] + shift[c]): batch normalisation with fixed statistics.
// VEC elements per thread and step; with VEC > 1 the host guarantees plane % VEC == 0 (a pack never
// straddles two channels) and 16-byte aligned tensors.
template <class T, int VEC>
__global__ __launch_bounds__(256) void channel_affine_kernel(size_t packs, int C, int plane_packs, int act, const T *__restrict__ x,
                                                             const float *__restrict__ scale, const float *__restrict__ shift, T *__restrict__ y)
{
    struct alignas(VEC * sizeof(T)) Pack {
        T v[VEC];
    };
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t k = (size_t)blockIdx.x * blockDim.x + threadIdx.x; k < packs; k += stride) {
        const int c = (int)((k / (size_t)plane_packs) % (size_t)C);
        const float sc = scale ? scale[c] : 1.0f, sh = shift ? shift[c] : 0.0f; // (x * 1 + sh rounds once, like x + sh)
        const Pack px = ((const Pack *)x)[k];
        Pack py;
#pragma unroll
        for (int e = 0; e < VEC; e++)
            store_plain(&py.v[e], apply_act(fmaf(to_float(px.v[e]), sc, sh), act));
        ((Pack *)y)[k] = py;
    }
}

// Softmax over dimension 1 of x[B][C][S] (S = 1 for a matrix): one wavefront per (b, s) column;
// max, sum of exp(x - max), then exp(x - max) / sum or, for the log variant, x - max - log(sum).
template <class T>
__global__ __launch_bounds__(256) void softmax_kernel(int B, int C, int S, int log_softmax, const T *__restrict__ x, T *__restrict__ y)
{
    const int lane = threadIdx.x & 63;
    const long long col = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (col >= (long long)B * S)
        return;
    const int b = (int)(col / S), sp = (int)(col - (long long)b * S);
    const T *xp = x + ((size_t)b * C) * S + sp;
    T *yp = y + ((size_t)b * C) * S + sp;
    float m = -3.402823466e+38f;
    for (int j = lane; j < C; j += 64)
        m = fmaxf(m, to_float(xp[(size_t)j * S]));
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1)
        m = fmaxf(m, __shfl_xor(m, off));
    float sum = 0.0f;
    for (int j = lane; j < C; j += 64)
        sum += expf(to_float(xp[(size_t)j * S]) - m);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1)
        sum += __shfl_xor(sum, off);
    if (log_softmax) {
        const float shift = -m - logf(sum);
        for (int j = lane; j < C; j += 64)
            store_plain(yp + (size_t)j * S, to_float(xp[(size_t)j * S]) + shift);
    } else {
        const float inv = 1.0f / sum;
        for (int j = lane; j < C; j += 64)
            store_plain(yp + (size_t)j * S, expf(to_float(xp[(size_t)j * S]) - m) * inv);
    }
}

} // namespace dlp

using namespace dlp;

struct dlp_pool2d_fwd {
    int kernel[2], pad[2], stride[2];
    int mode; // 0 max, 1 avg
    int count_include_pad;
    int global;
    int dtype;
    int channels_last; // global pooling: x is [image][pixel][channel]
};

static int pool_create(const int kernel[2], const int pad[2], const int stride[2], int mode, int cip, int global, int dtype,
                       dlp_pool2d_fwd **out)
{
    DLP_REQUIRE(out != nullptr, "null argument");
    *out = nullptr;
    if (dtype != DLP_FLOAT && dtype != DLP_BFLOAT16)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "pooling: float_data and bfloat16_data are implemented");
    dlp_pool2d_fwd *op = new (std::nothrow) dlp_pool2d_fwd();
    if (!op)
        return fail(DLP_ERR_RUNTIME, "out of host memory");
    for (int i = 0; i < 2; i++) {
        op->kernel[i] = kernel ? kernel[i] : 0;
        op->pad[i] = pad ? pad[i] : 0;
        op->stride[i] = stride ? stride[i] : 1;
    }
    op->mode = mode;
    op->count_include_pad = cip;
    op->global = global;
    op->dtype = dtype;
    if (!global) {
        for (int i = 0; i < 2; i++)
            if (op->kernel[i] <= 0 || op->stride[i] <= 0 || op->pad[i] < 0) {
                delete op;
                return fail(DLP_ERR_VALIDATION, "check failed: kernel > 0 && stride > 0 && pad >= 0");
            }
    }
    *out = op;
    return DLP_OK;
}

// rows x width units of U from a pitched source to a pitched destination (pitches in units); consecutive threads take consecutive
// units of a row
template <class U>
__global__ __launch_bounds__(256) void copy2d_kernel(U *__restrict__ dst, size_t dst_pitch, const U *__restrict__ src, size_t src_pitch, size_t width, size_t rows)
{
    const size_t total = width * rows;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const size_t r = i / width, c = i - r * width;
        dst[r * dst_pitch + c] = src[r * src_pitch + c];
    }
}

extern "C" {

int dlp_pool2d_output_size(int in_size, int kernel, int pad, int stride, int ceil_mode, int *out_size)
{
    DLP_REQUIRE(out_size != nullptr, "null argument");
    DLP_REQUIRE(kernel > 0 && stride > 0 && pad >= 0, "kernel/stride/pad");
    const int padded = in_size + pad * 2;
    DLP_REQUIRE(padded >= kernel, "padded input smaller than the pooling window"); // pool.hpp:20
    const int offset = ceil_mode ? (stride - 1) : 0;
    int size = (padded - kernel + offset) / stride + 1;
    if ((size - 1) * stride >= in_size + pad)
        size--;
    *out_size = size;
    return DLP_OK;
}

int dlp_pool2d_fwd_create_max(const int kernel[2], const int pad[2], const int stride[2], int dtype, dlp_pool2d_fwd **out)
{
    return pool_create(kernel, pad, stride, 0, 0, 0, dtype, out);
}

int dlp_pool2d_fwd_create_avg(const int kernel[2], const int pad[2], const int stride[2], int count_include_pad, int dtype,
                              dlp_pool2d_fwd **out)
{
    return pool_create(kernel, pad, stride, 1, count_include_pad != 0, 0, dtype, out);
}

int dlp_pool2d_fwd_create_global_max(int dtype, dlp_pool2d_fwd **out) { return pool_create(nullptr, nullptr, nullptr, 0, 0, 1, dtype, out); }

int dlp_pool2d_fwd_create_global_avg(int dtype, dlp_pool2d_fwd **out) { return pool_create(nullptr, nullptr, nullptr, 1, 0, 1, dtype, out); }

int dlp_pool2d_fwd_set_channels_last(dlp_pool2d_fwd *op, int on)
{
    DLP_REQUIRE(op != nullptr, "null argument");
    if (on && !op->global)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "channels-last input: global pooling only");
    op->channels_last = on ? 1 : 0;
    return DLP_OK;
}

int dlp_pool2d_fwd_enqueue(dlp_pool2d_fwd *op, const int x_shape[4], const int y_shape[4], const void *x, void *y, void *stream)
{
    DLP_REQUIRE(op != nullptr && x_shape != nullptr && y_shape != nullptr, "null argument");
    DLP_REQUIRE(x_shape[0] == y_shape[0] && x_shape[1] == y_shape[1], "batch / channels of input and output differ");
    const long long planes = (long long)x_shape[0] * x_shape[1];
    if (planes == 0)
        return DLP_OK;
    DLP_REQUIRE(x != nullptr && y != nullptr, "null tensor pointer");
    hipStream_t s = (hipStream_t)stream;
    if (op->global) {
        DLP_REQUIRE(y_shape[2] == 1 && y_shape[3] == 1, "global pooling output must be [B,C,1,1]");
        const long long plane_size = (long long)x_shape[2] * x_shape[3];
        DLP_REQUIRE(plane_size > 0 && plane_size < 0x7fffffffLL, "plane size");
        TimingScope ts("global_pooling", s);
        if (op->channels_last) {
            // four channels per thread where a pixel's channels come in fours and x is aligned for the wider loads
            const bool bf16 = op->dtype == DLP_BFLOAT16;
            const bool wide = x_shape[1] % 4 == 0 && ((uintptr_t)x & (bf16 ? 7 : 15)) == 0;
            const unsigned cl_grid = (unsigned)((planes / (wide ? 4 : 1) + 255) / 256);
            if (bf16 && wide)
                hipLaunchKernelGGL((global_pool_cl_kernel<bf16_t, 4>), dim3(cl_grid), dim3(256), 0, s, (const bf16_t *)x, (bf16_t *)y, x_shape[0], x_shape[1],
                                   (int)plane_size, op->mode);
            else if (bf16)
                hipLaunchKernelGGL((global_pool_cl_kernel<bf16_t, 1>), dim3(cl_grid), dim3(256), 0, s, (const bf16_t *)x, (bf16_t *)y, x_shape[0], x_shape[1],
                                   (int)plane_size, op->mode);
            else if (wide)
                hipLaunchKernelGGL((global_pool_cl_kernel<float, 4>), dim3(cl_grid), dim3(256), 0, s, (const float *)x, (float *)y, x_shape[0], x_shape[1],
                                   (int)plane_size, op->mode);
            else
                hipLaunchKernelGGL((global_pool_cl_kernel<float, 1>), dim3(cl_grid), dim3(256), 0, s, (const float *)x, (float *)y, x_shape[0], x_shape[1],
                                   (int)plane_size, op->mode);
            DLP_HIP_TRY(hipGetLastError());
            return DLP_OK;
        }
        const bool small = plane_size <= 64;
        const unsigned grid = (unsigned)((planes + (small ? 15 : 3)) / (small ? 16 : 4));
        if (op->dtype == DLP_BFLOAT16) {
            if (small)
                hipLaunchKernelGGL((global_pool_kernel<bf16_t, 16>), dim3(grid), dim3(256), 0, s, (const bf16_t *)x, (bf16_t *)y, planes, (int)plane_size,
                                   op->mode);
            else
                hipLaunchKernelGGL((global_pool_kernel<bf16_t, 64>), dim3(grid), dim3(256), 0, s, (const bf16_t *)x, (bf16_t *)y, planes, (int)plane_size,
                                   op->mode);
        } else {
            if (small)
                hipLaunchKernelGGL((global_pool_kernel<float, 16>), dim3(grid), dim3(256), 0, s, (const float *)x, (float *)y, planes, (int)plane_size,
                                   op->mode);
            else
                hipLaunchKernelGGL((global_pool_kernel<float, 64>), dim3(grid), dim3(256), 0, s, (const float *)x, (float *)y, planes, (int)plane_size,
                                   op->mode);
        }
    } else {
        // the output shape fixes ceil_mode; every window must start inside the padded input (pool.hpp:17-27)
        for (int i = 0; i < 2; i++) {
            DLP_REQUIRE(y_shape[2 + i] > 0, "empty pooling output");
            DLP_REQUIRE((y_shape[2 + i] - 1) * op->stride[i] < x_shape[2 + i] + op->pad[i], "output larger than the pooling geometry allows");
        }
        PoolArgs a;
        a.x = x;
        a.y = y;
        a.planes = (int)planes;
        a.H = x_shape[2];
        a.W = x_shape[3];
        a.OH = y_shape[2];
        a.OW = y_shape[3];
        a.kh = op->kernel[0];
        a.kw = op->kernel[1];
        a.ph = op->pad[0];
        a.pw = op->pad[1];
        a.sh = op->stride[0];
        a.sw = op->stride[1];
        a.mode = op->mode;
        a.count_include_pad = op->count_include_pad;
        const long long total = planes * a.OH * a.OW;
        DLP_REQUIRE(planes < 0x7fffffffLL && total < 0x7fffffffLL * 256, "tensor too large");
        TimingScope ts("pooling", s);
        if (a.mode == 0 && a.kh == 3 && a.kw == 3 && a.sh == 2 && a.sw == 2 && a.ph == 1 && a.pw == 1) {
            const int nstrips = (a.OH + kMaxStrip - 1) / kMaxStrip;
            if (a.W % 8 == 0 && a.OW * 2 == a.W && (((uintptr_t)x | (uintptr_t)y) & 15) == 0) {
                const int groups_per_row = a.OW / 4;
                const long long total_groups = planes * nstrips * groups_per_row;
                const long long wblocks = ((total_groups + 62) / 63 + 3) / 4;
                DLP_REQUIRE(wblocks < 0x7fffffffLL, "tensor too large");
                if (op->dtype == DLP_BFLOAT16)
                    hipLaunchKernelGGL(maxpool3x3s2p1_wide_kernel<bf16_t>, dim3((unsigned)wblocks), dim3(256), 0, s, a, nstrips, total_groups, groups_per_row);
                else
                    hipLaunchKernelGGL(maxpool3x3s2p1_wide_kernel<float>, dim3((unsigned)wblocks), dim3(256), 0, s, a, nstrips, total_groups, groups_per_row);
                DLP_HIP_TRY(hipGetLastError());
                return DLP_OK;
            }
            const long long total_cols = planes * nstrips * a.OW;
            const long long blocks = ((total_cols + 62) / 63 + 3) / 4;
            const size_t esize = dtype_size(op->dtype);
            const int pairs = a.W % 2 == 0 && ((uintptr_t)x & (2 * esize - 1)) == 0;
            if (op->dtype == DLP_BFLOAT16)
                hipLaunchKernelGGL(maxpool3x3s2p1_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, s, a, nstrips, total_cols, pairs);
            else
                hipLaunchKernelGGL(maxpool3x3s2p1_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, s, a, nstrips, total_cols, pairs);
        } else if (op->dtype == DLP_BFLOAT16)
            hipLaunchKernelGGL(pool2d_kernel<bf16_t>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, a);
        else
            hipLaunchKernelGGL(pool2d_kernel<float>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, a);
    }
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

void dlp_pool2d_fwd_destroy(dlp_pool2d_fwd *op) { delete op; }

static int eltwise_launch(int dtype, int operation, float coef1, float coef2, int activation, size_t n, const void *a, const void *b,
                          void *c, void *stream);

int dlp_copy2d_enqueue(void *dst, size_t dst_pitch, const void *src, size_t src_pitch, size_t width_bytes, size_t rows, void *stream)
{
    if (width_bytes == 0 || rows == 0)
        return DLP_OK;
    DLP_REQUIRE(dst != nullptr && src != nullptr, "null tensor pointer");
    DLP_REQUIRE(dst_pitch >= width_bytes && src_pitch >= width_bytes, "a row is longer than its pitch");
    hipStream_t st = (hipStream_t)stream;
    // the widest unit that every address of the copy is a multiple of
    const uintptr_t all = (uintptr_t)dst | (uintptr_t)src | dst_pitch | src_pitch | width_bytes;
    const size_t unit = (all & 15) == 0 ? 16 : (all & 3) == 0 ? 4 : (all & 1) == 0 ? 2 : 1;
    const size_t total = width_bytes / unit * rows;
    const unsigned blocks = (unsigned)std::min<size_t>((total + 255) / 256, 65536);
    TimingScope ts("copy", st);
    typedef uint32_t copy_u32x4 __attribute__((ext_vector_type(4)));
    if (unit == 16)
        hipLaunchKernelGGL(copy2d_kernel<copy_u32x4>, dim3(blocks), dim3(256), 0, st, (copy_u32x4 *)dst, dst_pitch / 16, (const copy_u32x4 *)src, src_pitch / 16,
                           width_bytes / 16, rows);
    else if (unit == 4)
        hipLaunchKernelGGL(copy2d_kernel<uint32_t>, dim3(blocks), dim3(256), 0, st, (uint32_t *)dst, dst_pitch / 4, (const uint32_t *)src, src_pitch / 4, width_bytes / 4, rows);
    else if (unit == 2)
        hipLaunchKernelGGL(copy2d_kernel<uint16_t>, dim3(blocks), dim3(256), 0, st, (uint16_t *)dst, dst_pitch / 2, (const uint16_t *)src, src_pitch / 2, width_bytes / 2, rows);
    else
        hipLaunchKernelGGL(copy2d_kernel<uint8_t>, dim3(blocks), dim3(256), 0, st, (uint8_t *)dst, dst_pitch, (const uint8_t *)src, src_pitch, width_bytes, rows);
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

int dlp_eltwise_fwd_enqueue(int operation, float coef1, float coef2, int activation, size_t n, const void *a, const void *b, void *c,
                            void *stream)
{
    return eltwise_launch(DLP_FLOAT, operation, coef1, coef2, activation, n, a, b, c, stream);
}

int dlp_eltwise_fwd_enqueue_dtype(int dtype, int operation, float coef1, float coef2, int activation, size_t n, const void *a,
                                  const void *b, void *c, void *stream)
{
    return eltwise_launch(dtype, operation, coef1, coef2, activation, n, a, b, c, stream);
}


int dlp_activation_fwd_enqueue(int dtype, int activation, size_t n, const void *x, void *y, void *stream)
{
    DLP_REQUIRE(dtype == DLP_FLOAT || dtype == DLP_BFLOAT16, "float_data and bfloat16_data are implemented");
    DLP_REQUIRE(activation >= DLP_ACT_IDENTITY && activation <= DLP_ACT_RELU6, "unknown activation");
    if (n == 0)
        return DLP_OK;
    DLP_REQUIRE(x != nullptr && y != nullptr, "null tensor pointer");
    hipStream_t st = (hipStream_t)stream;
    const int vec_ok = (((uintptr_t)x | (uintptr_t)y) & 15) == 0;
    const size_t per_block = 256 * (16 / dtype_size(dtype));
    size_t blocks = (n + per_block - 1) / per_block;
    if (blocks > 65536)
        blocks = 65536;
    TimingScope ts("activation", st);
    if (dtype == DLP_BFLOAT16)
        hipLaunchKernelGGL(activation_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, st, n, activation, (const bf16_t *)x, (bf16_t *)y, vec_ok);
    else
        hipLaunchKernelGGL(activation_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, st, n, activation, (const float *)x, (float *)y, vec_ok);
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

int dlp_pointwise_fwd_enqueue(int dtype, int operation, float p0, float p1, size_t n, const void *x, void *y, void *stream)
{
    DLP_REQUIRE(dtype == DLP_FLOAT || dtype == DLP_BFLOAT16, "float_data and bfloat16_data are implemented");
    DLP_REQUIRE(operation >= DLP_POINTWISE_THRESHOLD && operation <= DLP_POINTWISE_HARDTANH, "unknown pointwise operation");
    if (n == 0)
        return DLP_OK;
    DLP_REQUIRE(x != nullptr && y != nullptr, "null tensor pointer");
    hipStream_t st = (hipStream_t)stream;
    const int vec_ok = (((uintptr_t)x | (uintptr_t)y) & 15) == 0;
    const size_t per_block = 256 * (16 / dtype_size(dtype));
    size_t blocks = (n + per_block - 1) / per_block;
    if (blocks > 65536)
        blocks = 65536;
    TimingScope ts("activation", st);
    if (dtype == DLP_BFLOAT16)
        hipLaunchKernelGGL(pointwise_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, st, n, operation, p0, p1, (const bf16_t *)x, (bf16_t *)y, vec_ok);
    else
        hipLaunchKernelGGL(pointwise_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, st, n, operation, p0, p1, (const float *)x, (float *)y, vec_ok);
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

int dlp_channel_affine_fwd_enqueue(int dtype, int activation, int batch, int channels, int plane, const void *x, const float *scale,
                                   const float *shift, void *y, void *stream)
{
    DLP_REQUIRE(batch <= 0 || (scale != nullptr && shift != nullptr), "null tensor pointer");
    return dlp::channel_affine_launch(dtype, activation, batch, channels, plane, x, scale, shift, y, (hipStream_t)stream);
}

} // extern "C"

// y = act(x * scale[c] + shift[c]); a null scale is 1, a null shift 0 (bias and activation behind an operator that has no epilogue of its own)
int dlp::channel_affine_launch(int dtype, int activation, int batch, int channels, int plane, const void *x, const float *scale,
                               const float *shift, void *y, hipStream_t stream)
{
    DLP_REQUIRE(dtype == DLP_FLOAT || dtype == DLP_BFLOAT16, "float_data and bfloat16_data are implemented");
    DLP_REQUIRE(activation >= DLP_ACT_IDENTITY && activation <= DLP_ACT_RELU6, "unknown activation");
    DLP_REQUIRE(batch >= 0 && channels > 0 && plane > 0, "shape");
    if (batch == 0)
        return DLP_OK;
    DLP_REQUIRE(x != nullptr && y != nullptr, "null tensor pointer");
    const size_t n = (size_t)batch * channels * plane;
    hipStream_t st = (hipStream_t)stream;
    const int vec = 16 / (dtype == DLP_BFLOAT16 ? 2 : 4);
    const bool wide = plane % vec == 0 && (((uintptr_t)x | (uintptr_t)y) & 15) == 0;
    const size_t packs = wide ? n / vec : n;
    const int plane_packs = wide ? plane / vec : plane;
    size_t blocks = (packs + 255) / 256;
    if (blocks > 256 * 32)
        blocks = 256 * 32;
    TimingScope ts("channel_affine", st);
    if (dtype == DLP_BFLOAT16) {
        if (wide)
            hipLaunchKernelGGL((channel_affine_kernel<bf16_t, 8>), dim3((unsigned)blocks), dim3(256), 0, st, packs, channels, plane_packs,
                               activation, (const bf16_t *)x, scale, shift, (bf16_t *)y);
        else
            hipLaunchKernelGGL((channel_affine_kernel<bf16_t, 1>), dim3((unsigned)blocks), dim3(256), 0, st, packs, channels, plane_packs,
                               activation, (const bf16_t *)x, scale, shift, (bf16_t *)y);
    } else {
        if (wide)
            hipLaunchKernelGGL((channel_affine_kernel<float, 4>), dim3((unsigned)blocks), dim3(256), 0, st, packs, channels, plane_packs,
                               activation, (const float *)x, scale, shift, (float *)y);
        else
            hipLaunchKernelGGL((channel_affine_kernel<float, 1>), dim3((unsigned)blocks), dim3(256), 0, st, packs, channels, plane_packs,
                               activation, (const float *)x, scale, shift, (float *)y);
    }
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

extern "C" {

int dlp_softmax_fwd_enqueue(int dtype, int log_softmax, int batch, int classes, int inner, const void *x, void *y, void *stream)
{
    DLP_REQUIRE(dtype == DLP_FLOAT || dtype == DLP_BFLOAT16, "float_data and bfloat16_data are implemented");
    DLP_REQUIRE(batch >= 0 && classes > 0 && inner > 0, "shape");
    if (batch == 0)
        return DLP_OK;
    DLP_REQUIRE(x != nullptr && y != nullptr, "null tensor pointer");
    const long long cols = (long long)batch * inner;
    DLP_REQUIRE((cols + 3) / 4 < (1ll << 31), "too many columns");
    hipStream_t st = (hipStream_t)stream;
    TimingScope ts("softmax", st);
    if (dtype == DLP_BFLOAT16)
        hipLaunchKernelGGL(softmax_kernel<bf16_t>, dim3((unsigned)((cols + 3) / 4)), dim3(256), 0, st, batch, classes, inner, log_softmax,
                           (const bf16_t *)x, (bf16_t *)y);
    else
        hipLaunchKernelGGL(softmax_kernel<float>, dim3((unsigned)((cols + 3) / 4)), dim3(256), 0, st, batch, classes, inner, log_softmax,
                           (const float *)x, (float *)y);
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

} // extern "C"

static int eltwise_launch(int dtype, int operation, float coef1, float coef2, int activation, size_t n, const void *a, const void *b,
                          void *c, void *stream)
{
    if (dtype != DLP_FLOAT && dtype != DLP_BFLOAT16)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "elementwise: float_data and bfloat16_data are implemented");
    DLP_REQUIRE(operation >= 0 && operation <= 2, "unknown elementwise operation");
    DLP_REQUIRE(activation >= DLP_ACT_IDENTITY && activation <= DLP_ACT_RELU6, "unknown activation");
    if (n == 0)
        return DLP_OK;
    DLP_REQUIRE(a != nullptr && b != nullptr && c != nullptr, "null tensor pointer");
    size_t blocks = (n + 255) / 256;
    if (blocks > 256 * 32)
        blocks = 256 * 32;
    TimingScope ts("eltwise", (hipStream_t)stream);
    const bool aligned = (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) & 15) == 0;
    if (ELT_ONESHOT && aligned) {
        const size_t packs = n / (dtype == DLP_FLOAT ? 4 : 8);
        blocks = std::min<size_t>(std::max<size_t>(1, (packs + 255) / 256), (size_t)1 << 22);
    }
    hipStream_t st = (hipStream_t)stream;
    if (dtype == DLP_BFLOAT16) {
        if (aligned)
            hipLaunchKernelGGL(eltwise_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, st, n, operation, coef1, coef2, activation,
                               (const bf16_t *)a, (const bf16_t *)b, (bf16_t *)c);
        else
            hipLaunchKernelGGL(eltwise_scalar_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, st, n, operation, coef1, coef2,
                               activation, (const bf16_t *)a, (const bf16_t *)b, (bf16_t *)c);
    } else {
        if (aligned)
            hipLaunchKernelGGL(eltwise_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, st, n, operation, coef1, coef2, activation,
                               (const float *)a, (const float *)b, (float *)c);
        else
            hipLaunchKernelGGL(eltwise_scalar_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, st, n, operation, coef1, coef2,
                               activation, (const float *)a, (const float *)b, (float *)c);
    }
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

int dlp_eltwise_bcast_fwd_enqueue(int dtype, int operation, float coef1, float coef2, int activation, int rank, const int *a_shape, const int *b_shape,
                                  const void *a, const void *b, void *c, void *stream)
{
    if (dtype != DLP_FLOAT && dtype != DLP_BFLOAT16)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "elementwise: float_data and bfloat16_data are implemented");
    DLP_REQUIRE(operation >= 0 && operation <= 2, "unknown elementwise operation");
    DLP_REQUIRE(activation >= DLP_ACT_IDENTITY && activation <= DLP_ACT_RELU6, "unknown activation");
    DLP_REQUIRE(rank >= 1 && rank <= 8 && a_shape != nullptr && b_shape != nullptr, "rank 1 to 8 and both shapes are needed");
    // extents of the result; runs of dimensions in which both operands either follow the result or stay put collapse into one
    unsigned dims[8];
    long long sa[8], sb[8];
    int nd = 0;
    size_t total = 1;
    long long stride_a = 1, stride_b = 1; // element strides of the operands, built from the innermost dimension outwards
    int kind_prev = -1;
    for (int j = rank - 1; j >= 0; j--) {
        const int da = a_shape[j], db = b_shape[j];
        DLP_REQUIRE(da >= 0 && db >= 0 && (da == db || da == 1 || db == 1), "the shapes do not broadcast");
        const int dc = da == 1 ? db : da;
        total *= (size_t)dc;
        if (dc == 1)
            continue; // both operands have extent 1: no index, no stride
        const int kind = (da == dc ? 1 : 0) | (db == dc ? 2 : 0); // who moves along this dimension
        if (kind == kind_prev) { // same pattern as the dimension inside it: one longer dimension (strides stay the inner one's)
            dims[nd - 1] *= (unsigned)dc;
        } else {
            DLP_REQUIRE(nd < 8, "too many dimensions");
            dims[nd] = (unsigned)dc;
            sa[nd] = da == dc ? stride_a : 0;
            sb[nd] = db == dc ? stride_b : 0;
            nd++;
            kind_prev = kind;
        }
        stride_a *= da;
        stride_b *= db;
    }
    if (total == 0)
        return DLP_OK;
    DLP_REQUIRE(a != nullptr && b != nullptr && c != nullptr, "null tensor pointer");
    if (nd <= 1 && (nd == 0 || (sa[0] == 1 && sb[0] == 1)))
        return eltwise_launch(dtype, operation, coef1, coef2, activation, total, a, b, c, stream);
    if (nd > 4)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "elementwise: more than four runs of broadcast / plain dimensions");
    BcastArgs g;
    for (int d = 0; d < 4; d++) { // dims[] was filled innermost first; the kernel wants the innermost last
        const int src = 3 - d;
        g.dims[d] = src < nd ? dims[src] : 1u;
        g.sa[d] = src < nd ? sa[src] : 0;
        g.sb[d] = src < nd ? sb[src] : 0;
    }
    hipStream_t st = (hipStream_t)stream;
    const unsigned blocks = (unsigned)std::min<size_t>((total + 255) / 256, 256 * 32);
    TimingScope ts("eltwise", st);
    if (dtype == DLP_BFLOAT16)
        hipLaunchKernelGGL(eltwise_bcast_kernel<bf16_t>, dim3(blocks), dim3(256), 0, st, total, g, operation, coef1, coef2, activation, (const bf16_t *)a,
                           (const bf16_t *)b, (bf16_t *)c);
    else
        hipLaunchKernelGGL(eltwise_bcast_kernel<float>, dim3(blocks), dim3(256), 0, st, total, g, operation, coef1, coef2, activation, (const float *)a,
                           (const float *)b, (float *)c);
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

