// Depthwise (groups == channels) convolution forward for gfx950.
//
// Replaces the reference's Conv2DForwardDepthwiseSeparable / `conv` kernel
// (src/core/conv.cpp:436-510, src/kernels/depthwise_separable_conv.cl:20-105),
// which covers stride 1 only, and adds stride 2 (the reference falls back to a
// grouped GEMM with M = 1 there, src/core/conv.cpp:725-727).
//
// The op is HBM-bound (about 2 flop per byte), so no matrix cores: the kernel is
// organised around reading every input element once (plus a two-row halo per strip)
// and writing every output exactly once, in wide contiguous runs, with enough
// loads in flight per CU to cover the HBM latency.
//
// 3x3 kernel, lanes own output columns.  The (plane, row strip, column) triples of
// the whole tensor are laid on one flat axis; a wavefront covers 64 consecutive
// ones.  A lane produces a strip of 7 output rows of its column: it first issues
// the loads of ALL input rows the strip needs (9 at stride 1, 15 at stride 2), so a
// wavefront has 9-30 independent loads in flight, then computes.  Each lane loads
// only the input columns it owns; the columns to its left/right come from the
// neighbouring lanes through wavefront shuffles.  Lanes at the edge of the
// wavefront are halo lanes: they load and feed their neighbours but store
// nothing, and adjacent wavefronts overlap by the halo, so there is no
// divergent patch-up load.  Accumulation order is the reference's:
// sum = bias; sum = fma(k[dr][dc], x, sum) for dr, dc ascending.
//
// Other odd kernel sizes use a plain direct kernel.
#include "dlp_internal.hpp"

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
