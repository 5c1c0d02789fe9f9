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
// Structure: the 16 element-wise products become 16 independent GEMMs
//   M_e[Cout x T] = U_e[Cout x Cin] * V_e[Cin x T],   T = tiles of a batch chunk
// which run on the matrix cores through the implicit-GEMM kernel as ONE grouped
// launch (16 groups of a 1x1 "convolution" over a T x 1 image).  U, V and M live
// in the workspace; the batch is processed in chunks sized so that V and M of a
// chunk stay resident in the on-package caches between the three stages.
//   workspace = U (packed GEMM tile order) | V[16][Cin][Tcap] | M[16][Cout][Tcap]   (floats)
// All loads and stores of the transform kernels have consecutive lanes on
// consecutive tiles / channels, so HBM and workspace traffic is coalesced.
#include "dlp_internal.hpp"

namespace dlp {
namespace {

constexpr size_t kChunkBudgetBytes = 64u << 20; // V + M of one chunk

struct WinoShape {
    int B, C, N, H, W;
    int hh, hw;       // tiles per column / row
    int tiles_per_img;
    int chunk_imgs;   // images per chunk
    int tcap;         // tile capacity of a chunk = row stride of V and M
};

WinoShape wino_shape(const ConvGeom &g, const WinoPlan &plan, int batch)
{
    WinoShape s;
    s.B = batch;
    s.C = g.Cin;
    s.N = g.Cout;
    s.H = g.H;
    s.W = g.W;
    s.hh = (g.H + 1) / 2;
    s.hw = (g.W + 1) / 2;
    s.tiles_per_img = s.hh * s.hw;
    s.chunk_imgs = plan.chunk_imgs;
    s.tcap = plan.tcap;
    return s;
}

// U_e[n][c] = (G k G^T)[e], src/kernels/winograd_fwd.cl:103-135, written straight into
// the packed A layout of the GEMM stage: [e][m tile][K tile][k][m in tile], zero padded.
__global__ __launch_bounds__(256) void wino_filter_kernel(int N, int C, GemmPlan p, const float *__restrict__ w, float *__restrict__ U)
{
    const int npad = p.mtiles * p.BM, cpad = p.nkt * 16;
    const int idx = blockIdx.x * blockDim.x + threadIdx.x; // n * cpad + c over the padded domain
    if (idx >= npad * cpad)
        return;
    const int n = idx / cpad, c = idx - n * cpad;
    float u[16];
#pragma unroll
    for (int e = 0; e < 16; e++)
        u[e] = 0.0f;
    if (n < N && c < C) {
        const float *kp = w + ((size_t)n * C + c) * 9;
        float k[9];
#pragma unroll
        for (int i = 0; i < 9; i++)
            k[i] = kp[i];
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
    // group e, m tile n / BM, K tile c / 16 (1x1 "kernel": both K orders coincide)
    const size_t in_group = ((size_t)(n / p.BM) * p.nkt + c / 16) * (16 * p.BM) + (size_t)(c % 16) * p.BM + n % p.BM;
    const size_t estride = (size_t)p.mtiles * p.nkt * 16 * p.BM;
#pragma unroll
    for (int e = 0; e < 16; e++)
        U[(size_t)e * estride + in_group] = u[e];
}

// V[e][c][t] = (B^T d B)[e] for tile t of channel c, src/kernels/winograd_fwd.cl:35-69
__global__ __launch_bounds__(256) void wino_input_kernel(WinoShape s, int b0, int nb, const float *__restrict__ x, float *__restrict__ V)
{
    const int T = nb * s.tiles_per_img;
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; // c*T + t
    if (idx >= (long long)s.C * T)
        return;
    const int c = (int)(idx / T);
    const int t = (int)(idx - (long long)c * T);
    const int bl = t / s.tiles_per_img;
    const int rc = t - bl * s.tiles_per_img;
    const int row = (rc / s.hw) * 2 - 1;
    const int col = (rc % s.hw) * 2 - 1;
    const float *img = x + ((size_t)(b0 + bl) * s.C + c) * s.H * s.W;
    float a[4][4];
#pragma unroll
    for (int dr = 0; dr < 4; dr++) {
        const int yy = row + dr;
#pragma unroll
        for (int dc = 0; dc < 4; dc++) {
            const int xx = col + dc;
            a[dr][dc] = (yy >= 0 && yy < s.H && xx >= 0 && xx < s.W) ? img[(size_t)yy * s.W + xx] : 0.0f;
        }
    }
    float bta[4][4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        bta[0][j] = a[0][j] - a[2][j];
        bta[1][j] = a[1][j] + a[2][j];
        bta[2][j] = a[2][j] - a[1][j];
        bta[3][j] = a[1][j] - a[3][j];
    }
    const size_t estride = (size_t)s.C * s.tcap;
    float *vp = V + (size_t)c * s.tcap + t;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        vp[(size_t)(4 * i + 0) * estride] = bta[i][0] - bta[i][2];
        vp[(size_t)(4 * i + 1) * estride] = bta[i][1] + bta[i][2];
        vp[(size_t)(4 * i + 2) * estride] = bta[i][2] - bta[i][1];
        vp[(size_t)(4 * i + 3) * estride] = bta[i][1] - bta[i][3];
    }
}

// y tile = A^T m A, bias, activation, factor; src/kernels/winograd_fwd.cl:138-158,406-436
__global__ __launch_bounds__(256) void wino_output_kernel(WinoShape s, int b0, int nb, const float *__restrict__ M,
                                                          const float *__restrict__ bias, float *__restrict__ y, float factor, int act)
{
    const int T = nb * s.tiles_per_img;
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; // n*T + t
    if (idx >= (long long)s.N * T)
        return;
    const int n = (int)(idx / T);
    const int t = (int)(idx - (long long)n * T);
    const size_t estride = (size_t)s.N * s.tcap;
    const float *mp = M + (size_t)n * s.tcap + t;
    float m[16];
#pragma unroll
    for (int e = 0; e < 16; e++)
        m[e] = mp[(size_t)e * estride];
    float atp[2][4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        atp[0][j] = m[j] + m[4 + j] + m[8 + j];
        atp[1][j] = m[4 + j] - m[8 + j] - m[12 + j];
    }
    float o[4];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        o[2 * i + 0] = atp[i][0] + atp[i][1] + atp[i][2];
        o[2 * i + 1] = atp[i][1] - atp[i][2] - atp[i][3];
    }
    const float bv = bias ? bias[n] : 0.0f;
    const int bl = t / s.tiles_per_img;
    const int rc = t - bl * s.tiles_per_img;
    const int row = (rc / s.hw) * 2;
    const int col = (rc % s.hw) * 2;
    float *yp = y + (((size_t)(b0 + bl) * s.N + n) * s.H + row) * s.W + col;
#pragma unroll
    for (int dr = 0; dr < 2; dr++)
#pragma unroll
        for (int dc = 0; dc < 2; dc++)
            if (row + dr < s.H && col + dc < s.W)
                store_out(yp + (size_t)dr * s.W + dc, apply_act(o[2 * dr + dc] + bv, act), factor);
}

} // namespace

bool winograd_supported(const ConvGeom &g)
{
    return g.dtype == DLP_FLOAT && g.KH == 3 && g.KW == 3 && g.ph == 1 && g.pw == 1 && g.dh == 1 && g.dw == 1 && g.sh == 1 &&
           g.sw == 1 && g.groups == 1;
}

// Chunking, workspace size and the geometry of the grouped 1x1 "convolution"
// that runs the 16 GEMMs of a chunk; g.B is the batch hint given at create.
WinoPlan winograd_plan(const ConvGeom &g)
{
    WinoPlan p;
    const int tiles_per_img = ((g.H + 1) / 2) * ((g.W + 1) / 2);
    const size_t per_img = (size_t)16 * tiles_per_img * ((size_t)g.Cin + g.Cout) * sizeof(float);
    size_t imgs = kChunkBudgetBytes / (per_img ? per_img : 1);
    const size_t hint = g.B > 0 ? (size_t)g.B : 1;
    if (imgs < 1)
        imgs = 1;
    if (imgs > hint)
        imgs = hint;
    p.chunk_imgs = (int)imgs;
    p.tcap = p.chunk_imgs * tiles_per_img;
    ConvGeom &q = p.gemm;
    q.B = 1;
    q.Cin = 16 * g.Cin;
    q.H = p.tcap;
    q.W = 1;
    q.Cout = 16 * g.Cout;
    q.OH = p.tcap;
    q.OW = 1;
    q.KH = q.KW = 1;
    q.sh = q.sw = 1;
    q.ph = q.pw = 0;
    q.dh = q.dw = 1;
    q.groups = 16;
    q.dtype = DLP_FLOAT;
    p.gplan = conv_gemm_plan(q, DLP_ACT_IDENTITY);
    p.ws_bytes = p.gplan.wpack_bytes + sizeof(float) * 16 * (size_t)p.tcap * ((size_t)g.Cin + g.Cout);
    return p;
}

int winograd_launch(const ConvGeom &g, const WinoPlan &plan, const KTabEntry *gemm_ktab, const void *x, const void *w, void *y,
                    void *ws, size_t ws_bytes, const Epilogue &ep, hipStream_t stream)
{
    DLP_REQUIRE(winograd_supported(g), "geometry is not Winograd compatible");
    DLP_REQUIRE(ws != nullptr && ws_bytes >= plan.ws_bytes, "workspace smaller than workspace()");
    if (g.B == 0)
        return DLP_OK;
    const WinoShape s = wino_shape(g, plan, g.B);

    float *U = (float *)ws;
    float *V = (float *)((char *)ws + plan.gplan.wpack_bytes);
    float *Mw = V + (size_t)16 * g.Cin * s.tcap;

    {
        TimingScope ts("winograd_filter", stream);
        const int total = plan.gplan.mtiles * plan.gplan.BM * plan.gplan.nkt * 16;
        hipLaunchKernelGGL(wino_filter_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, g.Cout, g.Cin, plan.gplan, (const float *)w, U);
    }
    Epilogue none;
    none.bias = nullptr;
    none.factor = 0.0f;
    none.activation = DLP_ACT_IDENTITY;
    for (int b0 = 0; b0 < g.B; b0 += s.chunk_imgs) {
        const int nb = (g.B - b0 < s.chunk_imgs) ? g.B - b0 : s.chunk_imgs;
        const int T = nb * s.tiles_per_img;
        {
            TimingScope ts("winograd_input", stream);
            const long long total = (long long)g.Cin * T;
            hipLaunchKernelGGL(wino_input_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, s, b0, nb, (const float *)x, V);
        }
        int rc = conv_gemm_launch(plan.gemm, plan.gplan, gemm_ktab, V, U, Mw, none, stream, T);
        if (rc != DLP_OK)
            return rc;
        {
            TimingScope ts("winograd_output", stream);
            const long long total = (long long)g.Cout * T;
            hipLaunchKernelGGL(wino_output_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, s, b0, nb, Mw, ep.bias,
                               (float *)y, ep.factor, ep.activation);
        }
    }
    DLP_HIP_TRY(hipGetLastError());
    return DLP_OK;
}

} // namespace dlp
