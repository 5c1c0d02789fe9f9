/*
 * CPU oracle for the convolution forward hot path -- TEST INFRASTRUCTURE ONLY.
 * See dlp_oracle.h: this code is the checker, never the product.  Nothing in
 * the shipped library links, loads or calls it.
 *
 * Each function restates one piece of the dlprimitives CPU operator path and
 * cites the reference file:line it follows.
 *
 * Pinning status (what independently checks each function):
 *   orc_conv2d_output_shape  closed form + torch conv2d output shapes
 *   orc_apply_activation     reference golden vectors (tests/test_case_activation.json)
 *                            and the reference's own cpu_ops.hpp compiled into oracle/_ref
 *   orc_sgemm_nt             bit-exact against the reference's my_cblas compiled into
 *                            oracle/_ref; integer-exact property of tests/test_gemm.cpp
 *   orc_im2col/conv2d_forward independent 7-loop direct conv in double, torch conv2d,
 *                            1x1 == matmul, delta kernels == shifts
 *   orc_ip_forward           reference golden vectors (tests/test_case_inner_product.json)
 *   orc_winograd_forward     equals direct convolution to fp32 rounding; filter transform
 *                            against G k G^T computed in double with the published matrices
 *   orc_depthwise_forward    equals grouped convolution (groups == channels)
 */
#include "dlp_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <stdint.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* src/core/conv.cpp:17-29 */
int orc_conv2d_output_shape(const orc_conv2d_cfg *cfg, const int in_shape[4], int out_shape[4])
{
    if (in_shape[1] != cfg->channels_in)
        return -1;
    int ohw[2];
    for (int i = 0; i < 2; i++) {
        if (cfg->stride[i] <= 0)
            return -1;
        int num = in_shape[2 + i] + 2 * cfg->pad[i] - cfg->dilate[i] * (cfg->kernel[i] - 1) - 1;
        /* C integer division truncates toward zero exactly as the reference's does */
        ohw[i] = num / cfg->stride[i] + 1;
        if (ohw[i] <= 0)
            return -1;
    }
    out_shape[0] = in_shape[0];
    out_shape[1] = cfg->channels_out;
    out_shape[2] = ohw[0];
    out_shape[3] = ohw[1];
    return 0;
}

/* include/dlprim/cpu/cpu_ops.hpp:17-53 */
void orc_apply_activation(float *p, size_t n, int activation)
{
    switch (activation) {
    case ORC_ACT_IDENTITY:
        break;
    case ORC_ACT_RELU:
        for (size_t i = 0; i < n; i++)
            p[i] = p[i] < 0.0f ? 0.0f : p[i];
        break;
    case ORC_ACT_TANH:
        for (size_t i = 0; i < n; i++)
            p[i] = tanhf(p[i]);
        break;
    case ORC_ACT_SIGMOID:
        for (size_t i = 0; i < n; i++)
            p[i] = 1.0f / (1.0f + expf(-p[i]));
        break;
    case ORC_ACT_RELU6:
        for (size_t i = 0; i < n; i++) {
            float v = p[i] < 0.0f ? 0.0f : p[i];
            p[i] = v > 6.0f ? 6.0f : v;
        }
        break;
    }
}

/* src/my_blas/my_cblas.cpp:28-39 (beta), :63-74 (nt product), :88-103 (dispatch) */
void orc_sgemm_nt(int M, int N, int K, float alpha, const float *A, int lda,
                  const float *B, int ldb, float beta, float *C, int ldc)
{
    for (int r = 0; r < M; r++) {
        if (beta == 0.0f)
            memset(C + (size_t)ldc * r, 0, sizeof(float) * (size_t)N);
        else
            for (int c = 0; c < N; c++)
                C[(size_t)r * ldc + c] *= beta;
    }
    for (int r = 0; r < M; r++) {
        const float *a = A + (size_t)r * lda;
        for (int c = 0; c < N; c++) {
            const float *b = B + (size_t)c * ldb;
            /* accumulate through memory-order semantics: one rounding per term,
             * terms added in ascending k (volatile-free: -ffp-contract=off in the
             * Makefile keeps mul and add separate as in the reference's -O2 build) */
            float acc = C[(size_t)r * ldc + c];
            for (int k = 0; k < K; k++) {
                float av = a[k] * alpha;
                acc += av * b[k];
            }
            C[(size_t)r * ldc + c] = acc;
        }
    }
}

/* src/ops/conv2d.cpp:376-409 (generic branch; the specialised k/s/p branches
 * :282-343 produce the same matrix) */
void orc_im2col(const orc_conv2d_cfg *cfg, int cin_g, int H, int W, int OH, int OW,
                const float *img, float *mat)
{
    const int kh = cfg->kernel[0], kw = cfg->kernel[1];
    const int width = cin_g * kh * kw;
    for (int chan = 0; chan < cin_g; chan++) {
        for (int r = 0; r < OH; r++) {
            for (int c = 0; c < OW; c++) {
                float *m = mat + (size_t)(r * OW + c) * width + chan * kh * kw;
                int y0 = r * cfg->stride[0] - cfg->pad[0];
                int x0 = c * cfg->stride[1] - cfg->pad[1];
                for (int ky = 0; ky < kh; ky++) {
                    int y = y0 + ky * cfg->dilate[0];
                    for (int kx = 0; kx < kw; kx++) {
                        int x = x0 + kx * cfg->dilate[1];
                        float v = 0.0f;
                        if (y >= 0 && y < H && x >= 0 && x < W)
                            v = img[((size_t)chan * H + y) * W + x];
                        *m++ = v;
                    }
                }
            }
        }
    }
}

static int conv_cfg_ok(const orc_conv2d_cfg *cfg, const int in_shape[4], int out_shape[4])
{
    if (cfg->groups <= 0 || cfg->channels_in <= 0 || cfg->channels_out <= 0)
        return -1;
    /* src/ops/conv2d.cpp:105-106 */
    if (cfg->channels_in % cfg->groups != 0 || cfg->channels_out % cfg->groups != 0)
        return -1;
    return orc_conv2d_output_shape(cfg, in_shape, out_shape);
}

/* src/ops/conv2d.cpp:141-147 */
size_t orc_conv2d_workspace(const orc_conv2d_cfg *cfg, const int in_shape[4])
{
    int out[4];
    if (conv_cfg_ok(cfg, in_shape, out) != 0)
        return 0;
    size_t width = (size_t)(cfg->channels_in / cfg->groups) * cfg->kernel[0] * cfg->kernel[1];
    return (size_t)out[2] * out[3] * width * sizeof(float);
}

/* One image: src/ops/conv2d.cpp:452-473 */
static void conv_one_image(const orc_conv2d_cfg *cfg, const int in_shape[4], const int out[4],
                           const float *x_b, const float *w, const float *bias,
                           float *y_b, float *col)
{
    const int H = in_shape[2], W = in_shape[3];
    const int OH = out[2], OW = out[3];
    const int cin_g = cfg->channels_in / cfg->groups;
    const int cout_g = cfg->channels_out / cfg->groups;
    const int K = cin_g * cfg->kernel[0] * cfg->kernel[1];
    const int plane = OH * OW;
    for (int g = 0; g < cfg->groups; g++) {
        const float *img = x_b + (size_t)g * cin_g * H * W;
        float *omg = y_b + (size_t)g * cout_g * plane;
        orc_im2col(cfg, cin_g, H, W, OH, OW, img, col);
        orc_sgemm_nt(cout_g, plane, K, 1.0f, w + (size_t)g * cout_g * K, K, col, K, 0.0f, omg, plane);
        if (bias) {
            /* cblas_saxpy(plane, 1.0f, bias+i, 0, row, 1): row[j] += 1.0f * bias[i] */
            for (int i = 0; i < cout_g; i++) {
                float bv = 1.0f * bias[g * cout_g + i];
                float *row = omg + (size_t)i * plane;
                for (int j = 0; j < plane; j++)
                    row[j] += bv;
            }
        }
    }
}

/* src/ops/conv2d.cpp:421-425,437-474 */
int orc_conv2d_forward(const orc_conv2d_cfg *cfg, const int in_shape[4],
                       const float *x, const float *w, const float *bias,
                       float *y, void *ws, int activation)
{
    int out[4];
    if (conv_cfg_ok(cfg, in_shape, out) != 0)
        return -1;
    const size_t in_img = (size_t)in_shape[1] * in_shape[2] * in_shape[3];
    const size_t out_img = (size_t)out[1] * out[2] * out[3];
    for (int b = 0; b < in_shape[0]; b++)
        conv_one_image(cfg, in_shape, out, x + b * in_img, w, bias, y + b * out_img, (float *)ws);
    orc_apply_activation(y, out_img * (size_t)in_shape[0], activation);
    return 0;
}

int orc_conv2d_forward_mt(const orc_conv2d_cfg *cfg, const int in_shape[4],
                          const float *x, const float *w, const float *bias,
                          float *y, int activation, int threads)
{
    int out[4];
    if (conv_cfg_ok(cfg, in_shape, out) != 0)
        return -1;
    const size_t in_img = (size_t)in_shape[1] * in_shape[2] * in_shape[3];
    const size_t out_img = (size_t)out[1] * out[2] * out[3];
    const size_t ws_bytes = orc_conv2d_workspace(cfg, in_shape);
    int used = 1;
#ifdef _OPENMP
    if (threads <= 0)
        threads = omp_get_max_threads();
    if (threads > in_shape[0])
        threads = in_shape[0] > 0 ? in_shape[0] : 1;
    used = threads;
    int failed = 0;
#pragma omp parallel num_threads(threads)
    {
        float *col = (float *)malloc(ws_bytes ? ws_bytes : 4);
        if (!col) {
#pragma omp atomic write
            failed = 1;
        }
#pragma omp for schedule(dynamic, 1)
        for (int b = 0; b < in_shape[0]; b++) {
            if (col) {
                conv_one_image(cfg, in_shape, out, x + b * in_img, w, bias, y + b * out_img, col);
                orc_apply_activation(y + b * out_img, out_img, activation);
            }
        }
        free(col);
    }
    if (failed)
        return -1;
#else
    (void)threads;
    float *col = (float *)malloc(ws_bytes ? ws_bytes : 4);
    if (!col)
        return -1;
    orc_conv2d_forward(cfg, in_shape, x, w, bias, y, col, activation);
    free(col);
#endif
    return used;
}

/* src/my_blas/my_cblas.cpp:28-39 (beta), :41-51 (nn product: r, k, c loops) */
void orc_sgemm_nn(int M, int N, int K, float alpha, const float *A, int lda,
                  const float *B, int ldb, float beta, float *C, int ldc)
{
    for (int r = 0; r < M; r++) {
        if (beta == 0.0f)
            memset(C + (size_t)ldc * r, 0, sizeof(float) * (size_t)N);
        else
            for (int c = 0; c < N; c++)
                C[(size_t)r * ldc + c] *= beta;
    }
    for (int r = 0; r < M; r++)
        for (int k = 0; k < K; k++) {
            float av = A[(size_t)r * lda + k] * alpha;
            for (int c = 0; c < N; c++)
                C[(size_t)r * ldc + c] += av * B[(size_t)k * ldb + c];
        }
}

/* src/my_blas/my_cblas.cpp:28-39 (beta), :52-62 (tn product: k, r, c loops; A is K x M) */
void orc_sgemm_tn(int M, int N, int K, float alpha, const float *A, int lda,
                  const float *B, int ldb, float beta, float *C, int ldc)
{
    for (int r = 0; r < M; r++) {
        if (beta == 0.0f)
            memset(C + (size_t)ldc * r, 0, sizeof(float) * (size_t)N);
        else
            for (int c = 0; c < N; c++)
                C[(size_t)r * ldc + c] *= beta;
    }
    for (int k = 0; k < K; k++)
        for (int r = 0; r < M; r++) {
            float av = A[r + (size_t)lda * k] * alpha;
            for (int c = 0; c < N; c++)
                C[(size_t)r * ldc + c] += av * B[(size_t)k * ldb + c];
        }
}

/* Convolution2DBase::im2col<Col2ImOp>, src/ops/conv2d.cpp:262-278 (img += column entry, padding skipped)
 * over the generic walk :376-409: the adjoint of orc_im2col */
void orc_col2im(const orc_conv2d_cfg *cfg, int cin_g, int H, int W, int OH, int OW,
                float *img, const float *mat)
{
    const int kh = cfg->kernel[0], kw = cfg->kernel[1];
    const int width = cin_g * kh * kw;
    for (int chan = 0; chan < cin_g; chan++) {
        for (int r = 0; r < OH; r++) {
            for (int c = 0; c < OW; c++) {
                const float *m = mat + (size_t)(r * OW + c) * width + chan * kh * kw;
                int y0 = r * cfg->stride[0] - cfg->pad[0];
                int x0 = c * cfg->stride[1] - cfg->pad[1];
                for (int ky = 0; ky < kh; ky++) {
                    int y = y0 + ky * cfg->dilate[0];
                    for (int kx = 0; kx < kw; kx++) {
                        int x = x0 + kx * cfg->dilate[1];
                        float v = *m++;
                        if (y >= 0 && y < H && x >= 0 && x < W)
                            img[((size_t)chan * H + y) * W + x] += v;
                    }
                }
            }
        }
    }
}

/* Convolution2DBase::scale_cpu, src/ops/conv2d.cpp:411-419 */
static void scale_by(float *p, size_t n, float v)
{
    if (v == 0.0f)
        memset(p, 0, n * sizeof(float));
    else
        for (size_t i = 0; i < n; i++)
            p[i] *= v;
}

/* src/ops/conv2d.cpp:426-430 and the backward_data branch :485-498 */
int orc_conv2d_backward_data(const orc_conv2d_cfg *cfg, const int in_shape[4],
                             const float *dy, const float *w, float *dx, void *ws, float factor)
{
    int out[4];
    if (conv_cfg_ok(cfg, in_shape, out) != 0)
        return -1;
    const int H = in_shape[2], W = in_shape[3], OH = out[2], OW = out[3];
    const int cin_g = cfg->channels_in / cfg->groups, cout_g = cfg->channels_out / cfg->groups;
    const int K = cin_g * cfg->kernel[0] * cfg->kernel[1];
    const int plane = OH * OW;
    const size_t in_img = (size_t)in_shape[1] * H * W, out_img = (size_t)out[1] * plane;
    float *col = (float *)ws;
    scale_by(dx, in_img * (size_t)in_shape[0], factor);
    for (int b = 0; b < in_shape[0]; b++)
        for (int g = 0; g < cfg->groups; g++) {
            float *img = dx + b * in_img + (size_t)g * cin_g * H * W;
            const float *omg = dy + b * out_img + (size_t)g * cout_g * plane;
            /* col[plane x K] = omg^T[plane x cout_g] * kernel[cout_g x K] */
            orc_sgemm_tn(plane, K, cout_g, 1.0f, omg, plane, w + (size_t)g * cout_g * K, K, 0.0f, col, K);
            orc_col2im(cfg, cin_g, H, W, OH, OW, img, col);
        }
    return 0;
}

/* Conv2DBase::get_output_shape_transposed, src/core/conv.cpp:31-43 */
int orc_tconv2d_output_shape(const orc_conv2d_cfg *cfg, const int in_shape[4], const int output_pad[2], int out_shape[4])
{
    if (in_shape[1] != cfg->channels_in)
        return -1;
    for (int i = 0; i < 2; i++) {
        const int o = (in_shape[2 + i] - 1) * cfg->stride[i] - 2 * cfg->pad[i] + cfg->dilate[i] * (cfg->kernel[i] - 1) + output_pad[i] + 1;
        if (o <= 0)
            return -1;
        out_shape[2 + i] = o;
    }
    out_shape[0] = in_shape[0];
    out_shape[1] = cfg->channels_out;
    return 0;
}

/* TransposedConvolution2D::forward, CPU branch, src/ops/conv2d.cpp:760-778 and :798-801: the output is filled with the bias
 * (or zeros), the data-gradient pass of the convolution with swapped channels (:588-590) adds into it, the activation
 * runs over the whole tensor last.  cfg describes the transposed operator; w is [channels_in][channels_out / groups][kh][kw];
 * ws: orc_conv2d_workspace() bytes of the swapped convolution on the output shape. */
int orc_tconv2d_forward(const orc_conv2d_cfg *cfg, const int in_shape[4], const int output_pad[2], const float *x, const float *w,
                        const float *bias, float *y, void *ws, int activation)
{
    int out[4];
    if (orc_tconv2d_output_shape(cfg, in_shape, output_pad, out) != 0)
        return -1;
    orc_conv2d_cfg conv = *cfg;
    conv.channels_in = cfg->channels_out;
    conv.channels_out = cfg->channels_in;
    const size_t plane = (size_t)out[2] * out[3];
    float *p = y;
    for (int b = 0; b < out[0]; b++)
        for (int c = 0; c < out[1]; c++) {
            const float v = bias ? bias[c] : 0.0f;
            for (size_t k = 0; k < plane; k++)
                *p++ = v;
        }
    if (orc_conv2d_backward_data(&conv, out, x, w, y, ws, 1.0f) != 0)
        return -1;
    orc_apply_activation(y, (size_t)out[0] * out[1] * plane, activation);
    return 0;
}

/* src/ops/conv2d.cpp:431-435 and the backward_filter branch :475-484 */
int orc_conv2d_backward_filter(const orc_conv2d_cfg *cfg, const int in_shape[4],
                               const float *dy, const float *x, float *dw, void *ws, float factor)
{
    int out[4];
    if (conv_cfg_ok(cfg, in_shape, out) != 0)
        return -1;
    const int H = in_shape[2], W = in_shape[3], OH = out[2], OW = out[3];
    const int cin_g = cfg->channels_in / cfg->groups, cout_g = cfg->channels_out / cfg->groups;
    const int K = cin_g * cfg->kernel[0] * cfg->kernel[1];
    const int plane = OH * OW;
    const size_t in_img = (size_t)in_shape[1] * H * W, out_img = (size_t)out[1] * plane;
    float *col = (float *)ws;
    scale_by(dw, (size_t)cfg->channels_out * K, factor);
    for (int b = 0; b < in_shape[0]; b++)
        for (int g = 0; g < cfg->groups; g++) {
            const float *img = x + b * in_img + (size_t)g * cin_g * H * W;
            const float *omg = dy + b * out_img + (size_t)g * cout_g * plane;
            orc_im2col(cfg, cin_g, H, W, OH, OW, img, col);
            /* dK[cout_g x K] += omg[cout_g x plane] * col[plane x K] */
            orc_sgemm_nn(cout_g, K, plane, 1.0f, omg, plane, col, K, 1.0f, dw + (size_t)g * cout_g * K, K);
        }
    return 0;
}

/* BWBias::backward_cpu, src/ops/bwd_bias.cpp:34-60 */
void orc_bias_backward(int batch, int features, int plane, const float *dy, float *db, float beta)
{
    scale_by(db, (size_t)features, beta);
    for (int b = 0; b < batch; b++)
        for (int f = 0; f < features; f++)
            for (int p = 0; p < plane; p++)
                db[f] += *dy++;
}

/* src/kernels/sgemm.cl:707-710 (also winograd_fwd.cl:216-222,
 * depthwise_separable_conv.cl:96-101) */
void orc_apply_factor(float *y, const float *y_old, size_t n, float factor)
{
    if (factor == 0.0f)
        return;
    for (size_t i = 0; i < n; i++)
        y[i] = y_old[i] * factor + y[i];
}

static double act_f64(double v, int activation)
{
    switch (activation) {
    case ORC_ACT_RELU:
        return v < 0 ? 0 : v;
    case ORC_ACT_TANH:
        return tanh(v);
    case ORC_ACT_SIGMOID:
        return 1.0 / (1.0 + exp(-v));
    case ORC_ACT_RELU6:
        return v < 0 ? 0 : (v > 6 ? 6 : v);
    default:
        return v;
    }
}

/* Textbook NCHW cross-correlation: independent of im2col and sgemm. */
int orc_conv2d_direct_f64(const orc_conv2d_cfg *cfg, const int in_shape[4],
                          const float *x, const float *w, const float *bias,
                          double *y, int activation)
{
    int out[4];
    if (conv_cfg_ok(cfg, in_shape, out) != 0)
        return -1;
    const int B = in_shape[0], C = in_shape[1], H = in_shape[2], W = in_shape[3];
    const int O = out[1], OH = out[2], OW = out[3];
    const int cin_g = C / cfg->groups, cout_g = O / cfg->groups;
    const int kh = cfg->kernel[0], kw = cfg->kernel[1];
    for (int b = 0; b < B; b++)
        for (int o = 0; o < O; o++) {
            int g = o / cout_g;
            for (int oy = 0; oy < OH; oy++)
                for (int ox = 0; ox < OW; ox++) {
                    double acc = bias ? (double)bias[o] : 0.0;
                    for (int ci = 0; ci < cin_g; ci++)
                        for (int ky = 0; ky < kh; ky++) {
                            int iy = oy * cfg->stride[0] - cfg->pad[0] + ky * cfg->dilate[0];
                            if (iy < 0 || iy >= H)
                                continue;
                            for (int kx = 0; kx < kw; kx++) {
                                int ix = ox * cfg->stride[1] - cfg->pad[1] + kx * cfg->dilate[1];
                                if (ix < 0 || ix >= W)
                                    continue;
                                acc += (double)x[(((size_t)b * C + g * cin_g + ci) * H + iy) * W + ix] *
                                       (double)w[(((size_t)o * cin_g + ci) * kh + ky) * kw + kx];
                            }
                        }
                    y[(((size_t)b * O + o) * OH + oy) * OW + ox] = act_f64(acc, activation);
                }
        }
    return 0;
}

/* src/ops/inner_product.cpp:161-184 */
void orc_ip_forward(int batch, int inputs, int outputs, const float *x, const float *w,
                    const float *bias, float *y, int activation)
{
    orc_sgemm_nt(batch, outputs, inputs, 1.0f, x, inputs, w, inputs, 0.0f, y, outputs);
    if (bias) {
        for (int i = 0; i < batch; i++)
            for (int j = 0; j < outputs; j++)
                y[(size_t)i * outputs + j] += 1.0f * bias[j];
    }
    orc_apply_activation(y, (size_t)batch * outputs, activation);
}

/* src/kernels/winograd_fwd.cl:103-135: U = G k G^T with
 * G = [[1,0,0],[1/2,1/2,1/2],[1/2,-1/2,1/2],[0,0,1]], same operation order. */
static void wino_filter_one(const float *k, float *u)
{
    float gk[3][4]; /* gk[j][i] = (G k)[i][j] */
    for (int j = 0; j < 3; j++) {
        gk[j][0] = k[j];
        gk[j][1] = 0.5f * (k[j] + k[3 + j] + k[6 + j]);
        gk[j][2] = 0.5f * (k[j] - k[3 + j] + k[6 + j]);
        gk[j][3] = k[6 + j];
    }
    for (int i = 0; i < 4; i++) {
        u[4 * i + 0] = gk[0][i];
        u[4 * i + 1] = 0.5f * (gk[0][i] + gk[1][i] + gk[2][i]);
        u[4 * i + 2] = 0.5f * (gk[0][i] - gk[1][i] + gk[2][i]);
        u[4 * i + 3] = gk[2][i];
    }
}

/* src/kernels/winograd_fwd.cl:161-175; layout src/core/conv.cpp:229-232 */
void orc_winograd_filter_transform(int cout, int cin, const float *w, float *u)
{
    for (int n = 0; n < cout; n++)
        for (int c = 0; c < cin; c++)
            wino_filter_one(w + ((size_t)n * cin + c) * 9, u + ((size_t)n * cin + c) * 16);
}

/* src/kernels/winograd_fwd.cl:35-69: V = B^T d B,
 * B^T = [[1,0,-1,0],[0,1,1,0],[0,-1,1,0],[0,1,0,-1]] */
static void wino_input_one(const float a[4][4], float v[16])
{
    float bta[4][4];
    for (int j = 0; j < 4; j++) {
        bta[0][j] = a[0][j] - a[2][j];
        bta[1][j] = a[1][j] + a[2][j];
        bta[2][j] = a[2][j] - a[1][j];
        bta[3][j] = a[1][j] - a[3][j];
    }
    for (int i = 0; i < 4; i++) {
        v[4 * i + 0] = bta[i][0] - bta[i][2];
        v[4 * i + 1] = bta[i][1] + bta[i][2];
        v[4 * i + 2] = bta[i][2] - bta[i][1];
        v[4 * i + 3] = bta[i][1] - bta[i][3];
    }
}

/* src/kernels/winograd_fwd.cl:138-158: Y = A^T m A, A^T = [[1,1,1,0],[0,1,-1,-1]] */
static void wino_output_one(const float m[16], float o[4])
{
    float atp[2][4];
    for (int j = 0; j < 4; j++) {
        atp[0][j] = m[0 + j] + m[4 + j] + m[8 + j];
        atp[1][j] = m[4 + j] - m[8 + j] - m[12 + j];
    }
    for (int i = 0; i < 2; i++) {
        o[2 * i + 0] = atp[i][0] + atp[i][1] + atp[i][2];
        o[2 * i + 1] = atp[i][1] - atp[i][2] - atp[i][3];
    }
}

/* src/kernels/winograd_fwd.cl:241-441 and src/core/conv.cpp:233-274 */
int orc_winograd_forward(int B, int C, int N, int H, int W,
                         const float *x, const float *w, const float *bias,
                         float *y, float *u, int activation, float factor)
{
    if (B <= 0 || C <= 0 || N <= 0 || H <= 0 || W <= 0)
        return -1;
    orc_winograd_filter_transform(N, C, w, u);
    const int half_h = (H + 1) / 2, half_w = (W + 1) / 2;
    float *v = (float *)malloc(sizeof(float) * 16 * (size_t)C);
    if (!v)
        return -1;
    for (int b = 0; b < B; b++)
        for (int tr = 0; tr < half_h; tr++)
            for (int tc = 0; tc < half_w; tc++) {
                const int row = 2 * tr, col = 2 * tc;
                for (int c = 0; c < C; c++) {
                    float a[4][4];
                    for (int dr = 0; dr < 4; dr++)
                        for (int dc = 0; dc < 4; dc++) {
                            int yy = row - 1 + dr, xx = col - 1 + dc;
                            a[dr][dc] = (yy >= 0 && yy < H && xx >= 0 && xx < W)
                                            ? x[(((size_t)b * C + c) * H + yy) * W + xx]
                                            : 0.0f;
                        }
                    wino_input_one(a, v + (size_t)c * 16);
                }
                for (int n = 0; n < N; n++) {
                    float m[16];
                    for (int e = 0; e < 16; e++)
                        m[e] = 0.0f;
                    for (int c = 0; c < C; c++) {
                        const float *uu = u + ((size_t)n * C + c) * 16;
                        const float *vv = v + (size_t)c * 16;
                        for (int e = 0; e < 16; e++)
                            m[e] += uu[e] * vv[e];
                    }
                    float o[4];
                    wino_output_one(m, o);
                    for (int e = 0; e < 4; e++) {
                        if (bias)
                            o[e] += bias[n];
                    }
                    orc_apply_activation(o, 4, activation);
                    for (int dr = 0; dr < 2; dr++)
                        for (int dc = 0; dc < 2; dc++) {
                            if (row + dr >= H || col + dc >= W)
                                continue;
                            float *p = y + (((size_t)b * N + n) * H + row + dr) * W + col + dc;
                            float val = o[2 * dr + dc];
                            *p = (factor == 0.0f) ? val : (*p * factor + val);
                        }
                }
            }
    free(v);
    return 0;
}

/* src/kernels/depthwise_separable_conv.cl:20-105 (stride 1, pad = kern/2) */
int orc_depthwise_forward(int B, int C, int H, int W, int kern,
                          const float *x, const float *w, const float *bias,
                          float *y, int activation, float factor)
{
    if (kern % 2 != 1 || kern <= 0)
        return -1;
    const int pad = (kern - 1) / 2;
    for (int b = 0; b < B; b++)
        for (int d = 0; d < C; d++) {
            const float *img = x + ((size_t)b * C + d) * H * W;
            const float *kv = w + (size_t)d * kern * kern;
            float *out = y + ((size_t)b * C + d) * H * W;
            for (int r = 0; r < H; r++)
                for (int c = 0; c < W; c++) {
                    float sum = bias ? bias[d] : 0.0f;
                    for (int drk = 0; drk < kern; drk++)
                        for (int dck = 0; dck < kern; dck++) {
                            int yy = r - pad + drk, xx = c - pad + dck;
                            float iv = (yy >= 0 && yy < H && xx >= 0 && xx < W) ? img[(size_t)yy * W + xx] : 0.0f;
                            sum = fmaf(kv[drk * kern + dck], iv, sum); /* OpenCL mad() */
                        }
                    orc_apply_activation(&sum, 1, activation);
                    float *p = out + (size_t)r * W + c;
                    *p = (factor == 0.0f) ? sum : (factor * *p + sum);
                }
        }
    return 0;
}

/* include/dlprim/core/pool.hpp:17-27 */
int orc_pool_output_size(int in_size, int kernel, int pad, int stride, int ceil_mode)
{
    int padded = in_size + pad * 2;
    if (padded < kernel || stride <= 0)
        return -1;
    int offset = ceil_mode ? (stride - 1) : 0;
    int size = (padded - kernel + offset) / stride + 1;
    if ((size - 1) * stride >= in_size + pad)
        size--;
    return size;
}

/* src/ops/pooling.cpp:281-328; functors :116-145 (max: init -FLT_MAX; avg: sum then
 * * (1/(kh*kw)) on full windows, * (1/(dr*dc)) or / (dr_pad*dc_pad) on clipped ones) */
void orc_pool2d_forward(int planes, int H, int W, int OH, int OW, const int kernel[2], const int pad[2],
                        const int stride[2], int mode, int count_include_pad, const float *x, float *y)
{
    const float full_factor = 1.0f / (kernel[0] * kernel[1]);
    for (int p = 0; p < planes; p++, x += (size_t)H * W, y += (size_t)OH * OW)
        for (int orow = 0; orow < OH; orow++)
            for (int ocol = 0; ocol < OW; ocol++) {
                int row0 = orow * stride[0] - pad[0], col0 = ocol * stride[1] - pad[1];
                int row1 = row0 + kernel[0], col1 = col0 + kernel[1];
                int top = -pad[0] > row0 ? -pad[0] : row0, left = -pad[1] > col0 ? -pad[1] : col0;
                int dr_pad = (row1 < H + pad[0] ? row1 : H + pad[0]) - top;
                int dc_pad = (col1 < W + pad[1] ? col1 : W + pad[1]) - left;
                if (row0 < 0) row0 = 0;
                if (col0 < 0) col0 = 0;
                if (row1 > H) row1 = H;
                if (col1 > W) col1 = W;
                float val = mode == 0 ? -3.402823466e+38f : 0.0f;
                for (int r = row0; r < row1; r++)
                    for (int c = col0; c < col1; c++) {
                        float v = x[(size_t)r * W + c];
                        if (mode == 0)
                            val = val < v ? v : val;
                        else
                            val = val + v;
                    }
                if (mode != 0) {
                    int dr = row1 - row0, dc = col1 - col0;
                    if (dr == kernel[0] && dc == kernel[1])
                        val = val * full_factor;
                    else if (count_include_pad)
                        val = val / (dr_pad * dc_pad);
                    else
                        val = val * (1.0f / (dr * dc));
                }
                y[(size_t)orow * OW + ocol] = val;
            }
}

/* src/ops/pooling.cpp:427-452 */
void orc_global_pool_forward(size_t planes, size_t plane_size, int mode, const float *x, float *y)
{
    const float factor = 1.0f / plane_size;
    for (size_t i = 0; i < planes; i++, x += plane_size) {
        if (mode == 0) {
            float m = x[0];
            for (size_t j = 1; j < plane_size; j++)
                m = m < x[j] ? x[j] : m;
            y[i] = m;
        } else {
            float sum = 0;
            for (size_t j = 0; j < plane_size; j++)
                sum += x[j];
            y[i] = sum * factor;
        }
    }
}

/* src/ops/elementwise.cpp:517-559 (equal shapes: no broadcasting) */
void orc_eltwise_forward(size_t n, int op, float c1, float c2, int activation, const float *a, const float *b, float *c)
{
    const float w = c1 * c2;
    for (size_t i = 0; i < n; i++) {
        float x0 = a[i], x1 = b[i];
        if (op == 0)
            c[i] = x0 * c1 + x1 * c2;
        else if (op == 1)
            c[i] = x0 * x1 * w;
        else {
            float u = x0 * c1, v = x1 * c2;
            c[i] = u < v ? v : u;
        }
    }
    orc_apply_activation(c, n, activation);
}

float orc_bf16_round(float v)
{
    uint32_t bits;
    memcpy(&bits, &v, 4);
    if ((bits & 0x7fffffffu) > 0x7f800000u) { /* NaN stays NaN */
        bits |= 0x00400000u;
        bits &= 0xffff0000u;
    } else {
        uint32_t lsb = (bits >> 16) & 1u;
        bits += 0x7fffu + lsb;
        bits &= 0xffff0000u;
    }
    memcpy(&v, &bits, 4);
    return v;
}

void orc_bf16_round_array(float *p, size_t n)
{
    for (size_t i = 0; i < n; i++)
        p[i] = orc_bf16_round(p[i]);
}
