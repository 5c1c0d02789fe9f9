/*
 * CPU oracle for the convolution forward hot path -- TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of the dlprimitives CPU operators that the
 * HIP kernels are checked against.  It is never linked into, loaded by or
 * called from the shipped library: only tests, the smoke check and the
 * CPU-baseline leg of the benchmark use it, and there only as the checker.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the dlprimitives source tree).
 */
#ifndef DLP_ORACLE_H
#define DLP_ORACLE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* StandardActivations, include/dlprim/definitions.hpp:278-284 */
enum {
    ORC_ACT_IDENTITY = 0,
    ORC_ACT_RELU = 1,
    ORC_ACT_TANH = 2,
    ORC_ACT_SIGMOID = 3,
    ORC_ACT_RELU6 = 4
};

/* Convolution2DConfigBase, include/dlprim/definitions.hpp:313-321 */
typedef struct orc_conv2d_cfg {
    int channels_in;
    int channels_out;
    int kernel[2];
    int stride[2];
    int dilate[2];
    int pad[2];
    int groups;
} orc_conv2d_cfg;

/* Conv2DBase::get_output_shape, src/core/conv.cpp:17-29.
 * Returns 0 on success, -1 when the reference would throw ValidationError. */
int orc_conv2d_output_shape(const orc_conv2d_cfg *cfg, const int in_shape[4], int out_shape[4]);

/* cpu::apply_activation, include/dlprim/cpu/cpu_ops.hpp:17-53 */
void orc_apply_activation(float *p, size_t n, int activation);

/* my_cblas::cblas_sgemm (NoTrans x Trans branch), src/my_blas/my_cblas.cpp:28-39,63-74,88-103
 * C[M x N] = beta*C + alpha * A[M x K] * B[N x K]^T, k innermost, sequential fp32. */
void orc_sgemm_nt(int M, int N, int K, float alpha, const float *A, int lda,
                  const float *B, int ldb, float beta, float *C, int ldc);

/* Convolution2DBase::im2col<Im2ColOp>, generic branch, src/ops/conv2d.cpp:376-409.
 * img: one image, one group: [cin_g][H][W]; mat: [OH*OW][cin_g*KH*KW]. */
void orc_im2col(const orc_conv2d_cfg *cfg, int cin_g, int H, int W, int OH, int OW,
                const float *img, float *mat);

/* Convolution2D::forward_cpu, src/ops/conv2d.cpp:421-425,437-474.
 * x [B,Cin,H,W], w [Cout,Cin/g,KH,KW], bias [Cout] or NULL, y [B,Cout,OH,OW].
 * ws: scratch of at least orc_conv2d_workspace() bytes.
 * Returns 0, or -1 on invalid configuration. */
size_t orc_conv2d_workspace(const orc_conv2d_cfg *cfg, const int in_shape[4]);
int orc_conv2d_forward(const orc_conv2d_cfg *cfg, const int in_shape[4],
                       const float *x, const float *w, const float *bias,
                       float *y, void *ws, int activation);

/* Same arithmetic, images distributed over OpenMP threads (images are
 * independent, src/ops/conv2d.cpp:451); threads <= 0 means all cores.
 * Returns the number of threads used, or -1 on error. */
int orc_conv2d_forward_mt(const orc_conv2d_cfg *cfg, const int in_shape[4],
                          const float *x, const float *w, const float *bias,
                          float *y, int activation, int threads);

/* my_cblas::cblas_sgemm NoTrans x NoTrans and Trans x NoTrans, src/my_blas/my_cblas.cpp:41-62,88-103 */
void orc_sgemm_nn(int M, int N, int K, float alpha, const float *A, int lda,
                  const float *B, int ldb, float beta, float *C, int ldc);
void orc_sgemm_tn(int M, int N, int K, float alpha, const float *A, int lda,
                  const float *B, int ldb, float beta, float *C, int ldc);

/* Convolution2DBase::im2col<Col2ImOp>, src/ops/conv2d.cpp:262-278,376-409: img += the column matrix */
void orc_col2im(const orc_conv2d_cfg *cfg, int cin_g, int H, int W, int OH, int OW,
                float *img, const float *mat);

/* Convolution2D::backward_data_cpu / backward_filter_cpu, src/ops/conv2d.cpp:411-419,426-435,475-498.
 * dx = factor * dx + (gradient with respect to x); dw = factor * dw + (gradient with respect to w).
 * ws: scratch of at least orc_conv2d_workspace() bytes.  Returns 0, or -1 on invalid configuration. */
int orc_conv2d_backward_data(const orc_conv2d_cfg *cfg, const int in_shape[4],
                             const float *dy, const float *w, float *dx, void *ws, float factor);
/* TransposedConvolution2D (src/ops/conv2d.cpp:559-805): output shape (src/core/conv.cpp:31-43) and the CPU forward pass;
 * cfg describes the transposed operator, w is [channels_in][channels_out / groups][kh][kw] */
int orc_tconv2d_output_shape(const orc_conv2d_cfg *cfg, const int in_shape[4], const int output_pad[2], int out_shape[4]);
int orc_tconv2d_forward(const orc_conv2d_cfg *cfg, const int in_shape[4], const int output_pad[2], const float *x, const float *w,
                        const float *bias, float *y, void *ws, int activation);
int orc_conv2d_backward_filter(const orc_conv2d_cfg *cfg, const int in_shape[4],
                               const float *dy, const float *x, float *dw, void *ws, float factor);

/* BWBias::backward_cpu, src/ops/bwd_bias.cpp:34-60: db[f] = beta * db[f] + sum over batch and plane of dy */
void orc_bias_backward(int batch, int features, int plane, const float *dy, float *db, float beta);

/* The device-side `factor` contract, src/kernels/sgemm.cl:707-710:
 * y = factor != 0 ? y_old*factor + v : v, applied to an already activated v. */
void orc_apply_factor(float *y, const float *y_old, size_t n, float factor);

/* Independent 7-loop direct cross-correlation in double precision (textbook
 * definition, no im2col, no GEMM) -- used only to pin orc_conv2d_forward. */
int orc_conv2d_direct_f64(const orc_conv2d_cfg *cfg, const int in_shape[4],
                          const float *x, const float *w, const float *bias,
                          double *y, int activation);

/* InnerProduct::forward_cpu, src/ops/inner_product.cpp:161-184.
 * x [B,In], w [Out,In], bias [Out] or NULL, y [B,Out]. */
void orc_ip_forward(int batch, int inputs, int outputs, const float *x, const float *w,
                    const float *bias, float *y, int activation);

/* Winograd F(2x2,3x3) restated from the reference's OpenCL kernel (the CPU
 * path of the reference has no Winograd):
 *   filter transform  src/kernels/winograd_fwd.cl:103-135,161-175
 *   input transform   src/kernels/winograd_fwd.cl:35-69
 *   output transform  src/kernels/winograd_fwd.cl:138-158
 *   accumulation over channels in ascending order, :313-365
 *   bias, activation, scale_and_add  :406-436, :216-222
 * u: workspace of 16*Cin*Cout floats, layout u[(n*C+c)*16 + 4*i + j]
 * (src/core/conv.cpp:229-232). y is updated in place with `factor`. */
void orc_winograd_filter_transform(int cout, int cin, const float *w, float *u);
int orc_winograd_forward(int B, int C, int N, int H, int W,
                         const float *x, const float *w, const float *bias,
                         float *y, float *u, int activation, float factor);

/* Depthwise KxK stride-1 "conv" kernel, src/kernels/depthwise_separable_conv.cl:20-105:
 * sum starts at bias, fused multiply-add over (drk,dck), activation, scale. */
int orc_depthwise_forward(int B, int C, int H, int W, int kern,
                          const float *x, const float *w, const float *bias,
                          float *y, int activation, float factor);

/* ---- glue operators of the ResNet graphs (next rows after the convolution path) ---- */

/* core::calc_pooling_output_size, include/dlprim/core/pool.hpp:17-27; -1 on invalid */
int orc_pool_output_size(int in_size, int kernel, int pad, int stride, int ceil_mode);

/* Pooling2D::forward_cpu, src/ops/pooling.cpp:281-328 with the reduce functors :116-145.
 * mode 0 = max, 1 = avg; x [planes][H][W] -> y [planes][OH][OW] */
void orc_pool2d_forward(int planes, int H, int W, int OH, int OW, const int kernel[2], const int pad[2],
                        const int stride[2], int mode, int count_include_pad, const float *x, float *y);

/* GlobalPooling::forward_cpu, src/ops/pooling.cpp:427-452; mode 0 = max, 1 = avg */
void orc_global_pool_forward(size_t planes, size_t plane_size, int mode, const float *x, float *y);

/* Elementwise::forward_cpu for equal shapes, src/ops/elementwise.cpp:517-559:
 * op 0: a*c1 + b*c2; op 1: a*b*(c1*c2); op 2: max(a*c1, b*c2); then activation */
void orc_eltwise_forward(size_t n, int op, float c1, float c2, int activation, const float *a, const float *b, float *c);

/* bf16 helpers for the reduced-precision configuration: round-to-nearest-even
 * float -> bfloat16 -> float (the reference has no bf16 path; this defines the
 * storage rounding the HIP kernels use so tests can build matching inputs). */
float orc_bf16_round(float v);
void orc_bf16_round_array(float *p, size_t n);

#ifdef __cplusplus
}
#endif
#endif
