/* Runs every function of the CPU oracle on small, awkward shapes (odd sizes, padding larger than the image edge, groups,
 * dilation, strides, empty batches) so that an AddressSanitizer / UndefinedBehaviorSanitizer build of the oracle sees each
 * loop nest touch its first and last element.  No values are checked here (tests/test_oracle.py does that): the sanitizers
 * are the assertion.  Built by `make -C tests/cpp asan` together with oracle/dlp_oracle.c. */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../oracle/dlp_oracle.h"

static unsigned state = 12345u;
static float rnd(void)
{
    state = state * 1664525u + 1013904223u;
    return (float)((state >> 8) & 0xffff) / 32768.0f - 1.0f;
}
static float *tensor(size_t n)
{
    float *p = (float *)malloc((n ? n : 1) * sizeof(float)); /* exact size: one element past the end is a report */
    for (size_t i = 0; i < n; i++)
        p[i] = rnd();
    return p;
}

static int conv_case(int B, int cin, int cout, int kh, int kw, int s, int d, int ph, int pw, int g, int H, int W, int act)
{
    orc_conv2d_cfg c;
    memset(&c, 0, sizeof c);
    c.channels_in = cin;
    c.channels_out = cout;
    c.kernel[0] = kh, c.kernel[1] = kw;
    c.stride[0] = c.stride[1] = s;
    c.dilate[0] = c.dilate[1] = d;
    c.pad[0] = ph, c.pad[1] = pw;
    c.groups = g;
    const int in[4] = {B, cin, H, W};
    int out[4];
    if (orc_conv2d_output_shape(&c, in, out) != 0)
        return 1;
    const size_t nx = (size_t)B * cin * H * W, ny = (size_t)out[0] * out[1] * out[2] * out[3], nw = (size_t)cout * (cin / g) * kh * kw;
    float *x = tensor(nx), *w = tensor(nw), *b = tensor((size_t)cout), *y = tensor(ny), *dy = tensor(ny), *dx = tensor(nx), *dw = tensor(nw);
    double *y64 = (double *)malloc((ny ? ny : 1) * sizeof(double));
    void *ws = malloc(orc_conv2d_workspace(&c, in) + 1);
    int rc = orc_conv2d_forward(&c, in, x, w, b, y, ws, act);
    rc |= orc_conv2d_forward(&c, in, x, w, NULL, y, ws, 0);
    rc |= orc_conv2d_forward_mt(&c, in, x, w, b, y, act, 3) < 0;
    rc |= orc_conv2d_direct_f64(&c, in, x, w, b, y64, act);
    rc |= orc_conv2d_backward_data(&c, in, dy, w, dx, ws, 0.0f);
    rc |= orc_conv2d_backward_data(&c, in, dy, w, dx, ws, 0.5f);
    rc |= orc_conv2d_backward_filter(&c, in, dy, x, dw, ws, 0.0f);
    rc |= orc_conv2d_backward_filter(&c, in, dy, x, dw, ws, -1.0f);
    orc_bias_backward(out[0], out[1], out[2] * out[3], dy, b, 0.0f);
    orc_bias_backward(out[0], out[1], out[2] * out[3], dy, b, 1.0f);
    orc_apply_factor(y, dy, ny, 0.25f);
    orc_apply_activation(y, ny, act);
    free(x), free(w), free(b), free(y), free(dy), free(dx), free(dw), free(y64), free(ws);
    return rc;
}

static int tconv_case(int B, int cin, int cout, int k, int s, int p, int op, int g, int H, int W)
{
    orc_conv2d_cfg c;
    memset(&c, 0, sizeof c);
    c.channels_in = cin;
    c.channels_out = cout;
    c.kernel[0] = c.kernel[1] = k;
    c.stride[0] = c.stride[1] = s;
    c.dilate[0] = c.dilate[1] = 1;
    c.pad[0] = c.pad[1] = p;
    c.groups = g;
    const int in[4] = {B, cin, H, W}, opad[2] = {op, op};
    int out[4];
    if (orc_tconv2d_output_shape(&c, in, opad, out) != 0)
        return 1;
    const size_t nx = (size_t)B * cin * H * W, ny = (size_t)out[0] * out[1] * out[2] * out[3], nw = (size_t)cin * (cout / g) * k * k;
    float *x = tensor(nx), *w = tensor(nw), *b = tensor((size_t)cout), *y = tensor(ny);
    /* the forward pass of the transposed operator is the data gradient of the convolution with the channels swapped */
    orc_conv2d_cfg cc = c;
    cc.channels_in = cout;
    cc.channels_out = cin;
    void *ws = malloc(orc_conv2d_workspace(&cc, out) + 1);
    const int rc = orc_tconv2d_forward(&c, in, opad, x, w, b, y, ws, 1);
    free(x), free(w), free(b), free(y), free(ws);
    return rc;
}

int main(void)
{
    int rc = 0;
    rc |= conv_case(2, 3, 5, 3, 3, 1, 1, 1, 1, 1, 7, 9, 1);
    rc |= conv_case(1, 4, 6, 5, 3, 2, 1, 2, 1, 2, 11, 8, 4);
    rc |= conv_case(3, 6, 6, 3, 3, 2, 1, 1, 1, 6, 9, 9, 2);   /* depthwise, stride 2, odd size */
    rc |= conv_case(1, 2, 4, 3, 3, 1, 2, 2, 2, 1, 6, 5, 3);   /* dilation */
    rc |= conv_case(2, 8, 4, 1, 1, 2, 1, 0, 0, 1, 5, 5, 0);   /* 1x1 stride 2 */
    rc |= conv_case(1, 1, 1, 7, 7, 2, 1, 3, 3, 1, 8, 8, 1);
    rc |= conv_case(0, 3, 4, 3, 3, 1, 1, 1, 1, 1, 4, 4, 0);   /* empty batch */
    rc |= tconv_case(2, 4, 6, 3, 2, 1, 1, 2, 5, 4);
    rc |= tconv_case(1, 3, 2, 4, 2, 1, 0, 1, 3, 3);
    {   /* the three GEMM forms on sizes off every unroll */
        float *a = tensor(7 * 5), *b = tensor(5 * 9), *c = tensor(7 * 9);
        orc_sgemm_nt(7, 9, 5, 1.0f, a, 5, b, 5, 0.0f, c, 9);
        orc_sgemm_nn(7, 9, 5, 0.5f, a, 5, b, 9, 1.0f, c, 9);
        orc_sgemm_tn(5, 9, 7, 1.0f, a, 5, c, 9, 0.0f, b, 9);
        free(a), free(b), free(c);
    }
    {   /* inner product */
        float *x = tensor(3 * 11), *w = tensor(5 * 11), *b = tensor(5), *y = tensor(3 * 5);
        orc_ip_forward(3, 11, 5, x, w, b, y, 1);
        orc_ip_forward(3, 11, 5, x, w, NULL, y, 0);
        free(x), free(w), free(b), free(y);
    }
    {   /* Winograd on odd sizes, depthwise of the reference's kernel sizes */
        const int B = 2, C = 3, N = 5, H = 7, W = 5;
        float *x = tensor((size_t)B * C * H * W), *w = tensor((size_t)N * C * 9), *b = tensor(N), *y = tensor((size_t)B * N * H * W), *u = tensor((size_t)16 * C * N);
        orc_winograd_filter_transform(N, C, w, u);
        rc |= orc_winograd_forward(B, C, N, H, W, x, w, b, y, u, 1, 0.0f);
        rc |= orc_winograd_forward(B, C, N, H, W, x, w, NULL, y, u, 0, 0.5f);
        free(x), free(w), free(b), free(y), free(u);
        for (int k = 1; k <= 7; k += 2) {
            float *dx = tensor((size_t)2 * 4 * 6 * 9), *dwt = tensor((size_t)4 * k * k), *db = tensor(4), *dyy = tensor((size_t)2 * 4 * 6 * 9);
            rc |= orc_depthwise_forward(2, 4, 6, 9, k, dx, dwt, db, dyy, 4, 0.0f);
            rc |= orc_depthwise_forward(2, 4, 6, 9, k, dx, dwt, NULL, dyy, 0, 2.0f);
            free(dx), free(dwt), free(db), free(dyy);
        }
    }
    {   /* pooling with padding, ceil mode, both modes; global pooling; elementwise; bf16 rounding */
        const int k[2] = {3, 2}, p[2] = {1, 0}, s[2] = {2, 2};
        for (int ceil_mode = 0; ceil_mode < 2; ceil_mode++) {
            const int H = 7, W = 6, OH = orc_pool_output_size(H, k[0], p[0], s[0], ceil_mode), OW = orc_pool_output_size(W, k[1], p[1], s[1], ceil_mode);
            float *x = tensor((size_t)5 * H * W), *y = tensor((size_t)5 * OH * OW);
            for (int mode = 0; mode < 2; mode++)
                for (int cip = 0; cip < 2; cip++)
                    orc_pool2d_forward(5, H, W, OH, OW, k, p, s, mode, cip, x, y);
            free(x), free(y);
        }
        float *x = tensor(6 * 13), *y = tensor(6), *c = tensor(6 * 13);
        orc_global_pool_forward(6, 13, 0, x, y);
        orc_global_pool_forward(6, 13, 1, x, y);
        for (int op = 0; op < 3; op++)
            orc_eltwise_forward(6 * 13, op, 0.5f, -2.0f, op, x, x, c);
        orc_bf16_round_array(c, 6 * 13);
        c[0] = orc_bf16_round(3.14159f);
        for (int act = 0; act <= 4; act++)
            orc_apply_activation(x, 6 * 13, act);
        free(x), free(y), free(c);
    }
    printf(rc == 0 ? "oracle_sanitize: ok\n" : "oracle_sanitize: a call reported an error\n");
    return rc != 0;
}
