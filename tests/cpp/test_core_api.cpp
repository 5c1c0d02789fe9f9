// Exercises the C++ header layer the way dlprimitives' own callers use dlprim::core
// (tools/flops.cpp:594-671, src/ops/conv2d.cpp:160-183,235, src/ops/inner_product.cpp:98-104,158):
// Context -> Tensor -> Conv2DForward::create -> enqueue -> ExecutionContext::finish.
// Results are compared with a plain direct convolution computed here in double.
//
//   test_core_api host   : everything that needs no GPU (shapes, exceptions)
//   test_core_api <dev>  : the device checks on HIP device <dev> (default 0)
#include <dlprim/core/activation.hpp>
#include <dlprim/core/bias.hpp>
#include <dlprim/core/common.hpp>
#include <dlprim/core/conv.hpp>
#include <dlprim/core/interpolate.hpp>
#include <dlprim/core/ip.hpp>
#include <dlprim/core/loss.hpp>
#include <dlprim/core/pool.hpp>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <vector>

namespace dp = dlprim;

static int failures = 0;
#define EXPECT(cond)                                                      \
    do {                                                                  \
        if (!(cond)) {                                                    \
            std::printf("FAIL %s:%d %s\n", __FILE__, __LINE__, #cond);    \
            failures++;                                                   \
        }                                                                 \
    } while (0)

static double act(double v, dp::StandardActivations a)
{
    switch (a) {
    case dp::StandardActivations::relu: return v < 0 ? 0 : v;
    case dp::StandardActivations::relu6: return v < 0 ? 0 : (v > 6 ? 6 : v);
    case dp::StandardActivations::tanh: return std::tanh(v);
    case dp::StandardActivations::sigmoid: return 1 / (1 + std::exp(-v));
    default: return v;
    }
}

static void fill(dp::Tensor &t, std::mt19937 &rng, float lo, float hi)
{
    std::uniform_real_distribution<float> d(lo, hi);
    float *p = t.data<float>();
    for (size_t i = 0; i < t.shape().total_size(); i++)
        p[i] = d(rng);
}

static void host_checks()
{
    dp::Convolution2DConfigBase c;
    c.channels_in = 3;
    c.channels_out = 64;
    c.kernel[0] = c.kernel[1] = 7;
    c.stride[0] = c.stride[1] = 2;
    c.pad[0] = c.pad[1] = 3;
    dp::Shape out = dp::core::Conv2DBase::get_output_shape(c, dp::Shape(64, 3, 224, 224));
    EXPECT(out == dp::Shape(64, 64, 112, 112));
    bool thrown = false;
    try {
        dp::core::Conv2DBase::get_output_shape(c, dp::Shape(64, 4, 224, 224));
    } catch (dp::ValidationError const &) {
        thrown = true;
    }
    EXPECT(thrown);
    thrown = false;
    try {
        dp::Context cpu("cpu");
        dp::core::Conv2DSettings s(c, dp::Shape(1, 3, 8, 8), dp::float_data);
        dp::core::Conv2DForward::create(cpu, s, false);
    } catch (dp::NotImplementedError const &) {
        thrown = true;
    }
    EXPECT(thrown);
    dp::Shape s(2, 3, 4);
    EXPECT(s.size() == 3 && s.total_size() == 24 && s.size_no_batch() == 12 && s[-1] == 4);
    EXPECT(dp::size_of_data_type(dp::float_data) == 4 && dp::size_of_data_type(dp::bfloat16_data) == 2);
}

static void conv_case(dp::Context &ctx, dp::ExecutionContext &q, int B, int cin, int cout, int hw, int k, int stride, int pad, int groups,
                      bool bias, dp::StandardActivations a, char const *algo, char const *expect_algo, float factor)
{
    dp::Convolution2DConfigBase c;
    c.channels_in = cin;
    c.channels_out = cout;
    c.kernel[0] = c.kernel[1] = k;
    c.stride[0] = c.stride[1] = stride;
    c.pad[0] = c.pad[1] = pad;
    c.groups = groups;
    dp::Shape in(B, cin, hw, hw);
    dp::core::Conv2DSettings cfg(c, in, dp::float_data);
    std::unique_ptr<dp::core::Conv2DForward> conv = dp::core::Conv2DForward::create(ctx, cfg, bias, a, algo);
    EXPECT(std::strcmp(conv->algo(), expect_algo) == 0);
    dp::Shape os = dp::core::Conv2DBase::get_output_shape(c, in);
    dp::Tensor X(ctx, in), W(ctx, dp::Shape(cout, cin / groups, k, k)), Bv(ctx, dp::Shape(cout)), Y(ctx, os);
    size_t ws_size = conv->workspace();
    dp::Tensor ws(ctx, dp::Shape(ws_size ? ws_size : 1), dp::uint8_data);
    std::mt19937 rng(cin * 1000 + cout + hw);
    fill(X, rng, -1, 1);
    fill(W, rng, -0.3f, 0.3f);
    fill(Bv, rng, -0.1f, 0.1f);
    fill(Y, rng, -1, 1);
    std::vector<float> y_old(Y.data<float>(), Y.data<float>() + os.total_size());
    X.to_device(q);
    W.to_device(q);
    Bv.to_device(q);
    Y.to_device(q);
    conv->enqueue(X, W, bias ? &Bv : nullptr, Y, ws, factor, q);
    Y.to_host(q);
    q.finish();
    const int OH = int(os[2]), OW = int(os[3]), cg = cin / groups, og = cout / groups;
    const float *x = X.data<float>(), *w = W.data<float>(), *bv = Bv.data<float>(), *y = Y.data<float>();
    double worst = 0;
    for (int b = 0; b < B; b++)
        for (int o = 0; o < cout; o++)
            for (int oy = 0; oy < OH; oy++)
                for (int ox = 0; ox < OW; ox++) {
                    double acc = bias ? bv[o] : 0.0;
                    const int g = o / og;
                    for (int ci = 0; ci < cg; ci++)
                        for (int ky = 0; ky < k; ky++)
                            for (int kx = 0; kx < k; kx++) {
                                int iy = oy * stride - pad + ky, ix = ox * stride - pad + kx;
                                if (iy < 0 || iy >= hw || ix < 0 || ix >= hw)
                                    continue;
                                acc += double(x[((size_t(b) * cin + g * cg + ci) * hw + iy) * hw + ix]) * w[((size_t(o) * cg + ci) * k + ky) * k + kx];
                            }
                    size_t idx = ((size_t(b) * cout + o) * OH + oy) * OW + ox;
                    double want = act(acc, a) + double(factor) * y_old[idx];
                    double err = std::fabs(want - y[idx]) / (1.0 + std::fabs(want));
                    if (err > worst)
                        worst = err;
                }
    std::printf("conv %-20s b%d %d->%d @%d k%d s%d g%d factor %.2f : max err %.2e\n", expect_algo, B, cin, cout, hw, k, stride, groups, factor,
                worst);
    EXPECT(worst < 1e-4);
}

// Gradients the way Convolution2D::backward calls them (src/ops/conv2d.cpp:504-555): bias, filter, data,
// each accumulating with its own factor; checked against the definition of the gradients in double.
static void conv_backward_case(dp::Context &ctx, dp::ExecutionContext &q, int B, int cin, int cout, int hw, int k, int stride, int pad, int groups,
                               float factor)
{
    dp::Convolution2DConfigBase c;
    c.channels_in = cin;
    c.channels_out = cout;
    c.kernel[0] = c.kernel[1] = k;
    c.stride[0] = c.stride[1] = stride;
    c.pad[0] = c.pad[1] = pad;
    c.groups = groups;
    dp::Shape in(B, cin, hw, hw);
    dp::core::Conv2DSettings cfg(c, in, dp::float_data);
    dp::Shape os = dp::core::Conv2DBase::get_output_shape(c, in);
    std::unique_ptr<dp::core::Conv2DBackwardData> bd = dp::core::Conv2DBackwardData::create(ctx, cfg);
    std::unique_ptr<dp::core::Conv2DBackwardFilter> bf = dp::core::Conv2DBackwardFilter::create(ctx, cfg);
    std::unique_ptr<dp::core::BiasBackwardFilter> bb = dp::core::BiasBackwardFilter::create(ctx, os);
    const int cg = cin / groups, og = cout / groups, OH = int(os[2]), OW = int(os[3]);
    dp::Tensor X(ctx, in), W(ctx, dp::Shape(cout, cg, k, k)), dY(ctx, os), dX(ctx, in), dW(ctx, dp::Shape(cout, cg, k, k)), dB(ctx, dp::Shape(cout));
    size_t ws_size = std::max(std::max(bd->workspace(), bf->workspace()), bb->workspace());
    dp::Tensor ws(ctx, dp::Shape(ws_size ? ws_size : 1), dp::uint8_data);
    std::mt19937 rng(cin * 77 + cout + hw);
    fill(X, rng, -1, 1);
    fill(W, rng, -0.3f, 0.3f);
    fill(dY, rng, -1, 1);
    fill(dX, rng, -1, 1);
    fill(dW, rng, -1, 1);
    fill(dB, rng, -1, 1);
    std::vector<double> want_dx(in.total_size()), want_dw(W.shape().total_size()), want_db(cout);
    for (size_t i = 0; i < want_dx.size(); i++)
        want_dx[i] = double(factor) * dX.data<float>()[i];
    for (size_t i = 0; i < want_dw.size(); i++)
        want_dw[i] = double(factor) * dW.data<float>()[i];
    for (int i = 0; i < cout; i++)
        want_db[i] = double(factor) * dB.data<float>()[i];
    const float *x = X.data<float>(), *w = W.data<float>(), *dy = dY.data<float>();
    for (int b = 0; b < B; b++)
        for (int o = 0; o < cout; o++)
            for (int oy = 0; oy < OH; oy++)
                for (int ox = 0; ox < OW; ox++) {
                    const double g = dy[((size_t(b) * cout + o) * OH + oy) * OW + ox];
                    want_db[o] += g;
                    const int grp = o / og;
                    for (int ci = 0; ci < cg; ci++)
                        for (int ky = 0; ky < k; ky++)
                            for (int kx = 0; kx < k; kx++) {
                                int iy = oy * stride - pad + ky, ix = ox * stride - pad + kx;
                                if (iy < 0 || iy >= hw || ix < 0 || ix >= hw)
                                    continue;
                                const size_t xi = ((size_t(b) * cin + grp * cg + ci) * hw + iy) * hw + ix;
                                const size_t wi = ((size_t(o) * cg + ci) * k + ky) * k + kx;
                                want_dx[xi] += g * w[wi];
                                want_dw[wi] += g * x[xi];
                            }
                }
    for (dp::Tensor *t : {&X, &W, &dY, &dX, &dW, &dB})
        t->to_device(q);
    bb->enqueue(dY, dB, ws, factor, q);
    bf->enqueue(X, dW, dY, ws, factor, q);
    bd->enqueue(dX, W, dY, ws, factor, q);
    dX.to_host(q);
    dW.to_host(q);
    dB.to_host(q);
    q.finish();
    auto worst = [](std::vector<double> const &want, const float *got) {
        double scale = 1e-6, err = 0;
        for (double v : want)
            scale = std::max(scale, std::fabs(v));
        for (size_t i = 0; i < want.size(); i++)
            err = std::max(err, std::fabs(want[i] - got[i]) / scale);
        return err;
    };
    const double ex = worst(want_dx, dX.data<float>()), ew = worst(want_dw, dW.data<float>()), eb = worst(want_db, dB.data<float>());
    std::printf("conv backward (%s / %s) b%d %d->%d @%d k%d s%d g%d factor %.2f : max err dx %.2e dw %.2e db %.2e\n", bd->algo(), bf->algo(), B, cin, cout,
                hw, k, stride, groups, factor, ex, ew, eb);
    EXPECT(ex < 1e-4 && ew < 1e-4 && eb < 1e-4);
}

// Inner-product gradients as InnerProduct::backward calls them (src/ops/inner_product.cpp:186-240), against the definition in double.
static void ip_backward_case(dp::Context &ctx, dp::ExecutionContext &q, int B, int in, int out, float factor)
{
    dp::core::IPSettings cfg;
    cfg.inputs = in;
    cfg.outputs = out;
    cfg.optimal_batch_size = B;
    std::unique_ptr<dp::core::IPBackwardData> bd = dp::core::IPBackwardData::create(ctx, cfg);
    std::unique_ptr<dp::core::IPBackwardFilter> bf = dp::core::IPBackwardFilter::create(ctx, cfg);
    dp::Tensor X(ctx, dp::Shape(B, in)), W(ctx, dp::Shape(out, in)), dY(ctx, dp::Shape(B, out)), dX(ctx, dp::Shape(B, in)), dW(ctx, dp::Shape(out, in));
    std::mt19937 rng(in * 3 + out);
    fill(X, rng, -1, 1);
    fill(W, rng, -0.3f, 0.3f);
    fill(dY, rng, -1, 1);
    fill(dX, rng, -1, 1);
    fill(dW, rng, -1, 1);
    std::vector<double> want_dx(size_t(B) * in), want_dw(size_t(out) * in);
    for (size_t i = 0; i < want_dx.size(); i++)
        want_dx[i] = double(factor) * dX.data<float>()[i];
    for (size_t i = 0; i < want_dw.size(); i++)
        want_dw[i] = double(factor) * dW.data<float>()[i];
    for (int b = 0; b < B; b++)
        for (int o = 0; o < out; o++) {
            const double g = dY.data<float>()[size_t(b) * out + o];
            for (int i = 0; i < in; i++) {
                want_dx[size_t(b) * in + i] += g * W.data<float>()[size_t(o) * in + i];
                want_dw[size_t(o) * in + i] += g * X.data<float>()[size_t(b) * in + i];
            }
        }
    for (dp::Tensor *t : {&X, &W, &dY, &dX, &dW})
        t->to_device(q);
    for (int rep = 0; rep < 2; rep++) { // the second call reuses the operator's workspace
        if (rep == 1) {
            dX.to_device(q);
            dW.to_device(q);
        }
        bf->enqueue(X, dW, dY, factor, q);
        bd->enqueue(dX, W, dY, factor, q);
    }
    dX.to_host(q);
    dW.to_host(q);
    q.finish();
    double sx = 1e-6, sw = 1e-6, ex = 0, ew = 0;
    for (double v : want_dx)
        sx = std::max(sx, std::fabs(v));
    for (double v : want_dw)
        sw = std::max(sw, std::fabs(v));
    for (size_t i = 0; i < want_dx.size(); i++)
        ex = std::max(ex, std::fabs(want_dx[i] - dX.data<float>()[i]) / sx);
    for (size_t i = 0; i < want_dw.size(); i++)
        ew = std::max(ew, std::fabs(want_dw[i] - dW.data<float>()[i]) / sw);
    std::printf("ip backward b%d %d->%d factor %.2f : max err dx %.2e dw %.2e\n", B, in, out, factor, ex, ew);
    EXPECT(ex < 1e-4 && ew < 1e-4);
}

static void ip_case(dp::Context &ctx, dp::ExecutionContext &q, int B, int in, int out)
{
    dp::core::IPSettings cfg;
    cfg.inputs = in;
    cfg.outputs = out;
    cfg.optimal_batch_size = B;
    std::unique_ptr<dp::core::IPForward> ip = dp::core::IPForward::create(ctx, cfg, true, dp::StandardActivations::relu);
    dp::Tensor X(ctx, dp::Shape(B, in)), W(ctx, dp::Shape(out, in)), Bv(ctx, dp::Shape(out)), Y(ctx, dp::Shape(B, out));
    std::mt19937 rng(in + out);
    fill(X, rng, -1, 1);
    fill(W, rng, -0.1f, 0.1f);
    fill(Bv, rng, -0.1f, 0.1f);
    X.to_device(q);
    W.to_device(q);
    Bv.to_device(q);
    ip->enqueue(X, W, &Bv, Y, q);
    Y.to_host(q);
    q.finish();
    double worst = 0;
    for (int b = 0; b < B; b++)
        for (int o = 0; o < out; o++) {
            double acc = Bv.data<float>()[o];
            for (int i = 0; i < in; i++)
                acc += double(X.data<float>()[size_t(b) * in + i]) * W.data<float>()[size_t(o) * in + i];
            double want = acc < 0 ? 0 : acc;
            double err = std::fabs(want - Y.data<float>()[size_t(b) * out + o]) / (1.0 + std::fabs(want));
            if (err > worst)
                worst = err;
        }
    std::printf("ip b%d %d->%d : max err %.2e\n", B, in, out, worst);
    EXPECT(worst < 1e-4);
}

// Pooling2DForward the way src/ops/pooling.cpp:250-279 drives it: max 3x3 stride 2 pad 1 and global average
static void pool_case(dp::Context &ctx, dp::ExecutionContext &q)
{
    const int B = 2, C = 5, H = 9, W = 11;
    int k[2] = {3, 3}, p[2] = {1, 1}, s[2] = {2, 2};
    const int OH = dp::core::calc_pooling_output_size(H, 3, 1, 2, false), OW = dp::core::calc_pooling_output_size(W, 3, 1, 2, false);
    EXPECT(OH == 5 && OW == 6);
    EXPECT(dp::core::calc_pooling_output_size(7, 3, 1, 3, true) == 3 && dp::core::calc_pooling_output_size(5, 2, 0, 2, true) == 3);
    std::mt19937 rng(7);
    dp::Tensor X(ctx, dp::Shape(B, C, H, W)), Y(ctx, dp::Shape(B, C, OH, OW)), G(ctx, dp::Shape(B, C, 1, 1));
    fill(X, rng, -1, 1);
    X.to_device(q);
    auto mp = dp::core::Pooling2DForward::create_max_pooling(ctx, k, p, s);
    auto gp = dp::core::Pooling2DForward::create_global_avg_pooling(ctx, X.shape());
    EXPECT(mp->workspace() == 0);
    mp->enqueue(X, Y, q);
    gp->enqueue(X, G, q);
    Y.to_host(q);
    G.to_host(q);
    q.finish();
    double worst = 0;
    for (int bc = 0; bc < B * C; bc++) {
        const float *x = X.data<float>() + size_t(bc) * H * W;
        double sum = 0;
        for (int i = 0; i < H * W; i++)
            sum += x[i];
        worst = std::fmax(worst, std::fabs(sum / (H * W) - G.data<float>()[bc]));
        for (int oy = 0; oy < OH; oy++)
            for (int ox = 0; ox < OW; ox++) {
                float m = -INFINITY;
                for (int dy = 0; dy < 3; dy++)
                    for (int dx = 0; dx < 3; dx++) {
                        int yy = oy * 2 - 1 + dy, xx = ox * 2 - 1 + dx;
                        if (yy >= 0 && yy < H && xx >= 0 && xx < W)
                            m = std::fmax(m, x[yy * W + xx]);
                    }
                worst = std::fmax(worst, std::fabs(double(m) - Y.data<float>()[(size_t(bc) * OH + oy) * OW + ox]));
            }
    }
    std::printf("pooling max 3x3/2 + global avg : max err %.2e\n", worst);
    EXPECT(worst < 1e-6);
    bool thrown = false;
    try {
        dp::Tensor bad(ctx, dp::Shape(B, C, OH + 1, OW));
        mp->enqueue(X, bad, q);
    } catch (dp::ValidationError const &) {
        thrown = true;
    }
    EXPECT(thrown);
}

// the free functions of core/activation.hpp, loss.hpp, interpolate.hpp and SliceCopy of common.hpp against plain loops
static void tensor_function_case(dp::Context &ctx, dp::ExecutionContext &q)
{
    std::mt19937 rng(11);
    const int B = 6, C = 9;
    dp::Tensor X(ctx, dp::Shape(B, C)), A(ctx, dp::Shape(B, C)), L(ctx, dp::Shape(B, C)), lbl(ctx, dp::Shape(B), dp::int32_data);
    dp::Tensor rows(ctx, dp::Shape(B)), mean(ctx, dp::Shape(1));
    fill(X, rng, -2, 2);
    for (int b = 0; b < B; b++)
        lbl.data<int>()[b] = (b * 5 + 1) % C;
    X.to_device(q);
    lbl.to_device(q);
    dp::core::activation_forward(X, A, dp::StandardActivations::tanh, q);
    dp::core::softmax_forward(X, L, true, q);
    dp::core::nll_loss_forward(L, lbl, rows, false, 1.0f, q);
    dp::core::nll_loss_forward(L, lbl, mean, true, 1.0f / B, q);
    A.to_host(q);
    L.to_host(q);
    rows.to_host(q);
    mean.to_host(q);
    q.finish();
    double worst = 0, total = 0;
    for (int b = 0; b < B; b++) {
        double sum = 0;
        for (int c = 0; c < C; c++) {
            sum += std::exp(double(X.data<float>()[b * C + c]));
            worst = std::fmax(worst, std::fabs(std::tanh(double(X.data<float>()[b * C + c])) - A.data<float>()[b * C + c]));
        }
        const double want = std::log(sum) - X.data<float>()[b * C + lbl.data<int>()[b]];
        worst = std::fmax(worst, std::fabs(want - rows.data<float>()[b]));
        total += want;
    }
    worst = std::fmax(worst, std::fabs(total / B - mean.data<float>()[0]));
    std::printf("activation, log-softmax, nll loss : max err %.2e\n", worst);
    EXPECT(worst < 1e-5);

    // interpolate2d: nearest by 2 repeats every pixel; bilinear with align_corners keeps the corners
    dp::Tensor img(ctx, dp::Shape(2, 3, 4, 5)), up(ctx, dp::Shape(2, 3, 8, 10)), lin(ctx, dp::Shape(2, 3, 7, 9));
    fill(img, rng, -1, 1);
    img.to_device(q);
    dp::core::interpolate2d(img, up, 2.0, 2.0, dp::InterpolateType::nearest, false, q);
    dp::core::interpolate2d(img, lin, -1, -1, dp::InterpolateType::bilinear, true, q);
    up.to_host(q);
    lin.to_host(q);
    q.finish();
    bool same = true;
    for (int p = 0; p < 6; p++) {
        for (int r = 0; r < 8; r++)
            for (int c = 0; c < 10; c++)
                same = same && up.data<float>()[(p * 8 + r) * 10 + c] == img.data<float>()[(p * 4 + r / 2) * 5 + c / 2];
        same = same && std::fabs(lin.data<float>()[p * 63] - img.data<float>()[p * 20]) < 1e-6 &&
               std::fabs(lin.data<float>()[p * 63 + 62] - img.data<float>()[p * 20 + 19]) < 1e-6;
    }
    EXPECT(same);
    bool thrown = false;
    try {
        dp::core::interpolate2d(img, lin, 2.0, 2.0, dp::InterpolateType::nearest, false, q); // 7 x 9 is not int(4 * 2) x int(5 * 2)
    } catch (dp::ValidationError const &) {
        thrown = true;
    }
    EXPECT(thrown);

    // SliceCopy: channels 1..2 of img into channels 3..4 of a wider tensor
    dp::Tensor wide(ctx, dp::Shape(2, 6, 4, 5));
    std::fill(wide.data<float>(), wide.data<float>() + wide.shape().total_size(), -7.0f);
    wide.to_device(q);
    dp::core::SliceCopy copy(ctx);
    copy.tensor_slice_copy(1, 2, wide, 3, img, 1, 0.0f, q);
    wide.to_host(q);
    q.finish();
    same = true;
    for (int b = 0; b < 2; b++)
        for (int c = 0; c < 6; c++)
            for (int i = 0; i < 20; i++) {
                const float want = (c == 3 || c == 4) ? img.data<float>()[(b * 3 + c - 2) * 20 + i] : -7.0f;
                same = same && wide.data<float>()[(b * 6 + c) * 20 + i] == want;
            }
    EXPECT(same);
    std::printf("interpolate2d, SliceCopy : %s\n", same ? "ok" : "mismatch");
}

int main(int argc, char **argv)
{
    std::string dev = argc > 1 ? argv[1] : "0";
    try {
        host_checks();
        if (dev != "host") {
            dp::Context ctx(dev);
            std::printf("device: %s\n", ctx.name().c_str());
            dp::ExecutionContext q = ctx.make_execution_context();
            using A = dp::StandardActivations;
            conv_case(ctx, q, 2, 16, 32, 14, 3, 1, 1, 1, true, A::relu, "gemm", "gemm", 0.0f);
            conv_case(ctx, q, 2, 16, 32, 14, 3, 1, 1, 1, true, A::relu, "", "winograd", 0.0f);
            conv_case(ctx, q, 2, 3, 8, 20, 7, 2, 3, 1, false, A::identity, "", "gemm", 0.5f);
            conv_case(ctx, q, 3, 24, 24, 9, 3, 2, 1, 24, true, A::relu6, "", "depthwise_separable", 0.0f);
            conv_case(ctx, q, 1, 8, 6, 5, 1, 1, 0, 2, true, A::sigmoid, "winograd", "gemm", 0.0f); // incompatible request -> gemm
            conv_backward_case(ctx, q, 2, 16, 32, 14, 3, 1, 1, 1, 0.0f);
            conv_backward_case(ctx, q, 3, 6, 8, 13, 3, 2, 1, 2, 0.5f);
            conv_backward_case(ctx, q, 2, 24, 24, 9, 3, 1, 1, 24, 1.0f);
            conv_backward_case(ctx, q, 2, 3, 8, 20, 7, 2, 3, 1, 0.0f);
            ip_case(ctx, q, 5, 64, 10);
            ip_backward_case(ctx, q, 5, 64, 10, 0.0f);
            ip_backward_case(ctx, q, 70, 33, 129, 0.5f);
            ip_backward_case(ctx, q, 1, 512, 1000, 1.0f);
            pool_case(ctx, q);
            tensor_function_case(ctx, q);
            // sub-tensor views share memory: run on the second image of a batch-2 tensor
            dp::Tensor big(ctx, dp::Shape(2, 4, 6, 6));
            dp::Tensor second = big.sub_tensor(4 * 6 * 6, dp::Shape(1, 4, 6, 6));
            EXPECT(second.device_offset() == 144 && static_cast<char *>(second.device_ptr()) == static_cast<char *>(big.device_ptr()) + 576);
        }
    } catch (std::exception const &e) {
        std::printf("FAIL exception: %s\n", e.what());
        return 1;
    }
    if (failures) {
        std::printf("%d failure(s)\n", failures);
        return 1;
    }
    std::printf("ok\n");
    return 0;
}
