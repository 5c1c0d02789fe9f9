// dlprim::core::IPForward / IPBackwardData / IPBackwardFilter (InnerProduct) on the MI355X: same interface as
// dlprimitives' include/dlprim/core/ip.hpp:19-73, implemented over dlprim_hip.h.
#pragma once
#include <algorithm>
#include <memory>

#include "../context.hpp"
#include "../tensor.hpp"
#include "conv.hpp"

namespace dlprim {
namespace core {

struct IPSettings {
    int inputs = -1;             // number of input features
    int outputs = -1;            // output features
    int optimal_batch_size = -1; // expected batch size
    DataType dtype = float_data;
};

class IPForward {
public:
    virtual ~IPForward() {}
    // y[B,outputs] = act(x[B,inputs...] * w[outputs,inputs]^T + bias[outputs])
    virtual void enqueue(Tensor &x, Tensor &w, Tensor *bias, Tensor &y, ExecutionContext const &e) = 0;
    static std::unique_ptr<IPForward> create(Context &ctx, IPSettings const &config, bool bias,
                                             StandardActivations activation = StandardActivations::identity);
};

namespace details {
class IPForwardHip : public IPForward {
public:
    IPForwardHip(Context &ctx, IPSettings const &cfg, bool bias, StandardActivations activation) : cfg_(cfg)
    {
        if (ctx.is_cpu_context())
            throw NotImplementedError("core::IPForward needs a device context");
        ctx.select();
        dlp_ip_settings s;
        s.inputs = cfg.inputs;
        s.outputs = cfg.outputs;
        s.optimal_batch_size = cfg.optimal_batch_size;
        s.dtype = int(cfg.dtype);
        dlprim::details::check_status(dlp_ip_fwd_create(&s, bias ? 1 : 0, int(activation), &op_));
    }
    ~IPForwardHip() { dlp_ip_fwd_destroy(op_); }
    IPForwardHip(IPForwardHip const &) = delete;
    void operator=(IPForwardHip const &) = delete;

    void enqueue(Tensor &x, Tensor &w, Tensor *bias, Tensor &y, ExecutionContext const &e) override
    {
        DLPRIM_CHECK(int(x.shape().size_no_batch()) == cfg_.inputs);
        DLPRIM_CHECK(y.shape().size() == 2 && int(y.shape()[1]) == cfg_.outputs && y.shape()[0] == x.shape()[0]);
        dlprim::details::check_status(dlp_ip_fwd_enqueue(op_, int(x.shape()[0]), x.device_ptr(), w.device_ptr(),
                                                         bias ? bias->device_ptr() : nullptr, y.device_ptr(), e.stream()));
    }

private:
    IPSettings cfg_;
    dlp_ip_fwd *op_ = nullptr;
};
} // namespace details

inline std::unique_ptr<IPForward> IPForward::create(Context &ctx, IPSettings const &config, bool bias, StandardActivations activation)
{
    return std::unique_ptr<IPForward>(new details::IPForwardHip(ctx, config, bias, activation));
}

// Gradients of the inner product (include/dlprim/core/ip.hpp:47-73 in the reference):
//   dx[B,inputs] = factor * dx + dy[B,outputs] * w[outputs,inputs],   dw[outputs,inputs] = factor * dw + dy^T * x.
// An inner product is a 1x1 convolution over 1x1 images, so both run on the convolution gradients
// (the filter gradient's reduction over "pixels" is then the reduction over the batch).  enqueue has no
// workspace argument: the operator owns one, sized for the batch it sees.
class IPBackwardData {
public:
    virtual ~IPBackwardData() {}
    virtual void enqueue(Tensor &dx, Tensor &w, Tensor &dy, float factor, ExecutionContext const &e) = 0;
    static std::unique_ptr<IPBackwardData> create(Context &ctx, IPSettings const &config);
};

class IPBackwardFilter {
public:
    virtual ~IPBackwardFilter() {}
    virtual void enqueue(Tensor &x, Tensor &dw, Tensor &dy, float factor, ExecutionContext const &e) = 0;
    static std::unique_ptr<IPBackwardFilter> create(Context &ctx, IPSettings const &config);
};

namespace details {
inline Conv2DSettings ip_as_conv(IPSettings const &cfg, size_t batch)
{
    Convolution2DConfigBase c;
    c.channels_in = cfg.inputs;
    c.channels_out = cfg.outputs;
    return Conv2DSettings(c, Shape(batch, size_t(cfg.inputs), 1, 1), cfg.dtype);
}

class IPBackwardDataHip : public IPBackwardData {
public:
    IPBackwardDataHip(Context &ctx, IPSettings const &cfg) : ctx_(ctx), cfg_(cfg) { DLPRIM_CHECK(cfg.inputs > 0 && cfg.outputs > 0); }
    void enqueue(Tensor &dx, Tensor &w, Tensor &dy, float factor, ExecutionContext const &e) override
    {
        const size_t batch = dx.shape()[0];
        DLPRIM_CHECK(dx.shape().total_size() == batch * size_t(cfg_.inputs) && dy.shape().total_size() == batch * size_t(cfg_.outputs));
        if (batch != batch_) {
            op_ = Conv2DBackwardData::create(ctx_, ip_as_conv(cfg_, batch));
            ws_ = Tensor(ctx_, Shape(std::max<size_t>(op_->workspace(), 1)), uint8_data);
            batch_ = batch;
        }
        Tensor dx4 = dx.sub_tensor(0, Shape(batch, size_t(cfg_.inputs), 1, 1), dx.dtype());
        Tensor dy4 = dy.sub_tensor(0, Shape(batch, size_t(cfg_.outputs), 1, 1), dy.dtype());
        Tensor w4 = w.sub_tensor(0, Shape(size_t(cfg_.outputs), size_t(cfg_.inputs), 1, 1), w.dtype());
        op_->enqueue(dx4, w4, dy4, ws_, factor, e);
    }

private:
    Context ctx_;
    IPSettings cfg_;
    size_t batch_ = size_t(-1);
    std::unique_ptr<Conv2DBackwardData> op_;
    Tensor ws_;
};

class IPBackwardFilterHip : public IPBackwardFilter {
public:
    IPBackwardFilterHip(Context &ctx, IPSettings const &cfg) : ctx_(ctx), cfg_(cfg) { DLPRIM_CHECK(cfg.inputs > 0 && cfg.outputs > 0); }
    void enqueue(Tensor &x, Tensor &dw, Tensor &dy, float factor, ExecutionContext const &e) override
    {
        const size_t batch = x.shape()[0];
        DLPRIM_CHECK(x.shape().total_size() == batch * size_t(cfg_.inputs) && dy.shape().total_size() == batch * size_t(cfg_.outputs));
        if (batch != batch_) {
            op_ = Conv2DBackwardFilter::create(ctx_, ip_as_conv(cfg_, batch));
            ws_ = Tensor(ctx_, Shape(std::max<size_t>(op_->workspace(), 1)), uint8_data);
            batch_ = batch;
        }
        Tensor x4 = x.sub_tensor(0, Shape(batch, size_t(cfg_.inputs), 1, 1), x.dtype());
        Tensor dy4 = dy.sub_tensor(0, Shape(batch, size_t(cfg_.outputs), 1, 1), dy.dtype());
        Tensor dw4 = dw.sub_tensor(0, Shape(size_t(cfg_.outputs), size_t(cfg_.inputs), 1, 1), dw.dtype());
        op_->enqueue(x4, dw4, dy4, ws_, factor, e);
    }

private:
    Context ctx_;
    IPSettings cfg_;
    size_t batch_ = size_t(-1);
    std::unique_ptr<Conv2DBackwardFilter> op_;
    Tensor ws_;
};
} // namespace details

inline std::unique_ptr<IPBackwardData> IPBackwardData::create(Context &ctx, IPSettings const &config)
{
    if (!ctx.is_hip_context())
        throw ValidationError("core::IPBackwardData needs a device context");
    return std::unique_ptr<IPBackwardData>(new details::IPBackwardDataHip(ctx, config));
}

inline std::unique_ptr<IPBackwardFilter> IPBackwardFilter::create(Context &ctx, IPSettings const &config)
{
    if (!ctx.is_hip_context())
        throw ValidationError("core::IPBackwardFilter needs a device context");
    return std::unique_ptr<IPBackwardFilter>(new details::IPBackwardFilterHip(ctx, config));
}

} // namespace core
} // namespace dlprim
