// dlprim::core::Conv2DForward / Conv2DBackwardData / Conv2DBackwardFilter on the MI355X: same interface
// as dlprimitives' include/dlprim/core/conv.hpp:17-80, implemented over the C ABI in dlprim_hip.h.
#pragma once
#include <memory>
#include <string>

#include "../context.hpp"
#include "../tensor.hpp"

namespace dlprim {
namespace core {

struct Conv2DSettings : public Convolution2DConfigBase {
    Conv2DSettings(Conv2DSettings const &) = default;
    Conv2DSettings(Convolution2DConfigBase const &v, Shape s, DataType dt) : Convolution2DConfigBase(v), shape(s), dtype(dt) {}

    Shape shape; // input shape; the batch is a hint rather than a requirement
    DataType dtype = float_data;
};

namespace details {
inline dlp_conv2d_settings to_c(Convolution2DConfigBase const &c, Shape const &in, DataType dt)
{
    DLPRIM_CHECK(in.size() == 4);
    dlp_conv2d_settings s;
    s.channels_in = c.channels_in;
    s.channels_out = c.channels_out;
    for (int i = 0; i < 2; i++) {
        s.kernel[i] = c.kernel[i];
        s.stride[i] = c.stride[i];
        s.dilate[i] = c.dilate[i];
        s.pad[i] = c.pad[i];
    }
    s.groups = c.groups;
    for (int i = 0; i < 4; i++)
        s.shape[i] = int(in[i]);
    s.dtype = int(dt);
    return s;
}
} // namespace details

class Conv2DBase {
public:
    virtual ~Conv2DBase() {}
    virtual char const *algo() const = 0;
    virtual size_t workspace() { return 0; }
    static Shape get_output_shape(Convolution2DConfigBase const &config, Shape const &in)
    {
        dlp_conv2d_settings s = details::to_c(config, in, float_data);
        int out[4];
        dlprim::details::check_status(dlp_conv2d_output_shape(&s, s.shape, out));
        return Shape(size_t(out[0]), out[1], out[2], out[3]);
    }
    // output shape of the transposed convolution (src/core/conv.cpp:31-43 in the reference)
    static Shape get_output_shape_transposed(Convolution2DConfigBase const &config, Shape const &in, int output_pad[2])
    {
        dlp_conv2d_settings s = details::to_c(config, in, float_data);
        int out[4];
        dlprim::details::check_status(dlp_conv2d_transposed_output_shape(&s, s.shape, output_pad, out));
        return Shape(size_t(out[0]), out[1], out[2], out[3]);
    }
};

class Conv2DForward : public Conv2DBase {
public:
    virtual ~Conv2DForward() {}
    // y = factor != 0 ? factor * y + act(conv(x, w) + bias) : act(conv(x, w) + bias)
    // ws: uint8 tensor of at least workspace() bytes; asynchronous on e
    virtual void enqueue(Tensor &x, Tensor &w, Tensor *bias, Tensor &y, Tensor &ws, float factor, ExecutionContext const &e) = 0;
    // Not in the reference (default bodies, so that a class written against the reference's interface, which has
    // enqueue alone, still compiles): weights that stay constant between calls are transformed once into `packed`
    // (uint8 tensor of packed_size() bytes, may be empty when that is 0) and enqueue_packed reads them
    // from there; ws is then per-call scratch only (workspace() bytes are enough, operators that run
    // one after another may share it).  The defaults keep nothing: packed_size() is 0, pack() does
    // nothing and enqueue_packed() is enqueue().
    virtual size_t packed_size() { return 0; }
    virtual void pack(Tensor & /*w*/, Tensor & /*packed*/, ExecutionContext const & /*e*/) {}
    virtual void enqueue_packed(Tensor &x, Tensor &w, Tensor & /*packed*/, Tensor *bias, Tensor &y, Tensor &ws, float factor,
                                ExecutionContext const &e)
    {
        enqueue(x, w, bias, y, ws, factor, e);
    }
    // Not in the reference: y = act(conv + bias + factor * y) instead of factor * y + act(conv + bias), so that a
    // residual sum whose other branch is already in y costs no pass of its own.  The default refuses.
    virtual void accumulate_before_activation(bool on)
    {
        if (on)
            throw NotImplementedError("accumulate_before_activation is not implemented by this Conv2DForward");
    }
    // Not in the reference (its tensors are NCHW throughout): x is read / y is written as [image][row][column][channel]
    // (dlp_conv2d_fwd_set_channels_last; shapes stay [B, C, H, W]).  The default refuses.
    virtual void channels_last(bool x, bool y)
    {
        if (x || y)
            throw NotImplementedError("channels_last is not implemented by this Conv2DForward");
    }
    // Not in the reference (the pooling is an operator of its own there): y becomes the max pooling of the convolution's output,
    // [B, channels_out, PH, PW], and the convolution's own output is never written (dlp_conv2d_fwd_fuse_max_pool: the bfloat16
    // 7x7 stride-2 stem and its 3x3 stride-2 pad-1 pooling).  The default refuses.
    virtual void fuse_max_pool(int kernel, int stride, int pad, bool ceil_mode)
    {
        (void)kernel, (void)stride, (void)pad, (void)ceil_mode;
        throw NotImplementedError("fuse_max_pool is not implemented by this Conv2DForward");
    }
    static std::unique_ptr<Conv2DForward> create(Context &ctx, Conv2DSettings const &config, bool bias,
                                                 StandardActivations activation = StandardActivations::identity,
                                                 std::string const &algo = std::string());
};

namespace details {
class Conv2DForwardHip : public Conv2DForward {
public:
    Conv2DForwardHip(Context &ctx, Conv2DSettings const &config, bool bias, StandardActivations activation, std::string const &algo)
    {
        if (ctx.is_cpu_context())
            throw NotImplementedError("core::Conv2DForward needs a device context");
        ctx.select();
        dlp_conv2d_settings s = to_c(config, config.shape, config.dtype);
        dlprim::details::check_status(dlp_conv2d_fwd_create(&s, bias ? 1 : 0, int(activation), algo.c_str(), &op_));
    }
    ~Conv2DForwardHip() { dlp_conv2d_fwd_destroy(op_); }
    Conv2DForwardHip(Conv2DForwardHip const &) = delete;
    void operator=(Conv2DForwardHip const &) = delete;

    char const *algo() const override { return dlp_conv2d_fwd_algo(op_); }
    size_t workspace() override { return dlp_conv2d_fwd_workspace(op_); }
    void enqueue(Tensor &x, Tensor &w, Tensor *bias, Tensor &y, Tensor &ws, float factor, ExecutionContext const &e) override
    {
        DLPRIM_CHECK(x.shape().size() == 4);
        int xs[4];
        for (int i = 0; i < 4; i++)
            xs[i] = int(x.shape()[i]);
        const size_t ws_bytes = workspace() ? ws.memory_size() : 0;
        dlprim::details::check_status(dlp_conv2d_fwd_enqueue(op_, xs, x.device_ptr(), w.device_ptr(), bias ? bias->device_ptr() : nullptr,
                                                             y.device_ptr(), ws_bytes ? ws.device_ptr() : nullptr, ws_bytes, factor,
                                                             e.stream()));
    }

    void accumulate_before_activation(bool on) override { dlprim::details::check_status(dlp_conv2d_fwd_set_accumulate_first(op_, on ? 1 : 0)); }
    void channels_last(bool x, bool y) override { dlprim::details::check_status(dlp_conv2d_fwd_set_channels_last(op_, x ? 1 : 0, y ? 1 : 0)); }
    void fuse_max_pool(int kernel, int stride, int pad, bool ceil_mode) override
    {
        dlprim::details::check_status(dlp_conv2d_fwd_fuse_max_pool(op_, kernel, stride, pad, ceil_mode ? 1 : 0));
    }
    size_t packed_size() override { return dlp_conv2d_fwd_packed_bytes(op_); }
    void pack(Tensor &w, Tensor &packed, ExecutionContext const &e) override
    {
        dlprim::details::check_status(dlp_conv2d_fwd_pack(op_, w.device_ptr(), packed_size() ? packed.device_ptr() : nullptr, e.stream()));
    }
    void enqueue_packed(Tensor &x, Tensor &w, Tensor &packed, Tensor *bias, Tensor &y, Tensor &ws, float factor, ExecutionContext const &e) override
    {
        DLPRIM_CHECK(x.shape().size() == 4);
        int xs[4];
        for (int i = 0; i < 4; i++)
            xs[i] = int(x.shape()[i]);
        const size_t ws_bytes = workspace() ? ws.memory_size() : 0;
        dlprim::details::check_status(dlp_conv2d_fwd_enqueue_packed(op_, xs, x.device_ptr(), w.device_ptr(), packed_size() ? packed.device_ptr() : nullptr,
                                                                    bias ? bias->device_ptr() : nullptr, y.device_ptr(),
                                                                    ws_bytes ? ws.device_ptr() : nullptr, ws_bytes, factor, e.stream()));
    }

private:
    dlp_conv2d_fwd *op_ = nullptr;
};
} // namespace details

// dx = factor * dx + gradient with respect to x (include/dlprim/core/conv.hpp:60-68 in the reference)
class Conv2DBackwardData : public Conv2DBase {
public:
    virtual ~Conv2DBackwardData() {}
    virtual void enqueue(Tensor &dx, Tensor &w, Tensor &dy, Tensor &ws, float factor, ExecutionContext const &e) = 0;
    static std::unique_ptr<Conv2DBackwardData> create(Context &ctx, Conv2DSettings const &config, std::string const &algo = std::string());
};

// dw = factor * dw + gradient with respect to the filter (include/dlprim/core/conv.hpp:70-78 in the reference)
class Conv2DBackwardFilter : public Conv2DBase {
public:
    virtual ~Conv2DBackwardFilter() {}
    virtual void enqueue(Tensor &x, Tensor &dw, Tensor &dy, Tensor &ws, float factor, ExecutionContext const &e) = 0;
    static std::unique_ptr<Conv2DBackwardFilter> create(Context &ctx, Conv2DSettings const &config, std::string const &algo = std::string());
};

// The device half of the reference's TransposedConvolution2D operator (include/dlprim/ops/conv2d.hpp:96-171,
// TransposedConvolution2D::forward, src/ops/conv2d.cpp:741-805): y = act(transposed convolution of x with
// w [channels_in, channels_out / groups, kh, kw] + bias).  `config` describes the transposed operator (shape = shape of x).
class TransposedConv2DForward : public Conv2DBase {
public:
    TransposedConv2DForward(Context &ctx, Conv2DSettings const &config, int const output_pad[2], bool bias,
                            StandardActivations activation = StandardActivations::identity, std::string const &algo = std::string())
    {
        if (!ctx.is_hip_context())
            throw ValidationError("core::TransposedConv2DForward needs a device context");
        ctx.select();
        dlp_conv2d_settings s = details::to_c(config, config.shape, config.dtype);
        dlprim::details::check_status(dlp_tconv2d_fwd_create(&s, output_pad, bias ? 1 : 0, int(activation), algo.c_str(), &op_));
    }
    ~TransposedConv2DForward() { dlp_tconv2d_fwd_destroy(op_); }
    TransposedConv2DForward(TransposedConv2DForward const &) = delete;
    void operator=(TransposedConv2DForward const &) = delete;
    char const *algo() const override { return dlp_tconv2d_fwd_algo(op_); }
    size_t workspace() override { return dlp_tconv2d_fwd_workspace(op_); }
    void enqueue(Tensor &x, Tensor &w, Tensor *bias, Tensor &y, Tensor &ws, ExecutionContext const &e)
    {
        DLPRIM_CHECK(x.shape().size() == 4);
        int xs[4];
        for (int i = 0; i < 4; i++)
            xs[i] = int(x.shape()[i]);
        const size_t ws_bytes = workspace() ? ws.memory_size() : 0;
        dlprim::details::check_status(dlp_tconv2d_fwd_enqueue(op_, xs, x.device_ptr(), w.device_ptr(), bias ? bias->device_ptr() : nullptr, y.device_ptr(),
                                                              ws_bytes ? ws.device_ptr() : nullptr, ws_bytes, e.stream()));
    }

private:
    dlp_tconv2d_fwd *op_ = nullptr;
};

// A depthwise 3x3 convolution and the pointwise (1x1) convolution behind it as one operator: the tensor between them never
// reaches memory.  No counterpart in the reference, which runs two Conv2DForward operators; `config` describes the depthwise
// layer (groups = channels_in = channels_out, kernel 3, pad 1, stride 1 or 2, shape = shape of x).  supported() tells whether
// the device code takes the pair (and is faster than the two operators there); the constructor throws NotImplementedError otherwise.
class DepthwisePointwiseForward {
public:
    static bool supported(Conv2DSettings const &config, StandardActivations dw_activation, int channels_out, StandardActivations pw_activation)
    {
        dlp_conv2d_settings s = details::to_c(config, config.shape, config.dtype);
        return dlp_dwpw_fwd_supported(&s, int(dw_activation), channels_out, int(pw_activation)) != 0;
    }
    DepthwisePointwiseForward(Context &ctx, Conv2DSettings const &config, bool dw_bias, StandardActivations dw_activation, int channels_out,
                              bool pw_bias, StandardActivations pw_activation)
    {
        if (!ctx.is_hip_context())
            throw ValidationError("core::DepthwisePointwiseForward needs a device context");
        ctx.select();
        dlp_conv2d_settings s = details::to_c(config, config.shape, config.dtype);
        dlprim::details::check_status(dlp_dwpw_fwd_create(&s, dw_bias ? 1 : 0, int(dw_activation), channels_out, pw_bias ? 1 : 0, int(pw_activation), &op_));
    }
    ~DepthwisePointwiseForward() { dlp_dwpw_fwd_destroy(op_); }
    DepthwisePointwiseForward(DepthwisePointwiseForward const &) = delete;
    void operator=(DepthwisePointwiseForward const &) = delete;
    // y = pw_act(conv + pw_bias + factor * y) instead of factor * y + pw_act(conv + pw_bias)
    void accumulate_before_activation(bool on) { dlprim::details::check_status(dlp_dwpw_fwd_set_accumulate_first(op_, on ? 1 : 0)); }
    void enqueue(Tensor &x, Tensor &dw_w, Tensor *dw_bias, Tensor &pw_w, Tensor *pw_bias, Tensor &y, float factor, ExecutionContext const &e)
    {
        DLPRIM_CHECK(x.shape().size() == 4);
        int xs[4];
        for (int i = 0; i < 4; i++)
            xs[i] = int(x.shape()[i]);
        dlprim::details::check_status(dlp_dwpw_fwd_enqueue(op_, xs, x.device_ptr(), dw_w.device_ptr(), dw_bias ? dw_bias->device_ptr() : nullptr,
                                                           pw_w.device_ptr(), pw_bias ? pw_bias->device_ptr() : nullptr, y.device_ptr(), factor, e.stream()));
    }

private:
    dlp_dwpw_fwd *op_ = nullptr;
};

namespace details {
inline void shape4(Shape const &s, int (&out)[4])
{
    DLPRIM_CHECK(s.size() == 4);
    for (int i = 0; i < 4; i++)
        out[i] = int(s[i]);
}

class Conv2DBackwardDataHip : public Conv2DBackwardData {
public:
    Conv2DBackwardDataHip(Context &ctx, Conv2DSettings const &config, std::string const &algo)
    {
        if (!ctx.is_hip_context())
            throw ValidationError("core::Conv2DBackwardData needs a device context");
        ctx.select();
        dlp_conv2d_settings s = to_c(config, config.shape, config.dtype);
        dlprim::details::check_status(dlp_conv2d_bwd_data_create(&s, algo.c_str(), &op_));
    }
    ~Conv2DBackwardDataHip() { dlp_conv2d_bwd_data_destroy(op_); }
    Conv2DBackwardDataHip(Conv2DBackwardDataHip const &) = delete;
    void operator=(Conv2DBackwardDataHip const &) = delete;
    char const *algo() const override { return dlp_conv2d_bwd_data_algo(op_); }
    size_t workspace() override { return dlp_conv2d_bwd_data_workspace(op_); }
    void enqueue(Tensor &dx, Tensor &w, Tensor &dy, Tensor &ws, float factor, ExecutionContext const &e) override
    {
        int xs[4];
        shape4(dx.shape(), xs);
        const size_t ws_bytes = workspace() ? ws.memory_size() : 0;
        dlprim::details::check_status(dlp_conv2d_bwd_data_enqueue(op_, xs, dx.device_ptr(), w.device_ptr(), dy.device_ptr(),
                                                                  ws_bytes ? ws.device_ptr() : nullptr, ws_bytes, factor, e.stream()));
    }

private:
    dlp_conv2d_bwd_data *op_ = nullptr;
};

class Conv2DBackwardFilterHip : public Conv2DBackwardFilter {
public:
    Conv2DBackwardFilterHip(Context &ctx, Conv2DSettings const &config, std::string const &algo)
    {
        if (!ctx.is_hip_context())
            throw ValidationError("core::Conv2DBackwardFilter needs a device context");
        ctx.select();
        dlp_conv2d_settings s = to_c(config, config.shape, config.dtype);
        dlprim::details::check_status(dlp_conv2d_bwd_filter_create(&s, algo.c_str(), &op_));
    }
    ~Conv2DBackwardFilterHip() { dlp_conv2d_bwd_filter_destroy(op_); }
    Conv2DBackwardFilterHip(Conv2DBackwardFilterHip const &) = delete;
    void operator=(Conv2DBackwardFilterHip const &) = delete;
    char const *algo() const override { return dlp_conv2d_bwd_filter_algo(op_); }
    size_t workspace() override { return dlp_conv2d_bwd_filter_workspace(op_); }
    void enqueue(Tensor &x, Tensor &dw, Tensor &dy, Tensor &ws, float factor, ExecutionContext const &e) override
    {
        int xs[4];
        shape4(x.shape(), xs);
        const size_t ws_bytes = workspace() ? ws.memory_size() : 0;
        dlprim::details::check_status(dlp_conv2d_bwd_filter_enqueue(op_, xs, x.device_ptr(), dw.device_ptr(), dy.device_ptr(),
                                                                    ws_bytes ? ws.device_ptr() : nullptr, ws_bytes, factor, e.stream()));
    }

private:
    dlp_conv2d_bwd_filter *op_ = nullptr;
};
} // namespace details

inline std::unique_ptr<Conv2DBackwardData> Conv2DBackwardData::create(Context &ctx, Conv2DSettings const &config, std::string const &algo)
{
    return std::unique_ptr<Conv2DBackwardData>(new details::Conv2DBackwardDataHip(ctx, config, algo));
}

inline std::unique_ptr<Conv2DBackwardFilter> Conv2DBackwardFilter::create(Context &ctx, Conv2DSettings const &config, std::string const &algo)
{
    return std::unique_ptr<Conv2DBackwardFilter>(new details::Conv2DBackwardFilterHip(ctx, config, algo));
}

inline std::unique_ptr<Conv2DForward> Conv2DForward::create(Context &ctx, Conv2DSettings const &config, bool bias,
                                                            StandardActivations activation, std::string const &algo)
{
    return std::unique_ptr<Conv2DForward>(new details::Conv2DForwardHip(ctx, config, bias, activation, algo));
}

} // namespace core
} // namespace dlprim
