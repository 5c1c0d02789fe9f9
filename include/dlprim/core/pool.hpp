// dlprim::core::Pooling2DForward on the MI355X: same interface as dlprimitives'
// include/dlprim/core/pool.hpp:13-69 (forward part), implemented over dlprim_hip.h.
#pragma once
#include <memory>

#include "../context.hpp"
#include "../tensor.hpp"

namespace dlprim {
namespace core {

// output size of one pooled dimension; ceil_mode rounds the window count up but never
// starts a window in the bottom / right padding (include/dlprim/core/pool.hpp:17-27)
inline int calc_pooling_output_size(int in_size, int kernel, int pad, int stride, bool ceil_mode)
{
    int size = 0;
    dlprim::details::check_status(dlp_pool2d_output_size(in_size, kernel, pad, stride, ceil_mode ? 1 : 0, &size));
    return size;
}

class Pooling2DForward {
public:
    virtual ~Pooling2DForward() {}
    virtual size_t workspace() = 0;
    // X [B,C,H,W] -> Y [B,C,OH,OW]; OH/OW as calc_pooling_output_size gives them (either rounding);
    // the global variants need Y [B,C,1,1]
    virtual void enqueue(Tensor &X, Tensor &Y, ExecutionContext const &e) = 0;
    // Not in the reference: X is [image][row][column][channel] (global pooling only; shapes stay [B, C, H, W]).  The default refuses.
    virtual void channels_last(bool on)
    {
        if (on)
            throw NotImplementedError("channels_last is not implemented by this Pooling2DForward");
    }

    static std::unique_ptr<Pooling2DForward> create_max_pooling(Context &ctx, int kernel[2], int pad[2], int stride[2],
                                                                DataType dt = float_data);
    static std::unique_ptr<Pooling2DForward> create_avg_pooling(Context &ctx, int kernel[2], int pad[2], int stride[2],
                                                                bool count_include_pad = false, DataType dt = float_data);
    static std::unique_ptr<Pooling2DForward> create_global_max_pooling(Context &ctx, Shape const &in_shape, DataType dt = float_data);
    static std::unique_ptr<Pooling2DForward> create_global_avg_pooling(Context &ctx, Shape const &in_shape, DataType dt = float_data);
};

namespace details {
class Pooling2DForwardHip : public Pooling2DForward {
public:
    Pooling2DForwardHip(Context &ctx, dlp_pool2d_fwd *op) : op_(op)
    {
        if (ctx.is_cpu_context()) {
            dlp_pool2d_fwd_destroy(op);
            throw NotImplementedError("core::Pooling2DForward needs a device context");
        }
    }
    ~Pooling2DForwardHip() { dlp_pool2d_fwd_destroy(op_); }
    Pooling2DForwardHip(Pooling2DForwardHip const &) = delete;
    void operator=(Pooling2DForwardHip const &) = delete;

    size_t workspace() override { return 0; }
    void channels_last(bool on) override { dlprim::details::check_status(dlp_pool2d_fwd_set_channels_last(op_, on ? 1 : 0)); }
    void enqueue(Tensor &X, Tensor &Y, ExecutionContext const &e) override
    {
        DLPRIM_CHECK(X.shape().size() == 4 && Y.shape().size() == 4);
        int xs[4], ys[4];
        for (int i = 0; i < 4; i++) {
            xs[i] = int(X.shape()[i]);
            ys[i] = int(Y.shape()[i]);
        }
        dlprim::details::check_status(dlp_pool2d_fwd_enqueue(op_, xs, ys, X.device_ptr(), Y.device_ptr(), e.stream()));
    }

private:
    dlp_pool2d_fwd *op_ = nullptr;
};
} // namespace details

inline std::unique_ptr<Pooling2DForward> Pooling2DForward::create_max_pooling(Context &ctx, int kernel[2], int pad[2], int stride[2],
                                                                              DataType dt)
{
    ctx.select();
    dlp_pool2d_fwd *op = nullptr;
    dlprim::details::check_status(dlp_pool2d_fwd_create_max(kernel, pad, stride, int(dt), &op));
    return std::unique_ptr<Pooling2DForward>(new details::Pooling2DForwardHip(ctx, op));
}

inline std::unique_ptr<Pooling2DForward> Pooling2DForward::create_avg_pooling(Context &ctx, int kernel[2], int pad[2], int stride[2],
                                                                              bool count_include_pad, DataType dt)
{
    ctx.select();
    dlp_pool2d_fwd *op = nullptr;
    dlprim::details::check_status(dlp_pool2d_fwd_create_avg(kernel, pad, stride, count_include_pad ? 1 : 0, int(dt), &op));
    return std::unique_ptr<Pooling2DForward>(new details::Pooling2DForwardHip(ctx, op));
}

// in_shape is accepted for source compatibility; the kernel reads the shape at enqueue
inline std::unique_ptr<Pooling2DForward> Pooling2DForward::create_global_max_pooling(Context &ctx, Shape const &, DataType dt)
{
    ctx.select();
    dlp_pool2d_fwd *op = nullptr;
    dlprim::details::check_status(dlp_pool2d_fwd_create_global_max(int(dt), &op));
    return std::unique_ptr<Pooling2DForward>(new details::Pooling2DForwardHip(ctx, op));
}

inline std::unique_ptr<Pooling2DForward> Pooling2DForward::create_global_avg_pooling(Context &ctx, Shape const &, DataType dt)
{
    ctx.select();
    dlp_pool2d_fwd *op = nullptr;
    dlprim::details::check_status(dlp_pool2d_fwd_create_global_avg(int(dt), &op));
    return std::unique_ptr<Pooling2DForward>(new details::Pooling2DForwardHip(ctx, op));
}

} // namespace core
} // namespace dlprim
