// dlprim::core::BiasBackwardFilter on the MI355X: the interface of dlprimitives'
// include/dlprim/core/bias.hpp:16-35 over the C ABI in dlprim_hip.h.
#pragma once
#include <memory>

#include "../context.hpp"
#include "../tensor.hpp"

namespace dlprim {
namespace core {

// dw[f] = beta * dw[f] + sum of dy[b][f][...] over the batch and the plane
class BiasBackwardFilter {
public:
    virtual ~BiasBackwardFilter() {}
    virtual size_t workspace() = 0;
    virtual void enqueue(Tensor &dy, Tensor &dw, Tensor &ws, float beta, ExecutionContext const &e) = 0;
    // dy_shape: (B, features) for an inner product, (B, features, H, W) for a convolution
    static std::unique_ptr<BiasBackwardFilter> create(Context &ctx, Shape const &dy_shape, DataType dt = float_data);
};

namespace details {
class BiasBackwardFilterHip : public BiasBackwardFilter {
public:
    BiasBackwardFilterHip(Context &ctx, Shape const &dy_shape, DataType dt) : dtype_(dt)
    {
        if (!ctx.is_hip_context())
            throw ValidationError("core::BiasBackwardFilter needs a device context");
        DLPRIM_CHECK(dy_shape.size() >= 2);
    }
    size_t workspace() override { return 0; }
    void enqueue(Tensor &dy, Tensor &dw, Tensor &, float beta, ExecutionContext const &e) override
    {
        Shape const &s = dy.shape();
        DLPRIM_CHECK(s.size() >= 2 && dw.shape().total_size() == s[1]);
        const size_t planes = s[0] * s[1];
        dlprim::details::check_status(dlp_bias_bwd_enqueue(int(dtype_), int(s[0]), int(s[1]), int(planes ? s.total_size() / planes : 1), dy.device_ptr(),
                                                           static_cast<float *>(dw.device_ptr()), beta, e.stream()));
    }

private:
    DataType dtype_;
};
} // namespace details

inline std::unique_ptr<BiasBackwardFilter> BiasBackwardFilter::create(Context &ctx, Shape const &dy_shape, DataType dt)
{
    return std::unique_ptr<BiasBackwardFilter>(new details::BiasBackwardFilterHip(ctx, dy_shape, dt));
}

} // namespace core
} // namespace dlprim
