// dlprim::core::IPForward (InnerProduct) on the MI355X: same interface as
// dlprimitives' include/dlprim/core/ip.hpp:19-45, implemented over dlprim_hip.h.
#pragma once
#include <memory>

#include "../context.hpp"
#include "../tensor.hpp"

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

} // namespace core
} // namespace dlprim
