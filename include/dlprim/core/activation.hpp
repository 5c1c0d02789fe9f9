// dlprim::core::activation_forward on the MI355X: the function of dlprimitives'
// include/dlprim/core/activation.hpp:14-17 over the C ABI in dlprim_hip.h.
#pragma once
#include "../context.hpp"
#include "../tensor.hpp"

namespace dlprim {
namespace core {

// y = activation(x); y may be x
inline void activation_forward(Tensor &x, Tensor &y, StandardActivations activation, ExecutionContext const &e)
{
    DLPRIM_CHECK(x.shape().total_size() == y.shape().total_size() && x.dtype() == y.dtype());
    dlprim::details::check_status(dlp_activation_fwd_enqueue(int(x.dtype()), int(activation), x.shape().total_size(), x.device_ptr(), y.device_ptr(), e.stream()));
}

} // namespace core
} // namespace dlprim
