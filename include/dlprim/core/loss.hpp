// dlprim::core::softmax_forward and nll_loss_forward on the MI355X: the functions of dlprimitives'
// include/dlprim/core/loss.hpp:14-26 over the C ABI in dlprim_hip.h (forward only).
#pragma once
#include "../context.hpp"
#include "../tensor.hpp"

namespace dlprim {
namespace core {

// softmax (or its logarithm) over dimension 1 of x [batch, classes] or [batch, classes, inner] into y
inline void softmax_forward(Tensor &x, Tensor &y, bool log_softmax, ExecutionContext const &e)
{
    Shape const &s = x.shape();
    DLPRIM_CHECK((s.size() == 2 || s.size() == 3) && y.shape() == s && x.dtype() == y.dtype());
    dlprim::details::check_status(dlp_softmax_fwd_enqueue(int(x.dtype()), log_softmax ? 1 : 0, int(s[0]), int(s[1]), s.size() == 3 ? int(s[2]) : 1,
                                                  x.device_ptr(), y.device_ptr(), e.stream()));
}

// x [batch, classes] holds log-probabilities, label [batch] is float or int32; y[b] = -scale * x[b][label[b]], or with
// reduce their sum in y[0] (a mean is a sum with scale 1 / batch)
inline void nll_loss_forward(Tensor &x, Tensor &label, Tensor &y, bool reduce, float scale, ExecutionContext const &e)
{
    Shape const &s = x.shape();
    DLPRIM_CHECK(s.size() == 2 && label.shape().total_size() == s[0] && y.shape().total_size() == (reduce ? 1 : s[0]));
    DLPRIM_CHECK(x.dtype() == y.dtype());
    // the C entry point takes the reduction by name, as NLLLoss::forward uses this function (src/ops/nll_loss.cpp:95-101):
    // no reduction or a sum with scale 1, a mean with scale 1 / batch
    int mode = DLP_LOSS_REDUCE_NONE;
    if (reduce && scale == 1.0f / float(s[0]) && s[0] > 1)
        mode = DLP_LOSS_REDUCE_MEAN;
    else if (scale != 1.0f)
        throw NotImplementedError("nll_loss_forward takes scale 1, or 1 / batch with reduce");
    else if (reduce)
        mode = DLP_LOSS_REDUCE_SUM;
    dlprim::details::check_status(dlp_nll_loss_fwd_enqueue(int(x.dtype()), int(label.dtype()), mode, int(s[0]), int(s[1]), x.device_ptr(), label.device_ptr(),
                                                   y.device_ptr(), e.stream()));
}

} // namespace core
} // namespace dlprim
