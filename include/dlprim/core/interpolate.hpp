// dlprim::core::interpolate2d on the MI355X: the function of dlprimitives'
// include/dlprim/core/interpolate.hpp:14-17 over the C ABI in dlprim_hip.h (forward only).
#pragma once
#include "../context.hpp"
#include "../tensor.hpp"

namespace dlprim {

// numeric values as in the reference (include/dlprim/definitions.hpp:325-329); they go through the C ABI as ints
enum class InterpolateType { nearest = 0, nearest_exact = 1, bilinear = 2 };

namespace core {

// x [B, C, H, W] -> y [B, C, OH, OW].  scale_y / scale_x <= 0: the steps follow from the two sizes; otherwise the size of y
// must be int(size of x * scale)
inline void interpolate2d(Tensor &x, Tensor &y, double scale_y, double scale_x, InterpolateType method, bool align_corners, ExecutionContext const &e)
{
    Shape const &xs = x.shape(), &ys = y.shape();
    DLPRIM_CHECK(xs.size() == 4 && ys.size() == 4 && xs[0] == ys[0] && xs[1] == ys[1] && x.dtype() == y.dtype());
    dlprim::details::check_status(dlp_interpolate2d_fwd_enqueue(int(x.dtype()), int(method), align_corners ? 1 : 0, scale_y, scale_x, int(xs[0] * xs[1]), int(xs[2]),
                                                        int(xs[3]), int(ys[2]), int(ys[3]), x.device_ptr(), y.device_ptr(), e.stream()));
}

} // namespace core
} // namespace dlprim
