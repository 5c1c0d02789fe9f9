// dlprim::core::SliceCopy on the MI355X: the class of dlprimitives' include/dlprim/core/common.hpp:63-82
// over the C ABI in dlprim_hip.h, for target_scale 0 (what Concat::forward and Slice::forward pass).
#pragma once
#include "../context.hpp"
#include "../tensor.hpp"

namespace dlprim {
namespace core {

class SliceCopy {
public:
    explicit SliceCopy(Context &ctx, DataType dtype = float_data) : dtype_(dtype)
    {
        if (!ctx.is_hip_context())
            throw ValidationError("core::SliceCopy needs a device context");
    }
    // target[..., target_offset : target_offset + slice, ...] = source[..., source_offset : source_offset + slice, ...] along `dim`
    void tensor_slice_copy(int dim, size_t slice, Tensor &target, size_t target_offset, Tensor &source, size_t source_offset, float target_scale,
                           ExecutionContext const &e)
    {
        if (target_scale != 0.0f)
            throw NotImplementedError("SliceCopy with a target scale (the accumulation of the backward pass)");
        Shape const &t = target.shape(), &s = source.shape();
        DLPRIM_CHECK(t.size() == s.size() && dim >= 0 && dim < t.size());
        DLPRIM_CHECK(target.dtype() == dtype_ && source.dtype() == dtype_);
        DLPRIM_CHECK(target_offset + slice <= t[dim] && source_offset + slice <= s[dim]);
        size_t outer = 1, inner = size_t(size_of_data_type(dtype_));
        for (int j = 0; j < t.size(); j++) {
            DLPRIM_CHECK(j == dim || t[j] == s[j]);
            if (j < dim)
                outer *= t[j];
            else if (j > dim)
                inner *= t[j];
        }
        dlprim::details::check_status(dlp_copy2d_enqueue(static_cast<char *>(target.device_ptr()) + target_offset * inner, t[dim] * inner,
                                                 static_cast<const char *>(source.device_ptr()) + source_offset * inner, s[dim] * inner, slice * inner, outer,
                                                 e.stream()));
    }

private:
    DataType dtype_;
};

} // namespace core
} // namespace dlprim
