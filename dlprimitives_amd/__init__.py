"""MI355X (gfx950) implementation of dlprimitives' convolution forward hot path.

The product is the C-ABI library ``libdlprim_hip.so`` (declared in
``include/dlprim_hip.h``, built from ``dlprimitives_amd/csrc``) and the C++
header layer in ``include/dlprim/`` that keeps the ``dlprim::core`` names.
This package is the Python binding used by the tests and the benchmark: a
ctypes front end of the same C ABI, operating on torch device tensors.
"""
from .capi import (  # noqa: F401
    ACTIVATIONS,
    Conv2DBackwardData,
    Conv2DBackwardFilter,
    Conv2DForward,
    Conv2DSettings,
    DepthwisePointwiseForward,
    DlprimError,
    IPForward,
    IPSettings,
    NotImplementedErrorDlprim,
    Pooling2DForward,
    TransposedConv2DForward,
    ValidationError,
    activation_forward,
    bias_backward,
    build_library,
    channel_affine_forward,
    conv2d_output_shape,
    conv2d_transposed_output_shape,
    eltwise_forward,
    interpolate2d_forward,
    mse_loss_forward,
    nll_loss_forward,
    reduction_forward,
    slice_copy,
    softmax_loss_forward,
    lib,
    library_path,
    pointwise_forward,
    pool2d_output_size,
    softmax_forward,
    timing_count,
    timing_enable,
    timing_records,
    timing_reset,
)
