// InnerProduct forward on the matrix cores.
//
// Replaces the reference's IPForwardImpl / StandardSGEMM path
// (src/core/ip.cpp:15-50, src/gemm.cpp:240-345):
//   y[B x Out] = act(x[B x In] * w[Out x In]^T + bias[Out])
// This is the same GEMM as a 1x1 convolution over 1x1 images with
// Cin = In, Cout = Out and one "pixel" per batch row:
//   x[b][c] sits at element b*In + c      = NCHW [B, In, 1, 1]
//   y[b][o] sits at element b*Out + o     = NCHW [B, Out, 1, 1]
// so it runs through the implicit-GEMM kernel with that geometry; the bias is
// per output feature, which is the per-row (bias_M) epilogue of the conv form.
#include "dlp_internal.hpp"

namespace dlp {

ConvGeom ip_gemm_geom(int batch, int inputs, int outputs, int dtype)
{
    ConvGeom g;
    g.B = batch;
    g.Cin = inputs;
    g.H = 1;
    g.W = 1;
    g.Cout = outputs;
    g.OH = 1;
    g.OW = 1;
    g.KH = g.KW = 1;
    g.sh = g.sw = 1;
    g.ph = g.pw = 0;
    g.dh = g.dw = 1;
    g.groups = 1;
    g.dtype = dtype;
    return g;
}

} // namespace dlp
