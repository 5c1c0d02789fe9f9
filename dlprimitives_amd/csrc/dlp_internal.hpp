// Shared declarations of the gfx950 convolution forward path (host + device).
#pragma once
#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>
#include <string>

#include "../../include/dlprim_hip.h"

namespace dlp {

// Thread-local error message behind dlp_last_error().
void set_error(const std::string &msg);
int fail(int code, const std::string &msg);

#define DLP_HIP_TRY(expr)                                                                      \
    do {                                                                                       \
        hipError_t e__ = (expr);                                                               \
        if (e__ != hipSuccess)                                                                 \
            return ::dlp::fail(DLP_ERR_RUNTIME, std::string(#expr) + ": " + hipGetErrorString(e__)); \
    } while (0)

#define DLP_REQUIRE(cond, msg)                                    \
    do {                                                          \
        if (!(cond))                                              \
            return ::dlp::fail(DLP_ERR_VALIDATION, std::string("check failed: ") + #cond + " -- " + (msg)); \
    } while (0)

// Optional per-kernel timing (the analogue of dlprimitives' ExecutionContext::enable_timing,
// include/dlprim/context.hpp:23-94,180,237-243): when enabled, every kernel launch of the
// path is bracketed by a HIP event pair on its stream and recorded under a section name.
struct TimingScope {
    TimingScope(const char *section, hipStream_t stream);
    ~TimingScope();
    // which kernel the record is about: the host-side handle of the kernel launched inside this scope (what
    // hipLaunchKernelGGL is given); dlp_timing_get_kernel turns it into the name a profiler's kernel trace shows
    void kernel(const void *host_function);
    hipStream_t stream_;
    int index_;
};
// hipLaunchKernelGGL + TimingScope::kernel in one: launches `fn` and notes it in the record of `ts`
#define DLP_LAUNCH_TIMED(ts, fn, grid, block, lds, stream, ...)          \
    do {                                                                 \
        (ts).kernel(reinterpret_cast<const void *>(fn));                 \
        hipLaunchKernelGGL(fn, grid, block, lds, stream, __VA_ARGS__);   \
    } while (0)

// Compute units of the current device (256 on MI355X); cached after the first call.
int dlp_cu_count();

// Geometry of one forward convolution call (whole tensor, all groups).
struct ConvGeom {
    int B, Cin, H, W;
    int Cout, OH, OW;
    int KH, KW;
    int sh, sw, ph, pw, dh, dw;
    int groups;
    int dtype; // DLP_FLOAT / DLP_BFLOAT16 / DLP_HALF
    // tensor layouts of the implicit-GEMM convolution on the bf16 matrix instruction: x and / or y as [image][pixel][channel]
    // instead of [image][channel][pixel] (the reference knows the latter only: src/core/conv.cpp works on NCHW throughout)
    int x_channels_last = 0, y_channels_last = 0;
    int pool_ph = 0, pool_pw = 0; // > 0: the stem kernel runs a 3x3 stride-2 pad-1 max pooling behind the convolution, y is [B, Cout, pool_ph, pool_pw]
};

// Fused epilogue: v = act(acc + bias[c]); y = factor != 0 ? factor*y + v : v
// (src/kernels/sgemm.cl:658-672,707-710 in the reference).
// With accumulate_first the old value goes inside the activation: y = act(acc + bias[c] + factor*y)
// (a residual connection whose other branch already sits in y).
struct Epilogue {
    const float *bias; // nullptr when the op was created without bias
    float factor;
    int activation;
    int accumulate_first = 0;
};

__device__ __forceinline__ float apply_act(float v, int act)
{
    switch (act) {
    case DLP_ACT_RELU:
        return fmaxf(v, 0.0f);
    case DLP_ACT_TANH:
        return tanhf(v);
    case DLP_ACT_SIGMOID:
        return 1.0f / (1.0f + expf(-v));
    case DLP_ACT_RELU6:
        return fminf(fmaxf(v, 0.0f), 6.0f);
    default:
        return v;
    }
}

// min(max(v, lo), hi) for lo <= hi as one v_med3_f32 (fminf(fmaxf()) costs three vector instructions, and every
// vector-ALU instruction of an epilogue takes issue cycles from the matrix pipe); a NaN gives lo, as the pair does.
__device__ __forceinline__ float clamp_med3(float v, float lo, float hi) { return __builtin_amdgcn_fmed3f(v, lo, hi); }

__device__ __forceinline__ void store_out(float *p, float v, float factor)
{
    if (factor != 0.0f)
        *p = fmaf(*p, factor, v);
    else
        *p = v;
}

// bfloat16 storage element (bfloat16_data): the upper 16 bits of an IEEE float.
// Arithmetic is always done in fp32; conversion back rounds to nearest even.
struct bf16_t {
    uint16_t bits;
};

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return __builtin_bit_cast(float, (uint32_t)v.bits << 16); }

__device__ __forceinline__ bf16_t to_bf16(float f)
{
    // one v_cvt_pk_bf16_f32 on gfx950: round to nearest even, NaN stays NaN
    bf16_t r;
    r.bits = __builtin_bit_cast(uint16_t, (__bf16)f);
    return r;
}

__device__ __forceinline__ void store_out(bf16_t *p, float v, float factor)
{
    if (factor != 0.0f)
        v = fmaf(to_float(*p), factor, v);
    *p = to_bf16(v);
}

template <class T>
__device__ __forceinline__ void store_plain(T *p, float v);
template <>
__device__ __forceinline__ void store_plain<float>(float *p, float v)
{
    *p = v;
}
template <>
__device__ __forceinline__ void store_plain<bf16_t>(bf16_t *p, float v)
{
    *p = to_bf16(v);
}

inline size_t dtype_size(int dtype) { return dtype == DLP_FLOAT ? 4 : 2; }

// Division by a launch-time constant: q = (umulhi(n, magic) + n) >> shift == n / d for 0 <= n < 2^31.
inline void make_magic(uint32_t d, uint32_t &magic, uint32_t &shift)
{
    shift = 0;
    while ((1ull << shift) < d)
        shift++;
    magic = (uint32_t)(((1ull << 32) * ((1ull << shift) - d)) / d + 1);
}
__device__ __forceinline__ uint32_t fast_div(uint32_t n, uint32_t magic, uint32_t shift)
{
    return (__umulhi(n, magic) + n) >> shift;
}

// ---- implicit-GEMM convolution (conv_gemm.hip) ------------------------------
// Gather table entry (8 bytes).  Channel-major K order: one entry per k = {byte offset
// of tap (c,ky,kx) inside one image's group slice, tap bit or ky|kx<<8}.  Tap-major K
// order: two entries per K tile = {byte offset of (channel block, tap), tap bit, -, -}.
struct KTabEntry {
    int32_t offset;
    int32_t tap;
};

// K ordering: k = (c,ky,kx) with a per-element table, or one tap x 16 channels per K tile
// (the _BF16 orders feed bf16 operands to the bf16 matrix instruction, K tiles of 32: one tap x 32
// channels, or 32 consecutive k = (c,ky,kx) with the per-element table)
enum { GEMM_ORDER_CHANNEL = 0, GEMM_ORDER_TAP = 1, GEMM_ORDER_TAP_BF16 = 2, GEMM_ORDER_CHANNEL_BF16 = 3 };
// In-image test: one bit per tap (KH*KW <= 32) or separate row / column masks
enum { GEMM_MASK_TAPS = 1, GEMM_MASK_ROWCOL = 2 };

// Everything about a GEMM launch that is fixed by geometry + activation
// (the batch only changes the number of N tiles and the split-K factor).
struct GemmPlan {
    int order, mask;
    int tile, BM, BN;   // workgroup tile
    int M, K, nkt;      // per group: rows, reduction length, K tiles of 16
    int mtiles;         // ceil(M / BM)
    int patch;          // 1: stride-1 "same" convolution run by the LDS-patch kernel (tap-major packed weights)
    int stem;           // 1: 3-channel 7x7 stride-2 convolution run by conv_stem_f32_kernel (reads the weight tensor in place, nothing is packed)
    int wdirect;        // bf16 matrix-instruction path, 1x1: the kernel reads the weight tensor in place, nothing is packed
    int dense_pxl;      // bf16 matrix-instruction path, 1x1 stride 1 pad 0: input pixels per load of the dense loader (8, 4; 0 = gather)
    int dense_sx;       // ... 2: the dense loader on a 1x1 stride-2 convolution (dense_pxl output pixels = 2 * dense_pxl loaded)
    int pointwise;      // 1x1 stride-1 convolution with few output channels, fp32: conv_pointwise_f32_kernel (reads x and w in place)
    int patch_bf16;     // bf16 matrix-instruction path, stride-1 3x3 "same": pixels per load of the LDS-patch kernel (8, 4; 0 = gather)
    int pp_nbr;         // ... and the blocks of that many patch rows in its largest patch
    int xt;             // bf16 matrix-instruction path, neither dense nor patch: the input is first copied channels-last into the workspace
                        // ([image][pixel][channel], a 1x1 convolution's stride folded into the copy), so that a K tile of a pixel
                        // is 64 consecutive bytes and loads as 16-byte pieces instead of 32 two-byte gathers
    size_t wpack_bytes; // packed weights [group][m tile][K tile][16][BM] floats, 256-byte rounded
};
GemmPlan conv_gemm_plan(const ConvGeom &g, int activation);
size_t conv_gemm_ktab_entries(const ConvGeom &g);
// The table layout depends on the geometry AND on the activation the op was created with.
void conv_gemm_fill_ktab(const ConvGeom &g, int activation, KTabEntry *host_tab);
// Workspace (bytes) of a convolution run through this path: packed weights, plus the
// split-K partial sums when there are too few output tiles to fill the chip.
size_t conv_gemm_workspace_bytes(const ConvGeom &g, int activation);
// Repack [Cout][Cin/groups][KH][KW] weights into the tile order the kernel loads.
// part_ws/part_bytes: the workspace behind the packed weights that conv_gemm_launch will be given
// (the packing kernel clears the counters the launch keeps there).
// mode: both steps, the packing alone (weights that stay constant are packed once), or the counters alone.
enum { GEMM_PACK_AND_CLEAR = 0, GEMM_PACK_ONLY = 1, GEMM_CLEAR_ONLY = 2 };
// counters_owned: conv_gemm_launch will be given counters of the operator's own (see there): none are cleared here.
int conv_gemm_pack_weights(const ConvGeom &g, const GemmPlan &p, const void *w, void *wpacked, hipStream_t stream,
                           void *part_ws = nullptr, size_t part_bytes = 0, int mode = GEMM_PACK_AND_CLEAR, bool counters_owned = false);
// Tile counters a launch at this batch may use (0: none).  A caller that keeps that many zeroed ints per operator and
// hands them to conv_gemm_launch as own_counters saves the clearing before every launch: the kernels leave them at zero.
// Such an operator must not run on two streams at once.
bool conv_gemm_layouts_supported(const ConvGeom &g, int activation);
size_t conv_gemm_counter_count(const ConvGeom &g, const GemmPlan &p);
// n_valid >= 0 limits the GEMM N dimension (output pixels computed) below B*OH*OW.
// part_ws/part_bytes: optional split-K workspace; without it the launch runs unsplit.
// w: the weight tensor as the caller gave it (plans with wdirect read it in place when it is 16-byte aligned).
int conv_gemm_launch(const ConvGeom &g, const GemmPlan &p, const KTabEntry *dev_ktab, const void *x, const void *wpacked,
                     void *y, const Epilogue &ep, hipStream_t stream, int n_valid = -1, void *part_ws = nullptr,
                     size_t part_bytes = 0, const void *w = nullptr, int *own_counters = nullptr);

// ---- few-channel strided stem convolution (conv_stem.hip) ----------------------
bool conv_stem_supported(const ConvGeom &g);
// PH > 0: a 3x3 stride-2 pad-1 max pooling runs inside the kernel and y is the pooled [B, Cout, PH, PW] tensor (bfloat16 only)
bool conv_stem_pool_supported(const ConvGeom &g, int PH, int PW);
int conv_stem_launch(const ConvGeom &g, const void *x, const void *w, void *y, const Epilogue &ep, hipStream_t stream, int PH = 0, int PW = 0);

// ---- pointwise convolutions with few output channels (conv_pointwise.hip) --------
bool conv_pointwise_supported(const ConvGeom &g, int activation);
int conv_pointwise_launch(const ConvGeom &g, const void *x, const void *w, void *y, const Epilogue &ep, hipStream_t stream);

// ---- depthwise 3x3 + pointwise 1x1 in one launch (conv_dwpw.hip) ----------------
// g: the depthwise layer; M: filters of the pointwise layer; act1 / ep.activation: the two activations; bd: depthwise bias or null
bool conv_dwpw_supported(const ConvGeom &g, int M, int act1, int act2);
int conv_dwpw_launch(const ConvGeom &g, int M, const void *x, const void *wd, const float *bd, int act1, const void *wp, void *y, const Epilogue &ep,
                     hipStream_t stream);

// ---- depthwise (conv_depthwise.hip) ------------------------------------------
bool depthwise_supported(const ConvGeom &g);
int depthwise_launch(const ConvGeom &g, const void *x, const void *w, void *y, const Epilogue &ep, hipStream_t stream);

// ---- Winograd F(2x2,3x3) (conv_winograd.hip) ---------------------------------
struct WinoPlan {
    int Cpad, Npad;  // input / output channels rounded up to the kernel's K chunk / channel tile
    int chunk_imgs;  // images per launch (keeps 32-bit byte offsets in range)
    int stage_stride; // floats per channel of the LDS row staging buffer; 0 = patches gathered from global memory
    int stage_loads;  // staged variant: elements copied per thread and K chunk (8 or 16)
    size_t ws_bytes; // workspace() of the op: the transformed filter U[16][Cpad][Npad], fp32
};
bool winograd_supported(const ConvGeom &g);
WinoPlan winograd_plan(const ConvGeom &g);
// Workgroups of the fused kernel for the batch of g (when it fits one launch) with nob blocks of 32 output channels per workgroup,
// and the nob a launch takes (two where that leaves enough workgroups for the chip)
long long winograd_workgroups(const ConvGeom &g, const WinoPlan &plan, int nob);
int winograd_blocks_per_workgroup(const ConvGeom &g, const WinoPlan &plan);
// mode: filter transform and convolution, the transform alone (into ws), or the convolution on a ws transformed earlier
enum { WINO_FILTER_AND_RUN = 0, WINO_FILTER_ONLY = 1, WINO_RUN_ONLY = 2 };
int winograd_launch(const ConvGeom &g, const WinoPlan &plan, const void *x, const void *w, void *y, void *ws, size_t ws_bytes,
                    const Epilogue &ep, hipStream_t stream, int mode = WINO_FILTER_AND_RUN);

// ---- per-channel affine + activation (glue_ops.hip): y = act(x * scale[c] + shift[c]); null scale = 1, null shift = 0
int channel_affine_launch(int dtype, int activation, int batch, int channels, int plane, const void *x, const float *scale, const float *shift,
                          void *y, hipStream_t stream);

// ---- InnerProduct GEMM (ip_gemm.hip) ------------------------------------------
ConvGeom ip_gemm_geom(int batch, int inputs, int outputs, int dtype);
// Launch shape of the direct kernel (operands loaded from memory straight into matrix-instruction registers)
struct IpPlan {
    int nb;               // blocks of 32 batch rows per wavefront (1, 2, 4)
    int mblocks, nchunks; // tiles: blocks of 32 outputs x chunks of nb * 32 batch rows
    int ngroups, gps, S;  // groups of 8 (fp32) / 16 (bf16) k: in all, per K slice; K slices
    size_t cnt_bytes, part_bytes; // op-owned scratch: tile counters | partial sums
};
size_t ip_direct_scratch_bytes(int batch, int inputs, int outputs, int dtype, IpPlan *plan);
bool ip_direct_supported(int inputs, int dtype, const void *x, const void *w);
// counters: cnt_bytes of zeros (they are left zero); partials: part_bytes
int ip_direct_launch(int batch, int inputs, int outputs, int dtype, const void *x, const void *w, void *y, const Epilogue &ep, int *counters,
                     float *partials, hipStream_t stream);
// Large weight matrices at small batch: w streamed through LDS in 1 KB runs per row (same scratch layout and contract)
bool ip_stream_supported(int batch, int inputs, int outputs, int dtype, const void *x, const void *w);
void ip_stream_prepare(int dtype); // one-time set-up of the kernel on the current device (called when an operator is created)
size_t ip_stream_scratch_bytes(int batch, int inputs, int outputs, int dtype, IpPlan *plan);
int ip_stream_launch(int batch, int inputs, int outputs, int dtype, const void *x, const void *w, void *y, const Epilogue &ep, int *counters,
                     float *partials, hipStream_t stream);

} // namespace dlp
