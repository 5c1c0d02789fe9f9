/*
 * dlprim_hip.h -- C ABI of the MI355X (gfx950) convolution forward path.
 *
 * This is the boundary a dlprimitives build binds in place of its OpenCL
 * context / program-cache / kernel plumbing for Conv2DForward and IPForward.
 * Plain C: pointers, sizes and ints only.  Device pointers are ordinary HIP
 * device addresses, already advanced by the tensor's element offset.
 *
 * Every call returns DLP_OK or an error code; dlp_last_error() gives the
 * thread-local message (the C++ header layer in include/dlprim/ turns codes
 * back into dlprim::ValidationError / NotImplementedError exceptions).
 *
 * Citations (file:line) name the dlprimitives interface each entry replaces.
 */
#ifndef DLPRIM_HIP_H
#define DLPRIM_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DLP_OK 0
#define DLP_ERR_VALIDATION 1      /* dlprim::ValidationError, include/dlprim/definitions.hpp:54-60 */
#define DLP_ERR_NOT_IMPLEMENTED 2 /* dlprim::NotImplementedError, include/dlprim/definitions.hpp:46-52 */
#define DLP_ERR_RUNTIME 3         /* HIP runtime failure (the reference raises cl::Error) */

/* dlprim::DataType, include/dlprim/definitions.hpp:78-94 (same numeric values) */
#define DLP_FLOAT 3
#define DLP_HALF 2
#define DLP_BFLOAT16 10
#define DLP_INT32 19 /* int32_data: class labels of the losses */

/* dlprim::StandardActivations, include/dlprim/definitions.hpp:278-284 */
#define DLP_ACT_IDENTITY 0
#define DLP_ACT_RELU 1
#define DLP_ACT_TANH 2
#define DLP_ACT_SIGMOID 3
#define DLP_ACT_RELU6 4

/* core::Conv2DSettings = Convolution2DConfigBase + input shape + dtype,
 * include/dlprim/definitions.hpp:313-321, include/dlprim/core/conv.hpp:17-28.
 * shape[0] (batch) is a hint used for kernel selection, not a requirement. */
typedef struct dlp_conv2d_settings {
    int channels_in;
    int channels_out;
    int kernel[2];
    int stride[2];
    int dilate[2];
    int pad[2];
    int groups;
    int shape[4];
    int dtype;
} dlp_conv2d_settings;

/* core::IPSettings, include/dlprim/core/ip.hpp:19-24 */
typedef struct dlp_ip_settings {
    int inputs;
    int outputs;
    int optimal_batch_size;
    int dtype;
} dlp_ip_settings;

typedef struct dlp_conv2d_fwd dlp_conv2d_fwd; /* core::Conv2DForward object */
typedef struct dlp_ip_fwd dlp_ip_fwd;         /* core::IPForward object */

/* Thread-local message of the last failing call on this thread. */
const char *dlp_last_error(void);

/* ABI version of this library (major*100 + minor). */
int dlp_version(void);

/* ---- device plumbing: replaces dlprim::Context / ExecutionContext / cl::Buffer
 *      for this path (include/dlprim/context.hpp:128-299,309-431,
 *      include/dlprim/tensor.hpp:106-294) ------------------------------------ */
int dlp_device_count(int *count);
int dlp_set_device(int device);
int dlp_device_name(int device, char *buf, size_t buf_len);
int dlp_malloc(void **dev_ptr, size_t bytes);
int dlp_free(void *dev_ptr);
int dlp_memcpy_h2d(void *dst_dev, const void *src_host, size_t bytes, void *stream); /* Tensor::to_device */
int dlp_memcpy_d2h(void *dst_host, const void *src_dev, size_t bytes, void *stream); /* Tensor::to_host */
int dlp_stream_create(void **stream);   /* ExecutionContext's in-order queue */
int dlp_stream_sync(void *stream);      /* ExecutionContext::finish, context.hpp:216-220 */
int dlp_stream_destroy(void *stream);

/* ---- HIP graphs.  No counterpart in the reference (an OpenCL queue has no such thing); for callers whose
 *      step is bound by launch overhead (small batches, many small layers).  Between begin and end every
 *      enqueue on `stream` (a stream of its own, not the default one) is recorded instead of run; launch
 *      replays the recording on a stream.  The recording holds the pointers it was given: tensors,
 *      workspaces and operators must stay alive and in place.  Run one eager pass before capturing
 *      (dlp_ip_fwd_enqueue allocates its scratch buffer on first use), keep per-kernel timing off, and
 *      make no dlp_malloc / dlp_free / dlp_memcpy_* call on the capturing stream. -------------------- */
typedef struct dlp_graph dlp_graph;
int dlp_graph_capture_begin(void *stream);
int dlp_graph_capture_end(void *stream, dlp_graph **out);
int dlp_graph_launch(dlp_graph *graph, void *stream);
void dlp_graph_destroy(dlp_graph *graph);

/* ---- per-kernel timing: replaces ExecutionContext::enable_timing / TimingData
 *      (include/dlprim/context.hpp:23-94,180,237-243).  While enabled, every kernel
 *      launched by the calls below is bracketed by a HIP event pair on its stream and
 *      recorded under a section name ("conv_gemm", "pack_weights", "splitk_reduce",
 *      "sep_conv", "winograd_filter", "winograd_fused", "pooling", "global_pooling", "eltwise").
 *      dlp_timing_get waits for the record's kernel to finish. -------------------- */
int dlp_timing_enable(int on);
int dlp_timing_reset(void);
int dlp_timing_count(int *count);
int dlp_timing_get(int index, char *section, size_t section_len, float *milliseconds);
/* Name of the kernel a record is about, as a profiler's kernel trace lists it (template arguments included,
 * namespaces and parameter list left out), e.g. "conv_patch_f32_kernel<float, 3, 3, 192, 0>"; empty for
 * records of helper launches that do not note their kernel.  No counterpart in the reference, whose kernels
 * are named by the OpenCL program that holds them. */
int dlp_timing_get_kernel(int index, char *kernel, size_t kernel_len);

/* ---- Conv2DBase::get_output_shape, src/core/conv.cpp:17-29 ------------------ */
int dlp_conv2d_output_shape(const dlp_conv2d_settings *cfg, const int in_shape[4], int out_shape[4]);

/* ---- core::Conv2DForward::create, include/dlprim/core/conv.hpp:49-53,
 *      src/core/conv.cpp:704-729.  algo: NULL, "", "auto", "gemm", "winograd",
 *      "depthwise_separable"; a requested but incompatible algorithm falls back
 *      to "gemm" exactly as the reference does (:725-727).  The automatic
 *      choice ("" / "auto") differs from the reference's rule (:714-718) in one
 *      place: a Winograd-compatible fp32 convolution that the LDS-patch GEMM
 *      kernel serves (image at most 62 wide, Cin a multiple of 16, more than 32
 *      filters) stays "gemm" where that is the faster of the two on gfx950:
 *      with fewer than 64 input channels, with fewer than 128 and a filter count
 *      that is no multiple of 64, and when the batch of the settings leaves the
 *      Winograd kernel fewer than one and a half workgroups per compute unit;
 *      algo() reports what was chosen. ------ */
int dlp_conv2d_fwd_create(const dlp_conv2d_settings *cfg, int bias, int activation,
                          const char *algo, dlp_conv2d_fwd **out);

/* Conv2DBase::algo(), include/dlprim/core/conv.hpp:33 */
const char *dlp_conv2d_fwd_algo(const dlp_conv2d_fwd *op);

/* Conv2DBase::workspace() in bytes, include/dlprim/core/conv.hpp:34 */
size_t dlp_conv2d_fwd_workspace(const dlp_conv2d_fwd *op);

/* core::Conv2DForward::enqueue, include/dlprim/core/conv.hpp:48.
 * x [B,Cin,H,W], w [Cout,Cin/groups,KH,KW], bias [Cout] or NULL (must match the
 * `bias` flag given at create), y [B,Cout,OH,OW]; ws >= workspace() bytes;
 * y = factor != 0 ? factor*y + act(conv+bias) : act(conv+bias).
 * Asynchronous on `stream` (a hipStream_t, NULL = default stream).  The operator keeps
 * small device buffers of its own (tile counters that its kernels leave at zero), as the
 * reference's operators keep their kernels and buffers: do not enqueue one operator on two
 * streams at the same time.  A batch larger than the one in the shape given at create
 * allocates here. */
int dlp_conv2d_fwd_enqueue(dlp_conv2d_fwd *op, const int x_shape[4],
                           const void *x, const void *w, const void *bias, void *y,
                           void *ws, size_t ws_bytes, float factor, void *stream);

/* Weights that stay constant between calls (inference).  No counterpart in the reference, whose enqueue
 * takes the raw filter every time; dlp_conv2d_fwd_enqueue does the same and transforms the filter on
 * every call.  Here the caller transforms it once: `packed` is a device buffer of
 * dlp_conv2d_fwd_packed_bytes(op) bytes (0 for "depthwise_separable") that dlp_conv2d_fwd_pack fills
 * (tile-ordered weights of "gemm", the transformed filter of "winograd") and that
 * dlp_conv2d_fwd_enqueue_packed reads instead of transforming `w` again (`w` is still passed: 1x1
 * bf16 convolutions read it in place).  `ws` then only holds the per-call scratch: workspace() bytes
 * are always enough, and convolutions that run one after another on a stream may share it.  Pack
 * again after the weights change. */
size_t dlp_conv2d_fwd_packed_bytes(const dlp_conv2d_fwd *op);
int dlp_conv2d_fwd_pack(dlp_conv2d_fwd *op, const void *w, void *packed, void *stream);
int dlp_conv2d_fwd_enqueue_packed(dlp_conv2d_fwd *op, const int x_shape[4], const void *x, const void *w,
                                  const void *packed, const void *bias, void *y, void *ws, size_t ws_bytes,
                                  float factor, void *stream);

/* Residual connections.  No counterpart in the reference, where the sum is an Elementwise operator of
 * its own (src/ops/elementwise.cpp).  With `on`, enqueue computes y = act(conv + bias + factor * y)
 * instead of y = factor * y + act(conv + bias): when y already holds the other branch of a residual
 * block, factor 1 gives act(conv + bias + branch) in one pass.  "gemm" and "winograd". */
int dlp_conv2d_fwd_set_accumulate_first(dlp_conv2d_fwd *op, int on);

/* Tensor layouts.  No counterpart in the reference, whose tensors are [image][channel][row][column] throughout
 * (src/core/conv.cpp).  With x_channels_last (y_channels_last) the operator reads x (writes y, and reads the old y
 * of a factor) as [image][row][column][channel]; weights and bias keep their layout.  For chains of bfloat16
 * convolutions: on the bf16 matrix instruction a channels-last input is loaded the way the weights are (16-byte
 * pieces of one pixel's channels) instead of being transposed on the way in, and a channels-last output leaves in
 * runs of a whole tile of channels per pixel.  Served: algorithm "gemm", bfloat16_data, activations identity / relu /
 * relu6; x: input channels per group a multiple of 32 and x 16-byte aligned; y: output channels per group a multiple
 * of 8, y 16-byte aligned, factor 0 or accumulate_first.  Anything else: DLP_ERR_NOT_IMPLEMENTED, here or (alignment,
 * factor) from enqueue, and the operator stays as it was.  Call before workspace(): the workspace size depends on the
 * layout of x (no channels-last copy of the input is staged). */
int dlp_conv2d_fwd_set_channels_last(dlp_conv2d_fwd *op, int x_channels_last, int y_channels_last);

/* Max pooling inside the convolution.  No counterpart in the reference, where the pooling is an operator of its own
 * (src/ops/pooling.cpp).  After this call enqueue / enqueue_packed write y = max_pool(act(conv + bias)) -- the tensor
 * [B, channels_out, PH, PW] that Pooling2D with this kernel, stride and pad would make of the convolution's output -- and the
 * convolution's own output is never written: the stem of a ResNet leaves a quarter of the bytes and the pooling's pass is gone.
 * Values equal those of the two operators run one after the other.  Served: max pooling 3x3, stride 2, pad 1, ceil_mode 0, behind
 * the bfloat16 7x7 stride-2 convolution of 3 input channels (algorithm "gemm") whose image rows, output rows (up to 112 pixels) and
 * pooled rows are multiples of 8 pixels, activations identity / relu / relu6; at enqueue x and y 16-byte aligned and factor 0.
 * Anything else: DLP_ERR_NOT_IMPLEMENTED and the operator stays as it was.  Not together with channels-last tensors. */
int dlp_conv2d_fwd_fuse_max_pool(dlp_conv2d_fwd *op, int kernel, int stride, int pad, int ceil_mode);

void dlp_conv2d_fwd_destroy(dlp_conv2d_fwd *op);

/* ---- Depthwise 3x3 convolution followed by a pointwise (1x1) convolution in one launch.  No counterpart in the
 *      reference, where these are two Convolution2D operators ("depthwise_separable", then the 1x1 path of "gemm") with a
 *      tensor as large as x written and read back between them; here that tensor never reaches memory:
 *        t = dw_act(depthwise3x3(x, dw_w) + dw_bias),  y = pw_act(pw_w * t + pw_bias),  y = factor != 0 ? factor * y + that : that
 *      t is bit for bit what the depthwise operator alone would write; the pointwise sum is accumulated in fp32 like "gemm".
 *      `dw_cfg` describes the depthwise layer (groups = channels_in = channels_out, kernel 3, pad 1, stride 1 or 2, shape =
 *      shape of x); x [B,C,H,W], dw_w [C,1,3,3], dw_bias [C], pw_w [channels_out,C,1,1], pw_bias [channels_out],
 *      y [B,channels_out,OH,OW].  Served: float_data, images of at least 512 pixels and at most 56 wide whose output width is a
 *      multiple of 4 (of 2 at stride 2 up to 28 wide), C a multiple of 8, channels_out <= 128, activations identity / relu /
 *      relu6 -- the shapes where one launch beats the two operators (smaller images stay faster as two launches): create
 *      returns DLP_ERR_NOT_IMPLEMENTED otherwise (dlp_dwpw_fwd_supported tells beforehand) and the caller keeps the two
 *      operators.  No workspace. --------------------------------------------------------------------------------------- */
typedef struct dlp_dwpw_fwd dlp_dwpw_fwd;
int dlp_dwpw_fwd_supported(const dlp_conv2d_settings *dw_cfg, int dw_activation, int channels_out, int pw_activation);
int dlp_dwpw_fwd_create(const dlp_conv2d_settings *dw_cfg, int dw_bias, int dw_activation, int channels_out, int pw_bias,
                        int pw_activation, dlp_dwpw_fwd **out);
/* y = pw_act(conv + pw_bias + factor * y), as dlp_conv2d_fwd_set_accumulate_first */
int dlp_dwpw_fwd_set_accumulate_first(dlp_dwpw_fwd *op, int on);
int dlp_dwpw_fwd_enqueue(dlp_dwpw_fwd *op, const int x_shape[4], const void *x, const void *dw_w, const void *dw_bias,
                         const void *pw_w, const void *pw_bias, void *y, float factor, void *stream);
void dlp_dwpw_fwd_destroy(dlp_dwpw_fwd *op);

/* ---- Softmax::forward, src/ops/softmax.cpp:189-222 (core::softmax_forward, src/core/loss.cpp:13-40):
 *      softmax (or log-softmax) over dimension 1 of x[batch][classes][inner] (inner = 1 for a matrix);
 *      y may be x ------------------------------------------------------------------------------- */
int dlp_softmax_fwd_enqueue(int dtype, int log_softmax, int batch, int classes, int inner, const void *x, void *y, void *stream);

/* ---- core::Conv2DBackwardData, include/dlprim/core/conv.hpp:60-68, src/core/conv.cpp:113-163,299-367,
 *      512-590 (CPU contract: src/ops/conv2d.cpp:426-430,485-498):
 *      dx [B,Cin,H,W] = factor * dx + gradient of the convolution with respect to x, from
 *      w [Cout,Cin/groups,KH,KW] and dy [B,Cout,OH,OW].  `cfg` is the forward convolution's settings
 *      (shape = shape of x); algo as for the forward operator.  float_data only.
 *      ws >= workspace() bytes (sized for the batch in cfg->shape; a larger batch needs more when
 *      stride > 1).  Asynchronous on `stream`. ---------------------------------------------------- */
typedef struct dlp_conv2d_bwd_data dlp_conv2d_bwd_data;
int dlp_conv2d_bwd_data_create(const dlp_conv2d_settings *cfg, const char *algo, dlp_conv2d_bwd_data **out);
const char *dlp_conv2d_bwd_data_algo(const dlp_conv2d_bwd_data *op);
size_t dlp_conv2d_bwd_data_workspace(const dlp_conv2d_bwd_data *op);
int dlp_conv2d_bwd_data_enqueue(dlp_conv2d_bwd_data *op, const int x_shape[4], void *dx, const void *w,
                                const void *dy, void *ws, size_t ws_bytes, float factor, void *stream);
void dlp_conv2d_bwd_data_destroy(dlp_conv2d_bwd_data *op);

/* ---- TransposedConvolution2D::forward on a device, src/ops/conv2d.cpp:559-805 (operator declared in
 *      include/dlprim/ops/conv2d.hpp:96-171): y [B,Cout,OH,OW] = act(transposed convolution of x [B,Cin,H,W] with
 *      w [Cin,Cout/groups,KH,KW] + bias [Cout]).  As in the reference it is the data-gradient pass of the convolution with
 *      the channels swapped (:588-590,:693-699,:782), followed by bias and activation.  `cfg` describes the transposed
 *      operator itself (channels_in = channels of x, shape = shape of x, batch a hint); float_data only (:584).
 *      dlp_conv2d_transposed_output_shape is Conv2DBase::get_output_shape_transposed, src/core/conv.cpp:31-43:
 *      o = (i - 1) * stride - 2 * pad + dilate * (kernel - 1) + output_pad + 1. ------------------------------------ */
typedef struct dlp_tconv2d_fwd dlp_tconv2d_fwd;
int dlp_conv2d_transposed_output_shape(const dlp_conv2d_settings *cfg, const int in_shape[4], const int output_pad[2], int out_shape[4]);
int dlp_tconv2d_fwd_create(const dlp_conv2d_settings *cfg, const int output_pad[2], int bias, int activation, const char *algo,
                           dlp_tconv2d_fwd **out);
const char *dlp_tconv2d_fwd_algo(const dlp_tconv2d_fwd *op);
size_t dlp_tconv2d_fwd_workspace(const dlp_tconv2d_fwd *op);
int dlp_tconv2d_fwd_enqueue(dlp_tconv2d_fwd *op, const int x_shape[4], const void *x, const void *w, const void *bias, void *y,
                            void *ws, size_t ws_bytes, void *stream);
void dlp_tconv2d_fwd_destroy(dlp_tconv2d_fwd *op);

/* ---- core::Conv2DBackwardFilter, include/dlprim/core/conv.hpp:70-78, src/core/conv.cpp:165-220,
 *      369-434,592-669 (CPU contract: src/ops/conv2d.cpp:431-435,475-484):
 *      dw [Cout,Cin/groups,KH,KW] = factor * dw + gradient with respect to the filter, from
 *      x [B,Cin,H,W] and dy [B,Cout,OH,OW].  float_data only; ws >= workspace() bytes. ------------- */
typedef struct dlp_conv2d_bwd_filter dlp_conv2d_bwd_filter;
int dlp_conv2d_bwd_filter_create(const dlp_conv2d_settings *cfg, const char *algo, dlp_conv2d_bwd_filter **out);
const char *dlp_conv2d_bwd_filter_algo(const dlp_conv2d_bwd_filter *op);
size_t dlp_conv2d_bwd_filter_workspace(const dlp_conv2d_bwd_filter *op);
int dlp_conv2d_bwd_filter_enqueue(dlp_conv2d_bwd_filter *op, const int x_shape[4], const void *x, void *dw,
                                  const void *dy, void *ws, size_t ws_bytes, float factor, void *stream);
void dlp_conv2d_bwd_filter_destroy(dlp_conv2d_bwd_filter *op);

/* ---- core::BiasBackwardFilter::enqueue, include/dlprim/core/bias.hpp:16-35, src/core/bias.cpp (CPU contract:
 *      BWBias::backward_cpu, src/ops/bwd_bias.cpp:34-60): db[f] = beta * db[f] + sum over b, plane of
 *      dy[b][f][plane] ---------------------------------------------------------------------------- */
int dlp_bias_bwd_enqueue(int dtype, int batch, int features, int plane, const void *dy, float *db, float beta, void *stream);

/* ---- core::IPForward::create / enqueue, include/dlprim/core/ip.hpp:30-45,
 *      src/core/ip.cpp:15-50: y[B,Out] = act(x[B,In] * w[Out,In]^T + bias[Out]) */
int dlp_ip_fwd_create(const dlp_ip_settings *cfg, int bias, int activation, dlp_ip_fwd **out);
int dlp_ip_fwd_enqueue(dlp_ip_fwd *op, int batch, const void *x, const void *w,
                       const void *bias, void *y, void *stream);
void dlp_ip_fwd_destroy(dlp_ip_fwd *op);

/* dlp_ip_fwd_enqueue for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments, same
 * result bit for bit; the tile counters and K-slice partial sums that dlp_ip_fwd_enqueue keeps in a buffer
 * the operator allocates (and regrows for a larger batch) live here in one array of
 * DLP_IP_NO_ALLOC_SCRATCH_BYTES that the library holds on every device it runs on until the process ends.
 * The call makes no hipMalloc / hipFree and records no memset.  The array holds 64 KiB of tile counters and
 * 4 MiB of partial sums (4 KiB per tile of 32 outputs x 32 batch rows and K slice).  With rows on 16-byte
 * boundaries (the kernel that streams w through LDS) K is only cut while tiles x slices stay within 1024,
 * which keeps the partial sums within 4 MiB whatever the shape; other
 * alignments cut K more freely, and a batch x outputs that then needs more is a validation error that
 * names both sizes (e.g. 1026 -> 4096 at batch 160: 5 MiB).  bfloat16 rows of odd length are NotImplemented.
 * RULE: at most one call in flight per device.  All calls on one device share the array, whatever the operator: two
 * calls that overlap on one device (different streams, two threads, two recorded graphs replayed side by side) race on
 * the counters and partial sums, and nothing detects it; calls on one stream, or replays of graphs on one stream, are
 * ordered by the stream and do not. */
#define DLP_IP_NO_ALLOC_SCRATCH_BYTES (4 * 1024 * 1024 + 64 * 1024)
int dlp_ip_fwd_enqueue_no_alloc(dlp_ip_fwd *op, int batch, const void *x, const void *w,
                                const void *bias, void *y, void *stream);

/* ===== glue operators around the convolution path (forward only) ================= */

typedef struct dlp_pool2d_fwd dlp_pool2d_fwd; /* core::Pooling2DForward object */

/* core::calc_pooling_output_size, include/dlprim/core/pool.hpp:17-27 */
int dlp_pool2d_output_size(int in_size, int kernel, int pad, int stride, int ceil_mode, int *out_size);

/* core::Pooling2DForward::create_max_pooling / create_avg_pooling /
 * create_global_max_pooling / create_global_avg_pooling, include/dlprim/core/pool.hpp:38-69 */
int dlp_pool2d_fwd_create_max(const int kernel[2], const int pad[2], const int stride[2], int dtype, dlp_pool2d_fwd **out);
int dlp_pool2d_fwd_create_avg(const int kernel[2], const int pad[2], const int stride[2], int count_include_pad, int dtype,
                              dlp_pool2d_fwd **out);
int dlp_pool2d_fwd_create_global_max(int dtype, dlp_pool2d_fwd **out);
int dlp_pool2d_fwd_create_global_avg(int dtype, dlp_pool2d_fwd **out);

/* core::Pooling2DForward::enqueue(X, Y, e), include/dlprim/core/pool.hpp:36.
 * x [B,C,H,W] -> y [B,C,OH,OW]; the output shape (from dlp_pool2d_output_size, with or
 * without ceil_mode) is the caller's, as in the reference; global variants need [B,C,1,1]. */
int dlp_pool2d_fwd_enqueue(dlp_pool2d_fwd *op, const int x_shape[4], const int y_shape[4], const void *x, void *y, void *stream);
/* Global pooling of a channels-last x ([image][row][column][channel], as dlp_conv2d_fwd_set_channels_last writes it); x_shape stays
 * [B, C, H, W] and y is [B, C, 1, 1] either way.  No counterpart in the reference.  Other pooling: DLP_ERR_NOT_IMPLEMENTED. */
int dlp_pool2d_fwd_set_channels_last(dlp_pool2d_fwd *op, int on);
void dlp_pool2d_fwd_destroy(dlp_pool2d_fwd *op);

/* The copy behind Concat::forward and Slice::forward (core::SliceCopy::tensor_slice_copy with target_scale 0,
 * include/dlprim/core/common.hpp:63-82; src/ops/concat.cpp:66-84,150-171): `rows` runs of `width_bytes` bytes, the r-th from
 * src + r * src_pitch to dst + r * dst_pitch (pitches in bytes).  For a tensor split over axis `dim` into [outer][dim][inner]:
 * rows = outer, width = slice * inner elements, pitch = the tensor's dim * inner elements, offsets folded into the pointers. */
int dlp_copy2d_enqueue(void *dst, size_t dst_pitch, const void *src, size_t src_pitch, size_t width_bytes, size_t rows, void *stream);

/* Elementwise::forward for two tensors of equal shape, src/ops/elementwise.cpp:517-559:
 * operation 0 sum: c = act(coef1*a + coef2*b); 1 prod: act(a*b*coef1*coef2); 2 max: act(max(coef1*a, coef2*b)) */
#define DLP_ELTWISE_SUM 0
#define DLP_ELTWISE_PROD 1
#define DLP_ELTWISE_MAX 2
int dlp_eltwise_fwd_enqueue(int operation, float coef1, float coef2, int activation, size_t n, const void *a, const void *b, void *c,
                            void *stream);
/* same for tensors stored as `dtype` (DLP_FLOAT or DLP_BFLOAT16; arithmetic in fp32) */
int dlp_eltwise_fwd_enqueue_dtype(int dtype, int operation, float coef1, float coef2, int activation, size_t n, const void *a,
                                  const void *b, void *c, void *stream);
/* same with broadcasting (Elementwise::setup / forward, src/ops/elementwise.cpp:223,517-559; Shape broadcast rules of
 * src/shape.cpp:105-160): a_shape and b_shape have `rank` (1 to 8) extents each, padded with leading ones by the caller; in every
 * dimension the two extents are equal or one of them is 1; c has the larger extent of each dimension.  Runs of dimensions along which
 * the same operands move are treated as one; more than four such runs are NotImplemented. */
int dlp_eltwise_bcast_fwd_enqueue(int dtype, int operation, float coef1, float coef2, int activation, int rank, const int *a_shape,
                                  const int *b_shape, const void *a, const void *b, void *c, void *stream);

/* Activation::forward, src/ops/activation.cpp (cpu::apply_activation, include/dlprim/cpu/cpu_ops.hpp:17-53):
 * y = act(x) over n elements stored as `dtype`; x == y (in place) is allowed. */
int dlp_activation_fwd_enqueue(int dtype, int activation, size_t n, const void *x, void *y, void *stream);
/* Threshold / Abs / Hardtanh::forward (src/ops/pointwise.cpp:84-95,113-126,154-158; defaults threshold 0, min_val -1, max_val 1 in
 * include/dlprim/ops/pointwise.hpp:50,71-72): y = x > p0 ? 1 : 0 | y = |x| | y = max(p0, min(p1, x)); y may be x */
#define DLP_POINTWISE_THRESHOLD 0
#define DLP_POINTWISE_ABS 1
#define DLP_POINTWISE_HARDTANH 2
int dlp_pointwise_fwd_enqueue(int dtype, int operation, float p0, float p1, size_t n, const void *x, void *y, void *stream);

/* BatchNorm::forward with fixed statistics (predict mode / use_global_stats), src/ops/batch_normalization.cpp:161-232:
 * y[b][c][i] = act(x[b][c][i] * scale[c] + shift[c]) with scale = gamma / sqrt(var + eps), shift = beta - mean * scale
 * computed by the caller (fp32 device arrays of `channels` values); plane = H * W; x == y is allowed. */
int dlp_channel_affine_fwd_enqueue(int dtype, int activation, int batch, int channels, int plane, const void *x, const float *scale,
                                   const float *shift, void *y, void *stream);

/* core::interpolate2d, include/dlprim/core/interpolate.hpp:17 (src/core/interpolate.cpp:10-78, kernels of
 * src/kernels/interpolate_2d.cl): x [planes, src_h, src_w] -> y [planes, tgt_h, tgt_w], planes = batch * channels.
 * method as dlprim::InterpolateType (include/dlprim/definitions.hpp:325-329).  scale_y / scale_x <= 0: the steps follow from the
 * sizes; otherwise tgt = int(src * scale) is checked.  nearest: source index min(int((p + offset) * step), src - 1) with offset 0,
 * or 0.5 for nearest-exact; bilinear: source position max(step * (p + 0.5) - 0.5, 0), or p * (src - 1) / (tgt - 1) with
 * align_corners, and the two neighbours weighted by the fraction.  Bilinear blends along the row first and then between the two
 * rows, where the reference's kernel sums four weighted taps (src/kernels/interpolate_2d.cl:111-140): same value to within a few
 * ulp, not the same bits; nearest picks the reference's pixel exactly. */
#define DLP_INTERPOLATE_NEAREST 0
#define DLP_INTERPOLATE_NEAREST_EXACT 1
#define DLP_INTERPOLATE_BILINEAR 2
int dlp_interpolate2d_fwd_enqueue(int dtype, int method, int align_corners, double scale_y, double scale_x, int planes, int src_h,
                                  int src_w, int tgt_h, int tgt_w, const void *x, void *y, void *stream);

/* Reduction::forward, src/ops/reduction.cpp:96-111,300-361 (ReductionConfig::Method, include/dlprim/ops/reduction.hpp:16-21):
 * y = coefficient * sum over the dimensions with reduce[j] != 0 of x | x^2 | |x|; coefficient = output_scale, for mean
 * output_scale * (elements of y) / (elements of x).  shape and reduce have `rank` (1 to 8) entries; y holds the kept dimensions in
 * order (its shape with or without the reduced ones as extent 1 is the caller's).  Neighbouring dimensions that are all kept or all
 * reduced count as one group; more than three groups of either kind are NotImplemented (any tensor of rank <= 6 fits).  Sums are fp32;
 * the pieces of a long reduction are added in a fixed order, so results repeat bit for bit.  The workspace (device memory, size from
 * dlp_reduce_fwd_workspace, possibly 0) holds the pieces. */
#define DLP_REDUCE_SUM 0
#define DLP_REDUCE_SUMSQ 1
#define DLP_REDUCE_ABSSUM 2
#define DLP_REDUCE_MEAN 3
int dlp_reduce_fwd_workspace(int dtype, int method, int rank, const int *shape, const int *reduce, size_t *bytes);
int dlp_reduce_fwd_enqueue(int dtype, int method, float output_scale, int rank, const int *shape, const int *reduce, const void *x,
                           void *y, void *workspace, size_t workspace_bytes, void *stream);

/* The forward pass of the losses.  reduce as MSELossConfig / NLLLossConfig::Reduce (none, sum, mean). */
#define DLP_LOSS_REDUCE_NONE 0
#define DLP_LOSS_REDUCE_SUM 1
#define DLP_LOSS_REDUCE_MEAN 2
/* MSELoss::forward, src/ops/mse_loss.cpp:70-111: y[i] = (a[i] - b[i])^2 over n elements, or their sum / mean in y[0] */
int dlp_mse_loss_fwd_workspace(int dtype, int reduce, size_t n, size_t *bytes);
int dlp_mse_loss_fwd_enqueue(int dtype, int reduce, size_t n, const void *a, const void *b, void *y, void *workspace,
                             size_t workspace_bytes, void *stream);
/* core::nll_loss_forward, include/dlprim/core/loss.hpp:26 (NLLLoss::forward, src/ops/nll_loss.cpp:59-110; kernel
 * src/kernels/nll_loss_fwd.cl): x [batch, classes], labels [batch] stored as label_dtype (DLP_FLOAT or DLP_INT32);
 * y[b] = -x[b][label[b]], 0 for a label outside [0, classes), or the sum / mean over the batch in y[0] */
int dlp_nll_loss_fwd_enqueue(int dtype, int label_dtype, int reduce, int batch, int classes, const void *x, const void *labels,
                             void *y, void *stream);
/* SoftmaxWithLoss::forward, src/ops/softmax.cpp:134-155,224-244 (kernel src/kernels/softmax_with_loss.cl with CALC_LOSS 1):
 * y[0] = mean over the rows of -(x[b][label] - max_b - log(sum_c exp(x[b][c] - max_b))); a row whose label lies outside
 * [0, classes) adds 0, as in the reference's kernel.  The workspace holds one float per row. */
int dlp_softmax_loss_fwd_workspace(int batch, size_t *bytes);
int dlp_softmax_loss_fwd_enqueue(int dtype, int label_dtype, int batch, int classes, const void *x, const void *labels, void *y,
                                 void *workspace, size_t workspace_bytes, void *stream);

/* ===== data types ==================================================================
 * DLP_FLOAT: everything fp32, as in the reference (its conv/GEMM reject other types,
 * src/gemm.cpp:577,593).  DLP_BFLOAT16 (an extension): x, w, y of Conv2DForward and
 * IPForward and the tensors of the glue operators are stored as bfloat16; bias stays
 * fp32; products are accumulated in fp32 on the matrix cores and the epilogue runs in
 * fp32 before one round-to-nearest-even conversion of the result.  All three algorithms
 * serve it: "gemm" multiplies bf16 operands on the bf16 matrix instruction (products of bf16
 * values are exact in fp32), "winograd" transforms in fp32 and multiplies on the fp32 matrix
 * instruction, "depthwise_separable" computes in fp32.  With algo "" / "auto" a bf16
 * convolution runs "gemm" where the reference rule would pick "winograd". */

#ifdef __cplusplus
}
#endif
#endif
