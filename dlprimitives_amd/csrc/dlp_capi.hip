// C ABI of the gfx950 convolution forward path (see include/dlprim_hip.h).
//
// Host-side logic only: argument validation with the reference's rules,
// algorithm selection (src/core/conv.cpp:672-729 in the reference), ownership of
// the per-op gather tables, and dispatch to the HIP kernels.  There is no CPU
// fallback: every compute entry launches a device kernel or fails.
#include "dlp_internal.hpp"

#include <atomic>

#include <algorithm>

#include <cstdlib>
#include <cstring>
#include <cxxabi.h>
#include <mutex>
#include <new>
#include <vector>

namespace dlp {

static thread_local std::string g_last_error;

void set_error(const std::string &msg) { g_last_error = msg; }

int fail(int code, const std::string &msg)
{
    g_last_error = msg;
    return code;
}

namespace {
struct TimingRecord {
    const char *section;
    const void *kernel; // host-side handle of the kernel, or null
    hipStream_t stream;
    hipEvent_t start, stop;
};
std::mutex g_timing_mutex;
bool g_timing_enabled = false;
std::vector<TimingRecord> g_timing_records;
} // namespace

TimingScope::TimingScope(const char *section, hipStream_t stream) : stream_(stream), index_(-1)
{
    std::lock_guard<std::mutex> lock(g_timing_mutex);
    if (!g_timing_enabled)
        return;
    TimingRecord r;
    r.section = section;
    r.kernel = nullptr;
    r.stream = stream;
    if (hipEventCreate(&r.start) != hipSuccess)
        return;
    if (hipEventCreate(&r.stop) != hipSuccess) {
        (void)hipEventDestroy(r.start);
        return;
    }
    (void)hipEventRecord(r.start, stream);
    index_ = (int)g_timing_records.size();
    g_timing_records.push_back(r);
}

TimingScope::~TimingScope()
{
    if (index_ < 0)
        return;
    std::lock_guard<std::mutex> lock(g_timing_mutex);
    if (index_ < (int)g_timing_records.size())
        (void)hipEventRecord(g_timing_records[index_].stop, stream_);
}

int dlp_cu_count()
{
    // per device: every GPU of a process may be a different part
    constexpr int kMaxDevices = 64;
    static std::atomic<int> cus[kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return 256;
    int n = cus[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        cus[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

void TimingScope::kernel(const void *host_function)
{
    if (index_ < 0)
        return;
    std::lock_guard<std::mutex> lock(g_timing_mutex);
    if (index_ < (int)g_timing_records.size())
        g_timing_records[index_].kernel = host_function;
}

} // namespace dlp

using namespace dlp;

enum ConvAlgo { ALGO_GEMM = 0, ALGO_WINOGRAD = 1, ALGO_DEPTHWISE = 2 };

struct dlp_conv2d_fwd {
    dlp_conv2d_settings cfg;
    bool bias;
    int activation;
    ConvAlgo algo;
    int device;
    KTabEntry *ktab; // device gather table of the GEMM stage
    WinoPlan wino;
    size_t workspace;
    int packed_layout[6]; // of the last dlp_conv2d_fwd_pack: order, BM, K tiles, m tiles, patch, in-place
    int accumulate_first; // y = act(conv + bias + factor * y) instead of factor * y + act(conv + bias)
    int x_channels_last, y_channels_last; // tensor layouts of the gemm algorithm on bf16 tensors (dlp_conv2d_fwd_set_channels_last)
    int max_pool;                         // a 3x3 stride-2 pad-1 max pooling runs behind the convolution (dlp_conv2d_fwd_fuse_max_pool)
    int *counters;        // GEMM stage: tile counters of split-K / stream-K launches, zero between launches
    size_t counter_count;
};

// The operator's own tile counters, enough for this batch (they only ever grow; a larger batch than any before
// allocates anew, which waits for the kernels that use the old ones).
static int own_counters(dlp_conv2d_fwd *op, const ConvGeom &g, const GemmPlan &plan, int **out)
{
    const size_t need = conv_gemm_counter_count(g, plan);
    if (need > op->counter_count) {
        if (op->counters)
            (void)hipFree(op->counters);
        op->counters = nullptr;
        op->counter_count = 0;
        DLP_HIP_TRY(hipMalloc((void **)&op->counters, need * sizeof(int)));
        DLP_HIP_TRY(hipMemset(op->counters, 0, need * sizeof(int)));
        op->counter_count = need;
    }
    *out = op->counters;
    return DLP_OK;
}

static size_t round256(size_t v) { return (v + 255) / 256 * 256; }

static int make_geom(const dlp_conv2d_settings &c, const int x_shape[4], ConvGeom &g);
// geometry of an operator's convolution on an input of this shape, with the operator's tensor layouts
static int op_geom(const dlp_conv2d_fwd *op, const int x_shape[4], ConvGeom &g)
{
    const int rc = make_geom(op->cfg, x_shape, g);
    g.x_channels_last = op->x_channels_last;
    g.y_channels_last = op->y_channels_last;
    if (op->max_pool) { // sizes as Pooling2D with ceil_mode false computes them
        g.pool_ph = (g.OH + 2 - 3) / 2 + 1;
        g.pool_pw = (g.OW + 2 - 3) / 2 + 1;
    }
    return rc;
}

struct dlp_ip_fwd {
    dlp_ip_settings cfg;
    bool bias;
    int activation;
    int device;
    KTabEntry *ktab;
    GemmPlan plan;
    void *wpacked; // op-owned: IPForward::enqueue has no workspace argument
    void *scratch; // direct kernel: tile counters + K-slice partial sums, grown to the largest batch seen
    size_t scratch_bytes, scratch_cnt_bytes;
};

static int upload_ktab(const ConvGeom &g, int activation, KTabEntry **out)
{
    const size_t n = conv_gemm_ktab_entries(g);
    std::vector<KTabEntry> host(n ? n : 1);
    conv_gemm_fill_ktab(g, activation, host.data());
    KTabEntry *dev = nullptr;
    DLP_HIP_TRY(hipMalloc((void **)&dev, host.size() * sizeof(KTabEntry)));
    hipError_t e = hipMemcpy(dev, host.data(), host.size() * sizeof(KTabEntry), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        (void)hipFree(dev);
        return fail(DLP_ERR_RUNTIME, std::string("hipMemcpy(gather table): ") + hipGetErrorString(e));
    }
    *out = dev;
    return DLP_OK;
}

static bool valid_activation(int a) { return a >= DLP_ACT_IDENTITY && a <= DLP_ACT_RELU6; }

// Conv2DBase::get_output_shape, src/core/conv.cpp:17-29
static int output_shape(const dlp_conv2d_settings *cfg, const int in[4], int out[4])
{
    DLP_REQUIRE(cfg != nullptr && in != nullptr && out != nullptr, "null argument");
    DLP_REQUIRE(in[1] == cfg->channels_in, "input channels differ from channels_in");
    for (int i = 0; i < 2; i++) {
        DLP_REQUIRE(cfg->kernel[i] > 0 && cfg->stride[i] > 0 && cfg->dilate[i] > 0 && cfg->pad[i] >= 0, "kernel/stride/dilate/pad");
        int o = (in[2 + i] + 2 * cfg->pad[i] - cfg->dilate[i] * (cfg->kernel[i] - 1) - 1) / cfg->stride[i] + 1;
        DLP_REQUIRE(o > 0, "empty output");
        out[2 + i] = o;
    }
    out[0] = in[0];
    out[1] = cfg->channels_out;
    return DLP_OK;
}

static int make_geom(const dlp_conv2d_settings &c, const int x_shape[4], ConvGeom &g)
{
    int out[4];
    int rc = output_shape(&c, x_shape, out);
    if (rc != DLP_OK)
        return rc;
    g.B = x_shape[0];
    g.Cin = c.channels_in;
    g.H = x_shape[2];
    g.W = x_shape[3];
    g.Cout = c.channels_out;
    g.OH = out[2];
    g.OW = out[3];
    g.KH = c.kernel[0];
    g.KW = c.kernel[1];
    g.sh = c.stride[0];
    g.sw = c.stride[1];
    g.ph = c.pad[0];
    g.pw = c.pad[1];
    g.dh = c.dilate[0];
    g.dw = c.dilate[1];
    g.groups = c.groups;
    g.dtype = c.dtype;
    return DLP_OK;
}

// ---- the entry point that allocates nothing ----------------------------------------------------------------
// The tile counters and K-slice partial sums of ip_direct_kernel live in a device array of this library instead of
// an op-owned hipMalloc buffer.  Every device the library runs on holds its own copy of the array until the process
// ends; host code must never hand the array's name to a kernel (on the host it is a stand-in, not a device address):
// the address on the current device comes from hipGetSymbolAddress, once per device, and is kept in g_scratch_ptr.
static __device__ __align__(256) unsigned char scratch[DLP_IP_NO_ALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
constexpr size_t kNoAllocCounterBytes = 64 * 1024; // front of the array: tile counters; the rest: partial sums
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices];

// address of `scratch` on the current device (looked up on first use, with that device current)
int scratch_on_current_device(void **out)
{
    int device = -1;
    DLP_HIP_TRY(hipGetDevice(&device));
    DLP_REQUIRE(device >= 0 && device < kMaxDevices, "device index beyond the table of scratch addresses");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        void *ptr = nullptr;
        DLP_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr)
            return fail(DLP_ERR_RUNTIME, "hipGetSymbolAddress gave no address for the scratch array");
        g_scratch_ptr[device] = ptr;
    }
    *out = g_scratch_ptr[device];
    return DLP_OK;
}

// a fill kernel, not hipMemsetAsync: the call may be recorded into a HIP graph
__global__ void clear_ints_kernel(int *p, int n)
{
    const int i = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (i < n)
        p[i] = 0;
}
} // namespace

extern "C" {

const char *dlp_last_error(void) { return g_last_error.c_str(); }

int dlp_version(void) { return 100; }

int dlp_timing_enable(int on)
{
    std::lock_guard<std::mutex> lock(g_timing_mutex);
    g_timing_enabled = on != 0;
    return DLP_OK;
}

int dlp_timing_reset(void)
{
    std::lock_guard<std::mutex> lock(g_timing_mutex);
    for (TimingRecord &r : g_timing_records) {
        (void)hipEventDestroy(r.start);
        (void)hipEventDestroy(r.stop);
    }
    g_timing_records.clear();
    return DLP_OK;
}

int dlp_timing_count(int *count)
{
    DLP_REQUIRE(count != nullptr, "null argument");
    std::lock_guard<std::mutex> lock(g_timing_mutex);
    *count = (int)g_timing_records.size();
    return DLP_OK;
}

int dlp_timing_get(int index, char *section, size_t section_len, float *milliseconds)
{
    DLP_REQUIRE(section != nullptr && section_len > 0 && milliseconds != nullptr, "null argument");
    std::lock_guard<std::mutex> lock(g_timing_mutex);
    DLP_REQUIRE(index >= 0 && index < (int)g_timing_records.size(), "timing record index out of range");
    const TimingRecord &r = g_timing_records[index];
    DLP_HIP_TRY(hipEventSynchronize(r.stop));
    DLP_HIP_TRY(hipEventElapsedTime(milliseconds, r.start, r.stop));
    std::strncpy(section, r.section, section_len - 1);
    section[section_len - 1] = 0;
    return DLP_OK;
}

int dlp_timing_get_kernel(int index, char *kernel, size_t kernel_len)
{
    DLP_REQUIRE(kernel != nullptr && kernel_len > 0, "null argument");
    std::lock_guard<std::mutex> lock(g_timing_mutex);
    DLP_REQUIRE(index >= 0 && index < (int)g_timing_records.size(), "timing record index out of range");
    const TimingRecord &r = g_timing_records[index];
    std::string name;
    if (r.kernel) {
        const char *mangled = hipKernelNameRefByPtr(r.kernel, r.stream);
        if (mangled) {
            int status = 0;
            char *plain = abi::__cxa_demangle(mangled, nullptr, nullptr, &status);
            name = (status == 0 && plain) ? plain : mangled;
            std::free(plain);
            // as a kernel trace prints it: no namespaces, no parameter list
            if (!name.empty() && name.back() == ')') { // the parameter list: back to the parenthesis that matches the last one
                int depth = 0;
                for (size_t i = name.size(); i-- > 0;) {
                    depth += name[i] == ')' ? 1 : name[i] == '(' ? -1 : 0;
                    if (depth == 0) {
                        name.erase(i);
                        break;
                    }
                }
            }
            if (name.compare(0, 5, "void ") == 0)
                name.erase(0, 5);
            for (const char *ns : {"dlp::(anonymous namespace)::", "(anonymous namespace)::", "dlp::"}) {
                const std::string n(ns);
                for (size_t at; (at = name.find(n)) != std::string::npos;)
                    name.erase(at, n.size());
            }
        }
    }
    std::strncpy(kernel, name.c_str(), kernel_len - 1);
    kernel[kernel_len - 1] = 0;
    return DLP_OK;
}

int dlp_device_count(int *count)
{
    DLP_REQUIRE(count != nullptr, "null argument");
    DLP_HIP_TRY(hipGetDeviceCount(count));
    return DLP_OK;
}

int dlp_set_device(int device)
{
    DLP_HIP_TRY(hipSetDevice(device));
    return DLP_OK;
}

int dlp_device_name(int device, char *buf, size_t buf_len)
{
    DLP_REQUIRE(buf != nullptr && buf_len > 0, "null argument");
    hipDeviceProp_t prop;
    DLP_HIP_TRY(hipGetDeviceProperties(&prop, device));
    std::string s = std::string(prop.name) + " (" + prop.gcnArchName + ")";
    std::strncpy(buf, s.c_str(), buf_len - 1);
    buf[buf_len - 1] = 0;
    return DLP_OK;
}

int dlp_malloc(void **dev_ptr, size_t bytes)
{
    DLP_REQUIRE(dev_ptr != nullptr, "null argument");
    *dev_ptr = nullptr;
    if (bytes == 0)
        return DLP_OK;
    DLP_HIP_TRY(hipMalloc(dev_ptr, bytes));
    return DLP_OK;
}

int dlp_free(void *dev_ptr)
{
    if (dev_ptr)
        DLP_HIP_TRY(hipFree(dev_ptr));
    return DLP_OK;
}

int dlp_memcpy_h2d(void *dst_dev, const void *src_host, size_t bytes, void *stream)
{
    if (bytes == 0)
        return DLP_OK;
    DLP_HIP_TRY(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
    DLP_HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return DLP_OK;
}

int dlp_memcpy_d2h(void *dst_host, const void *src_dev, size_t bytes, void *stream)
{
    if (bytes == 0)
        return DLP_OK;
    DLP_HIP_TRY(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
    DLP_HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return DLP_OK;
}

int dlp_stream_create(void **stream)
{
    DLP_REQUIRE(stream != nullptr, "null argument");
    hipStream_t s;
    DLP_HIP_TRY(hipStreamCreate(&s)); // default priority
    *stream = (void *)s;
    return DLP_OK;
}

int dlp_stream_sync(void *stream)
{
    DLP_HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return DLP_OK;
}

int dlp_stream_destroy(void *stream)
{
    if (stream)
        DLP_HIP_TRY(hipStreamDestroy((hipStream_t)stream));
    return DLP_OK;
}

// ---- HIP graphs: record what a stream is given once, replay it with one launch ----
struct dlp_graph {
    hipGraph_t graph;
    hipGraphExec_t exec;
};

int dlp_graph_capture_begin(void *stream)
{
    DLP_REQUIRE(stream != nullptr, "capture needs a stream of its own (not the default stream)");
    {
        std::lock_guard<std::mutex> lock(g_timing_mutex);
        DLP_REQUIRE(!g_timing_enabled, "per-kernel timing records events: switch it off before capturing");
    }
    // relaxed: other threads of the process (a framework's allocator) may keep calling the runtime meanwhile
    DLP_HIP_TRY(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeRelaxed));
    return DLP_OK;
}

int dlp_graph_capture_end(void *stream, dlp_graph **out)
{
    DLP_REQUIRE(stream != nullptr && out != nullptr, "null argument");
    *out = nullptr;
    hipGraph_t graph = nullptr;
    DLP_HIP_TRY(hipStreamEndCapture((hipStream_t)stream, &graph));
    if (!graph)
        return fail(DLP_ERR_RUNTIME, "stream capture produced no graph");
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(graph);
        return fail(DLP_ERR_RUNTIME, std::string("hipGraphInstantiate: ") + hipGetErrorString(e));
    }
    dlp_graph *g = new (std::nothrow) dlp_graph();
    if (!g) {
        (void)hipGraphExecDestroy(exec);
        (void)hipGraphDestroy(graph);
        return fail(DLP_ERR_RUNTIME, "out of host memory");
    }
    g->graph = graph;
    g->exec = exec;
    *out = g;
    return DLP_OK;
}

int dlp_graph_launch(dlp_graph *g, void *stream)
{
    DLP_REQUIRE(g != nullptr, "null argument");
    DLP_HIP_TRY(hipGraphLaunch(g->exec, (hipStream_t)stream));
    return DLP_OK;
}

void dlp_graph_destroy(dlp_graph *g)
{
    if (!g)
        return;
    (void)hipGraphExecDestroy(g->exec);
    (void)hipGraphDestroy(g->graph);
    delete g;
}

int dlp_conv2d_output_shape(const dlp_conv2d_settings *cfg, const int in_shape[4], int out_shape[4])
{
    return output_shape(cfg, in_shape, out_shape);
}

int dlp_conv2d_fwd_create(const dlp_conv2d_settings *cfg, int bias, int activation, const char *algo, dlp_conv2d_fwd **out)
{
    DLP_REQUIRE(cfg != nullptr && out != nullptr, "null argument");
    *out = nullptr;
    DLP_REQUIRE(cfg->channels_in > 0 && cfg->channels_out > 0 && cfg->groups > 0, "channels/groups must be positive");
    // src/ops/conv2d.cpp:105-106
    DLP_REQUIRE(cfg->channels_in % cfg->groups == 0 && cfg->channels_out % cfg->groups == 0, "channels not divisible by groups");
    DLP_REQUIRE(valid_activation(activation), "unknown activation");
    // The reference checks dtype == float_data (src/gemm.cpp:593).  Here bfloat16_data is
    // also accepted: x, w, y are stored as bf16, bias stays fp32, all arithmetic is fp32
    // (all three algorithms serve it).
    if (cfg->dtype != DLP_FLOAT && cfg->dtype != DLP_BFLOAT16)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "Conv2DForward: float_data and bfloat16_data are implemented");
    std::string al = algo ? algo : "";
    DLP_REQUIRE(al == "" || al == "auto" || al == "gemm" || al == "winograd" || al == "depthwise_separable", "unknown algorithm name");

    ConvGeom g;
    int rc = make_geom(*cfg, cfg->shape, g);
    if (rc != DLP_OK)
        return rc;

    // src/core/conv.cpp:704-729: requested-but-incompatible silently becomes gemm.
    // The depthwise kernel here also covers stride 2, which the reference's does not.
    const bool win = winograd_supported(g);
    const bool dsc = depthwise_supported(g);
    const bool auto_algo = al == "" || al == "auto";
    ConvAlgo chosen = ALGO_GEMM;
    // bf16 tensors whose GEMM runs on the bf16 matrix instruction are faster there than through
    // Winograd (whose transforms force fp32 matrix instructions): automatic choice keeps gemm
    const GemmPlan gplan = conv_gemm_plan(g, activation);
    const bool bf16_mfma = gplan.order >= GEMM_ORDER_TAP_BF16;
    // Where the reference rule would pick Winograd (src/core/conv.cpp:714-718), the automatic choice here keeps "gemm" for layers that
    // the LDS-patch kernel serves and that (a) have fewer than 64 input channels, or fewer than 128 with a filter count off 64 (the
    // Winograd kernel then gives a workgroup 32 output channels: 130 against 126 us on 64->64 at 56x56, batch 64), or (b) leave the
    // Winograd kernel fewer than one and a half workgroups per compute unit at the batch of the settings.  Whole layers, weights
    // transformed in the call, cold tensors, gemm / winograd, at batch 64: 64->64 at 56x56 150 / 125 us, 128->128 at 28x28 129 / 108,
    // 256->256 at 14x14 123 / 97, 512->512 at 7x7 124 / 105; at batch 16: 49 / 40, 45 / 39, 47 / 46 (200 workgroups), 48 / 77 (128).
    const int cin_g = cfg->channels_in / cfg->groups;
    bool gemm_faster = false;
    if (gplan.patch && win) {
        const WinoPlan wp = winograd_plan(g);
        const long long wgs = winograd_workgroups(g, wp, winograd_blocks_per_workgroup(g, wp));
        gemm_faster = cin_g < 64 || (cin_g < 128 && cfg->channels_out % 64 != 0) || wgs * 2 < 3ll * dlp_cu_count();
    }
    if ((al == "winograd" && win) || (auto_algo && win && !bf16_mfma && !gemm_faster && cfg->channels_in >= 8 && cfg->channels_out >= 8))
        chosen = ALGO_WINOGRAD;
    else if ((al == "depthwise_separable" && dsc) || (auto_algo && dsc))
        chosen = ALGO_DEPTHWISE;

    dlp_conv2d_fwd *op = new (std::nothrow) dlp_conv2d_fwd();
    if (!op)
        return fail(DLP_ERR_RUNTIME, "out of host memory");
    op->cfg = *cfg;
    op->bias = bias != 0;
    op->activation = activation;
    op->algo = chosen;
    op->ktab = nullptr;
    op->workspace = 0;
    for (int i = 0; i < 6; i++)
        op->packed_layout[i] = -1;
    op->accumulate_first = 0;
    op->x_channels_last = 0;
    op->y_channels_last = 0;
    op->max_pool = 0;
    op->counters = nullptr;
    op->counter_count = 0;
    if (hipGetDevice(&op->device) != hipSuccess)
        op->device = 0;
    if (chosen == ALGO_GEMM) {
        op->workspace = conv_gemm_workspace_bytes(g, activation);
        rc = upload_ktab(g, activation, &op->ktab);
        int *unused = nullptr;
        if (rc == DLP_OK) // counters for the batch of the hint, so that a first call inside a stream capture allocates nothing
            rc = own_counters(op, g, conv_gemm_plan(g, activation), &unused);
    } else if (chosen == ALGO_WINOGRAD) {
        op->wino = winograd_plan(g);
        op->workspace = op->wino.ws_bytes;
    }
    if (rc != DLP_OK) {
        delete op;
        return rc;
    }
    *out = op;
    return DLP_OK;
}

const char *dlp_conv2d_fwd_algo(const dlp_conv2d_fwd *op)
{
    if (!op)
        return "";
    switch (op->algo) {
    case ALGO_WINOGRAD:
        return "winograd";
    case ALGO_DEPTHWISE:
        return "depthwise_separable";
    default:
        return "gemm";
    }
}

size_t dlp_conv2d_fwd_workspace(const dlp_conv2d_fwd *op) { return op ? op->workspace : 0; }

int dlp_conv2d_fwd_enqueue(dlp_conv2d_fwd *op, const int x_shape[4], const void *x, const void *w, const void *bias, void *y,
                           void *ws, size_t ws_bytes, float factor, void *stream)
{
    DLP_REQUIRE(op != nullptr && x_shape != nullptr, "null argument");
    DLP_REQUIRE(x_shape[0] >= 0, "negative batch");
    // the op is specialised for the H x W it was created with (the reference
    // re-runs setup_algo when they change, src/ops/conv2d.cpp:200-209)
    DLP_REQUIRE(x_shape[1] == op->cfg.channels_in && x_shape[2] == op->cfg.shape[2] && x_shape[3] == op->cfg.shape[3],
                "input shape differs from the shape given at create (only the batch may change)");
    // bias pointer present iff created with bias (src/gemm.cpp:526-533)
    DLP_REQUIRE((bias != nullptr) == op->bias, "bias pointer must be given exactly when the op was created with bias");
    ConvGeom g;
    int rc = op_geom(op, x_shape, g);
    if (rc != DLP_OK)
        return rc;
    if (g.B == 0)
        return DLP_OK;
    DLP_REQUIRE(x != nullptr && w != nullptr && y != nullptr, "null tensor pointer");
    Epilogue ep;
    ep.bias = (const float *)bias;
    ep.factor = factor;
    ep.activation = op->activation;
    ep.accumulate_first = op->accumulate_first;
    hipStream_t s = (hipStream_t)stream;
    switch (op->algo) {
    case ALGO_WINOGRAD:
        return winograd_launch(g, op->wino, x, w, y, ws, ws_bytes, ep, s);
    case ALGO_DEPTHWISE:
        return depthwise_launch(g, x, w, y, ep, s);
    default: {
        // workspace = packed weights | split-K partial sums
        const GemmPlan plan = conv_gemm_plan(g, op->activation);
        DLP_REQUIRE(ws != nullptr && ws_bytes >= plan.wpack_bytes, "workspace smaller than workspace()");
        const size_t used = round256(plan.wpack_bytes);
        void *part = ws_bytes > used ? (char *)ws + used : nullptr;
        int *counters = nullptr;
        rc = own_counters(op, g, plan, &counters);
        if (rc != DLP_OK)
            return rc;
        rc = conv_gemm_pack_weights(g, plan, w, ws, s, part, part ? ws_bytes - used : 0, GEMM_PACK_AND_CLEAR, true);
        if (rc != DLP_OK)
            return rc;
        return conv_gemm_launch(g, plan, op->ktab, x, ws, y, ep, s, -1, part, part ? ws_bytes - used : 0, w, counters);
    }
    }
}

// ---- weights that stay constant between calls: transformed once into a buffer of the caller ----
static void layout_of(const GemmPlan &p, int (&sig)[6])
{
    sig[0] = p.order;
    sig[1] = p.BM;
    sig[2] = p.nkt;
    sig[3] = p.mtiles;
    sig[4] = p.patch;
    sig[5] = p.wdirect;
}

int dlp_conv2d_fwd_set_accumulate_first(dlp_conv2d_fwd *op, int on)
{
    DLP_REQUIRE(op != nullptr, "null argument");
    if (on && op->algo == ALGO_DEPTHWISE)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "accumulation before the activation: algorithms gemm and winograd");
    op->accumulate_first = on ? 1 : 0;
    return DLP_OK;
}

int dlp_conv2d_fwd_set_channels_last(dlp_conv2d_fwd *op, int x_channels_last, int y_channels_last)
{
    DLP_REQUIRE(op != nullptr, "null argument");
    x_channels_last = x_channels_last ? 1 : 0;
    y_channels_last = y_channels_last ? 1 : 0;
    if (x_channels_last == op->x_channels_last && y_channels_last == op->y_channels_last)
        return DLP_OK;
    if ((x_channels_last || y_channels_last) && op->max_pool)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "channels-last tensors: not with a max pooling inside the convolution");
    if ((x_channels_last || y_channels_last) && op->algo != ALGO_GEMM)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "channels-last tensors: algorithm gemm on bfloat16_data only");
    ConvGeom g;
    int rc = make_geom(op->cfg, op->cfg.shape, g);
    if (rc != DLP_OK)
        return rc;
    g.x_channels_last = x_channels_last;
    g.y_channels_last = y_channels_last;
    if (!conv_gemm_layouts_supported(g, op->activation))
        return fail(DLP_ERR_NOT_IMPLEMENTED, "channels-last tensors: served by the bf16 matrix-instruction kernels only (bfloat16_data, relu-like or no "
                                             "activation, input channels per group in multiples of 32 for x, output channels per group in eights for y)");
    // the gather table and the workspace depend on the layout of x: build them anew
    KTabEntry *ktab = nullptr;
    rc = upload_ktab(g, op->activation, &ktab);
    if (rc != DLP_OK)
        return rc;
    if (op->ktab)
        (void)hipFree(op->ktab); // synchronises with the launches that still read the old table
    op->ktab = ktab;
    op->x_channels_last = x_channels_last;
    op->y_channels_last = y_channels_last;
    op->workspace = conv_gemm_workspace_bytes(g, op->activation);
    return DLP_OK;
}

int dlp_conv2d_fwd_fuse_max_pool(dlp_conv2d_fwd *op, int kernel, int stride, int pad, int ceil_mode)
{
    DLP_REQUIRE(op != nullptr, "null argument");
    ConvGeom g;
    const int rc = make_geom(op->cfg, op->cfg.shape, g);
    if (rc != DLP_OK)
        return rc;
    const int ph = (g.OH + 2 - 3) / 2 + 1, pw = (g.OW + 2 - 3) / 2 + 1;
    if (kernel != 3 || stride != 2 || pad != 1 || ceil_mode || op->algo != ALGO_GEMM || op->x_channels_last || op->y_channels_last ||
        op->activation == DLP_ACT_TANH || op->activation == DLP_ACT_SIGMOID || !conv_stem_pool_supported(g, ph, pw))
        return fail(DLP_ERR_NOT_IMPLEMENTED, "max pooling inside the convolution: 3x3 stride 2 pad 1 (floor mode) behind the bfloat16 7x7 stride-2 "
                                             "convolution of 3 channels, rows of the image, of y and of the pooled y in multiples of 8 (y up to 112 wide), "
                                             "relu-like or no activation");
    op->max_pool = 1;
    return DLP_OK;
}

size_t dlp_conv2d_fwd_packed_bytes(const dlp_conv2d_fwd *op)
{
    if (!op)
        return 0;
    if (op->algo == ALGO_WINOGRAD)
        return round256(op->wino.ws_bytes);
    if (op->algo == ALGO_DEPTHWISE)
        return 0;
    ConvGeom g;
    if (op_geom(op, op->cfg.shape, g) != DLP_OK)
        return 0;
    return round256(conv_gemm_plan(g, op->activation).wpack_bytes);
}

int dlp_conv2d_fwd_pack(dlp_conv2d_fwd *op, const void *w, void *packed, void *stream)
{
    DLP_REQUIRE(op != nullptr && w != nullptr, "null argument");
    if (op->algo == ALGO_DEPTHWISE)
        return DLP_OK; // the kernel reads the filter as it is
    DLP_REQUIRE(packed != nullptr, "null buffer for the packed weights");
    ConvGeom g;
    int rc = op_geom(op, op->cfg.shape, g);
    if (rc != DLP_OK)
        return rc;
    if (op->algo == ALGO_WINOGRAD) {
        Epilogue ep = {nullptr, 0.0f, op->activation};
        return winograd_launch(g, op->wino, nullptr, w, nullptr, packed, op->wino.ws_bytes, ep, (hipStream_t)stream, WINO_FILTER_ONLY);
    }
    const GemmPlan plan = conv_gemm_plan(g, op->activation);
    layout_of(plan, op->packed_layout);
    return conv_gemm_pack_weights(g, plan, w, packed, (hipStream_t)stream, nullptr, 0, GEMM_PACK_ONLY);
}

int dlp_conv2d_fwd_enqueue_packed(dlp_conv2d_fwd *op, const int x_shape[4], const void *x, const void *w, const void *packed, const void *bias,
                                  void *y, void *ws, size_t ws_bytes, float factor, void *stream)
{
    DLP_REQUIRE(op != nullptr && x_shape != nullptr, "null argument");
    DLP_REQUIRE(x_shape[0] >= 0, "negative batch");
    DLP_REQUIRE(x_shape[1] == op->cfg.channels_in && x_shape[2] == op->cfg.shape[2] && x_shape[3] == op->cfg.shape[3],
                "input shape differs from the shape given at create (only the batch may change)");
    DLP_REQUIRE((bias != nullptr) == op->bias, "bias pointer must be given exactly when the op was created with bias");
    ConvGeom g;
    int rc = op_geom(op, x_shape, g);
    if (rc != DLP_OK)
        return rc;
    if (g.B == 0)
        return DLP_OK;
    DLP_REQUIRE(x != nullptr && w != nullptr && y != nullptr, "null tensor pointer");
    Epilogue ep;
    ep.bias = (const float *)bias;
    ep.factor = factor;
    ep.activation = op->activation;
    ep.accumulate_first = op->accumulate_first;
    hipStream_t s = (hipStream_t)stream;
    switch (op->algo) {
    case ALGO_WINOGRAD:
        DLP_REQUIRE(packed != nullptr, "null buffer of packed weights");
        return winograd_launch(g, op->wino, x, w, y, const_cast<void *>(packed), op->wino.ws_bytes, ep, s, WINO_RUN_ONLY);
    case ALGO_DEPTHWISE:
        return depthwise_launch(g, x, w, y, ep, s);
    default: {
        const GemmPlan plan = conv_gemm_plan(g, op->activation);
        int sig[6];
        layout_of(plan, sig);
        for (int i = 0; i < 6; i++)
            DLP_REQUIRE(sig[i] == op->packed_layout[i], "the weights were packed for another tile plan (pack again for this batch)");
        DLP_REQUIRE(packed != nullptr, "null buffer of packed weights");
        void *part = ws_bytes > 0 ? ws : nullptr;
        int *counters = nullptr;
        rc = own_counters(op, g, plan, &counters);
        if (rc != DLP_OK)
            return rc;
        // fp32 1x1 convolutions could read w in place, but the packed tiles are there and load faster: no w, no in-place reading
        const void *w_arg = (plan.wdirect && plan.order < GEMM_ORDER_TAP_BF16 && !plan.pointwise) ? nullptr : w;
        return conv_gemm_launch(g, plan, op->ktab, x, packed, y, ep, s, -1, part, ws_bytes, w_arg, counters);
    }
    }
}

void dlp_conv2d_fwd_destroy(dlp_conv2d_fwd *op)
{
    if (!op)
        return;
    if (op->ktab)
        (void)hipFree(op->ktab);
    if (op->counters)
        (void)hipFree(op->counters);
    delete op;
}

// ---- depthwise 3x3 + pointwise 1x1 in one launch (conv_dwpw.hip) ----
struct dlp_dwpw_fwd {
    dlp_conv2d_settings cfg; // the depthwise layer
    int channels_out;        // filters of the pointwise layer
    bool dw_bias, pw_bias;
    int dw_activation, pw_activation;
    int accumulate_first;
};

int dlp_dwpw_fwd_supported(const dlp_conv2d_settings *dw_cfg, int dw_activation, int channels_out, int pw_activation)
{
    if (!dw_cfg || !valid_activation(dw_activation) || !valid_activation(pw_activation) || channels_out <= 0)
        return 0;
    if (dw_cfg->channels_in <= 0 || dw_cfg->groups <= 0 || dw_cfg->channels_in % dw_cfg->groups != 0 || dw_cfg->channels_out % dw_cfg->groups != 0)
        return 0;
    ConvGeom g;
    if (make_geom(*dw_cfg, dw_cfg->shape, g) != DLP_OK)
        return 0;
    return conv_dwpw_supported(g, channels_out, dw_activation, pw_activation) ? 1 : 0;
}

int dlp_dwpw_fwd_create(const dlp_conv2d_settings *dw_cfg, int dw_bias, int dw_activation, int channels_out, int pw_bias, int pw_activation,
                        dlp_dwpw_fwd **out)
{
    DLP_REQUIRE(dw_cfg != nullptr && out != nullptr, "null argument");
    *out = nullptr;
    DLP_REQUIRE(dw_cfg->channels_in > 0 && dw_cfg->channels_out > 0 && dw_cfg->groups > 0 && channels_out > 0, "channels/groups must be positive");
    DLP_REQUIRE(dw_cfg->channels_in % dw_cfg->groups == 0 && dw_cfg->channels_out % dw_cfg->groups == 0, "channels not divisible by groups");
    DLP_REQUIRE(valid_activation(dw_activation) && valid_activation(pw_activation), "unknown activation");
    ConvGeom g;
    int rc = make_geom(*dw_cfg, dw_cfg->shape, g);
    if (rc != DLP_OK)
        return rc;
    if (!conv_dwpw_supported(g, channels_out, dw_activation, pw_activation))
        return fail(DLP_ERR_NOT_IMPLEMENTED,
                    "fused depthwise + pointwise: float_data, depthwise 3x3 with padding 1 and stride 1 or 2 on images of at least 512 pixels and at most "
                    "56 wide (output width a multiple of 4, or of 2 at stride 2 up to 28 wide), channels a multiple of 8, at most 128 filters, "
                    "identity / relu / relu6; run the two operators separately otherwise");
    dlp_dwpw_fwd *op = new (std::nothrow) dlp_dwpw_fwd();
    if (!op)
        return fail(DLP_ERR_RUNTIME, "out of host memory");
    op->cfg = *dw_cfg;
    op->channels_out = channels_out;
    op->dw_bias = dw_bias != 0;
    op->pw_bias = pw_bias != 0;
    op->dw_activation = dw_activation;
    op->pw_activation = pw_activation;
    op->accumulate_first = 0;
    *out = op;
    return DLP_OK;
}

int dlp_dwpw_fwd_set_accumulate_first(dlp_dwpw_fwd *op, int on)
{
    DLP_REQUIRE(op != nullptr, "null argument");
    op->accumulate_first = on ? 1 : 0;
    return DLP_OK;
}

int dlp_dwpw_fwd_enqueue(dlp_dwpw_fwd *op, const int x_shape[4], const void *x, const void *dw_w, const void *dw_bias, const void *pw_w,
                         const void *pw_bias, void *y, float factor, void *stream)
{
    DLP_REQUIRE(op != nullptr && x_shape != nullptr, "null argument");
    DLP_REQUIRE(x_shape[0] >= 0, "negative batch");
    DLP_REQUIRE(x_shape[1] == op->cfg.channels_in && x_shape[2] == op->cfg.shape[2] && x_shape[3] == op->cfg.shape[3],
                "input shape differs from the shape given at create (only the batch may change)");
    DLP_REQUIRE((dw_bias != nullptr) == op->dw_bias && (pw_bias != nullptr) == op->pw_bias,
                "bias pointers must be given exactly when the op was created with that bias");
    ConvGeom g;
    int rc = make_geom(op->cfg, x_shape, g);
    if (rc != DLP_OK)
        return rc;
    if (g.B == 0)
        return DLP_OK;
    DLP_REQUIRE(x != nullptr && dw_w != nullptr && pw_w != nullptr && y != nullptr, "null tensor pointer");
    Epilogue ep;
    ep.bias = (const float *)pw_bias;
    ep.factor = factor;
    ep.activation = op->pw_activation;
    ep.accumulate_first = op->accumulate_first;
    return conv_dwpw_launch(g, op->channels_out, x, dw_w, (const float *)dw_bias, op->dw_activation, pw_w, y, ep, (hipStream_t)stream);
}

void dlp_dwpw_fwd_destroy(dlp_dwpw_fwd *op) { delete op; }

int dlp_ip_fwd_create(const dlp_ip_settings *cfg, int bias, int activation, dlp_ip_fwd **out)
{
    DLP_REQUIRE(cfg != nullptr && out != nullptr, "null argument");
    *out = nullptr;
    DLP_REQUIRE(cfg->inputs > 0 && cfg->outputs > 0, "inputs/outputs must be positive");
    DLP_REQUIRE(valid_activation(activation), "unknown activation");
    // float_data as in the reference (src/gemm.cpp:577), plus bfloat16_data storage (fp32 bias and arithmetic)
    if (cfg->dtype != DLP_FLOAT && cfg->dtype != DLP_BFLOAT16)
        return fail(DLP_ERR_NOT_IMPLEMENTED, "IPForward: float_data and bfloat16_data are implemented");
    dlp_ip_fwd *op = new (std::nothrow) dlp_ip_fwd();
    if (!op)
        return fail(DLP_ERR_RUNTIME, "out of host memory");
    op->cfg = *cfg;
    op->bias = bias != 0;
    op->activation = activation;
    op->ktab = nullptr;
    if (hipGetDevice(&op->device) != hipSuccess)
        op->device = 0;
    const ConvGeom g1 = ip_gemm_geom(1, cfg->inputs, cfg->outputs, cfg->dtype);
    op->plan = conv_gemm_plan(g1, activation);
    op->wpacked = nullptr;
    op->scratch = nullptr;
    op->scratch_bytes = op->scratch_cnt_bytes = 0;
    int rc = upload_ktab(g1, activation, &op->ktab);
    if (rc == DLP_OK) { // set-up of dlp_ip_fwd_enqueue_no_alloc on this device, so that its first call may sit inside a stream capture
        void *unused = nullptr;
        rc = scratch_on_current_device(&unused);
    }
    if (rc != DLP_OK) {
        if (op->ktab)
            (void)hipFree(op->ktab);
        delete op;
        return rc;
    }
    ip_stream_prepare(cfg->dtype);
    *out = op;
    return DLP_OK;
}

int dlp_ip_fwd_enqueue(dlp_ip_fwd *op, int batch, const void *x, const void *w, const void *bias, void *y, void *stream)
{
    DLP_REQUIRE(op != nullptr, "null argument");
    DLP_REQUIRE(batch >= 0, "negative batch");
    DLP_REQUIRE((bias != nullptr) == op->bias, "bias pointer must be given exactly when the op was created with bias");
    if (batch == 0)
        return DLP_OK;
    DLP_REQUIRE(x != nullptr && w != nullptr && y != nullptr, "null tensor pointer");
    Epilogue ep;
    ep.bias = (const float *)bias;
    ep.factor = 0.0f; // src/core/ip.cpp:38
    ep.activation = op->activation;
    if (ip_direct_supported(op->cfg.inputs, op->cfg.dtype, x, w)) {
        IpPlan ip;
        // large weight matrices stream through LDS (ip_stream_kernel); the scratch layout is the same for both kernels
        const bool streamed = ip_stream_supported(batch, op->cfg.inputs, op->cfg.outputs, op->cfg.dtype, x, w);
        const size_t need = streamed ? ip_stream_scratch_bytes(batch, op->cfg.inputs, op->cfg.outputs, op->cfg.dtype, &ip)
                                     : ip_direct_scratch_bytes(batch, op->cfg.inputs, op->cfg.outputs, op->cfg.dtype, &ip);
        (void)need;
        // op-owned scratch = [counters | partial sums]; both regions only ever grow, and the counter region keeps
        // its place so that no partial sum is ever written where a later, larger batch expects zeroed counters
        if (ip.cnt_bytes > op->scratch_cnt_bytes || ip.part_bytes > op->scratch_bytes - op->scratch_cnt_bytes) {
            // first call, or a larger batch than any before: hipFree waits for the kernels that use the old buffer
            const size_t cnt_bytes = std::max(ip.cnt_bytes, op->scratch_cnt_bytes);
            const size_t part_bytes = std::max(ip.part_bytes, op->scratch_bytes - op->scratch_cnt_bytes);
            if (op->scratch)
                (void)hipFree(op->scratch);
            op->scratch = nullptr;
            op->scratch_bytes = op->scratch_cnt_bytes = 0;
            DLP_HIP_TRY(hipMalloc(&op->scratch, cnt_bytes + part_bytes));
            DLP_HIP_TRY(hipMemset(op->scratch, 0, cnt_bytes));
            op->scratch_bytes = cnt_bytes + part_bytes;
            op->scratch_cnt_bytes = cnt_bytes;
        }
        if (streamed)
            return ip_stream_launch(batch, op->cfg.inputs, op->cfg.outputs, op->cfg.dtype, x, w, y, ep, (int *)op->scratch,
                                    (float *)((char *)op->scratch + op->scratch_cnt_bytes), (hipStream_t)stream);
        return ip_direct_launch(batch, op->cfg.inputs, op->cfg.outputs, op->cfg.dtype, x, w, y, ep, (int *)op->scratch,
                                (float *)((char *)op->scratch + op->scratch_cnt_bytes), (hipStream_t)stream);
    }
    const ConvGeom g = ip_gemm_geom(batch, op->cfg.inputs, op->cfg.outputs, op->cfg.dtype);
    // the packed copy of w (about the size of w) exists only for operators that ever come here: bf16 rows of odd length
    if (!op->wpacked)
        DLP_HIP_TRY(hipMalloc(&op->wpacked, op->plan.wpack_bytes));
    int rc = conv_gemm_pack_weights(g, op->plan, w, op->wpacked, (hipStream_t)stream);
    if (rc != DLP_OK)
        return rc;
    return conv_gemm_launch(g, op->plan, op->ktab, x, op->wpacked, y, ep, (hipStream_t)stream, -1, nullptr, 0, w);
}

int dlp_ip_fwd_enqueue_no_alloc(dlp_ip_fwd *op, int batch, const void *x, const void *w, const void *bias, void *y, void *stream)
{
    DLP_REQUIRE(op != nullptr, "null argument");
    DLP_REQUIRE(batch >= 0, "negative batch");
    DLP_REQUIRE((bias != nullptr) == op->bias, "bias pointer must be given exactly when the op was created with bias");
    if (batch == 0)
        return DLP_OK;
    DLP_REQUIRE(x != nullptr && w != nullptr && y != nullptr, "null tensor pointer");
    if (!ip_direct_supported(op->cfg.inputs, op->cfg.dtype, x, w))
        return fail(DLP_ERR_NOT_IMPLEMENTED, "dlp_ip_fwd_enqueue_no_alloc: bfloat16 rows must have an even length and dword-aligned tensors");
    IpPlan ip;
    const bool streamed = ip_stream_supported(batch, op->cfg.inputs, op->cfg.outputs, op->cfg.dtype, x, w); // the kernel dlp_ip_fwd_enqueue takes
    if (streamed)
        ip_stream_scratch_bytes(batch, op->cfg.inputs, op->cfg.outputs, op->cfg.dtype, &ip);
    else
        ip_direct_scratch_bytes(batch, op->cfg.inputs, op->cfg.outputs, op->cfg.dtype, &ip);
    // (an unsplit K uses neither counters nor partial sums)
    if (ip.S > 1 && (ip.cnt_bytes > kNoAllocCounterBytes || ip.part_bytes > (size_t)DLP_IP_NO_ALLOC_SCRATCH_BYTES - kNoAllocCounterBytes))
        return fail(DLP_ERR_VALIDATION, "dlp_ip_fwd_enqueue_no_alloc: this batch x outputs needs " + std::to_string(ip.cnt_bytes) + " + " +
                                            std::to_string(ip.part_bytes) + " bytes of scratch, the library's array holds " +
                                            std::to_string(kNoAllocCounterBytes) + " + " +
                                            std::to_string((size_t)DLP_IP_NO_ALLOC_SCRATCH_BYTES - kNoAllocCounterBytes) +
                                            " (use dlp_ip_fwd_enqueue)");
    void *base = nullptr;
    int rc = scratch_on_current_device(&base);
    if (rc != DLP_OK)
        return rc;
    Epilogue ep;
    ep.bias = (const float *)bias;
    ep.factor = 0.0f;
    ep.activation = op->activation;
    int *counters = (int *)base;
    float *partials = (float *)((char *)base + kNoAllocCounterBytes);
    if (ip.S > 1) {
        // the array keeps what the last call left: the counters of this launch start from zero whatever that was
        const int n = ip.mblocks * ip.nchunks;
        hipLaunchKernelGGL(clear_ints_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, counters, n);
        DLP_HIP_TRY(hipGetLastError());
    }
    if (streamed)
        return ip_stream_launch(batch, op->cfg.inputs, op->cfg.outputs, op->cfg.dtype, x, w, y, ep, counters, partials, (hipStream_t)stream);
    return ip_direct_launch(batch, op->cfg.inputs, op->cfg.outputs, op->cfg.dtype, x, w, y, ep, counters, partials, (hipStream_t)stream);
}

void dlp_ip_fwd_destroy(dlp_ip_fwd *op)
{
    if (!op)
        return;
    if (op->ktab)
        (void)hipFree(op->ktab);
    if (op->wpacked)
        (void)hipFree(op->wpacked);
    if (op->scratch)
        (void)hipFree(op->scratch);
    delete op;
}

} // extern "C"

