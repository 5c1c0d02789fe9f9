// Device peak probes used only to put the roofline numbers in context:
// an MFMA-only loop (no memory traffic) and a streaming copy.  Not part of the
// operator ABI; built as a separate library, libdlp_microbench.so.
#include <hip/hip_runtime.h>
#include <cstdio>

typedef float f32x16 __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void mfma_f32_loop(float *out, int iters, float a0, float b0)
{
    f32x16 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
    float a = a0 + threadIdx.x, b = b0;
    for (int i = 0; i < iters; i++) {
        c0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c3, 0, 0, 0);
    }
    float s = 0;
    for (int r = 0; r < 16; r++)
        s += c0[r] + c1[r] + c2[r] + c3[r];
    if (s == 12345.678f) // never true: keeps the result alive without a store per thread
        out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

__global__ __launch_bounds__(256) void mfma_bf16_loop(float *out, int iters, float a0, float b0)
{
    f32x16 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
    bf16x8 a, b;
    for (int i = 0; i < 8; i++) {
        a[i] = (__bf16)(a0 + threadIdx.x + i);
        b[i] = (__bf16)(b0 + i);
    }
    for (int i = 0; i < iters; i++) {
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
    }
    float s = 0;
    for (int r = 0; r < 16; r++)
        s += c0[r] + c1[r] + c2[r] + c3[r];
    if (s == 12345.678f)
        out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// ---- streaming kernels -------------------------------------------------------------------------------------------------
// What was measured on MI355X and shapes these probes: (1) one 16-byte piece per thread in a grid as large as the tensor is the
// fastest plain form (2 GiB copy 6.2 TB/s; four or eight pieces per thread 5.7 / 5.4, a persistent grid of 8 workgroups per CU 5.5);
// (2) a grid-stride loop
// whose stride is a power of two (4096 workgroups x 4 KB = 16 MiB) keeps every workgroup on the same memory channels: a
// write-only kernel of that form reaches 3.9 TB/s where the one-piece-per-thread form reaches 6.9; (3) non-temporal loads and
// stores help below ~100 MB, where the end-of-kernel write-back of the dirty L2 lines is a large share of a launch (38 MB copy
// 8.7 -> 7.4 us), and when several pieces per thread are under way; (4) read-only peaks at 7.1 TB/s with non-temporal loads.
// The probes run each form and report the fastest, which is the yardstick ("tuned copy") the bandwidth-bound kernels are held to.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <bool NT> __device__ __forceinline__ u32x4 ld16(const u32x4 *p) { return NT ? __builtin_nontemporal_load(p) : *p; }
template <bool NT> __device__ __forceinline__ void st16(u32x4 *p, u32x4 v)
{
    if (NT)
        __builtin_nontemporal_store(v, p);
    else
        *p = v;
}

// reads n_in and writes n_out 16-byte pieces (the sizes may differ, as for a strided convolution): U pieces per thread and
// direction, consecutive threads on consecutive pieces, grid sized to the larger tensor
template <int U, int T, bool NT>
__global__ __launch_bounds__(T) void stream_kernel(const u32x4 *__restrict__ src, size_t n_in, u32x4 *__restrict__ dst, size_t n_out)
{
    const size_t base = (size_t)blockIdx.x * (U * T) + threadIdx.x;
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const size_t i = base + (size_t)u * T;
        v[u] = u32x4{1, 2, 3, 4};
        if (i < n_in)
            v[u] = ld16<NT>(src + i);
    }
    if (n_out == 0) { // read-only: keep the loads alive without a store per thread
        unsigned s = 0;
#pragma unroll
        for (int u = 0; u < U; u++)
            s |= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
        if (s == 0x12345679u)
            dst[0] = v[0];
        return;
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        const size_t i = base + (size_t)u * T;
        if (i < n_out)
            st16<NT>(dst + i, v[u]);
    }
}

// the untuned form kept for comparison: 4096 workgroups walk the tensor with a stride of 16 MiB
__global__ __launch_bounds__(256) void stream_gridstride_kernel(const u32x4 *__restrict__ src, size_t n_in, u32x4 *__restrict__ dst, size_t n_out)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const size_t n = n_in > n_out ? n_in : n_out;
    for (; i < n; i += stride) {
        u32x4 v = {1, 2, 3, 4};
        if (i < n_in)
            v = src[i];
        if (i < n_out)
            dst[i] = v;
    }
}

enum { FORM_U1 = 0, FORM_U1_NT_1024 = 1, FORM_U4_NT = 2, FORM_U8_NT = 3, FORM_GRIDSTRIDE = 4, FORM_MEMCPY = 5, N_FORMS = 6 };
static const char *const kFormNames[N_FORMS] = {"1 piece per thread", "1 piece per thread, 1024 threads, non-temporal", "4 pieces per thread, non-temporal",
                                                "8 pieces per thread, non-temporal", "grid-stride loop, stride 16 MiB", "hipMemcpyAsync device to device"};

static void launch_form(int form, const void *src, size_t in_bytes, void *dst, size_t out_bytes)
{
    const size_t n_in = in_bytes / 16, n_out = out_bytes / 16;
    const size_t n = n_in > n_out ? n_in : n_out;
    const u32x4 *s = (const u32x4 *)src;
    u32x4 *d = (u32x4 *)dst;
    switch (form) {
    case FORM_U1:
        stream_kernel<1, 256, false><<<(unsigned)((n + 255) / 256), 256>>>(s, n_in, d, n_out);
        break;
    case FORM_U1_NT_1024:
        stream_kernel<1, 1024, true><<<(unsigned)((n + 1023) / 1024), 1024>>>(s, n_in, d, n_out);
        break;
    case FORM_U4_NT:
        stream_kernel<4, 256, true><<<(unsigned)((n + 1023) / 1024), 256>>>(s, n_in, d, n_out);
        break;
    case FORM_U8_NT:
        stream_kernel<8, 256, true><<<(unsigned)((n + 2047) / 2048), 256>>>(s, n_in, d, n_out);
        break;
    case FORM_GRIDSTRIDE:
        stream_gridstride_kernel<<<256 * 16, 256>>>(s, n_in, d, n_out);
        break;
    default:
        (void)hipMemcpyAsync(dst, src, in_bytes < out_bytes ? in_bytes : out_bytes, hipMemcpyDeviceToDevice, 0);
    }
}

static float time_ms(hipStream_t s, hipEvent_t e0, hipEvent_t e1)
{
    float ms = 0;
    (void)hipEventSynchronize(e1);
    (void)hipEventElapsedTime(&ms, e0, e1);
    (void)s;
    return ms;
}

extern "C" {

// fp32 MFMA throughput in TFLOP/s with `waves_per_simd` wavefronts resident per SIMD.
int dlp_probe_mfma_f32(int waves_per_simd, double *tflops)
{
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, 0) != hipSuccess)
        return 1;
    const int cus = prop.multiProcessorCount;
    const int blocks = cus * waves_per_simd; // 256 threads = 4 waves = one per SIMD
    const int iters = 20000;
    float *out = nullptr;
    if (hipMalloc(&out, (size_t)blocks * 256 * 4) != hipSuccess)
        return 1;
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    mfma_f32_loop<<<blocks, 256>>>(out, 1000, 1.0f, 2.0f);
    (void)hipEventRecord(e0, 0);
    mfma_f32_loop<<<blocks, 256>>>(out, iters, 1.0f, 2.0f);
    (void)hipEventRecord(e1, 0);
    float ms = time_ms(0, e0, e1);
    double flops = (double)blocks * 4 /*waves*/ * iters * 4 /*mfma*/ * 4096.0;
    *tflops = flops / (ms * 1e-3) / 1e12;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(out);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}

// bf16 MFMA (32x32x16, fp32 accumulate) throughput in TFLOP/s.
int dlp_probe_mfma_bf16(int waves_per_simd, double *tflops)
{
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, 0) != hipSuccess)
        return 1;
    const int blocks = prop.multiProcessorCount * waves_per_simd;
    const int iters = 40000;
    float *out = nullptr;
    if (hipMalloc(&out, (size_t)blocks * 256 * 4) != hipSuccess)
        return 1;
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    mfma_bf16_loop<<<blocks, 256>>>(out, 1000, 1.0f, 2.0f);
    (void)hipEventRecord(e0, 0);
    mfma_bf16_loop<<<blocks, 256>>>(out, iters, 1.0f, 2.0f);
    (void)hipEventRecord(e1, 0);
    float ms = time_ms(0, e0, e1);
    double flops = (double)blocks * 4 * iters * 4 * (2.0 * 32 * 32 * 16);
    *tflops = flops / (ms * 1e-3) / 1e12;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(out);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}

// Mean launch time (microseconds) of one streaming form that reads in_bytes and writes out_bytes (either may be 0).  The launches
// run back to back, each on its own pair of buffers out of a ring that is larger than the 256 MB last-level cache, so every
// launch starts cold, as a layer in a network does; one event pair brackets all of them (an event between two launches makes the
// first one write back its part of the L2 before it ends, which a kernel inside a network does not).
static int time_form(int form, char *ring, size_t pair, size_t in_bytes, size_t out_bytes, int nbuf, int reps, double *us)
{
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    for (int r = -nbuf; r < reps; r++) { // one untimed pass over the ring first
        char *base = ring + pair * (size_t)((r + nbuf) % nbuf);
        if (r == 0)
            (void)hipEventRecord(e0, 0);
        launch_form(form, base, in_bytes, base + in_bytes, out_bytes);
    }
    (void)hipEventRecord(e1, 0);
    (void)hipEventSynchronize(e1);
    float total_ms = 0;
    (void)hipEventElapsedTime(&total_ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    *us = (double)total_ms * 1e3 / reps;
    return hipGetLastError() == hipSuccess ? 0 : 1;
}

// What streaming kernels reach on tensors of a given size: reads in_bytes, writes out_bytes (0: read-only / write-only).
// us[f] = mean launch time of form f (see kFormNames; a form that does not apply is left at 0), *best = the fastest kernel form
// (hipMemcpyAsync and the grid-stride loop are reported but never "best": the first is not a kernel of ours, the second is the
// untuned form).  Returns 0 on success.
int dlp_probe_stream_forms(size_t in_bytes, size_t out_bytes, double *us, int *best)
{
    in_bytes = (in_bytes + 15) / 16 * 16;
    out_bytes = (out_bytes + 15) / 16 * 16;
    const size_t pair = (in_bytes + out_bytes + 255) / 256 * 256;
    if (pair == 0)
        return 1;
    const size_t ring_bytes = pair >= ((size_t)1 << 30) ? pair : (size_t)768 << 20;
    int nbuf = (int)(ring_bytes / pair);
    if (nbuf < 1)
        nbuf = 1;
    if (nbuf > 64)
        nbuf = 64;
    char *ring = nullptr;
    if (hipMalloc(&ring, pair * nbuf) != hipSuccess)
        return 1;
    (void)hipMemset(ring, 1, pair * nbuf);
    const int reps = pair >= ((size_t)1 << 30) ? 6 : (3 * nbuf > 40 ? 3 * nbuf : 40);
    int rc = 0;
    *best = -1;
    for (int f = 0; f < N_FORMS && rc == 0; f++) {
        us[f] = 0;
        if (f == FORM_MEMCPY && (in_bytes != out_bytes))
            continue;
        rc = time_form(f, ring, pair, in_bytes, out_bytes, nbuf, reps, &us[f]);
        if (f < FORM_GRIDSTRIDE && (*best < 0 || us[f] < us[*best]))
            *best = f;
    }
    (void)hipFree(ring);
    return rc;
}

const char *dlp_probe_stream_form_name(int form) { return form >= 0 && form < N_FORMS ? kFormNames[form] : ""; }
int dlp_probe_stream_form_count(void) { return N_FORMS; }
}
