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

__global__ __launch_bounds__(256) void copy_f4(const float4 *__restrict__ src, float4 *__restrict__ dst, size_t n)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride)
        dst[i] = src[i];
}

__global__ __launch_bounds__(256) void read_f4(const float4 *__restrict__ src, float *out, size_t n)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    float4 s = {0, 0, 0, 0};
    for (; i < n; i += stride) {
        const float4 v = src[i];
        s.x += v.x;
        s.y += v.y;
        s.z += v.z;
        s.w += v.w;
    }
    if (s.x + s.y + s.z + s.w == 12345.678f) // never true for the probe's data
        out[0] = 1.0f;
}

__global__ __launch_bounds__(256) void write_f4(float4 *__restrict__ dst, size_t n)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    const float4 v = {1, 2, 3, 4};
    for (; i < n; i += stride)
        dst[i] = v;
}

// reads n_in and writes n_out 16-byte pieces (the sizes may differ, as for a strided convolution): one piece per thread and
// direction, 32-bit index, no loop -- the plainest streaming kernel there is
__global__ __launch_bounds__(256) void read_write_f4(const float4 *__restrict__ src, int n_in, float4 *__restrict__ dst, int n_out)
{
    const int i = (int)(blockIdx.x * 256 + threadIdx.x);
    float4 v = {0, 0, 0, 0};
    if (i < n_in)
        v = src[i];
    if (i < n_out)
        dst[i] = v;
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

// streaming copy bandwidth in GB/s (read + write bytes) over `mbytes` MiB per direction.
int dlp_probe_copy(int mbytes, double *gbs)
{
    size_t bytes = (size_t)mbytes << 20;
    float4 *a = nullptr, *b = nullptr;
    if (hipMalloc(&a, bytes) != hipSuccess || hipMalloc(&b, bytes) != hipSuccess)
        return 1;
    (void)hipMemset(a, 1, bytes);
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    size_t n = bytes / 16;
    copy_f4<<<256 * 16, 256>>>(a, b, n);
    (void)hipEventRecord(e0, 0);
    const int reps = 10;
    for (int r = 0; r < reps; r++)
        copy_f4<<<256 * 16, 256>>>(a, b, n);
    (void)hipEventRecord(e1, 0);
    float ms = time_ms(0, e0, e1);
    *gbs = 2.0 * bytes * reps / (ms * 1e-3) / 1e9;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(a);
    (void)hipFree(b);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}

// What a plain streaming kernel reaches on tensors of a given size: reads in_bytes, writes out_bytes (16-byte
// accesses, one piece per thread and direction).  The launches run back
// to back, each on its own pair of buffers out of a ring that is larger than the 256 MB last-level cache, so every
// launch starts cold, as a layer in a network does; one event pair brackets all of them (an event between two
// launches makes the first one write back its part of the L2 before it ends, which a kernel inside a network does not).
// gbs = (in_bytes + out_bytes) / mean launch time; us = that mean time in microseconds.
int dlp_probe_copy_sized(size_t in_bytes, size_t out_bytes, double *gbs, double *us)
{
    in_bytes = (in_bytes + 15) / 16 * 16;
    out_bytes = (out_bytes + 15) / 16 * 16;
    const size_t pair = in_bytes + out_bytes;
    if (pair == 0)
        return 1;
    int nbuf = (int)(((size_t)768 << 20) / pair) + 1;
    if (nbuf < 2)
        nbuf = 2;
    if (nbuf > 64)
        nbuf = 64;
    char *ring = nullptr;
    if (hipMalloc(&ring, pair * nbuf) != hipSuccess)
        return 1;
    (void)hipMemset(ring, 1, pair * nbuf);
    const int reps = 3 * nbuf > 40 ? 3 * nbuf : 40;
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    const size_t n_in = in_bytes / 16, n_out = out_bytes / 16;
    const size_t n = n_in > n_out ? n_in : n_out;
    if (n >= ((size_t)1 << 31))
        return 1;
    const size_t blocks = (n + 255) / 256;
    for (int r = -nbuf; r < reps; r++) { // one untimed pass over the ring first
        char *base = ring + pair * (size_t)((r + nbuf) % nbuf);
        if (r == 0)
            (void)hipEventRecord(e0, 0);
        read_write_f4<<<(unsigned)blocks, 256>>>((const float4 *)base, (int)n_in, (float4 *)(base + in_bytes), (int)n_out);
    }
    (void)hipEventRecord(e1, 0);
    (void)hipEventSynchronize(e1);
    float total_ms = 0;
    (void)hipEventElapsedTime(&total_ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(ring);
    const double mean_ms = (double)total_ms / reps;
    *us = mean_ms * 1e3;
    *gbs = (double)pair / (mean_ms * 1e-3) / 1e9;
    return hipGetLastError() == hipSuccess ? 0 : 1;
}

// read-only (write != 0: write-only) streaming bandwidth in GB/s over `mbytes` MiB
int dlp_probe_stream(int mbytes, int write, double *gbs)
{
    size_t bytes = (size_t)mbytes << 20;
    float4 *a = nullptr;
    float *o = nullptr;
    if (hipMalloc(&a, bytes) != hipSuccess || hipMalloc(&o, 4) != hipSuccess)
        return 1;
    (void)hipMemset(a, 1, bytes);
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    size_t n = bytes / 16;
    const int reps = 10;
    for (int r = 0; r <= reps; r++) {
        if (r == 1)
            (void)hipEventRecord(e0, 0);
        if (write)
            write_f4<<<256 * 16, 256>>>(a, n);
        else
            read_f4<<<256 * 16, 256>>>(a, o, n);
    }
    (void)hipEventRecord(e1, 0);
    float ms = time_ms(0, e0, e1);
    *gbs = 1.0 * bytes * reps / (ms * 1e-3) / 1e9;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(a);
    (void)hipFree(o);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}
}
