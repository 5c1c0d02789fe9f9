// Device peak probes used only to put the roofline numbers in context:
// an MFMA-only loop (no memory traffic) and a streaming copy.  Not part of the
// operator ABI; built as a separate library, libdlp_microbench.so.
#include <hip/hip_runtime.h>
#include <type_traits>
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


// ---- one K step of a 128 x 128 x 32 bf16 tile in a four-wavefront workgroup, piece by piece --------------------------------
// What LDS and the matrix pipe sustain together: 8 v_mfma_f32_32x32x16_bf16 per wavefront (2 x 2 blocks of 32 x 32, two halves of
// the K tile), their operands as 8 ds_read_b128 per lane (32 KB per workgroup), the next tile as 4 ds_write_b128 per lane (16 KB),
// one barrier.  Tiles lie in LDS as rows of 64 bytes whose 16-byte pieces are XOR-swizzled with the row number: reads (one row
// per lane) and stores (four lanes per row) are free of bank conflicts.
// PARTS: 1 LDS reads, 2 LDS stores, 4 barrier, 8 matrix instructions, 16 the tiles come from memory (an L2-resident buffer,
// requested three steps ahead), 32 with 16: the weight tile goes from memory straight into the operand registers (4 x 1 wavefronts
// of 32 x 128) and only the pixel tile passes through LDS.
typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));
template <int PARTS>
__global__ __launch_bounds__(256) void tile_step_kernel(int iters, float *out, const unsigned char *src, unsigned src_mask)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char step_lds[];
    constexpr int TILE = 128 * 64;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, h = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;
    for (int i = tid; i < 4 * TILE / 4; i += 256)
        ((unsigned *)step_lds)[i] = 0x3f803f80u;
    __syncthreads();
    auto at = [&](int tile, int buf, int row, int piece) { return step_lds + (buf * 2 + tile) * TILE + row * 64 + ((piece ^ ((row >> 2) & 3)) * 16); };
    const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void *)src, 0, src_mask + 1, 0x00020000);
    const unsigned pos = (blockIdx.x * 2654435761u) & src_mask & ~16383u; // this workgroup's stream of 16 KB tile pairs
    probe_f32x16 acc[4];
    for (int j = 0; j < 4; j++)
        for (int q = 0; q < 16; q++)
            acc[j][q] = 0.f;
    u32x4 regs[3][4];
    const u32x4 fill = {1u, 2u, 3u, 4u};
    for (int q = 0; q < 3; q++)
        for (int j = 0; j < 4; j++)
            regs[q][j] = fill;
    probe_bf16x8 fa[2][2], fb[2][2], fw[3][2], fp[2][4];
    auto request = [&](auto set, int t) {
        constexpr int S = decltype(set)::value;
        const unsigned soff = (pos + (unsigned)t * 16384u) & src_mask;
        if (PARTS & 32) { // weight operands of this wavefront's 32 rows + its two pieces of the pixel tile
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++)
                fw[S][s2] = __builtin_bit_cast(probe_bf16x8, __builtin_amdgcn_raw_buffer_load_b128(r, (unsigned)((wave * 32 + l32) * 64 + h * 16), soff + s2 * 32, 0));
#pragma unroll
            for (int j = 0; j < 2; j++)
                regs[S][j] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (unsigned)(tid * 16 + j * 4096), soff + 8192, 0));
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++)
                regs[S][j] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (unsigned)(tid * 16 + j * 4096), soff, 0));
        }
    };
    auto step = [&](auto set, int it) {
        constexpr int S = decltype(set)::value;
        const int buf = it & 1;
        if (PARTS & 1) {
            if (PARTS & 32) {
#pragma unroll
                for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        fp[s2][j] = *(const probe_bf16x8 *)at(1, buf, j * 32 + l32, s2 * 2 + h);
            } else {
#pragma unroll
                for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        fa[s2][i] = *(const probe_bf16x8 *)at(0, buf, wm * 64 + i * 32 + l32, s2 * 2 + h);
                        fb[s2][i] = *(const probe_bf16x8 *)at(1, buf, wn * 64 + i * 32 + l32, s2 * 2 + h);
                    }
            }
        }
        if (PARTS & 8) {
            if (PARTS & 32) {
#pragma unroll
                for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw[S][s2], fp[s2][j], acc[j], 0, 0, 0);
            } else {
#pragma unroll
                for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
                    for (int i = 0; i < 2; i++)
#pragma unroll
                        for (int j = 0; j < 2; j++)
                            acc[i * 2 + j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[s2][i], fb[s2][j], acc[i * 2 + j], 0, 0, 0);
            }
        } else {
            asm volatile("" ::"v"(fa[0][0]), "v"(fa[0][1]), "v"(fa[1][0]), "v"(fa[1][1]), "v"(fb[0][0]), "v"(fb[0][1]), "v"(fb[1][0]), "v"(fb[1][1]));
        }
        if (PARTS & 2) { // the tile of the next step, from the registers that were requested three steps ago
            constexpr int N = (PARTS & 32) ? 2 : 4;
#pragma unroll
            for (int j = 0; j < N; j++) {
                const int idx = tid + j * 256, tile = (PARTS & 32) ? 1 : idx >> 9, row = (idx >> 2) & 127;
                *(u32x4 *)at(tile, buf ^ 1, row, idx & 3) = regs[(S + 1) % 3][j];
            }
        }
        if (PARTS & 16)
            request(std::integral_constant<int, (S + 1) % 3>{}, it + 4);
        if (PARTS & 4)
            __syncthreads();
        else
            asm volatile("" ::: "memory");
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    if (PARTS & 16) {
        request(I0{}, 0);
        request(I1{}, 1);
        request(I2{}, 2);
    }
    for (int it = 0; it < iters; it += 3) {
        step(I0{}, it);
        step(I1{}, it + 1);
        step(I2{}, it + 2);
    }
    float sum = 0.f;
    for (int j = 0; j < 4; j++)
        for (int q = 0; q < 16; q++)
            sum += acc[j][q];
    if (sum == 123.456f)
        out[tid] = sum;
}

template <int PARTS>
static int run_tile_step(int wgs_per_cu, double *ns_per_step)
{
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, 0) != hipSuccess)
        return 1;
    const int cus = prop.multiProcessorCount, iters = 6000;
    // LDS per workgroup fixes how many share a compute unit
    const int lds = wgs_per_cu <= 1 ? 150 * 1024 : wgs_per_cu == 2 ? 75 * 1024 : 50 * 1024;
    float *out = nullptr;
    unsigned char *src = nullptr;
    const unsigned src_bytes = 2u << 20;
    if (hipMalloc(&out, 4096) != hipSuccess || hipMalloc(&src, src_bytes) != hipSuccess)
        return 1;
    (void)hipMemset(src, 0x3f, src_bytes);
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    int rc = hipFuncSetAttribute((const void *)tile_step_kernel<PARTS>, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess;
    if (!rc) {
        tile_step_kernel<PARTS><<<cus * wgs_per_cu, 256, lds>>>(300, out, src, src_bytes - 1);
        (void)hipEventRecord(e0);
        tile_step_kernel<PARTS><<<cus * wgs_per_cu, 256, lds>>>(iters, out, src, src_bytes - 1);
        (void)hipEventRecord(e1);
        rc = hipDeviceSynchronize() != hipSuccess;
        float ms = 0.f;
        (void)hipEventElapsedTime(&ms, e0, e1);
        *ns_per_step = ms * 1e6 / iters;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(out);
    (void)hipFree(src);
    return rc;
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

// Time per K step of a 128 x 128 x 32 bf16 tile (2 * 128 * 128 * 32 flop) in a four-wavefront workgroup, `wgs_per_cu` (1..3) of them
// per compute unit, for one of the forms of tile_step_kernel (see dlp_probe_tile_step_name).  Returns 0 on success.
static const char *kStepNames[] = {"matrix instructions only",
                                   "matrix instructions + operand reads from LDS",
                                   "... + barrier",
                                   "... + next tile stored to LDS",
                                   "LDS stores + barrier alone (16 KB per step)",
                                   "LDS reads + barrier alone (32 KB per step)",
                                   "whole step, both tiles from memory (L2) through registers and LDS",
                                   "whole step, weights from memory straight into registers, pixels through LDS"};
int dlp_probe_tile_step(int form, int wgs_per_cu, double *ns_per_step)
{
    switch (form) {
    case 0: return run_tile_step<8>(wgs_per_cu, ns_per_step);
    case 1: return run_tile_step<9>(wgs_per_cu, ns_per_step);
    case 2: return run_tile_step<13>(wgs_per_cu, ns_per_step);
    case 3: return run_tile_step<15>(wgs_per_cu, ns_per_step);
    case 4: return run_tile_step<6>(wgs_per_cu, ns_per_step);
    case 5: return run_tile_step<5>(wgs_per_cu, ns_per_step);
    case 6: return run_tile_step<31>(wgs_per_cu, ns_per_step);
    case 7: return run_tile_step<63>(wgs_per_cu, ns_per_step);
    default: return 1;
    }
}
const char *dlp_probe_tile_step_name(int form) { return form >= 0 && form < 8 ? kStepNames[form] : ""; }
int dlp_probe_tile_step_count(void) { return 8; }
}
