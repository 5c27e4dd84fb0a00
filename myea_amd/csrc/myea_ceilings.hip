// Two measured ceilings for the roofline figures: what this device does on a loop of nothing but FP32 MFMAs, and on a
// streaming triad.  Both are measured, not looked up: clocks under load and the memory system's real read + write rate sit
// below the published peaks, and a kernel's fraction of the measured ceiling says how much of ITS inefficiency is left.
// No counterpart in the reference.
#include <hip/hip_runtime.h>

#include "myea_kernels.h"

namespace myea {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));

// every wavefront issues back-to-back v_mfma_f32_32x32x2_f32 on register operands: four independent accumulators, so the
// matrix pipe never waits for a result
__global__ __launch_bounds__(256) void ceiling_mfma_kernel(float *out, int iterations, float a, float b)
{
    f32x16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
    const float x = a + threadIdx.x * 1e-6f, y = b;
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(x, y, acc[i], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += acc[i][r];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

typedef float f32x4 __attribute__((ext_vector_type(4)));

// a[i] = b[i] + scalar * c[i] on 16-byte elements: two reads and one write per element, each address touched once.  Shaped like
// the optimizer update it is a yardstick for: one element per lane and no loop (a grid of n / 256 workgroups keeps more
// requests in flight than a few resident workgroups that loop), the store non-temporal since nothing reads it back.
__global__ __launch_bounds__(256) void ceiling_triad_kernel(f32x4 *__restrict__ a, const f32x4 *__restrict__ b, const f32x4 *__restrict__ c, float scalar, size_t n4)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n4) {
        const f32x4 x = b[i], y = c[i];
        __builtin_nontemporal_store(f32x4{x[0] + scalar * y[0], x[1] + scalar * y[1], x[2] + scalar * y[2], x[3] + scalar * y[3]}, &a[i]);
    }
}

struct EventPair {
    hipEvent_t a = nullptr, b = nullptr;
    ~EventPair() { if (a) (void)hipEventDestroy(a); if (b) (void)hipEventDestroy(b); }
};

}  // namespace
}  // namespace myea

extern "C" int myea_hip_ceiling_mfma_f32(void *stream, int iterations, int repeats, double *tflops)
{
    using namespace myea;
    if (!tflops || iterations < 1 || iterations > 10000000 || repeats < 1 || repeats > 100) { set_last_error("ceiling_mfma_f32: bad argument"); return MYEA_E_INVALID; }
    hipStream_t s = static_cast<hipStream_t>(stream);
    int dev = 0;
    hipDeviceProp_t prop;
    MYEA_HIP_TRY(hipGetDevice(&dev));
    MYEA_HIP_TRY(hipGetDeviceProperties(&prop, dev));
    const int blocks = prop.multiProcessorCount * 2;   // two wavefronts per SIMD
    float *out = nullptr;
    MYEA_HIP_TRY(hipMalloc(&out, (size_t)blocks * 256 * sizeof(float)));
    EventPair ev;
    hipError_t e = hipEventCreate(&ev.a);
    if (e == hipSuccess) e = hipEventCreate(&ev.b);
    float best = 0.f;
    if (e == hipSuccess) {
        hipLaunchKernelGGL(ceiling_mfma_kernel, dim3((unsigned)blocks), dim3(256), 0, s, out, iterations / 10 + 1, 1.f, 2.f);   // clocks up
        for (int r = 0; r < repeats && e == hipSuccess; ++r) {
            e = hipEventRecord(ev.a, s);
            hipLaunchKernelGGL(ceiling_mfma_kernel, dim3((unsigned)blocks), dim3(256), 0, s, out, iterations, 1.f, 2.f);
            if (e == hipSuccess) e = hipGetLastError();
            if (e == hipSuccess) e = hipEventRecord(ev.b, s);
            if (e == hipSuccess) e = hipEventSynchronize(ev.b);
            float ms = 0.f;
            if (e == hipSuccess) e = hipEventElapsedTime(&ms, ev.a, ev.b);
            if (e == hipSuccess && (best == 0.f || ms < best)) best = ms;
        }
    }
    (void)hipFree(out);
    if (e != hipSuccess) return hip_fail(e, "ceiling_mfma_f32");
    const double flop = (double)blocks * 4.0 * (double)iterations * 16.0 * (32.0 * 32.0 * 2.0 * 2.0);
    *tflops = flop / ((double)best * 1e-3) / 1e12;
    return MYEA_OK;
}

extern "C" int myea_hip_ceiling_hbm_triad(void *stream, size_t bytes_per_array, int repeats, double *gigabytes_per_second)
{
    using namespace myea;
    if (!gigabytes_per_second || bytes_per_array < (1u << 20) || bytes_per_array > ((size_t)8 << 30) || bytes_per_array % 16 || repeats < 1 || repeats > 100) {
        set_last_error("ceiling_hbm_triad: bad argument");
        return MYEA_E_INVALID;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    int dev = 0;
    hipDeviceProp_t prop;
    MYEA_HIP_TRY(hipGetDevice(&dev));
    MYEA_HIP_TRY(hipGetDeviceProperties(&prop, dev));
    f32x4 *a = nullptr, *b = nullptr, *c = nullptr;
    hipError_t e = hipMalloc(&a, bytes_per_array);
    if (e == hipSuccess) e = hipMalloc(&b, bytes_per_array);
    if (e == hipSuccess) e = hipMalloc(&c, bytes_per_array);
    EventPair ev;
    if (e == hipSuccess) e = hipEventCreate(&ev.a);
    if (e == hipSuccess) e = hipEventCreate(&ev.b);
    if (e == hipSuccess) e = hipMemsetAsync(b, 0, bytes_per_array, s);
    if (e == hipSuccess) e = hipMemsetAsync(c, 0, bytes_per_array, s);
    const size_t n4 = bytes_per_array / 16;
    const unsigned blocks = (unsigned)((n4 + 255) / 256);
    float best = 0.f;
    if (e == hipSuccess) {
        hipLaunchKernelGGL(ceiling_triad_kernel, dim3(blocks), dim3(256), 0, s, a, b, c, 0.5f, n4);
        for (int r = 0; r < repeats && e == hipSuccess; ++r) {
            e = hipEventRecord(ev.a, s);
            hipLaunchKernelGGL(ceiling_triad_kernel, dim3(blocks), dim3(256), 0, s, a, b, c, 0.5f, n4);
            if (e == hipSuccess) e = hipGetLastError();
            if (e == hipSuccess) e = hipEventRecord(ev.b, s);
            if (e == hipSuccess) e = hipEventSynchronize(ev.b);
            float ms = 0.f;
            if (e == hipSuccess) e = hipEventElapsedTime(&ms, ev.a, ev.b);
            if (e == hipSuccess && (best == 0.f || ms < best)) best = ms;
        }
    }
    if (a) (void)hipFree(a);
    if (b) (void)hipFree(b);
    if (c) (void)hipFree(c);
    if (e != hipSuccess) return hip_fail(e, "ceiling_hbm_triad");
    *gigabytes_per_second = 3.0 * (double)bytes_per_array / ((double)best * 1e-3) / 1e9;
    return MYEA_OK;
}
