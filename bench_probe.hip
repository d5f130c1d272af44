// Matrix-core ceiling probe: a loop of independent v_mfma_f32_16x16x32_bf16 (the instruction of the product kernels;
// v_mfma_f32_32x32x16_bf16 sustains 10 % less under the power cap) with no memory traffic at all, on
// every SIMD of the device, for a fixed number of launches.  With random bf16 operands it shows the rate the part
// sustains under its power cap when the matrix cores do nothing but multiply realistic data; with constant operands
// (little switching activity) it reaches the nominal clock.  Used by the benchmark to put the product kernels'
// MFMA throughput next to what the hardware can hold, not to compute anything.
// Built into bench_probe.so, which only bench.py loads: the layer library does not contain it.
#include <hip/hip_runtime.h>

typedef __attribute__((ext_vector_type(8))) __bf16 probe_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float probe_f32x4_t;

#define PROBE_ACC 32  // 32 x 4 accumulator registers: the 128 of a wave of the product kernels

__global__ __launch_bounds__(512) void mfma_probe_kernel(float *out, int iters, int random_operands)
{
    probe_f32x4_t acc[PROBE_ACC];
#pragma unroll
    for (int i = 0; i < PROBE_ACC; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][r] = 0.0f;
    probe_bf16x8_t a[8], b[8];
    unsigned h = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            h = h * 1664525u + 1013904223u;
            a[i][q] = (__bf16)(random_operands ? ((int)((h >> 8) % 2001u) - 1000) * 1e-3f : 1.0f);
            h = h * 1664525u + 1013904223u;
            b[i][q] = (__bf16)(random_operands ? ((int)((h >> 8) % 2001u) - 1000) * 1e-3f : 1.0f);
        }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < PROBE_ACC; ++i)
            acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i & 7], b[i >> 3], acc[i], 0, 0, 0);  // the kernels' order: 8 x 4 pieces
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < PROBE_ACC; ++i) s += acc[i][0];
    if (s == 12345.678f) out[0] = s;  // keeps the loop alive
}

// Bf16 matrix-core rate in TFLOP/s that `device` sustains over `launches` launches of about 2.5 ms (the first quarter
// untimed).  random_operands != 0: random bf16 values (the rate under the power cap); 0: constants (the nominal clock).
// Returns 0, or the HIP error code.
extern "C" int bench_probe_mfma(int device, int random_operands, int launches, float *tflops)
{
    if (!tflops || launches < 4) return (int)hipErrorInvalidValue;
    hipDeviceProp_t prop;
    hipError_t e = hipSetDevice(device);
    if (e == hipSuccess) e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return (int)e;
    const int num_cus = prop.multiProcessorCount, iters = 10000, warm = launches / 4;
    float *scratch = nullptr;
    hipStream_t s = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    e = hipMalloc((void **)&scratch, 4);
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    for (int i = 0; e == hipSuccess && i < launches; ++i) {
        if (i == warm) e = hipEventRecord(e0, s);
        hipLaunchKernelGGL(mfma_probe_kernel, dim3(num_cus), dim3(512), 0, s, scratch, iters, random_operands);
    }
    if (e == hipSuccess) e = hipGetLastError();
    if (e == hipSuccess) e = hipEventRecord(e1, s);
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    float ms = 0.0f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (s) (void)hipStreamDestroy(s);
    if (scratch) (void)hipFree(scratch);
    if (e != hipSuccess) return (int)e;
    // 8 waves per workgroup, 2 x 16 x 16 x 32 FLOP per MFMA
    const double flop = (double)iters * PROBE_ACC * 8.0 * num_cus * 16384.0;
    *tflops = (float)(flop * (launches - warm) / (ms * 1e-3) / 1e12);
    return 0;
}
