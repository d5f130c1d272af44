// Matrix-core ceiling probe: a loop of independent v_mfma_f32_32x32x16_bf16 with no memory traffic at all, on
// every SIMD of the device, for a fixed number of launches.  With random bf16 operands it shows the rate the part
// sustains under its power cap when the matrix cores do nothing but multiply realistic data; with constant operands
// (little switching activity) it reaches the nominal clock.  Used by the benchmark to put the product kernels'
// MFMA throughput next to what the hardware can hold, not to compute anything.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 probe_bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float probe_f32x16_t;

#define PROBE_ACC 8

__global__ __launch_bounds__(512) void mfma_probe_kernel(float *out, int iters, int random_operands)
{
    probe_f32x16_t acc[PROBE_ACC];
#pragma unroll
    for (int i = 0; i < PROBE_ACC; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
    probe_bf16x8_t a[PROBE_ACC], b[PROBE_ACC];
    unsigned h = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
#pragma unroll
    for (int i = 0; i < PROBE_ACC; ++i)
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
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[(i + 3) % PROBE_ACC], acc[i], 0, 0, 0);
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < PROBE_ACC; ++i) s += acc[i][0];
    if (s == 12345.678f) out[0] = s;  // keeps the loop alive
}

// launches the probe `launches` times (about 2.5 ms each at full rate) and returns the FLOP count of one launch
hipError_t launch_mfma_probe(float *scratch, int num_cus, int random_operands, int launches, hipStream_t s, double *flop_per_launch)
{
    const int iters = 20000;
    for (int i = 0; i < launches; ++i)
        hipLaunchKernelGGL(mfma_probe_kernel, dim3(num_cus), dim3(512), 0, s, scratch, iters, random_operands);
    *flop_per_launch = (double)iters * PROBE_ACC * 8.0 * num_cus * 32768.0;  // 8 waves per workgroup, 2 x 32 x 32 x 16 per MFMA
    return hipGetLastError();
}
