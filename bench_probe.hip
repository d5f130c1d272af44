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


// ---- k-step probe --------------------------------------------------------------------------------------------------
// The inner loop of the product kernels without the kernels around it: per 32-k step and workgroup 256 MFMAs
// (16x16x32 bf16) on fragments read from LDS (ds_read_b128, double-buffered in registers), one barrier, and optionally
// the 32 KiB of direct global->LDS loads that refill the stage just consumed (ring of five 32 KiB stages, three steps
// of loads in flight).  Two shapes: 8 waves of 128 x 64 (two per SIMD, the product kernels' shape: 12 fragment reads per
// 32 MFMAs) and 4 waves of 128 x 128 (one per SIMD: 16 reads per 64 MFMAs, a third less LDS traffic).  The loads walk
// cyclic streams of `stream_kib` KiB of random bf16 values; `share` consecutive workgroups of an XCD walk the same stream
// in step, so 1 / share of the loads miss the XCD's L2, and the streams together either fit the last-level cache or not.
// It shows what this loop structure sustains under the power cap when nothing else (epilogues, ragged tiles, item
// switches) is in the way.
#define KP_STAGE 32768
#define KP_NSTAGE 5

__device__ __forceinline__ void kp_dma16(const void *sbase, uint32_t voff, uint32_t lds_base)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0" ::"s"(sbase), "v"(voff), "s"(lds_base) : "memory");
}

__global__ void kp_fill_kernel(uint16_t *p, size_t n)
{
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        unsigned h = (unsigned)i * 2654435761u + 12345u;
        h ^= h >> 15;
        h *= 2246822519u;
        h ^= h >> 13;
        const __bf16 b = (__bf16)(((int)(h % 2001u) - 1000) * 1e-3f);
        p[i] = *(const uint16_t *)&b;
    }
}

template <int WAVES, int LOADS>
__global__ __launch_bounds__(WAVES * 64) void kstep_probe_kernel(const unsigned char *__restrict__ src, float *out, int steps,
                                                                 int share, int stream_steps)
{
    extern __shared__ __attribute__((aligned(1024))) unsigned char kp_smem[];
    constexpr int NC = WAVES == 4 ? 8 : 4;  // B fragments per wave
    constexpr int NR = 8 + NC;              // LDS reads per step
    constexpr int NL = 32 / WAVES;          // direct loads per wave and step
    constexpr int NG = 8 * NC / 4;          // groups of 4 MFMAs
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)kp_smem;
    unsigned h = tid * 2654435761u + blockIdx.x * 40503u + 12345u;
    for (int i = tid; i < KP_NSTAGE * KP_STAGE / 2; i += WAVES * 64) {
        h = h * 1664525u + 1013904223u;
        ((__bf16 *)kp_smem)[i] = (__bf16)(((int)((h >> 8) % 2001u) - 1000) * 1e-3f);
    }
    __syncthreads();
    // stream of this workgroup: workgroup w runs on XCD w % 8; `share` consecutive workgroups of an XCD share one
    const size_t stream = (size_t)(blockIdx.x & 7) * (32 / share) + (size_t)((blockIdx.x >> 3) & 31) / share;
    const unsigned char *base = src + stream * (size_t)stream_steps * KP_STAGE;
    {
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)(uint64_t)base), hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)base >> 32));
        base = (const unsigned char *)(((uint64_t)hi << 32) | lo);
    }
    const uint32_t voff = wave * 1024 + lane * 16;
    const int l16 = lane & 15, lq = lane >> 4;
    const uint32_t pa = (uint32_t)(l16 * 64 + ((lq ^ (((l16 >> 1) ^ (l16 >> 3)) & 3)) << 4));
    probe_f32x4_t acc[8][NC];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < NC; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;
    probe_bf16x8_t fa0[8], fb0[NC], fa1[8], fb1[NC];
#pragma unroll
    for (int i = 0; i < 8; ++i) fa0[i] = fa1[i] = *(const probe_bf16x8_t *)(kp_smem + pa + i * 2048);
#pragma unroll
    for (int i = 0; i < NC; ++i) fb0[i] = fb1[i] = *(const probe_bf16x8_t *)(kp_smem + 16384 + pa + i * 1024 + (wave & 1) * 8192);
    int cur = 0, kc = 0;  // ring stage, step within the stream
#define KP_READ(QA, QB, stage, r)                                                                                       \
    do {                                                                                                                \
        const unsigned char *sp = kp_smem + (stage) * KP_STAGE;                                                          \
        if ((r) < NC) QB[(r) % NC] = *(const probe_bf16x8_t *)(sp + 16384 + pa + ((r) % NC) * 1024 + (wave & 1) * 8192);  \
        else QA[((r) - NC) & 7] = *(const probe_bf16x8_t *)(sp + pa + (((r) - NC) & 7) * 2048 + ((wave >> 1) & 1) * 1024); \
    } while (0)
#define KP_STEP(PA, PB, QA, QB)                                                                                         \
    do {                                                                                                                \
        const int nxt = cur + 1 == KP_NSTAGE ? 0 : cur + 1;                                                              \
        __builtin_amdgcn_sched_barrier(0);                                                                              \
        _Pragma("unroll") for (int g = 0; g < NG; ++g)                                                                   \
        {                                                                                                               \
            _Pragma("unroll") for (int r = 0; r < NR; ++r) if (r * (NG / 2) / NR == g) KP_READ(QA, QB, nxt, r);          \
            if (LOADS) {                                                                                                \
                _Pragma("unroll") for (int l = 0; l < NL; ++l) if (l * NG / NL == g)                                     \
                    kp_dma16(base, (uint32_t)kc * KP_STAGE + l * (WAVES * 1024) + voff,                                  \
                             lds0 + cur * KP_STAGE + wave * 1024 + l * (WAVES * 1024));                                  \
            }                                                                                                           \
            _Pragma("unroll") for (int u = 0; u < 4; ++u)                                                                \
            {                                                                                                           \
                const int m = g * 4 + u;                                                                                \
                acc[m / NC][m % NC] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(PB[m % NC], PA[m / NC], acc[m / NC][m % NC], 0, 0, 0); \
            }                                                                                                           \
            __builtin_amdgcn_sched_barrier(0);                                                                          \
        }                                                                                                               \
        if (LOADS) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(3 * NL) : "memory");                              \
        else asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                                         \
        __syncthreads();                                                                                                \
        cur = nxt;                                                                                                      \
        kc = kc + 1 == stream_steps ? 0 : kc + 1;                                                                       \
    } while (0)
    for (int kt = 0; kt < steps; kt += 2) {
        KP_STEP(fa0, fb0, fa1, fb1);
        KP_STEP(fa1, fb1, fa0, fb0);
    }
#undef KP_STEP
#undef KP_READ
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < NC; ++j) s += acc[i][j][0];
    if (s == 12345.678f) out[0] = s;  // keeps the loop alive
}

// MFMA rate in TFLOP/s of the k-step loop on `device`.  waves: 4 or 8 per workgroup; loads: 0 = fragments and barrier only,
// 1 = with the direct loads; share: 1, 2, 4, 8, 16 or 32 workgroups of an XCD per stream; stream_kib: length of a stream in
// KiB (a multiple of 32; 256 / share streams exist, at most 2 GiB in all).  Every address the kernel forms lies inside
// the buffer allocated here: stream index < 256 / share, offset inside a stream < stream_kib KiB.
// Returns 0, or the HIP error code.
extern "C" int bench_probe_kstep(int device, int waves, int loads, int share, int stream_kib, int launches, float *tflops)
{
    if (!tflops || launches < 4 || (waves != 4 && waves != 8) || share < 1 || share > 32 || (share & (share - 1)) != 0 ||
        stream_kib < 32 || stream_kib % 32 != 0)
        return (int)hipErrorInvalidValue;
    const size_t streams = 256 / (size_t)share, bytes = streams * (size_t)stream_kib * 1024;
    if (bytes > ((size_t)2 << 30) || (size_t)stream_kib * 1024 > ((size_t)1 << 31)) return (int)hipErrorInvalidValue;
    hipDeviceProp_t prop;
    hipError_t e = hipSetDevice(device);
    if (e == hipSuccess) e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return (int)e;
    const int n_wg = prop.multiProcessorCount < 256 ? prop.multiProcessorCount / 8 * 8 : 256;  // stream index uses 8 x 32
    if (n_wg < 8) return (int)hipErrorInvalidValue;
    const int steps = 4000, warm = launches / 4;
    unsigned char *src = nullptr;
    float *scratch = nullptr;
    hipStream_t s = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    e = hipMalloc((void **)&src, bytes);
    if (e == hipSuccess) e = hipMalloc((void **)&scratch, 4);
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    const void *fn = waves == 4 ? (loads ? (const void *)kstep_probe_kernel<4, 1> : (const void *)kstep_probe_kernel<4, 0>)
                                : (loads ? (const void *)kstep_probe_kernel<8, 1> : (const void *)kstep_probe_kernel<8, 0>);
    if (e == hipSuccess) e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, KP_NSTAGE * KP_STAGE);
    if (e == hipSuccess) {
        hipLaunchKernelGGL(kp_fill_kernel, dim3(4096), dim3(256), 0, s, (uint16_t *)src, bytes / 2);
        e = hipGetLastError();
    }
    const int stream_steps = stream_kib / 32;
    for (int i = 0; e == hipSuccess && i < launches; ++i) {
        if (i == warm) e = hipEventRecord(e0, s);
        if (waves == 4 && loads) hipLaunchKernelGGL((kstep_probe_kernel<4, 1>), dim3(n_wg), dim3(256), KP_NSTAGE * KP_STAGE, s, src, scratch, steps, share, stream_steps);
        else if (waves == 4) hipLaunchKernelGGL((kstep_probe_kernel<4, 0>), dim3(n_wg), dim3(256), KP_NSTAGE * KP_STAGE, s, src, scratch, steps, share, stream_steps);
        else if (loads) hipLaunchKernelGGL((kstep_probe_kernel<8, 1>), dim3(n_wg), dim3(512), KP_NSTAGE * KP_STAGE, s, src, scratch, steps, share, stream_steps);
        else hipLaunchKernelGGL((kstep_probe_kernel<8, 0>), dim3(n_wg), dim3(512), KP_NSTAGE * KP_STAGE, s, src, scratch, steps, share, stream_steps);
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
    if (src) (void)hipFree(src);
    if (e != hipSuccess) return (int)e;
    const double flop = (double)steps * 256.0 * 16384.0 * n_wg;  // 256 MFMAs of 2 x 16 x 16 x 32 per step and workgroup
    *tflops = (float)(flop * (launches - warm) / (ms * 1e-3) / 1e12);
    return 0;
}
