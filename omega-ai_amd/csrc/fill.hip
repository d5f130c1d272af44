// Seeded synthetic data and dtype conversion on the device.
//
// Generator: counter-based SplitMix64 feeding a Box-Muller transform evaluated in double with
// only +,-,*,/ and sqrt (each a single correctly rounded IEEE operation, contraction disabled),
// so the values are the same bit for bit wherever the same recipe is evaluated:
//   key = mix(seed ^ mix(stream*G2 + 1));  h1 = mix(key + G*(2i+1));  h2 = mix(key + G*(2i+2))
//   u = ((h1>>11)+1)*2^-53;  r = sqrt(-2 ln u);  th = ((h2>>8)&(2^53-1))*2^-53*pi/4
//   z = r * (bit62(h2) ? sin th : cos th) * (bit63(h2) ? -1 : 1);  value = (float)(z*std)
// ln: u = m*2^e with m in [sqrt(1/2),sqrt(2)), ln m = 2 atanh((m-1)/(m+1)) as an 11-term odd series;
// sin/cos: Taylor series to th^19 / th^18 on [0,pi/4).
#include "common.h"

#define GAMMA 0x9E3779B97F4A7C15ULL
#define GAMMA2 0xD1342543DE82EF95ULL

__host__ __device__ static inline uint64_t mix64(uint64_t z)
{
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

__device__ static const double INV_ODD[11] = {
    0x1.0000000000000p+0, 0x1.5555555555555p-2, 0x1.999999999999ap-3, 0x1.2492492492492p-3,
    0x1.c71c71c71c71cp-4, 0x1.745d1745d1746p-4, 0x1.3b13b13b13b14p-4, 0x1.1111111111111p-4,
    0x1.e1e1e1e1e1e1ep-5, 0x1.af286bca1af28p-5, 0x1.8618618618618p-5};
__device__ static const double INV_FACT[20] = {
    0x1.0000000000000p+0,  0x1.0000000000000p+0,  0x1.0000000000000p-1,  0x1.5555555555555p-3,
    0x1.5555555555555p-5,  0x1.1111111111111p-7,  0x1.6c16c16c16c17p-10, 0x1.a01a01a01a01ap-13,
    0x1.a01a01a01a01ap-16, 0x1.71de3a556c734p-19, 0x1.27e4fb7789f5cp-22, 0x1.ae64567f544e4p-26,
    0x1.1eed8eff8d898p-29, 0x1.6124613a86d09p-33, 0x1.93974a8c07c9dp-37, 0x1.ae7f3e733b81fp-41,
    0x1.ae7f3e733b81fp-45, 0x1.952c77030ad4ap-49, 0x1.6827863b97d97p-53, 0x1.2f49b46814157p-57};

// This file is compiled with -ffp-contract=off: every operator below is one rounding.
__device__ static float normal_at(uint64_t key, uint64_t i, double std)
{
    const uint64_t h1 = mix64(key + GAMMA * (2ULL * i + 1ULL));
    const uint64_t h2 = mix64(key + GAMMA * (2ULL * i + 2ULL));
    const double u = (double)((h1 >> 11) + 1ULL) * 0x1.0p-53;
    // frexp by bit manipulation: u is a positive normal number in [2^-53, 1]
    const uint64_t ub = (uint64_t)__double_as_longlong(u);
    int e = (int)((ub >> 52) & 0x7ff) - 1022;
    double m = __longlong_as_double((long long)((ub & 0x000fffffffffffffULL) | 0x3fe0000000000000ULL));  // [0.5,1)
    if (m < 0x1.6a09e667f3bcdp-1) { m = m * 2.0; e -= 1; }
    const double s = (m - 1.0) / (m + 1.0);
    const double s2 = s * s;
    double p = INV_ODD[10];
#pragma unroll
    for (int k = 9; k >= 0; --k) p = p * s2 + INV_ODD[k];
    const double ln = (double)e * 0x1.62e42fefa39efp-1 + 2.0 * s * p;
    const double r = sqrt(-2.0 * ln);
    const double th = (double)((h2 >> 8) & ((1ULL << 53) - 1ULL)) * 0x1.0p-53 * 0x1.921fb54442d18p-1;
    const double t2 = th * th;
    double c = INV_FACT[18], sn = INV_FACT[19];
#pragma unroll
    for (int k = 8; k >= 0; --k) {
        c = INV_FACT[2 * k] - t2 * c;
        sn = INV_FACT[2 * k + 1] - t2 * sn;
    }
    sn = th * sn;
    double z = r * (((h2 >> 62) & 1ULL) ? sn : c);
    if ((h2 >> 63) & 1ULL) z = -z;
    return (float)(z * std);
}

__global__ __launch_bounds__(256) void fill_normal_kernel(void *out, uint64_t n, uint64_t key, double std,
                                                          uint64_t first, int dtype)
{
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t j = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; j < n; j += stride) {
        const float v = normal_at(key, first + j, std);
        if (dtype == OMEGA_DTYPE_BF16) ((bf16_t *)out)[j] = f32_to_bf16(v);
        else ((float *)out)[j] = v;
    }
}

hipError_t launch_fill_normal(void *dptr, uint64_t n, uint64_t seed, uint64_t stream_id, double std, uint64_t first,
                              int dtype, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    const uint64_t key = mix64(seed ^ mix64(stream_id * GAMMA2 + 1ULL));
    uint64_t blocks = (n + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    hipLaunchKernelGGL(fill_normal_kernel, dim3((unsigned)blocks), dim3(256), 0, s, dptr, n, key, std, first, dtype);
    return hipGetLastError();
}

__global__ __launch_bounds__(256) void convert_kernel(void *dst, int dst_dtype, const void *src, int src_dtype, uint64_t n)
{
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t j = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; j < n; j += stride) {
        const float v = src_dtype == OMEGA_DTYPE_BF16 ? bf16_to_f32(((const bf16_t *)src)[j]) : ((const float *)src)[j];
        if (dst_dtype == OMEGA_DTYPE_BF16) ((bf16_t *)dst)[j] = f32_to_bf16(v);
        else ((float *)dst)[j] = v;
    }
}

hipError_t launch_convert(void *dst, int dst_dtype, const void *src, int src_dtype, uint64_t n, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    uint64_t blocks = (n + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    hipLaunchKernelGGL(convert_kernel, dim3((unsigned)blocks), dim3(256), 0, s, dst, dst_dtype, src, src_dtype, n);
    return hipGetLastError();
}
