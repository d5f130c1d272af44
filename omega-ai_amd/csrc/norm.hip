// Row statistics of the RMSNorm in front of the layer (block form): rms[t] = sqrtf(sum_k x[t,k]^2 / d + 1e-6f),
// with the sum taken exactly as rmsnorm_forward_kernel2 takes it
// (J/engine/nn/layer/normalization/gpu/RMSKernel.cu:185-223): 32 lanes per row, lane l adds x[i]*x[i] for
// i = l, l+32, ... in index order with one fused multiply-add per step, then an xor butterfly (16, 8, 4, 2, 1) over
// the 32 partial sums.  The normalised row (x/rms)*weight is never written: the router and the gather apply it to
// the rows they read anyway (norm_apply in common.h), and the combine adds x back.
//
// One workgroup = 8 rows x 32 lanes.  The rows come in with 16-byte loads, pass through LDS as fp32 and are read
// back lane-strided (32 consecutive floats per row and step: no bank conflicts); chunks of NORM_DC columns keep the
// order of every lane's additions (chunk boundaries are multiples of 32).
// This file is compiled with -ffp-contract=off; the only fused operation is the explicit fmaf.
#include "common.h"

#define NORM_ROWS 8
#define NORM_DC 2048  // columns per staged chunk: 8 rows x 2048 x 4 B = 64 KiB of LDS

template <bool XBF>
__global__ __launch_bounds__(256) void rms_stats_kernel(const void *__restrict__ x, int T, int d, float *__restrict__ rms)
{
    __shared__ __attribute__((aligned(16))) float xs[NORM_ROWS][NORM_DC];
    const int tid = threadIdx.x;
    const int r = tid >> 5, l = tid & 31;
    const int t0 = blockIdx.x * NORM_ROWS;
    const bool vec_ok = (d % 8 == 0) && ((uintptr_t)x % 16 == 0);
    float s = 0.0f;
    for (int c0 = 0; c0 < d; c0 += NORM_DC) {
        const int cw = min(NORM_DC, d - c0);  // columns of this chunk
        // stage: 8 consecutive columns per thread and pass
        for (int i = tid * 8; i < NORM_ROWS * NORM_DC; i += 256 * 8) {
            const int rr = i / NORM_DC, cc = i % NORM_DC;
            const int t = t0 + rr;
            float v[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) v[q] = 0.0f;
            if (t < T && cc < cw) {
                const size_t off = (size_t)t * d + c0 + cc;
                if (vec_ok && cc + 8 <= cw) {
                    if (XBF) {
                        const uint4 u = *(const uint4 *)((const bf16_t *)x + off);
                        v[0] = __uint_as_float(u.x << 16); v[1] = __uint_as_float(u.x & 0xffff0000u);
                        v[2] = __uint_as_float(u.y << 16); v[3] = __uint_as_float(u.y & 0xffff0000u);
                        v[4] = __uint_as_float(u.z << 16); v[5] = __uint_as_float(u.z & 0xffff0000u);
                        v[6] = __uint_as_float(u.w << 16); v[7] = __uint_as_float(u.w & 0xffff0000u);
                    } else {
                        const float4 a = *(const float4 *)((const float *)x + off);
                        const float4 b = *(const float4 *)((const float *)x + off + 4);
                        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
                        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
                    }
                } else {
#pragma unroll
                    for (int q = 0; q < 8; ++q)
                        if (cc + q < cw)
                            v[q] = XBF ? bf16_to_f32(((const bf16_t *)x)[off + q]) : ((const float *)x)[off + q];
                }
            }
            *(float4 *)&xs[rr][cc] = make_float4(v[0], v[1], v[2], v[3]);
            *(float4 *)&xs[rr][cc + 4] = make_float4(v[4], v[5], v[6], v[7]);
        }
        __syncthreads();
        // columns beyond the row are zero: fmaf(0, 0, s) leaves s unchanged
        const int steps = (cw + 31) / 32;
#pragma unroll 8
        for (int j = 0; j < steps; ++j) {
            const float v = xs[r][l + 32 * j];
            s = fmaf(v, v, s);
        }
        __syncthreads();
    }
#pragma unroll
    for (int m = 16; m >= 1; m >>= 1) s = s + __shfl_xor(s, m, 32);
    const int t = t0 + r;
    if (l == 0 && t < T) rms[t] = sqrtf(s / (float)d + 1e-6f);
}

hipError_t launch_rms_stats(const omega_moe *m, const void *x, int T, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const int grid = ceil_div(T, NORM_ROWS);
    if (c.dtype == OMEGA_DTYPE_BF16)
        hipLaunchKernelGGL(rms_stats_kernel<true>, dim3(grid), dim3(256), 0, s, x, T, c.d, m->rms);
    else
        hipLaunchKernelGGL(rms_stats_kernel<false>, dim3(grid), dim3(256), 0, s, x, T, c.d, m->rms);
    return hipGetLastError();
}
