// RMSNorm in front of the layer (block form): rms[t] = sqrtf(sum_k x[t,k]^2 / d + 1e-6f), h[t,k] = (x[t,k] / rms[t]) * w[k],
// with the sum taken exactly as rmsnorm_forward_kernel2 takes it
// (J/engine/nn/layer/normalization/gpu/RMSKernel.cu:185-223): 32 lanes per row, lane l adds x[i]*x[i] for
// i = l, l+32, ... in index order with one fused multiply-add per step, then an xor butterfly (16, 8, 4, 2, 1) over
// the 32 partial sums.  h is written once, in the layer's storage type (rounded to bf16 in bf16 layers), and is what
// the router and the gather read; the residual x is added back by the combine kernel.
//
// One workgroup = 8 rows x 32 lanes.  The rows come in with 16-byte loads, pass through LDS as fp32 and are read
// back lane-strided (32 consecutive floats per row and step: no bank conflicts); chunks of NORM_DC columns keep the
// order of every lane's additions (chunk boundaries are multiples of 32).  The second pass re-reads the rows (they
// are still in L2) and writes h with 16-byte stores.
// This file is compiled with -ffp-contract=off; the only fused operation is the explicit fmaf.
#include "common.h"

#define NORM_ROWS 8
#define NORM_DC 2048  // columns per staged chunk: 8 rows x 2048 x 4 B = 64 KiB of LDS

// h == nullptr: statistics only
template <bool XBF>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const void *__restrict__ x, const float *__restrict__ gamma, int T,
                                                      int d, float *__restrict__ rms, void *__restrict__ h)
{
    __shared__ float rms_s[NORM_ROWS];
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
    const float my = sqrtf(s / (float)d + 1e-6f);
    if (l == 0) {
        rms_s[r] = my;
        if (t < T) rms[t] = my;
    }
    if (h == nullptr) return;
    __syncthreads();
    // second pass: 8 consecutive columns per thread and step
    const int per_row = (d + 7) / 8;
    for (int i = tid; i < NORM_ROWS * per_row; i += 256) {
        const int rr = i / per_row, cc = (i % per_row) * 8;
        const int tt = t0 + rr;
        if (tt >= T) continue;
        const float rv = rms_s[rr];
        const size_t off = (size_t)tt * d + cc;
        float v[8], g[8];
        const bool full = vec_ok && ((uintptr_t)h % 16 == 0) && ((uintptr_t)gamma % 16 == 0) && cc + 8 <= d;
        if (full) {
            const float4 g0 = *(const float4 *)(gamma + cc), g1 = *(const float4 *)(gamma + cc + 4);
            g[0] = g0.x; g[1] = g0.y; g[2] = g0.z; g[3] = g0.w; g[4] = g1.x; g[5] = g1.y; g[6] = g1.z; g[7] = g1.w;
            if (XBF) {
                const uint4 u = *(const uint4 *)((const bf16_t *)x + off);
                v[0] = __uint_as_float(u.x << 16); v[1] = __uint_as_float(u.x & 0xffff0000u);
                v[2] = __uint_as_float(u.y << 16); v[3] = __uint_as_float(u.y & 0xffff0000u);
                v[4] = __uint_as_float(u.z << 16); v[5] = __uint_as_float(u.z & 0xffff0000u);
                v[6] = __uint_as_float(u.w << 16); v[7] = __uint_as_float(u.w & 0xffff0000u);
            } else {
                const float4 a = *(const float4 *)((const float *)x + off), b = *(const float4 *)((const float *)x + off + 4);
                v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
            }
#pragma unroll
            for (int q = 0; q < 8; ++q) v[q] = norm_apply<XBF>(v[q], rv, g[q]);
            if (XBF) {
                uint4 o;
                o.x = (__float_as_uint(v[0]) >> 16) | (__float_as_uint(v[1]) & 0xffff0000u);
                o.y = (__float_as_uint(v[2]) >> 16) | (__float_as_uint(v[3]) & 0xffff0000u);
                o.z = (__float_as_uint(v[4]) >> 16) | (__float_as_uint(v[5]) & 0xffff0000u);
                o.w = (__float_as_uint(v[6]) >> 16) | (__float_as_uint(v[7]) & 0xffff0000u);
                *(uint4 *)((bf16_t *)h + off) = o;
            } else {
                *(float4 *)((float *)h + off) = make_float4(v[0], v[1], v[2], v[3]);
                *(float4 *)((float *)h + off + 4) = make_float4(v[4], v[5], v[6], v[7]);
            }
        } else {
            for (int q = 0; q < 8 && cc + q < d; ++q) {
                const float xv = XBF ? bf16_to_f32(((const bf16_t *)x)[off + q]) : ((const float *)x)[off + q];
                const float hv = norm_apply<XBF>(xv, rv, gamma[cc + q]);
                if (XBF) ((bf16_t *)h)[off + q] = f32_to_bf16(hv);
                else ((float *)h)[off + q] = hv;
            }
        }
    }
}

hipError_t launch_rmsnorm(const omega_moe *m, const void *x, int T, void *h, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const int grid = ceil_div(T, NORM_ROWS);
    if (c.dtype == OMEGA_DTYPE_BF16)
        hipLaunchKernelGGL(rmsnorm_kernel<true>, dim3(grid), dim3(256), 0, s, x, m->gamma, T, c.d, m->rms, h);
    else
        hipLaunchKernelGGL(rmsnorm_kernel<false>, dim3(grid), dim3(256), 0, s, x, m->gamma, T, c.d, m->rms, h);
    return hipGetLastError();
}

// ---- backward of the pre-norm (block form) ----
// rmsnorm_backward_kernel2 (J/engine/nn/layer/normalization/gpu/RMSKernel.cu:226-277): per row, with the forward's rms,
//   drms = sum_i x[i]*dh[i]*w[i] (lane l adds i = l, l+32, ... in order: product x*dh, then one fused multiply-add with w;
//          xor butterfly over the 32 lanes) * (-1 / (rms^3 * C))
//   dx[i] = dh[i]*w[i]/rms + drms*x[i]   (+ resid[i]: the gradient that bypasses the norm, Tensor_OP().add(norm2.diff, delta),
//          J/engine/nn/layer/llama/LlamaTransformerBlock.java:157-158), rounded once in bf16 layers
// 8 rows x 32 lanes per workgroup, rows read straight from memory (this kernel moves 4 rows of T x d once).
template <bool XBF>
__global__ __launch_bounds__(256) void rmsnorm_backward_kernel(const void *__restrict__ x, const void *__restrict__ dh,
                                                               const float *__restrict__ gamma, const float *__restrict__ rms,
                                                               const void *__restrict__ resid, int T, int d, void *__restrict__ dx)
{
    const int r = threadIdx.x >> 5, l = threadIdx.x & 31;
    const int t = blockIdx.x * NORM_ROWS + r;
    if (t >= T) return;  // whole 32-lane groups leave together; the shuffles below stay within a group
    const size_t base = (size_t)t * d;
    auto ld = [&](const void *p, int i) {
        return XBF ? bf16_to_f32(((const bf16_t *)p)[base + i]) : ((const float *)p)[base + i];
    };
    float s = 0.0f;
    for (int i = l; i < d; i += 32) {
        const float pr = ld(x, i) * ld(dh, i);
        s = fmaf(pr, gamma[i], s);
    }
#pragma unroll
    for (int m = 16; m >= 1; m >>= 1) s = s + __shfl_xor(s, m, 32);
    const float rv = rms[t];
    const float drms = s * (-1.0f / (rv * rv * rv * (float)d));
    for (int i = l; i < d; i += 32) {
        const float a = ld(dh, i) * gamma[i];
        const float q = a / rv;
        float v = fmaf(drms, ld(x, i), q);
        if (resid != nullptr) v = v + ld(resid, i);
        if (XBF) ((bf16_t *)dx)[base + i] = f32_to_bf16(v);
        else ((float *)dx)[base + i] = v;
    }
}

// dgamma[c] = sum_t (x[t,c]/rms[t]) * dh[t,c]: partial sums over 32 slices of the rows (fixed order, no atomics; the
// reference accumulates with atomicAdd in no defined order), then their sum.
template <bool XBF>
__global__ __launch_bounds__(256) void rmsnorm_dgamma_partial_kernel(const void *__restrict__ x, const void *__restrict__ dh,
                                                                     const float *__restrict__ rms, int T, int d, int tslice,
                                                                     float *__restrict__ part)
{
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= d) return;
    const int t0 = blockIdx.y * tslice, t1 = min(T, t0 + tslice);
    float acc = 0.0f;
    for (int t = t0; t < t1; ++t) {
        const size_t o = (size_t)t * d + c;
        const float xv = XBF ? bf16_to_f32(((const bf16_t *)x)[o]) : ((const float *)x)[o];
        const float gv = XBF ? bf16_to_f32(((const bf16_t *)dh)[o]) : ((const float *)dh)[o];
        const float n = xv / rms[t];
        const float pr = n * gv;
        acc = acc + pr;
    }
    part[(size_t)blockIdx.y * d + c] = acc;
}

__global__ __launch_bounds__(256) void rmsnorm_dgamma_reduce_kernel(const float *__restrict__ part, int nslices, int d,
                                                                    float *__restrict__ dgamma)
{
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= d) return;
    float s = 0.0f;
    for (int q = 0; q < nslices; ++q) s = s + part[(size_t)q * d + c];
    dgamma[c] = s;
}

// dx = resid + rmsnorm backward of dh; dgamma into m->dgamma (partials in m->bw_gpart: at least 32 x d floats)
hipError_t launch_rmsnorm_backward(const omega_moe *m, const void *x, const void *dh, const void *resid, int T, void *dx,
                                   hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const int grid = ceil_div(T, NORM_ROWS);
    const int tslice = ceil_div(T, 32), nsl = ceil_div(T, tslice);
    const dim3 pg(ceil_div(c.d, 256), nsl);
    if (c.dtype == OMEGA_DTYPE_BF16) {
        hipLaunchKernelGGL(rmsnorm_backward_kernel<true>, dim3(grid), dim3(256), 0, s, x, dh, m->gamma, m->rms, resid, T, c.d, dx);
        hipLaunchKernelGGL(rmsnorm_dgamma_partial_kernel<true>, pg, dim3(256), 0, s, x, dh, m->rms, T, c.d, tslice, m->bw_gpart);
    } else {
        hipLaunchKernelGGL(rmsnorm_backward_kernel<false>, dim3(grid), dim3(256), 0, s, x, dh, m->gamma, m->rms, resid, T, c.d, dx);
        hipLaunchKernelGGL(rmsnorm_dgamma_partial_kernel<false>, pg, dim3(256), 0, s, x, dh, m->rms, T, c.d, tslice, m->bw_gpart);
    }
    hipLaunchKernelGGL(rmsnorm_dgamma_reduce_kernel, dim3(ceil_div(c.d, 256)), dim3(256), 0, s, (const float *)m->bw_gpart, nsl,
                       c.d, m->dgamma);
    return hipGetLastError();
}
