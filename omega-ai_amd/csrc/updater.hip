// AdamW step of the layer's parameters: the Updater branch of FullyLayer.update
// (J/engine/nn/layer/FullyLayer.java:569-590 -> AdamW.update, J/engine/updater/AdamW.java:69-92 ->
// AdamWKernel.updateW / updateB, J/engine/updater/gpu/AdamWKernel.java:177-195,380-399 -> adamw_kernel,
// J/engine/updater/gpu/updater.cu:31-52).  Built without contraction: every operation below rounds once, where it is
// written, so the result is the same bits as the same formula on any IEEE machine.
#include "common.h"
#include "pack.h"

// lerp(start, end, weight) = fma(weight, end, fma(-weight, start, start)) (updater.cu:31-33); the decay term and the
// final step are written as the fused operations the source's expression shape offers to the CUDA compiler
__device__ __forceinline__ float adamw_elem(float w, float g, float &m, float &v, const omega_adamw &p)
{
    m = fmaf(p.beta1, m, fmaf(-p.beta1, g, g));
    const float g2 = g * g;
    v = fmaf(p.beta2, v, fmaf(-p.beta2, g2, g2));
    const float mh = m / p.b1c, vh = v / p.b2c;
    const float t = fmaf(p.wd, w, mh / (sqrtf(vh) + p.eps));
    return fmaf(-p.lr, t, w);
}

// fp32 tensors: group blockIdx.y of `n` elements at w + y*wstride, its gradient and moments at + y*gstride
__global__ __launch_bounds__(256) void adamw_f32_kernel(float *__restrict__ w, size_t wstride, const float *__restrict__ grad,
                                                        float *__restrict__ mw, float *__restrict__ vw, size_t gstride, size_t n,
                                                        omega_adamw p)
{
    w += blockIdx.y * wstride;
    grad += blockIdx.y * gstride;
    mw += blockIdx.y * gstride;
    vw += blockIdx.y * gstride;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        float m = mw[i], v = vw[i];
        w[i] = adamw_elem(w[i], grad[i], m, v, p);
        mw[i] = m;
        vw[i] = v;
    }
}

// bf16 expert weights: the step is taken on the fp32 master, the packed bf16 image is re-rounded from it.  One thread
// per 16-byte chunk (8 consecutive columns of one row) of the image of expert blockIdx.y; master, gradient and
// moments share one layout.
__global__ __launch_bounds__(256) void adamw_packed_kernel(float *__restrict__ master, const float *__restrict__ grad,
                                                           float *__restrict__ mw, float *__restrict__ vw, size_t stride,
                                                           unsigned char *__restrict__ packed, size_t pstride, int R, int K,
                                                           omega_adamw p)
{
    const int g = blockIdx.y, nch = K >> 3, KT = K >> 5;
    const size_t base = (size_t)g * stride;
    unsigned char *pg = packed + (size_t)g * pstride;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < (size_t)R * nch; i += (size_t)gridDim.x * 256) {
        const int r = (int)(i / nch), ch = (int)(i % nch);
        const size_t o = base + (size_t)r * K + ch * 8;
        float wv[8], mv[8], vv[8], gv[8];
        *(float4 *)&wv[0] = *(const float4 *)(master + o);
        *(float4 *)&wv[4] = *(const float4 *)(master + o + 4);
        *(float4 *)&mv[0] = *(const float4 *)(mw + o);
        *(float4 *)&mv[4] = *(const float4 *)(mw + o + 4);
        *(float4 *)&vv[0] = *(const float4 *)(vw + o);
        *(float4 *)&vv[4] = *(const float4 *)(vw + o + 4);
        *(float4 *)&gv[0] = *(const float4 *)(grad + o);
        *(float4 *)&gv[4] = *(const float4 *)(grad + o + 4);
#pragma unroll
        for (int q = 0; q < 8; ++q) wv[q] = adamw_elem(wv[q], gv[q], mv[q], vv[q], p);
        *(float4 *)(master + o) = *(const float4 *)&wv[0];
        *(float4 *)(master + o + 4) = *(const float4 *)&wv[4];
        *(float4 *)(mw + o) = *(const float4 *)&mv[0];
        *(float4 *)(mw + o + 4) = *(const float4 *)&mv[4];
        *(float4 *)(vw + o) = *(const float4 *)&vv[0];
        *(float4 *)(vw + o + 4) = *(const float4 *)&vv[4];
        uint4 u;
        u.x = (uint32_t)f32_to_bf16(wv[0]) | ((uint32_t)f32_to_bf16(wv[1]) << 16);
        u.y = (uint32_t)f32_to_bf16(wv[2]) | ((uint32_t)f32_to_bf16(wv[3]) << 16);
        u.z = (uint32_t)f32_to_bf16(wv[4]) | ((uint32_t)f32_to_bf16(wv[5]) << 16);
        u.w = (uint32_t)f32_to_bf16(wv[6]) | ((uint32_t)f32_to_bf16(wv[7]) << 16);
        *(uint4 *)(pg + pk_chunk_off(r, ch >> 2, ch & 3, KT)) = u;
    }
}

// the bf16 gate weight: row-major
__global__ __launch_bounds__(256) void adamw_rows_bf16_kernel(float *__restrict__ master, const float *__restrict__ grad,
                                                              float *__restrict__ mw, float *__restrict__ vw,
                                                              bf16_t *__restrict__ w, size_t n, omega_adamw p)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        float m = mw[i], v = vw[i];
        const float nw = adamw_elem(master[i], grad[i], m, v, p);
        master[i] = nw;
        mw[i] = m;
        vw[i] = v;
        w[i] = f32_to_bf16(nw);
    }
}

static inline unsigned grid_for(size_t n, unsigned cap)
{
    const size_t b = (n + 255) / 256;
    return (unsigned)(b < cap ? (b ? b : 1) : cap);
}

// mw, vw (and master for bf16 layers) are laid out like the gradient block that starts at m->dWg
hipError_t launch_update_adamw(const omega_moe *m, float *master, float *mw, float *vw, const omega_adamw &p, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const size_t HD = (size_t)c.H * c.d, nWg = (size_t)c.E * c.d;
    const size_t o_bg = m->dbg - m->dWg, o_gm = m->dgamma - m->dWg, o13 = m->dW13 - m->dWg, o2 = m->dW2 - m->dWg;
    const bool bf = c.dtype == OMEGA_DTYPE_BF16;
    if (bf)
        hipLaunchKernelGGL(adamw_rows_bf16_kernel, dim3(grid_for(nWg, 1024)), dim3(256), 0, s, master, (const float *)m->dWg, mw,
                           vw, (bf16_t *)m->Wg, nWg, p);
    else
        hipLaunchKernelGGL(adamw_f32_kernel, dim3(grid_for(nWg, 1024)), dim3(256), 0, s, (float *)m->Wg, (size_t)0,
                           (const float *)m->dWg, mw, vw, (size_t)0, nWg, p);
    if (c.has_gate_bias)
        hipLaunchKernelGGL(adamw_f32_kernel, dim3(grid_for(c.E, 1024)), dim3(256), 0, s, m->bg, (size_t)0, (const float *)m->dbg,
                           mw + o_bg, vw + o_bg, (size_t)0, (size_t)c.E, p);
    if (m->gamma_set)
        hipLaunchKernelGGL(adamw_f32_kernel, dim3(grid_for(c.d, 1024)), dim3(256), 0, s, m->gamma, (size_t)0,
                           (const float *)m->dgamma, mw + o_gm, vw + o_gm, (size_t)0, (size_t)c.d, p);
    if (bf) {
        const dim3 grid(512, m->G);
        hipLaunchKernelGGL(adamw_packed_kernel, grid, dim3(256), 0, s, master + o13, (const float *)m->dW13, mw + o13, vw + o13,
                           2 * HD, (unsigned char *)m->W1, HD * 2, c.H, c.d, p);
        hipLaunchKernelGGL(adamw_packed_kernel, grid, dim3(256), 0, s, master + o13 + HD, (const float *)m->dW13 + HD,
                           mw + o13 + HD, vw + o13 + HD, 2 * HD, (unsigned char *)m->W3, HD * 2, c.H, c.d, p);
        hipLaunchKernelGGL(adamw_packed_kernel, grid, dim3(256), 0, s, master + o2, (const float *)m->dW2, mw + o2, vw + o2, HD,
                           (unsigned char *)m->W2, HD * 2, c.d, c.H, p);
    } else {
        const dim3 grid(grid_for(HD, 512), m->G);
        hipLaunchKernelGGL(adamw_f32_kernel, grid, dim3(256), 0, s, (float *)m->W1, HD, (const float *)m->dW13, mw + o13,
                           vw + o13, 2 * HD, HD, p);
        hipLaunchKernelGGL(adamw_f32_kernel, grid, dim3(256), 0, s, (float *)m->W3, HD, (const float *)m->dW13 + HD,
                           mw + o13 + HD, vw + o13 + HD, 2 * HD, HD, p);
        hipLaunchKernelGGL(adamw_f32_kernel, grid, dim3(256), 0, s, (float *)m->W2, HD, (const float *)m->dW2, mw + o2, vw + o2,
                           HD, HD, p);
    }
    return hipGetLastError();
}
