// Grouped expert SwiGLU products in fp32 (the parity configuration): plain LDS-tiled FMA kernels.
//   up    a[r,h] = silu(xg[r,:].W1g[h,:]) * (xg[r,:].W3g[h,:])     silu(v) = v/(1+exp(-v))
//   down  y[r,c] = a[r,:].W2g[c,:]
// (J/engine/nn/layer/llama/LlamaMLPLayer.java:117-130; silu J/engine/nn/layer/active/gpu/activeFunction.cu:172-179;
//  product J/engine/ad/op/gpu/OPKernel.cu:1103-1110; y = x W^T with W [out,in], J/engine/nn/layer/FullyLayer.java:181,235.)
// Row tiles come from the tile list written by the dispatch stage: a tile never straddles two experts.
#include "common.h"

#define FBM 64
#define FBN 64
#define FBK 16

int experts_f32_tile_m(void) { return FBM; }

// C[rows x N] = A[rows x Kd] * B[N x Kd]^T for one (row tile, column tile); FUSED adds the second
// weight matrix and the SwiGLU epilogue.  256 threads, 4x4 outputs each.
template <bool FUSED>
__global__ __launch_bounds__(256) void experts_f32_kernel(const float *__restrict__ Axg, const float *__restrict__ Ax,
                                                          const float *__restrict__ Wa, const float *__restrict__ Wb,
                                                          float *__restrict__ Cout, const omega_tile *__restrict__ tiles,
                                                          const int32_t *__restrict__ tile_meta, int N, int Kd)
{
    const int mt = blockIdx.y;
    if (mt >= tile_meta[0]) return;
    const omega_tile tl = tiles[mt];
    const int n0 = blockIdx.x * FBN;
    const float *A = (FUSED && tl.xrow0 >= 0) ? Ax + (size_t)tl.xrow0 * Kd : Axg + (size_t)tl.row0 * Kd;
    const float *B1 = Wa + (size_t)tl.g * N * Kd;
    const float *B2 = FUSED ? Wb + (size_t)tl.g * N * Kd : nullptr;

    __shared__ float As[FBK][FBM + 4];
    __shared__ float Bs1[FBK][FBN + 4];
    __shared__ float Bs2[FUSED ? FBK : 1][FBN + 4];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    float acc1[4][4] = {}, acc2[4][4] = {};

    for (int k0 = 0; k0 < Kd; k0 += FBK) {
        for (int idx = tid; idx < FBM * FBK; idx += 256) {
            const int r = idx / FBK, kk = idx % FBK;
            const int k = k0 + kk;
            As[kk][r] = (r < tl.rows && k < Kd) ? A[(size_t)r * Kd + k] : 0.0f;
            const int n = n0 + r;
            const bool ok = n < N && k < Kd;
            Bs1[kk][r] = ok ? B1[(size_t)n * Kd + k] : 0.0f;
            if (FUSED) Bs2[kk][r] = ok ? B2[(size_t)n * Kd + k] : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < FBK; ++kk) {
            float av[4], b1[4], b2[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                b1[j] = Bs1[kk][tx * 4 + j];
                if (FUSED) b2[j] = Bs2[kk][tx * 4 + j];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc1[i][j] = fmaf(av[i], b1[j], acc1[i][j]);
                    if (FUSED) acc2[i][j] = fmaf(av[i], b2[j], acc2[i][j]);
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = ty * 4 + i;
        if (r >= tl.rows) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = acc1[i][j];
            if (FUSED) v = (v / (1.0f + expf(-v))) * acc2[i][j];
            Cout[(size_t)(tl.row0 + r) * N + n] = v;
        }
    }
}

hipError_t launch_experts_f32(const omega_moe *m, const void *x, int T, int which, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    (void)T;
    if (which == 0) {
        dim3 grid(ceil_div(c.H, FBN), m->max_m_tiles);
        hipLaunchKernelGGL(experts_f32_kernel<true>, grid, dim3(256), 0, s, (const float *)m->xg, (const float *)x,
                           (const float *)m->W1, (const float *)m->W3, (float *)m->a, m->tiles, m->tile_meta, c.H, c.d);
    } else {
        dim3 grid(ceil_div(c.d, FBN), m->max_m_tiles);
        hipLaunchKernelGGL(experts_f32_kernel<false>, grid, dim3(256), 0, s, (const float *)m->a, (const float *)nullptr,
                           (const float *)m->W2, (const float *)nullptr, m->y, m->tiles, m->tile_meta, c.d, c.H);
    }
    return hipGetLastError();
}
