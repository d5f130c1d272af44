// Grouped expert SwiGLU products in fp32 on the matrix cores (v_mfma_f32_32x32x2_f32, fp32 operands and accumulators).
//   up    a[r,h] = silu(xg[r,:].W1g[h,:]) * (xg[r,:].W3g[h,:])     silu(v) = v/(1+exp(-v))
//   down  y[r,c] = a[r,:].W2g[c,:]
// (J/engine/nn/layer/llama/LlamaMLPLayer.java:117-130; silu J/engine/nn/layer/active/gpu/activeFunction.cu:172-179;
//  product J/engine/ad/op/gpu/OPKernel.cu:1103-1110; y = x W^T with W [out,in], J/engine/nn/layer/FullyLayer.java:181,235;
//  the reference's product is a cuBLAS sgemm on the tensor cores, J/engine/gpu/GPUOP.java:395,405-417.)
// Row tiles come from the tile list written by the dispatch stage: a tile never straddles two experts.
//
// One workgroup = 4 waves = one 64 x 64 output tile, each wave a 32 x 32 block (two accumulator blocks for the up
// product: W1 and W3 against the same rows, so silu(h1)*h3 is applied in registers).  Operands are staged through LDS
// k-major (As[k][row], Bs[k][col]) in steps of 32 k, so a lane's MFMA operands - A[row l32][k], B[k][col l32] for
// k = 2*kk + lane/32 - are conflict-free 4-byte reads; the next step's rows travel from memory in registers while the
// current step is multiplied.  Any d, H and alignment: rows that are 16-byte aligned take 16-byte loads (VEC), the
// others scalar ones; everything past the edges of the tile is zero.
#include "common.h"

#define FBM 64
#define FBN 64
#define FBK 32

typedef __attribute__((ext_vector_type(16))) float f32x16_t;

int experts_f32_tile_m(void) { return FBM; }

// Stage of one operand: 64 rows x 32 k.  Thread t carries two pieces of 4 consecutive k: rows t/8 and t/8 + 32,
// k = 4*(t%8) ...
template <bool VEC>
__device__ __forceinline__ void f32_fetch(const float *__restrict__ M, int rows, int Kd, int k0, int tid, float4 (&v)[2])
{
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int r = (tid >> 3) + 32 * u, k = k0 + 4 * (tid & 7);
        float4 q = {0.0f, 0.0f, 0.0f, 0.0f};
        if (r < rows) {
            const float *p = M + (size_t)r * Kd + k;
            if (VEC) {
                if (k < Kd) q = *(const float4 *)p;  // Kd % 4 == 0: a piece lies wholly inside or outside
            } else {
                if (k + 0 < Kd) q.x = p[0];
                if (k + 1 < Kd) q.y = p[1];
                if (k + 2 < Kd) q.z = p[2];
                if (k + 3 < Kd) q.w = p[3];
            }
        }
        v[u] = q;
    }
}

__device__ __forceinline__ void f32_stash(float (*S)[FBM + 1], int tid, const float4 (&v)[2])
{
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int r = (tid >> 3) + 32 * u, k = 4 * (tid & 7);
        S[k + 0][r] = v[u].x;
        S[k + 1][r] = v[u].y;
        S[k + 2][r] = v[u].z;
        S[k + 3][r] = v[u].w;
    }
}

// C[rows x N] = A[rows x Kd] * B[N x Kd]^T for one (row tile, column tile); FUSED adds the second
// weight matrix and the SwiGLU epilogue.
template <bool FUSED, bool VEC>
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
    const float *B1 = Wa + ((size_t)tl.g * N + n0) * Kd;
    const float *B2 = FUSED ? Wb + ((size_t)tl.g * N + n0) * Kd : nullptr;
    const int brows = min(FBN, N - n0);

    __shared__ float As[FBK][FBM + 1];
    __shared__ float Bs1[FBK][FBN + 1];
    __shared__ float Bs2[FUSED ? FBK : 1][FBN + 1];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, kh = lane >> 5;
    const int wr = wave >> 1, wc = wave & 1;  // this wave's 32 x 32 block of the tile

    f32x16_t acc1, acc2;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc1[r] = acc2[r] = 0.0f;

    float4 va[2], vb1[2], vb2[2];
    f32_fetch<VEC>(A, tl.rows, Kd, 0, tid, va);
    f32_fetch<VEC>(B1, brows, Kd, 0, tid, vb1);
    if (FUSED) f32_fetch<VEC>(B2, brows, Kd, 0, tid, vb2);
    for (int k0 = 0; k0 < Kd; k0 += FBK) {
        f32_stash(As, tid, va);
        f32_stash(Bs1, tid, vb1);
        if (FUSED) f32_stash(Bs2, tid, vb2);
        __syncthreads();
        if (k0 + FBK < Kd) {  // the next step's rows travel while this one is multiplied
            f32_fetch<VEC>(A, tl.rows, Kd, k0 + FBK, tid, va);
            f32_fetch<VEC>(B1, brows, Kd, k0 + FBK, tid, vb1);
            if (FUSED) f32_fetch<VEC>(B2, brows, Kd, k0 + FBK, tid, vb2);
        }
#pragma unroll
        for (int kk = 0; kk < FBK / 2; ++kk) {
            const float a = As[2 * kk + kh][wr * 32 + l32];
            const float b1 = Bs1[2 * kk + kh][wc * 32 + l32];
            acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b1, acc1, 0, 0, 0);
            if (FUSED) {
                const float b2 = Bs2[2 * kk + kh][wc * 32 + l32];
                acc2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b2, acc2, 0, 0, 0);
            }
        }
        __syncthreads();
    }
    // lane: column l32 of the block; register r -> row 8*(r/4) + 4*kh + r%4
    const int n = n0 + wc * 32 + l32;
    if (n >= N) return;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int row = wr * 32 + 8 * (r >> 2) + 4 * kh + (r & 3);
        if (row >= tl.rows) continue;
        float v = acc1[r];
        if (FUSED) v = (v / (1.0f + expf(-v))) * acc2[r];
        Cout[(size_t)(tl.row0 + row) * N + n] = v;
    }
}

hipError_t launch_experts_f32(const omega_moe *m, const void *x, int T, int which, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    (void)T;
    if (which == 0) {
        dim3 grid(ceil_div(c.H, FBN), m->max_m_tiles);
        const bool vec = c.d % 4 == 0 && (((uintptr_t)x | (uintptr_t)m->xg | (uintptr_t)m->W1 | (uintptr_t)m->W3) % 16) == 0;
        if (vec)
            hipLaunchKernelGGL((experts_f32_kernel<true, true>), grid, dim3(256), 0, s, (const float *)m->xg, (const float *)x,
                               (const float *)m->W1, (const float *)m->W3, (float *)m->a, m->tiles, m->tile_meta, c.H, c.d);
        else
            hipLaunchKernelGGL((experts_f32_kernel<true, false>), grid, dim3(256), 0, s, (const float *)m->xg, (const float *)x,
                               (const float *)m->W1, (const float *)m->W3, (float *)m->a, m->tiles, m->tile_meta, c.H, c.d);
    } else {
        dim3 grid(ceil_div(c.d, FBN), m->max_m_tiles);
        const bool vec = c.H % 4 == 0 && (((uintptr_t)m->a | (uintptr_t)m->W2) % 16) == 0;
        if (vec)
            hipLaunchKernelGGL((experts_f32_kernel<false, true>), grid, dim3(256), 0, s, (const float *)m->a, (const float *)nullptr,
                               (const float *)m->W2, (const float *)nullptr, m->y, m->tiles, m->tile_meta, c.d, c.H);
        else
            hipLaunchKernelGGL((experts_f32_kernel<false, false>), grid, dim3(256), 0, s, (const float *)m->a, (const float *)nullptr,
                               (const float *)m->W2, (const float *)nullptr, m->y, m->tiles, m->tile_meta, c.d, c.H);
    }
    return hipGetLastError();
}
