// Backward pass of the layer: gradients of the input, the gate and every expert for an output gradient dout [T,d],
// composed from the backward steps of the reference primitives the forward pass is built from:
//   linear layer   diffW = delta^T . input (overwritten), diff = delta . W, diffB = column sums of delta
//                  (FullyLayer.diff, J/engine/nn/layer/FullyLayer.java:292-334)
//   SwiGLU wiring  w2 back; dh3 = d(a) * silu(h1); dh1 = silu'(h1) applied to d(a) * h3; input gradient = w1's + w3's
//                  (LlamaMLPLayer.diff, J/engine/nn/layer/llama/LlamaMLPLayer.java:139-158)
//   SiLU           diff = delta * s * (1 + x * (1 - s)), s = 1/(1+exp(-x))
//                  (silu_backward, J/engine/nn/layer/active/gpu/activeFunction.cu:182-190)
//   softmax        sum = sum_e out*delta; diff = (delta - sum) * out   (softmax_back, J/engine/gpu/SoftmaxKernel.cu:101-112)
// The routing of the forward pass (ids, permutation, row tiles) is reused as it was left in the workspace, together
// with the activations a and the expert outputs y; h1 and h3 are recomputed.  Expert rows keep their forward places:
// dy, dh1, dh3 and dxg are indexed by the same physical rows as xg, a and y.
//
// bf16 layers run every product on the matrix-core kernel of the forward pass (launch_backward_bf16 at the end of this
// file; the products themselves are described in experts_bf16.hip, their tables and the transposes in dispatch.hip).
// fp32 layers (the parity configuration) use the plain LDS-tiled FMA kernels below:
//   bw_combine_kernel   dy[r,:] = w[t,j] * dout[t,:],  dw[t,j] = dout[t,:] . y[r,:]
//   bw_rows_f32_kernel  row-tiled grouped products over the forward tile list (h1/h3, d(a) + SwiGLU backward, dxg)
//   bw_wgrad_f32_kernel dW_g = A_g^T . B_g over the rows of group g
//   bw_router_kernel    combine weights -> (renormalisation) -> selected probabilities -> softmax -> dlogits
//   bw_dx_kernel        dx[t,:] = sum_j dxg[row(t,j),:] + shared rows + dlogits[t,:] . Wg
#include "common.h"
#include "pack.h"

#define GBM 64
#define GBN 64
#define GBK 16

__device__ __forceinline__ float block_sum_256(float v, float *red)
{
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    const int wave = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

// One workgroup per token.  Shared experts take dout rows directly (their combine weight is 1).
__global__ __launch_bounds__(256) void bw_combine_kernel(const float *__restrict__ dout, const float *__restrict__ y,
                                                         const int32_t *__restrict__ dstp, const float *__restrict__ w,
                                                         int K, int d, float *__restrict__ dy, float *__restrict__ dw)
{
    __shared__ float red[4];
    const int t = blockIdx.x;
    const float *g = dout + (size_t)t * d;
    for (int j = 0; j < K; ++j) {
        const int r = dstp[(size_t)t * K + j];
        const float wv = w[(size_t)t * K + j];
        float part = 0.0f;
        for (int c = threadIdx.x; c < d; c += 256) {
            const float gv = g[c];
            dy[(size_t)r * d + c] = wv * gv;
            part = fmaf(gv, y[(size_t)r * d + c], part);
        }
        const float tot = block_sum_256(part, red);
        if (threadIdx.x == 0) dw[(size_t)t * K + j] = tot;
    }
}

// C[r, n] = sum_k A[r, k] * B_g(k, n) for the rows of one row tile (group g = the tile's expert).
// BKN = false: B_g is [N, Kd] (k contiguous: "x W^T");  BKN = true: B_g is [Kd, N] (n contiguous: "delta W").
// A rows: Atok + xrow0*Kd for a shared-expert tile when Atok is given, else Aphys + row0*Kd.
// EPI 0: C1 = acc.  EPI 1: C1 += acc.  EPI 2: acc is d(a); with h1 = C1[r,n], h3 = C2[r,n] writes, in place,
// C1 = dh1 = acc*h3 * s*(1 + h1*(1-s)) and C2 = dh3 = acc * h1*s, s = 1/(1+exp(-h1)).
template <bool BKN, int EPI>
__global__ __launch_bounds__(256) void bw_rows_f32_kernel(const float *__restrict__ Aphys, const float *__restrict__ Atok,
                                                          const float *__restrict__ Bw, float *__restrict__ C1,
                                                          float *__restrict__ C2, const omega_tile *__restrict__ tiles,
                                                          const int32_t *__restrict__ tile_meta, int N, int Kd)
{
    const int mt = blockIdx.y;
    if (mt >= tile_meta[0]) return;
    const omega_tile tl = tiles[mt];
    const int n0 = blockIdx.x * GBN;
    const float *A = (Atok && tl.xrow0 >= 0) ? Atok + (size_t)tl.xrow0 * Kd : Aphys + (size_t)tl.row0 * Kd;
    const float *B = Bw + (size_t)tl.g * N * Kd;

    __shared__ float As[GBK][GBM + 4];
    __shared__ float Bs[GBK][GBN + 4];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    float acc[4][4] = {};

    for (int k0 = 0; k0 < Kd; k0 += GBK) {
        for (int idx = tid; idx < GBM * GBK; idx += 256) {
            const int r = idx / GBK, kk = idx % GBK;
            const int k = k0 + kk;
            As[kk][r] = (r < tl.rows && k < Kd) ? A[(size_t)r * Kd + k] : 0.0f;
            if (!BKN) {
                const int n = n0 + r;
                Bs[kk][r] = (n < N && k < Kd) ? B[(size_t)n * Kd + k] : 0.0f;
            }
        }
        if (BKN) {
            for (int idx = tid; idx < GBN * GBK; idx += 256) {
                const int kk = idx / GBN, nn = idx % GBN;
                const int k = k0 + kk, n = n0 + nn;
                Bs[kk][nn] = (n < N && k < Kd) ? B[(size_t)k * N + n] : 0.0f;
            }
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GBK; ++kk) {
            float av[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) bv[j] = Bs[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
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
            const size_t o = (size_t)(tl.row0 + r) * N + n;
            if (EPI == 0) C1[o] = acc[i][j];
            else if (EPI == 1) C1[o] = C1[o] + acc[i][j];
            else {
                const float h1 = C1[o], h3 = C2[o], da = acc[i][j];
                const float sg = 1.0f / (1.0f + expf(-h1));
                C2[o] = da * (h1 * sg);
                C1[o] = (da * h3) * sg * (1.0f + h1 * (1.0f - sg));
            }
        }
    }
}

// dW_g[m, n] = sum over the rows r of group g of A[r, m] * B[r, n]  (diffW = delta^T . input); always written, so a group
// without rows gets zeros.  grid (ceil(N/64), ceil(M/64), groups).  Rows of group g: physical rows from
// tile_meta[1+g]*bm, counts[g] of them for a routed expert, T for a shared one; a shared group reads token rows
// 0..T-1 of Atok / Btok when those are given.
// gstride: floats between the outputs of consecutive groups.
__global__ __launch_bounds__(256) void bw_wgrad_f32_kernel(const float *__restrict__ Aphys, const float *__restrict__ Atok,
                                                           const float *__restrict__ Bphys, const float *__restrict__ Btok,
                                                           float *__restrict__ dW, size_t gstride,
                                                           const int32_t *__restrict__ tile_meta,
                                                           const int32_t *__restrict__ counts, int E, int T, int bm,
                                                           int M, int N)
{
    const int g = blockIdx.z;
    const int rows = g < E ? counts[g] : T, row0 = tile_meta[1 + g] * bm;
    const bool shared = g >= E;
    const float *A = (shared && Atok) ? Atok : Aphys + (size_t)row0 * M;
    const float *B = (shared && Btok) ? Btok : Bphys + (size_t)row0 * N;
    const int m0 = blockIdx.y * GBM, n0 = blockIdx.x * GBN;

    __shared__ float As[GBK][GBM + 4];
    __shared__ float Bs[GBK][GBN + 4];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    float acc[4][4] = {};
    for (int r0 = 0; r0 < rows; r0 += GBK) {
        for (int idx = tid; idx < GBK * GBM; idx += 256) {
            const int rr = idx / GBM, cc = idx % GBM;
            const int r = r0 + rr;
            As[rr][cc] = (r < rows && m0 + cc < M) ? A[(size_t)r * M + m0 + cc] : 0.0f;
            Bs[rr][cc] = (r < rows && n0 + cc < N) ? B[(size_t)r * N + n0 + cc] : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GBK; ++kk) {
            float av[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) bv[j] = Bs[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
        }
        __syncthreads();
    }
    float *out = dW + (size_t)g * gstride;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int mm = m0 + ty * 4 + i;
        if (mm >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) out[(size_t)mm * N + n] = acc[i][j];
        }
    }
}

// One thread per token: dw -> gradient of the selected probabilities (through the renormalisation w = q / sum q when
// enabled) -> softmax_back over the E experts.  Only the selected experts have a non-zero probability gradient, so
// sum_e p_e*dp_e runs over the K slots.
__global__ __launch_bounds__(256) void bw_router_kernel(const float *__restrict__ probs, const int32_t *__restrict__ ids,
                                                        const float *__restrict__ w, const float *__restrict__ dw, int T,
                                                        int E, int K, int renorm, float *__restrict__ dlogits)
{
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t >= T) return;
    const float *p = probs + (size_t)t * E;
    const int32_t *id = ids + (size_t)t * K;
    float S = 1.0f, dot = 0.0f;
    if (renorm) {
        S = 0.0f;
        for (int j = 0; j < K; ++j) S += p[id[j]];
        for (int j = 0; j < K; ++j) dot = fmaf(dw[(size_t)t * K + j], w[(size_t)t * K + j], dot);
    }
    float sum = 0.0f;
    for (int j = 0; j < K; ++j) {
        float g = dw[(size_t)t * K + j];
        if (renorm) g = (g - dot) / S;
        sum = fmaf(p[id[j]], g, sum);
    }
    float *dl = dlogits + (size_t)t * E;
    for (int e = 0; e < E; ++e) dl[e] = (0.0f - sum) * p[e];
    for (int j = 0; j < K; ++j) {
        float g = dw[(size_t)t * K + j];
        if (renorm) g = (g - dot) / S;
        dl[id[j]] = (g - sum) * p[id[j]];
    }
}

// Gate weight gradient dWg[e,k] = sum_t dlogits[t,e] * x[t,k] (diffW = delta^T . input) in two steps, both with a fixed
// order of additions: partial sums over slices of the tokens, then their sum.  Workgroup (column chunk of 256, token
// slice, expert chunk of 32): a thread owns one column and up to 32 experts; the slice's dlogits pass through LDS.
#define GW_EC 32
template <bool XBF>
__global__ __launch_bounds__(256) void bw_gate_partial_kernel(const float *__restrict__ dlogits, const void *__restrict__ x,
                                                              int T, int d, int E, int tslice, float *__restrict__ part)
{
    __shared__ __attribute__((aligned(16))) float dl[64][GW_EC];
    const int k = blockIdx.x * 256 + threadIdx.x, e0 = blockIdx.z * GW_EC;
    const int t0 = blockIdx.y * tslice, t1 = min(T, t0 + tslice);
    float acc[GW_EC];
#pragma unroll
    for (int e = 0; e < GW_EC; ++e) acc[e] = 0.0f;
    for (int tb = t0; tb < t1; tb += 64) {
        __syncthreads();
        for (int i = threadIdx.x; i < 64 * GW_EC; i += 256) {
            const int tt = tb + i / GW_EC, e = e0 + i % GW_EC;
            dl[i / GW_EC][i % GW_EC] = (tt < t1 && e < E) ? dlogits[(size_t)tt * E + e] : 0.0f;
        }
        __syncthreads();
        if (k < d) {
            const int n = min(64, t1 - tb);
            for (int tt = 0; tt < n; ++tt) {
                const float xv = XBF ? bf16_to_f32(((const bf16_t *)x)[(size_t)(tb + tt) * d + k])
                                     : ((const float *)x)[(size_t)(tb + tt) * d + k];
#pragma unroll
                for (int e4 = 0; e4 < GW_EC / 4; ++e4) {  // the whole wave reads the same 16 bytes: one broadcast read
                    const float4 v = *(const float4 *)&dl[tt][e4 * 4];
                    acc[e4 * 4 + 0] = fmaf(v.x, xv, acc[e4 * 4 + 0]);
                    acc[e4 * 4 + 1] = fmaf(v.y, xv, acc[e4 * 4 + 1]);
                    acc[e4 * 4 + 2] = fmaf(v.z, xv, acc[e4 * 4 + 2]);
                    acc[e4 * 4 + 3] = fmaf(v.w, xv, acc[e4 * 4 + 3]);
                }
            }
        }
    }
    if (k < d)
#pragma unroll
        for (int e = 0; e < GW_EC; ++e)
            if (e0 + e < E) part[((size_t)blockIdx.y * E + e0 + e) * d + k] = acc[e];
}

__global__ __launch_bounds__(256) void bw_gate_reduce_kernel(const float *__restrict__ part, int nslices, size_t n,
                                                             float *__restrict__ dWg)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float s = 0.0f;
    for (int q = 0; q < nslices; ++q) s += part[(size_t)q * n + i];
    dWg[i] = s;
}

#define GW_SLICES 32
static hipError_t launch_gate_wgrad(const omega_moe *m, const void *x, int T, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const int tslice = ceil_div(ceil_div(T, GW_SLICES), 64) * 64, nsl = ceil_div(T, tslice);
    const dim3 grid(ceil_div(c.d, 256), nsl, ceil_div(c.E, GW_EC));
    if (c.dtype == OMEGA_DTYPE_BF16)
        hipLaunchKernelGGL(bw_gate_partial_kernel<true>, grid, dim3(256), 0, s, (const float *)m->bw_dlogits, x, T, c.d, c.E,
                           tslice, m->bw_gpart);
    else
        hipLaunchKernelGGL(bw_gate_partial_kernel<false>, grid, dim3(256), 0, s, (const float *)m->bw_dlogits, x, T, c.d, c.E,
                           tslice, m->bw_gpart);
    const size_t n = (size_t)c.E * c.d;
    hipLaunchKernelGGL(bw_gate_reduce_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const float *)m->bw_gpart, nsl,
                       n, m->dWg);
    return hipGetLastError();
}

// dbg[e] = sum_t dlogits[t,e]: one workgroup per expert.
__global__ __launch_bounds__(256) void bw_gate_bias_kernel(const float *__restrict__ dlogits, int T, int E,
                                                           float *__restrict__ dbg)
{
    __shared__ float red[4];
    const int e = blockIdx.x;
    float part = 0.0f;
    for (int t = threadIdx.x; t < T; t += 256) part += dlogits[(size_t)t * E + e];
    const float tot = block_sum_256(part, red);
    if (threadIdx.x == 0) dbg[e] = tot;
}

// dx[t,:] = sum_j dxg[row(t,j),:] (slot order) + shared-expert rows + dlogits[t,:] . Wg.  One workgroup per DX_TT
// tokens and 512 columns (a thread owns two adjacent columns): a gate weight is read once for the DX_TT tokens.
// XBF: Wg and dx are bf16 (one rounding of the fp32 sum).  d must be even.
#define DX_TT 8
template <bool XBF>
__global__ __launch_bounds__(256) void bw_dx_kernel(const float *__restrict__ dxg, const int32_t *__restrict__ dstp,
                                                    const float *__restrict__ dlogits, const void *__restrict__ Wg,
                                                    const int32_t *__restrict__ tile_meta, int T, int K, int d, int E, int Es,
                                                    int bm, void *__restrict__ dx)
{
    extern __shared__ __attribute__((aligned(16))) float dl[];  // [E][DX_TT]
    const int t0 = blockIdx.x * DX_TT, nt = min(DX_TT, T - t0);
    for (int i = threadIdx.x; i < E * DX_TT; i += 256) {
        const int e = i / DX_TT, tt = i % DX_TT;
        dl[i] = tt < nt ? dlogits[(size_t)(t0 + tt) * E + e] : 0.0f;
    }
    __syncthreads();
    const int c = (blockIdx.y * 256 + threadIdx.x) * 2;
    if (c >= d) return;
    float g0[DX_TT], g1[DX_TT];
#pragma unroll
    for (int tt = 0; tt < DX_TT; ++tt) g0[tt] = g1[tt] = 0.0f;
    for (int e = 0; e < E; ++e) {
        float w0, w1;
        if (XBF) {
            const uint32_t u = *(const uint32_t *)((const bf16_t *)Wg + (size_t)e * d + c);
            w0 = __uint_as_float(u << 16);
            w1 = __uint_as_float(u & 0xffff0000u);
        } else {
            const float2 f = *(const float2 *)((const float *)Wg + (size_t)e * d + c);
            w0 = f.x;
            w1 = f.y;
        }
        const float4 da = *(const float4 *)&dl[e * DX_TT], db = *(const float4 *)&dl[e * DX_TT + 4];
        const float dv[DX_TT] = {da.x, da.y, da.z, da.w, db.x, db.y, db.z, db.w};
#pragma unroll
        for (int tt = 0; tt < DX_TT; ++tt) {
            g0[tt] = fmaf(dv[tt], w0, g0[tt]);
            g1[tt] = fmaf(dv[tt], w1, g1[tt]);
        }
    }
#pragma unroll
    for (int tt = 0; tt < DX_TT; ++tt) {
        if (tt >= nt) break;
        const int t = t0 + tt;
        float a0 = 0.0f, a1 = 0.0f;
        for (int j = 0; j < K; ++j) {
            const float2 v = *(const float2 *)(dxg + (size_t)dstp[(size_t)t * K + j] * d + c);
            a0 += v.x;
            a1 += v.y;
        }
        for (int s = 0; s < Es; ++s) {
            const float2 v = *(const float2 *)(dxg + ((size_t)tile_meta[1 + E + s] * bm + t) * d + c);
            a0 += v.x;
            a1 += v.y;
        }
        a0 += g0[tt];
        a1 += g1[tt];
        if (XBF) *(uint32_t *)((bf16_t *)dx + (size_t)t * d + c) = (uint32_t)f32_to_bf16(a0) | ((uint32_t)f32_to_bf16(a1) << 16);
        else *(float2 *)((float *)dx + (size_t)t * d + c) = make_float2(a0, a1);
    }
}

// bf16 layers (d is a multiple of 256): four adjacent columns per thread (16-byte loads of the fp32 rows, 8-byte loads
// of the gate weights), the row indices of the workgroup's tokens staged in LDS so that the loads of a token's rows do
// not wait for index loads one by one.  Same sums in the same order as bw_dx_kernel.
__global__ __launch_bounds__(256) void bw_dx4_bf16_kernel(const float *__restrict__ dxg, const int32_t *__restrict__ dstp,
                                                          const float *__restrict__ dlogits, const bf16_t *__restrict__ Wg,
                                                          const int32_t *__restrict__ tile_meta, int T, int K, int d, int E,
                                                          int Es, int bm, bf16_t *__restrict__ dx)
{
    extern __shared__ __attribute__((aligned(16))) float dl[];  // [E][DX_TT], then the row indices [DX_TT][K]
    int *rows_s = (int *)(dl + E * DX_TT);
    const int t0 = blockIdx.x * DX_TT, nt = min(DX_TT, T - t0);
    for (int i = threadIdx.x; i < E * DX_TT; i += 256) {
        const int e = i / DX_TT, tt = i % DX_TT;
        dl[i] = tt < nt ? dlogits[(size_t)(t0 + tt) * E + e] : 0.0f;
    }
    for (int i = threadIdx.x; i < nt * K; i += 256) rows_s[i] = dstp[(size_t)t0 * K + i];
    __syncthreads();
    const int c = (blockIdx.y * 256 + threadIdx.x) * 4;
    if (c >= d) return;
    float g[4][DX_TT];
#pragma unroll
    for (int v = 0; v < 4; ++v)
#pragma unroll
        for (int tt = 0; tt < DX_TT; ++tt) g[v][tt] = 0.0f;
    for (int e = 0; e < E; ++e) {
        const uint2 u = *(const uint2 *)(Wg + (size_t)e * d + c);
        const float w[4] = {__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                            __uint_as_float(u.y & 0xffff0000u)};
        const float4 da = *(const float4 *)&dl[e * DX_TT], db = *(const float4 *)&dl[e * DX_TT + 4];
        const float dv[DX_TT] = {da.x, da.y, da.z, da.w, db.x, db.y, db.z, db.w};
#pragma unroll
        for (int tt = 0; tt < DX_TT; ++tt)
#pragma unroll
            for (int v = 0; v < 4; ++v) g[v][tt] = fmaf(dv[tt], w[v], g[v][tt]);
    }
#pragma unroll
    for (int tt = 0; tt < DX_TT; ++tt) {
        if (tt >= nt) break;
        const int t = t0 + tt;
        float a[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int j0 = 0; j0 < K; j0 += 8) {
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)  // slots past K re-read the last row and are not added
                v[u] = *(const float4 *)(dxg + (size_t)rows_s[tt * K + min(j0 + u, K - 1)] * d + c);
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (j0 + u < K) { a[0] += v[u].x; a[1] += v[u].y; a[2] += v[u].z; a[3] += v[u].w; }
        }
        for (int s = 0; s < Es; ++s) {
            const float4 v = *(const float4 *)(dxg + ((size_t)tile_meta[1 + E + s] * bm + t) * d + c);
            a[0] += v.x; a[1] += v.y; a[2] += v.z; a[3] += v.w;
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) a[q] += g[q][tt];
        uint2 o;
        o.x = (uint32_t)f32_to_bf16(a[0]) | ((uint32_t)f32_to_bf16(a[1]) << 16);
        o.y = (uint32_t)f32_to_bf16(a[2]) | ((uint32_t)f32_to_bf16(a[3]) << 16);
        *(uint2 *)(dx + (size_t)t * d + c) = o;
    }
}

// fp32 layers whose width is odd: one workgroup per token, one column per thread and step
__global__ __launch_bounds__(256) void bw_dx_scalar_kernel(const float *__restrict__ dxg, const int32_t *__restrict__ dstp,
                                                           const float *__restrict__ dlogits, const float *__restrict__ Wg,
                                                           const int32_t *__restrict__ tile_meta, int K, int d, int E, int Es,
                                                           int bm, float *__restrict__ dx)
{
    const int t = blockIdx.x;
    extern __shared__ float dl[];  // E floats
    for (int e = threadIdx.x; e < E; e += 256) dl[e] = dlogits[(size_t)t * E + e];
    __syncthreads();
    for (int c = threadIdx.x; c < d; c += 256) {
        float acc = 0.0f;
        for (int j = 0; j < K; ++j) acc += dxg[(size_t)dstp[(size_t)t * K + j] * d + c];
        for (int s = 0; s < Es; ++s) acc += dxg[((size_t)tile_meta[1 + E + s] * bm + t) * d + c];
        float gs = 0.0f;
        for (int e = 0; e < E; ++e) gs = fmaf(dl[e], Wg[(size_t)e * d + c], gs);
        dx[(size_t)t * d + c] = acc + gs;
    }
}

// dst += scale * src (accGrad: axpy_gpu, J/engine/nn/layer/FullyLayer.java:593-607);  w -= lr * g (update without an updater,
// FullyLayer.java:581-586)
__global__ __launch_bounds__(256) void bw_axpy_kernel(float *__restrict__ dst, const float *__restrict__ src, float scale, size_t n)
{
    // 16-byte accesses when both pointers allow them
    if ((((uintptr_t)dst | (uintptr_t)src) & 15) == 0) {
        const size_t n4 = n >> 2;
        float4 *d4 = (float4 *)dst;
        const float4 *s4 = (const float4 *)src;
        for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (size_t)gridDim.x * 256) {
            float4 v = d4[i];
            const float4 u = s4[i];
            v.x = fmaf(scale, u.x, v.x); v.y = fmaf(scale, u.y, v.y); v.z = fmaf(scale, u.z, v.z); v.w = fmaf(scale, u.w, v.w);
            d4[i] = v;
        }
        if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
            const size_t i = (n4 << 2) + threadIdx.x;
            dst[i] = fmaf(scale, src[i], dst[i]);
        }
        return;
    }
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) dst[i] = fmaf(scale, src[i], dst[i]);
}

__global__ __launch_bounds__(256) void bw_zero_kernel(float *__restrict__ dst, size_t n)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) dst[i] = 0.0f;
}

// a fill kernel, not a memset node: safe inside a captured graph
hipError_t launch_zero_f32(float *dst, size_t n, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    const int grid = (int)((n + 255) / 256 < 1024 ? (n + 255) / 256 : 1024);
    hipLaunchKernelGGL(bw_zero_kernel, dim3(grid), dim3(256), 0, s, dst, n);
    return hipGetLastError();
}

hipError_t launch_axpy_f32(float *dst, const float *src, float scale, size_t n, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    const int grid = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
    hipLaunchKernelGGL(bw_axpy_kernel, dim3(grid), dim3(256), 0, s, dst, src, scale, n);
    return hipGetLastError();
}

// ---- global gradient norm and clipping (Network.clipGradNorm, J/engine/nn/network/Network.java:379-432) ----
// Sum of squares in two fixed-order stages (vectorL2NormKernel, J/engine/gpu/GlobalNormKernel.cu:3-30, adds its block
// sums with atomicAdd in arrival order; here the same data always gives the same bits): a thread sums its grid-stride
// elements in fp32, the workgroup and then one last workgroup add those in double.
#define SUMSQ_WG (OMEGA_SUMSQ_SLOTS - 1)
__global__ __launch_bounds__(256) void bw_sumsq_partial_kernel(const float *__restrict__ src, size_t n, double *__restrict__ part)
{
    __shared__ double red[256];
    // 16 bytes per load, four independent sums per thread; the last n % 4 elements go to the first thread
    float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
    const size_t n4 = n >> 2;
    const float4 *src4 = (const float4 *)src;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (size_t)gridDim.x * 256) {
        const float4 v = src4[i];
        a0 = fmaf(v.x, v.x, a0);
        a1 = fmaf(v.y, v.y, a1);
        a2 = fmaf(v.z, v.z, a2);
        a3 = fmaf(v.w, v.w, a3);
    }
    if (blockIdx.x == 0 && threadIdx.x == 0)
        for (size_t i = n4 << 2; i < n; ++i) a0 = fmaf(src[i], src[i], a0);
    red[threadIdx.x] = ((double)a0 + (double)a1) + ((double)a2 + (double)a3);
    __syncthreads();
    for (int h = 128; h > 0; h >>= 1) {
        if ((int)threadIdx.x < h) red[threadIdx.x] += red[threadIdx.x + h];
        __syncthreads();
    }
    if (threadIdx.x == 0) part[blockIdx.x] = red[0];
}

__global__ __launch_bounds__(256) void bw_sumsq_final_kernel(const double *__restrict__ part, int np, double *__restrict__ out)
{
    __shared__ double red[256];
    double acc = 0.0;
    for (int i = threadIdx.x; i < np; i += 256) acc += part[i];
    red[threadIdx.x] = acc;
    __syncthreads();
    for (int h = 128; h > 0; h >>= 1) {
        if ((int)threadIdx.x < h) red[threadIdx.x] += red[threadIdx.x + h];
        __syncthreads();
    }
    if (threadIdx.x == 0) out[0] = red[0];
}

// part: SUMSQ_WG + 1 doubles; the result lands in part[SUMSQ_WG]
hipError_t launch_sumsq_f32(const float *src, size_t n, double *part, hipStream_t s)
{
    const size_t want = (n / 4 + 255) / 256;
    const int grid = (int)(want < SUMSQ_WG ? want : SUMSQ_WG);
    hipLaunchKernelGGL(bw_sumsq_partial_kernel, dim3(grid > 0 ? grid : 1), dim3(256), 0, s, src, n, part);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(bw_sumsq_final_kernel, dim3(1), dim3(256), 0, s, (const double *)part, grid > 0 ? grid : 1, part + SUMSQ_WG);
    return hipGetLastError();
}

// dst *= coef, one rounding per element (TensorOP.mul(diffW, clip_coef, diffW), Network.java:416-431)
__global__ __launch_bounds__(256) void bw_scale_kernel(float *__restrict__ dst, float coef, size_t n)
{
    const size_t n4 = n >> 2;
    float4 *d4 = (float4 *)dst;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (size_t)gridDim.x * 256) {
        float4 v = d4[i];
        v.x *= coef; v.y *= coef; v.z *= coef; v.w *= coef;
        d4[i] = v;
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) dst[(n4 << 2) + threadIdx.x] *= coef;
}

hipError_t launch_scale_f32(float *dst, float coef, size_t n, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    const int grid = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
    hipLaunchKernelGGL(bw_scale_kernel, dim3(grid), dim3(256), 0, s, dst, coef, n);
    return hipGetLastError();
}

// ---- update of bf16 layers: fp32 master copies of the weights, the layer's bf16 copies re-rounded from them ----
// One thread per 16-byte chunk (8 consecutive columns of one row) of the packed tile image of expert blockIdx.y.
// init != 0: master = weight (first update after the weights were set); else master -= lr * grad, weight = bf16(master).
__global__ __launch_bounds__(256) void bw_update_packed_kernel(float *__restrict__ master, size_t mstride,
                                                               const float *__restrict__ grad, size_t gstride,
                                                               unsigned char *__restrict__ packed, size_t pstride, int R, int K,
                                                               float lr, int init)
{
    const int g = blockIdx.y, nch = K >> 3, KT = K >> 5;
    float *mg = master + (size_t)g * mstride;
    const float *gg = grad + (size_t)g * gstride;
    unsigned char *pg = packed + (size_t)g * pstride;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < (size_t)R * nch; i += (size_t)gridDim.x * 256) {
        const int r = (int)(i / nch), ch = (int)(i % nch);
        uint4 *pk = (uint4 *)(pg + pk_chunk_off(r, ch >> 2, ch & 3, KT));
        float4 *mp = (float4 *)(mg + (size_t)r * K + ch * 8);
        if (init) {
            const uint4 u = *pk;
            mp[0] = make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                                __uint_as_float(u.y & 0xffff0000u));
            mp[1] = make_float4(__uint_as_float(u.z << 16), __uint_as_float(u.z & 0xffff0000u), __uint_as_float(u.w << 16),
                                __uint_as_float(u.w & 0xffff0000u));
        } else {
            const float4 *gp = (const float4 *)(gg + (size_t)r * K + ch * 8);
            float4 a = mp[0], b = mp[1];
            const float4 ga = gp[0], gb = gp[1];
            a.x = fmaf(-lr, ga.x, a.x); a.y = fmaf(-lr, ga.y, a.y); a.z = fmaf(-lr, ga.z, a.z); a.w = fmaf(-lr, ga.w, a.w);
            b.x = fmaf(-lr, gb.x, b.x); b.y = fmaf(-lr, gb.y, b.y); b.z = fmaf(-lr, gb.z, b.z); b.w = fmaf(-lr, gb.w, b.w);
            mp[0] = a;
            mp[1] = b;
            uint4 o;
            o.x = (uint32_t)f32_to_bf16(a.x) | ((uint32_t)f32_to_bf16(a.y) << 16);
            o.y = (uint32_t)f32_to_bf16(a.z) | ((uint32_t)f32_to_bf16(a.w) << 16);
            o.z = (uint32_t)f32_to_bf16(b.x) | ((uint32_t)f32_to_bf16(b.y) << 16);
            o.w = (uint32_t)f32_to_bf16(b.z) | ((uint32_t)f32_to_bf16(b.w) << 16);
            *pk = o;
        }
    }
}

// the gate weight: row-major bf16
__global__ __launch_bounds__(256) void bw_update_rows_bf16_kernel(float *__restrict__ master, const float *__restrict__ grad,
                                                                  bf16_t *__restrict__ w, size_t n, float lr, int init)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        if (init) master[i] = bf16_to_f32(w[i]);
        else {
            const float v = fmaf(-lr, grad[i], master[i]);
            master[i] = v;
            w[i] = f32_to_bf16(v);
        }
    }
}

// masters laid out like the gradient block: mWg at `master`, mW13 and mW2 at the offsets of dW13 and dW2
hipError_t launch_update_bf16(const omega_moe *m, float *master, float lr, int init, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const size_t HD = (size_t)c.H * c.d;
    float *mW13 = master + (m->dW13 - m->dWg), *mW2 = master + (m->dW2 - m->dWg);
    const size_t nWg = (size_t)c.E * c.d;
    hipLaunchKernelGGL(bw_update_rows_bf16_kernel, dim3((unsigned)((nWg + 255) / 256 < 1024 ? (nWg + 255) / 256 : 1024)), dim3(256), 0,
                       s, master, (const float *)m->dWg, (bf16_t *)m->Wg, nWg, lr, init);
    const dim3 grid(512, m->G);
    hipLaunchKernelGGL(bw_update_packed_kernel, grid, dim3(256), 0, s, mW13, 2 * HD, (const float *)m->dW13, 2 * HD,
                       (unsigned char *)m->W1, HD * 2, c.H, c.d, lr, init);
    hipLaunchKernelGGL(bw_update_packed_kernel, grid, dim3(256), 0, s, mW13 + HD, 2 * HD, (const float *)m->dW13 + HD, 2 * HD,
                       (unsigned char *)m->W3, HD * 2, c.H, c.d, lr, init);
    hipLaunchKernelGGL(bw_update_packed_kernel, grid, dim3(256), 0, s, mW2, HD, (const float *)m->dW2, HD,
                       (unsigned char *)m->W2, HD * 2, c.d, c.H, lr, init);
    return hipGetLastError();
}

hipError_t launch_backward_f32(const omega_moe *m, const void *xv, const void *doutv, int T, void *dxv, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const float *x = (const float *)xv, *dout = (const float *)doutv;
    const float *xg = (const float *)m->xg, *a = (const float *)m->a;
    const float *W1 = (const float *)m->W1, *W3 = (const float *)m->W3, *W2 = (const float *)m->W2;
    const int G = m->G;
    hipError_t e;
    // probabilities of the forward pass (the router leaves ids and w as they are: same inputs, same arithmetic)
    if ((e = launch_router(m, x, T, nullptr, m->bw_probs, s)) != hipSuccess) return e;
    hipLaunchKernelGGL(bw_combine_kernel, dim3(T), dim3(256), 0, s, dout, m->y, m->dstp, m->w, c.K, c.d, m->bw_dy, m->bw_dw);
    // h1, h3 (recomputed), then d(a) = dy . W2 with the SwiGLU backward in its epilogue: bw_h1 <- dh1, bw_h3 <- dh3
    const dim3 gH(ceil_div(c.H, GBN), m->max_m_tiles), gD(ceil_div(c.d, GBN), m->max_m_tiles);
    hipLaunchKernelGGL((bw_rows_f32_kernel<false, 0>), gH, dim3(256), 0, s, xg, x, W1, m->bw_h1, (float *)nullptr, m->tiles,
                       m->tile_meta, c.H, c.d);
    hipLaunchKernelGGL((bw_rows_f32_kernel<false, 0>), gH, dim3(256), 0, s, xg, x, W3, m->bw_h3, (float *)nullptr, m->tiles,
                       m->tile_meta, c.H, c.d);
    hipLaunchKernelGGL((bw_rows_f32_kernel<true, 2>), gH, dim3(256), 0, s, (const float *)m->bw_dy, dout, W2, m->bw_h1,
                       m->bw_h3, m->tiles, m->tile_meta, c.H, c.d);
    // dxg = dh1 . W1 + dh3 . W3
    hipLaunchKernelGGL((bw_rows_f32_kernel<true, 0>), gD, dim3(256), 0, s, (const float *)m->bw_h1, (const float *)nullptr,
                       W1, m->bw_dxg, (float *)nullptr, m->tiles, m->tile_meta, c.d, c.H);
    hipLaunchKernelGGL((bw_rows_f32_kernel<true, 1>), gD, dim3(256), 0, s, (const float *)m->bw_h3, (const float *)nullptr,
                       W3, m->bw_dxg, (float *)nullptr, m->tiles, m->tile_meta, c.d, c.H);
    // weight gradients: dW2 = dy^T a [d,H]; dW1 = dh1^T xg, dW3 = dh3^T xg [H,d]
    const size_t HD = (size_t)c.H * c.d;
    hipLaunchKernelGGL(bw_wgrad_f32_kernel, dim3(ceil_div(c.H, GBN), ceil_div(c.d, GBM), G), dim3(256), 0, s,
                       (const float *)m->bw_dy, dout, a, (const float *)nullptr, m->dW2, HD, m->tile_meta, m->counts, c.E, T,
                       m->bm, c.d, c.H);
    hipLaunchKernelGGL(bw_wgrad_f32_kernel, dim3(ceil_div(c.d, GBN), ceil_div(c.H, GBM), G), dim3(256), 0, s,
                       (const float *)m->bw_h1, (const float *)nullptr, xg, x, m->dW13, 2 * HD, m->tile_meta, m->counts, c.E,
                       T, m->bm, c.H, c.d);
    hipLaunchKernelGGL(bw_wgrad_f32_kernel, dim3(ceil_div(c.d, GBN), ceil_div(c.H, GBM), G), dim3(256), 0, s,
                       (const float *)m->bw_h3, (const float *)nullptr, xg, x, m->dW13 + HD, 2 * HD, m->tile_meta, m->counts,
                       c.E, T, m->bm, c.H, c.d);
    // router and gate
    hipLaunchKernelGGL(bw_router_kernel, dim3(ceil_div(T, 256)), dim3(256), 0, s, (const float *)m->bw_probs, m->ids, m->w,
                       (const float *)m->bw_dw, T, c.E, c.K, c.renorm, m->bw_dlogits);
    if ((e = launch_gate_wgrad(m, x, T, s)) != hipSuccess) return e;
    if (c.has_gate_bias)
        hipLaunchKernelGGL(bw_gate_bias_kernel, dim3(c.E), dim3(256), 0, s, (const float *)m->bw_dlogits, T, c.E, m->dbg);
    if (c.d % 2 == 0 && ((uintptr_t)dxv % 8) == 0)
        hipLaunchKernelGGL(bw_dx_kernel<false>, dim3(ceil_div(T, DX_TT), ceil_div(c.d, 512)), dim3(256),
                           c.E * DX_TT * sizeof(float), s, (const float *)m->bw_dxg, m->dstp, (const float *)m->bw_dlogits,
                           (const void *)m->Wg, m->tile_meta, T, c.K, c.d, c.E, c.Es, m->bm, dxv);
    else
        hipLaunchKernelGGL(bw_dx_scalar_kernel, dim3(T), dim3(256), c.E * sizeof(float), s, (const float *)m->bw_dxg, m->dstp,
                           (const float *)m->bw_dlogits, (const float *)m->Wg, m->tile_meta, c.K, c.d, c.E, c.Es, m->bm,
                           (float *)dxv);
    return hipGetLastError();
}


// ------------------------------------------------------------------------------------------ bf16 layers
// One workgroup per token: dy rows (bf16, packed tile image) and dw; with shared experts also the packed copy of dout
// their products read.
__global__ __launch_bounds__(256) void bw_combine_bf16_kernel(const uint4 *__restrict__ dout, const float *__restrict__ y,
                                                              const int32_t *__restrict__ dstp, const float *__restrict__ w,
                                                              int K, int d, unsigned char *__restrict__ dy16,
                                                              unsigned char *__restrict__ dys16, float *__restrict__ dw)
{
    __shared__ float red[4];
    const int t = blockIdx.x, nch = d >> 3, KT = d >> 5;
    for (int j = 0; j < K; ++j) {
        const int r = dstp[(size_t)t * K + j];
        const float wv = w[(size_t)t * K + j];
        float part = 0.0f;
        for (int ch = threadIdx.x; ch < nch; ch += 256) {
            const uint4 u = dout[(size_t)t * nch + ch];
            const uint32_t uw[4] = {u.x, u.y, u.z, u.w};
            const float4 y0 = *(const float4 *)(y + (size_t)r * d + ch * 8), y1 = *(const float4 *)(y + (size_t)r * d + ch * 8 + 4);
            const float yv[8] = {y0.x, y0.y, y0.z, y0.w, y1.x, y1.y, y1.z, y1.w};
            uint32_t ow[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float g0 = __uint_as_float(uw[q] << 16), g1 = __uint_as_float(uw[q] & 0xffff0000u);
                part = fmaf(g0, yv[2 * q], part);
                part = fmaf(g1, yv[2 * q + 1], part);
                ow[q] = (uint32_t)f32_to_bf16(wv * g0) | ((uint32_t)f32_to_bf16(wv * g1) << 16);
            }
            *(uint4 *)(dy16 + pk_chunk_off(r, ch >> 2, ch & 3, KT)) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
        }
        const float tot = block_sum_256(part, red);
        if (threadIdx.x == 0) dw[(size_t)t * K + j] = tot;
    }
    if (dys16 != nullptr)
        for (int ch = threadIdx.x; ch < nch; ch += 256)
            *(uint4 *)(dys16 + pk_chunk_off(t, ch >> 2, ch & 3, KT)) = dout[(size_t)t * nch + ch];
}

// The weight gradients of a group without rows are zero; the product kernels have no items for it.
// A block that this kernel zeroed and nothing has written since (the group stayed without rows) is left alone:
// st_in[g] == 1 says so; every workgroup writes the group's new state to st_out (a second array, so that no workgroup
// of this launch reads what another one wrote).  force: the states are not to be trusted (the gradients were
// overwritten from the accumulators).
__global__ __launch_bounds__(256) void bw_zero_empty_kernel(const int32_t *__restrict__ counts, int E, int T,
                                                            float *__restrict__ dW13, float *__restrict__ dW2, size_t HD,
                                                            const int32_t *__restrict__ st_in, int32_t *__restrict__ st_out,
                                                            int force)
{
    const int g = blockIdx.x;
    const bool has_rows = (g < E ? counts[g] : T) > 0;
    const bool known_zero = !has_rows && !force && st_in[g] == 1;
    if (blockIdx.y == 0 && threadIdx.x == 0) st_out[g] = has_rows ? 0 : 1;
    if (has_rows || known_zero) return;
    float4 *p13 = (float4 *)(dW13 + (size_t)g * 2 * HD), *p2 = (float4 *)(dW2 + (size_t)g * HD);
    const float4 z = {0.0f, 0.0f, 0.0f, 0.0f};
    for (size_t i = (size_t)blockIdx.y * 256 + threadIdx.x; i < HD / 4; i += (size_t)gridDim.y * 256) {
        p13[i] = z;
        p13[HD / 4 + i] = z;
        p2[i] = z;
    }
}

hipError_t launch_backward_bf16(const omega_moe *m, const void *x, const void *dout, int T, void *dx, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const int G = m->G;
    const size_t HD = (size_t)c.H * c.d;
    hipError_t e;
#define STEP(expr) if ((e = (expr)) != hipSuccess) return e
    if (!m->rec_valid) STEP(launch_router(m, x, T, nullptr, m->bw_probs, s));  // a training forward kept the probabilities
    STEP(launch_backward_tables(m, T, s));
    hipLaunchKernelGGL(bw_combine_bf16_kernel, dim3(T), dim3(256), 0, s, (const uint4 *)dout, (const float *)m->y, m->dstp, m->w,
                       c.K, c.d, (unsigned char *)m->bw_dy16, (unsigned char *)m->bw_dys16, m->bw_dw);
    STEP(hipGetLastError());
    // h1, h3 (recomputed) as block records; d(a) = dy . W2 with the SwiGLU backward in its epilogue -> dh1 | dh3;
    // dxg = dh1 . W1 + dh3 . W3 as one product over the 2H columns of dh
    if (!m->rec_valid)
        STEP(launch_product_bf16(m, MODE_UPRAW, m->xg, m->xs, m->W1, m->W3, m->bw_h1, m->bw_h3, nullptr, m->wq_up, c.H, c.d, s));
    STEP(launch_product_bf16(m, MODE_DA, m->bw_dy16, m->bw_dys16, m->W2T, nullptr, m->bw_dh16, m->bw_h1, m->bw_h3, m->wq_da,
                             c.H, c.d, s));
    // (the forward's down table: where it holds k slices, their partial results go through y_slabs like the forward's)
    const bool sliced = m->down_ks_max > 1 || m->down_tail_ks > 1;
    STEP(launch_product_bf16(m, MODE_DOWN, m->bw_dh16, nullptr, m->W13T, nullptr, m->bw_dxg, sliced ? (void *)m->y_slabs : nullptr,
                             nullptr, m->wq_down, c.d, 2 * c.H, s));
    if (sliced) STEP(launch_down_slab_reduce(m, m->bw_dxg, s));
    // weight gradients: the experts' rows become the K axis of transposed images
    STEP(launch_transpose_groups(m, m->bw_dy16, m->bw_dys16, c.d, m->bw_dyT, T, s));
    STEP(launch_transpose_groups(m, m->a, nullptr, c.H, m->bw_aT, T, s));
    STEP(launch_transpose_groups(m, m->xg, m->xs, c.d, m->bw_xgT, T, s));
    STEP(launch_transpose_groups(m, m->bw_dh16, nullptr, 2 * c.H, m->bw_dhT, T, s));
    STEP(launch_product_bf16(m, MODE_WGRAD, m->bw_dyT, nullptr, m->bw_aT, nullptr, m->dW2, nullptr, nullptr, m->wq_w2, c.H,
                             m->bw_ksteps_cap * 32, s));
    STEP(launch_product_bf16(m, MODE_WGRAD, m->bw_dhT, nullptr, m->bw_xgT, nullptr, m->dW13, nullptr, nullptr, m->wq_w13, c.d,
                             m->bw_ksteps_cap * 32, s));
    hipLaunchKernelGGL(bw_zero_empty_kernel, dim3(G, 128), dim3(256), 0, s, m->counts, c.E, T, m->dW13, m->dW2, HD,
                       (const int32_t *)(m->bw_zero_state + (m->bw_zero_phase ? G : 0)), m->bw_zero_state + (m->bw_zero_phase ? 0 : G),
                       m->bw_zero_valid ? 0 : 1);
    // router and gate
    hipLaunchKernelGGL(bw_router_kernel, dim3(ceil_div(T, 256)), dim3(256), 0, s, (const float *)m->bw_probs, m->ids, m->w,
                       (const float *)m->bw_dw, T, c.E, c.K, c.renorm, m->bw_dlogits);
    STEP(launch_gate_wgrad(m, x, T, s));
    if (c.has_gate_bias)
        hipLaunchKernelGGL(bw_gate_bias_kernel, dim3(c.E), dim3(256), 0, s, (const float *)m->bw_dlogits, T, c.E, m->dbg);
    hipLaunchKernelGGL(bw_dx4_bf16_kernel, dim3(ceil_div(T, DX_TT), ceil_div(c.d, 1024)), dim3(256),
                       (c.E * DX_TT + DX_TT * c.K) * sizeof(float), s, (const float *)m->bw_dxg, m->dstp,
                       (const float *)m->bw_dlogits, (const bf16_t *)m->Wg, m->tile_meta, T, c.K, c.d, c.E, c.Es, m->bm,
                       (bf16_t *)dx);
#undef STEP
    return hipGetLastError();
}
