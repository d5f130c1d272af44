// Combine: out[t,:] = sum_j w[t,j] * y[row of pair t*K+j,:] in slot order, then + the shared experts' rows
// (rows are the physical rows the dispatch stage assigned; shared expert s owns rows first_tile[E+s]*bm + t).
// One wave per token; each lane owns 4 (fp32 out) or 8 (bf16 out) consecutive columns, read from the
// fp32 rows of y with 16-byte loads; products and sums are separate fp32 operations in slot order
// (this file is compiled with -ffp-contract=off), the weighted sum of add_mul_kernel
// (J/engine/gpu/BaseKernel.cu:228-241) generalised to K terms; shared rows are added as add_kernel
// (J/engine/ad/op/gpu/OPKernel.cu:359-366).  No atomics: every output element has one writer.
#include "common.h"

#define MAXK 64

// KU: slots whose rows are fetched together before any of them is used (all loads of a group are in flight at
// once; slots beyond K re-read the last row and are ignored).
// resid != nullptr (block form): the row of x is added to the fp32 sum before the output is rounded
// (Tensor_OP().add(mlp out, tmp1, tmp2), J/engine/nn/layer/llama/LlamaTransformerBlock.java:136).
// NT: the rows of y are read with non-temporal loads.  They are read exactly once; when y is larger than the last-level
// cache (256 MiB) letting them pass it by is worth 13 % (8192 tokens, 64 experts: 0.143 -> 0.125 ms; 16384 tokens, 128
// experts: 0.260 -> 0.225 ms), below that size nothing.
template <int VEC, bool BF16, int KU, bool NT>
__global__ __launch_bounds__(256) void combine_kernel(const float *__restrict__ y, const int32_t *__restrict__ dst,
                                                      const float *__restrict__ w, int T, int K, int d, int Es,
                                                      const int32_t *__restrict__ tile_meta, int E, int bm,
                                                      const void *__restrict__ resid, void *__restrict__ out, int split)
{
    // `split` waves share a token, each taking d / split consecutive columns (more waves, more loads in flight, when
    // the batch has few tokens for the compute units there are)
    const int lane = threadIdx.x & 63;
    const int wv = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int t = wv / split, part = wv - t * split;
    if (t >= T) return;
    const int dc = d / split;
    // lane j < K holds row index and weight of slot j; broadcast through cross-lane reads
    int myrow = 0;
    float myw = 0.0f;
    if (lane < K) {
        myrow = dst[(size_t)t * K + lane];
        myw = w[(size_t)t * K + lane];
    }
    // every lane makes every trip (lanes past the row's end work on column 0 and store nothing): the cross-lane reads
    // of the slot rows and weights below must find their source lanes active
    for (int cb = part * dc; cb < (part + 1) * dc; cb += 64 * VEC) {
        const bool on = cb + lane * VEC < (part + 1) * dc;
        const int c0 = on ? cb + lane * VEC : 0;
        float acc[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;
        for (int j0 = 0; j0 < K; j0 += KU) {
            float4 buf[KU][VEC / 4];
#pragma unroll
            for (int u = 0; u < KU; ++u) {
                const int row = __shfl(myrow, min(j0 + u, K - 1), 64);
                const float4 *src = (const float4 *)(y + (size_t)row * d + c0);
#pragma unroll
                for (int q = 0; q < VEC / 4; ++q) {
                    if (NT) {
                        typedef float v4f __attribute__((ext_vector_type(4)));
                        const v4f t4 = __builtin_nontemporal_load((const v4f *)(src + q));
                        buf[u][q] = make_float4(t4.x, t4.y, t4.z, t4.w);
                    } else {
                        buf[u][q] = src[q];
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < KU; ++u) {
                if (j0 + u < K) {
                    const float wj = __shfl(myw, j0 + u, 64);
#pragma unroll
                    for (int q = 0; q < VEC / 4; ++q) {
                        const float4 v4 = buf[u][q];
                        float term;
                        term = wj * v4.x; acc[q * 4 + 0] = acc[q * 4 + 0] + term;
                        term = wj * v4.y; acc[q * 4 + 1] = acc[q * 4 + 1] + term;
                        term = wj * v4.z; acc[q * 4 + 2] = acc[q * 4 + 2] + term;
                        term = wj * v4.w; acc[q * 4 + 3] = acc[q * 4 + 3] + term;
                    }
                }
            }
        }
        for (int s = 0; s < Es; ++s) {
            const float4 *src = (const float4 *)(y + ((size_t)tile_meta[1 + E + s] * bm + t) * d + c0);
#pragma unroll
            for (int q = 0; q < VEC / 4; ++q) {
                const float4 v4 = src[q];
                acc[q * 4 + 0] = acc[q * 4 + 0] + v4.x;
                acc[q * 4 + 1] = acc[q * 4 + 1] + v4.y;
                acc[q * 4 + 2] = acc[q * 4 + 2] + v4.z;
                acc[q * 4 + 3] = acc[q * 4 + 3] + v4.w;
            }
        }
        if (resid != nullptr) {
            if (BF16) {
                const uint4 u = *(const uint4 *)((const bf16_t *)resid + (size_t)t * d + c0);
                const uint32_t uu[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                for (int v = 0; v < VEC / 2; ++v) {
                    acc[2 * v] = acc[2 * v] + __uint_as_float(uu[v] << 16);
                    acc[2 * v + 1] = acc[2 * v + 1] + __uint_as_float(uu[v] & 0xffff0000u);
                }
            } else {
                const float4 r4 = *(const float4 *)((const float *)resid + (size_t)t * d + c0);
                acc[0] = acc[0] + r4.x; acc[1] = acc[1] + r4.y; acc[2] = acc[2] + r4.z; acc[3] = acc[3] + r4.w;
            }
        }
        if (!on) continue;
        if (BF16) {
            uint32_t pk[VEC / 2];
#pragma unroll
            for (int v = 0; v < VEC / 2; ++v)
                pk[v] = (uint32_t)f32_to_bf16(acc[2 * v]) | ((uint32_t)f32_to_bf16(acc[2 * v + 1]) << 16);
            uint4 o = {pk[0], pk[1], pk[2], pk[3]};
            *(uint4 *)((bf16_t *)out + (size_t)t * d + c0) = o;
        } else {
            float4 o = {acc[0], acc[1], acc[2], acc[3]};
            *(float4 *)((float *)out + (size_t)t * d + c0) = o;
        }
    }
}

// Any d: scalar columns.
template <bool BF16>
__global__ __launch_bounds__(256) void combine_scalar_kernel(const float *__restrict__ y, const int32_t *__restrict__ dst,
                                                             const float *__restrict__ w, int T, int K, int d, int Es,
                                                             const int32_t *__restrict__ tile_meta, int E, int bm,
                                                             const void *__restrict__ resid, void *__restrict__ out)
{
    const int t = blockIdx.x;
    for (int c = threadIdx.x; c < d; c += 256) {
        float acc = 0.0f;
        for (int j = 0; j < K; ++j) {
            const float term = w[(size_t)t * K + j] * y[(size_t)dst[(size_t)t * K + j] * d + c];
            acc = acc + term;
        }
        for (int s = 0; s < Es; ++s) acc = acc + y[((size_t)tile_meta[1 + E + s] * bm + t) * d + c];
        if (resid != nullptr)
            acc = acc + (BF16 ? bf16_to_f32(((const bf16_t *)resid)[(size_t)t * d + c]) : ((const float *)resid)[(size_t)t * d + c]);
        if (BF16) ((bf16_t *)out)[(size_t)t * d + c] = f32_to_bf16(acc);
        else ((float *)out)[(size_t)t * d + c] = acc;
    }
}

hipError_t launch_combine(const omega_moe *m, int T, void *out, const void *resid, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const bool bf = c.dtype == OMEGA_DTYPE_BF16;
    const int vec = bf ? 8 : 4;
    if (c.d % vec == 0 && (((uintptr_t)out | (uintptr_t)resid) % 16) == 0 && c.K <= MAXK) {
        const bool nt = (size_t)T * (c.K + c.Es) * c.d * 4 > OMEGA_LLC_BYTES;
        // several waves per token, each with a share of the columns, until the launch has 256 waves per compute unit:
        // more loads in flight (4096 tokens x 4096 columns: 36.3 -> 30.6 us with 8 waves per token; 64 tokens:
        // 12.0 -> 6.9 us; 8192 tokens x 2048 columns x 8 rows: 122.6 -> 113.8 us with 4; 16384 tokens: 228 -> 210 us)
        int split = 1;
        while (split < 8 && (long long)T * split < 256LL * m->ctx->num_cus && c.d % (64 * vec * split * 2) == 0) split *= 2;
#define COMBINE_LAUNCH2(KUV, NTV)                                                                                      \
    do {                                                                                                              \
        if (bf)                                                                                                       \
            hipLaunchKernelGGL((combine_kernel<8, true, KUV, NTV>), dim3(ceil_div(T * split, 4)), dim3(256), 0, s, m->y, m->dstp, m->w, \
                               T, c.K, c.d, c.Es, m->tile_meta, c.E, m->bm, resid, out, split);                              \
        else                                                                                                          \
            hipLaunchKernelGGL((combine_kernel<4, false, KUV, NTV>), dim3(ceil_div(T * split, 4)), dim3(256), 0, s, m->y, m->dstp, \
                               m->w, T, c.K, c.d, c.Es, m->tile_meta, c.E, m->bm, resid, out, split);                        \
    } while (0)
#define COMBINE_LAUNCH(KUV)              \
    do {                                 \
        if (nt) COMBINE_LAUNCH2(KUV, true); \
        else COMBINE_LAUNCH2(KUV, false);   \
    } while (0)
        if (c.K <= 2) COMBINE_LAUNCH(2);
        else if (c.K <= 4) COMBINE_LAUNCH(4);
        else COMBINE_LAUNCH(8);
#undef COMBINE_LAUNCH
#undef COMBINE_LAUNCH2
    } else {
        if (bf)
            hipLaunchKernelGGL(combine_scalar_kernel<true>, dim3(T), dim3(256), 0, s, m->y, m->dstp, m->w, T, c.K, c.d,
                               c.Es, m->tile_meta, c.E, m->bm, resid, out);
        else
            hipLaunchKernelGGL(combine_scalar_kernel<false>, dim3(T), dim3(256), 0, s, m->y, m->dstp, m->w, T, c.K, c.d,
                               c.Es, m->tile_meta, c.E, m->bm, resid, out);
    }
    return hipGetLastError();
}
