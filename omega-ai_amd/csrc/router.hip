// Router: gate projection, row softmax, wave-level top-k, per-token-tile expert histogram.
//
// One workgroup (256 threads) routes a tile of 32 tokens.
//  phase 1  logits[t,e] = sum_k x[t,k]*Wg[e,k] (+bg[e]): one lane per (token, expert); x and Wg are
//           staged through LDS in chunks of 64 k.  EXACT mode adds the products one k at a time with
//           a separate multiply and add (this file is compiled with -ffp-contract=off), which is the
//           summation order of the reference's CPU dot (J/common/utils/MatrixOperation.java:1472-1478);
//           FAST mode uses fused multiply-adds (same order, one rounding per step).
//  phase 2  softmax as the reference's thread-per-row kernel (J/engine/gpu/SoftmaxKernel.cu:4-24, CPU twin
//           J/engine/gpu/SoftmaxKernel.java:69-87): max, e=(float)exp((double)(z-max)), sum in expert order,
//           divide -- the experts of a token live in the lanes of a wave (or of an 8/16/32-lane group),
//           the ordered sum is taken through cross-lane reads;
//           top-k: K rounds of a cross-lane (value,index) butterfly arg-max, "greater value, or equal
//           value and lower index" so ties go to the lowest expert; winners are masked out.
//  phase 3  LDS-atomic histogram of the selected experts, flushed as row `tile` of tile_counts[.,E].
#include "common.h"

#define TOK_TILE ROUTER_TOK_TILE
#define KC 64

template <int EP>
__global__ __launch_bounds__(256) void router_kernel(const void *__restrict__ x, int dtype, const void *__restrict__ Wg,
                                                     const float *__restrict__ bg, int T, int d, int E, int K,
                                                     int renorm, int exact, int32_t *__restrict__ ids,
                                                     float *__restrict__ wout, int32_t *__restrict__ tile_counts,
                                                     float *__restrict__ logits_out, float *__restrict__ probs_out)
{
    constexpr int NT = TOK_TILE * EP / 256;  // tokens per thread in phase 1
    constexpr int TPP = 256 / EP;            // tokens per pass
    constexpr int GS = EP < 64 ? EP : 64;    // lanes that share one token in phase 2
    constexpr int VPL = EP / GS;             // experts per lane in phase 2
    __shared__ float xs[TOK_TILE][KC + 1];
    __shared__ float ws[EP][KC + 1];
    __shared__ float lg[TOK_TILE][EP];
    __shared__ int hist[EP];

    const int tid = threadIdx.x;
    const int tile = blockIdx.x;
    const int t0 = tile * TOK_TILE;
    const int e1 = tid % EP, tg = tid / EP;
    if (tid < EP) hist[tid] = 0;

    float acc[NT];
#pragma unroll
    for (int i = 0; i < NT; ++i) acc[i] = 0.0f;

    for (int k0 = 0; k0 < d; k0 += KC) {
        const int kend = min(KC, d - k0);
        {   // x tile: 32 tokens x 64 k, 8 consecutive k per thread
            const int tt = tid >> 3, ks = (tid & 7) * 8;
            const int t = t0 + tt;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int k = k0 + ks + j;
                float v = 0.0f;
                if (t < T && k < d)
                    v = dtype == OMEGA_DTYPE_BF16 ? bf16_to_f32(((const bf16_t *)x)[(size_t)t * d + k])
                                                  : ((const float *)x)[(size_t)t * d + k];
                xs[tt][ks + j] = v;
            }
        }
        for (int idx = tid; idx < EP * KC; idx += 256) {
            const int e = idx / KC, kk = idx % KC;
            const int k = k0 + kk;
            float v = 0.0f;
            if (e < E && k < d)
                v = dtype == OMEGA_DTYPE_BF16 ? bf16_to_f32(((const bf16_t *)Wg)[(size_t)e * d + k])
                                              : ((const float *)Wg)[(size_t)e * d + k];
            ws[e][kk] = v;
        }
        __syncthreads();
        if (exact) {
            for (int k = 0; k < kend; ++k) {
                const float wv = ws[e1][k];
#pragma unroll
                for (int i = 0; i < NT; ++i) {
                    const float prod = xs[tg + i * TPP][k] * wv;
                    acc[i] = acc[i] + prod;
                }
            }
        } else {
            for (int k = 0; k < kend; ++k) {
                const float wv = ws[e1][k];
#pragma unroll
                for (int i = 0; i < NT; ++i) acc[i] = fmaf(xs[tg + i * TPP][k], wv, acc[i]);
            }
        }
        __syncthreads();
    }
    {
        const float b = (bg != nullptr && e1 < E) ? bg[e1] : 0.0f;
#pragma unroll
        for (int i = 0; i < NT; ++i) {
            const float z = bg != nullptr ? acc[i] + b : acc[i];
            lg[tg + i * TPP][e1] = z;
            const int t = t0 + tg + i * TPP;
            if (logits_out != nullptr && t < T && e1 < E) logits_out[(size_t)t * E + e1] = z;
        }
    }
    __syncthreads();

    // ---- phase 2: each wave owns 8 tokens; GS lanes share a token ----
    const int lane = tid & 63, wave = tid >> 6;
    const int sub = lane % GS, grp = lane / GS;
    constexpr int TOK_PER_PASS = 64 / GS;
    constexpr int PASSES = 8 / TOK_PER_PASS;
    for (int pass = 0; pass < PASSES; ++pass) {
        const int tt = wave * 8 + pass * TOK_PER_PASS + grp;
        const int t = t0 + tt;
        if (t >= T) continue;  // uniform over the GS lanes that exchange data
        float v[VPL], p[VPL];
        float mx = -INFINITY;
#pragma unroll
        for (int q = 0; q < VPL; ++q) {
            const int e = sub + q * GS;
            v[q] = e < E ? lg[tt][e] : -INFINITY;
            mx = fmaxf(mx, v[q]);
        }
#pragma unroll
        for (int m = GS / 2; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, GS));
#pragma unroll
        for (int q = 0; q < VPL; ++q) {
            const int e = sub + q * GS;
            p[q] = e < E ? (float)exp((double)(v[q] - mx)) : 0.0f;
        }
        float s = 0.0f;
#pragma unroll
        for (int q = 0; q < VPL; ++q)
            for (int l = 0; l < GS; ++l) {
                const float ev = __shfl(p[q], l, GS);
                if (l + q * GS < E) s = s + ev;
            }
#pragma unroll
        for (int q = 0; q < VPL; ++q) {
            const int e = sub + q * GS;
            p[q] = p[q] / s;
            if (probs_out != nullptr && e < E) probs_out[(size_t)t * E + e] = p[q];
            if (e >= E) p[q] = -1.0f;  // never selected: probabilities are >= 0
        }
        int myid = 0;
        float myw = 0.0f;
        for (int j = 0; j < K; ++j) {
            float bv = p[0];
            int bi = sub;
#pragma unroll
            for (int q = 1; q < VPL; ++q)
                if (p[q] > bv) { bv = p[q]; bi = sub + q * GS; }
#pragma unroll
            for (int m = GS / 2; m >= 1; m >>= 1) {
                const float ov = __shfl_xor(bv, m, GS);
                const int oi = __shfl_xor(bi, m, GS);
                if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
            }
            if (sub == j) { myid = bi; myw = bv; }
#pragma unroll
            for (int q = 0; q < VPL; ++q)
                if (bi == sub + q * GS) p[q] = -1.0f;
        }
        if (renorm) {
            float rs = 0.0f;
            for (int j = 0; j < K; ++j) rs = rs + __shfl(myw, j, GS);
            myw = myw / rs;
        }
        if (sub < K) {
            ids[(size_t)t * K + sub] = myid;
            wout[(size_t)t * K + sub] = myw;
            atomicAdd(&hist[myid], 1);
        }
    }
    __syncthreads();
    for (int e = tid; e < E; e += 256) tile_counts[(size_t)tile * E + e] = hist[e];
}

hipError_t launch_router(const omega_moe *m, const void *x, int T, float *logits_out, float *probs_out, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const int tiles = ceil_div(T, TOK_TILE);
    const int exact = c.router_mode == OMEGA_ROUTER_EXACT;
    const float *bg = c.has_gate_bias ? m->bg : nullptr;
#define ROUTER_LAUNCH(EPV)                                                                                         \
    hipLaunchKernelGGL(router_kernel<EPV>, dim3(tiles), dim3(256), 0, s, x, c.dtype, m->Wg, bg, T, c.d, c.E, c.K,   \
                       c.renorm, exact, m->ids, m->w, m->tile_counts, logits_out, probs_out)
    if (c.E <= 8) ROUTER_LAUNCH(8);
    else if (c.E <= 16) ROUTER_LAUNCH(16);
    else if (c.E <= 32) ROUTER_LAUNCH(32);
    else if (c.E <= 64) ROUTER_LAUNCH(64);
    else if (c.E <= 128) ROUTER_LAUNCH(128);
    else ROUTER_LAUNCH(256);
#undef ROUTER_LAUNCH
    return hipGetLastError();
}
