// Router: gate projection, row softmax, wave-level top-k, per-token-tile expert histogram.
//
// One workgroup routes a tile of TT tokens: 32 (256 threads), or 16 for layers with at most 16 experts (one thread per
// token and expert, 128 or 256 threads: the sums are bound by LDS reads per compute unit, so such a layer spreads its
// tokens over twice as many workgroups).
//  phase 1  logits[t,e] = sum_k x[t,k]*Wg[e,k] (+bg[e]): one lane per (token, expert); x and Wg are
//           staged through LDS in chunks of 64..256 k.  EXACT mode adds the products one k at a time with
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
// FAST mode of bf16 layers with more than 16 experts takes phase 1 to the matrix cores (router_mfma_kernel below).
// bf16 layers with at most 16 experts and at most one tile per compute unit take router_pipe_kernel: phase 1 is then as
// long as one chain of d dependent multiply-adds, and separate staging waves keep everything else out of the waves that
// run the chains (Mixtral shape: 4096 tokens 33 -> 29 us, 64 tokens 27 -> 22 us; of the 22, 11 are the chain itself at
// 6.25 clocks a term and 6.5 are launch, the first loads and phases 2 and 3).
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 rt_bf16x8;
typedef __attribute__((ext_vector_type(16))) float rt_f32x16;

#define ROUTER_EPT(EP) ((EP) >= 128 ? 4 : (EP) >= 32 ? 2 : 1)
// MFMA form of the exact sums (bf16 layers with more than 16 experts): a unit = 16 tokens x 64 experts, one
// v_mfma_f32_16x16x1_4b_f32 per k; a workgroup of 32 tokens has 2 * ceil(EP/64) units, dealt to its 4 waves
#define ROUTER_MU(EP) ((EP) > 128 ? 2 : 1)
// token tile and threads per workgroup for EP (padded) experts
#define ROUTER_TT(EP) ((EP) <= 16 ? 16 : 32)
#define ROUTER_NTHR(EP) ((EP) <= 8 ? 128 : 256)
// k per staged chunk for at most 16 experts: with 16-token tiles the sums of a 256-k chunk take less time than the
// next chunk's loads need to arrive, and the kernel is bound by one memory latency per chunk: 512-k chunks halve their
// number (Mixtral shape, 4096 tokens: 32-token tiles 42 us; 16-token tiles 54 us with 256-k chunks, 34 us with 512)
#define ROUTER_KC_SMALL 512
int router_tok_tile(int E) { return E <= 16 ? 16 : 32; }

// Phase 1 for the tokens t0.. of one workgroup: acc[x*NT + i] = logit of (token tg + i*TPP, expert e1 + x*EL), bias
// not yet added.  A thread owns EPT experts (2 from 128 experts on: each x value read from LDS then feeds two sums,
// which halves the LDS reads per multiply-add) and NT tokens.
// EP: experts padded to a power of two; KC: k per staged chunk (larger for few experts, where one chunk in
// flight per workgroup would otherwise leave the kernel waiting on memory latency).
// XBF: x and Wg are stored as bf16 (else fp32).  FAST_IO: rows are 16-byte aligned and d is a multiple of KC, so
// every load is a whole 16-byte vector; rows beyond T or E are redirected to the last valid row (their sums are
// never used), which keeps the loads free of branches - and with that really asynchronous: a load issued inside
// a divergent branch makes the compiler wait for all earlier ones first.
// MFMA: the sums run on the matrix cores instead (macc; acc is not touched): v_mfma_f32_16x16x1_4b_f32 takes ONE k per
// instruction - D = C + a*b per element, one product and one addition - so a chain of them over k = 0, 1, 2, ... is
// the sequential sum, term for term: with bf16 operands every product is exact in fp32 and the addition rounds once,
// exactly as the fused multiply-add of the vector path does.  A unit of 16 tokens x 64 experts is four 16 x 16 blocks
// (lane l supplies x[token l % 16][k] and Wg[expert l of the unit][k]); the chain of one unit keeps a SIMD's matrix
// pipe busy at twice the rate of the vector units, and a lane reads 32 bytes of LDS per 4 k instead of 128.
template <int EP, int KC, bool EXACT, bool XBF, bool FAST_IO, bool MFMA = false>
__device__ __forceinline__ void router_sums(const void *__restrict__ x, const void *__restrict__ Wg, int T, int d, int E,
                                            int t0, float (*xs)[KC + 4], float (*ws)[KC + 4],
                                            float (&acc)[ROUTER_TT(EP) * EP / ROUTER_NTHR(EP)], rt_f32x16 (&macc)[ROUTER_MU(EP)])
{
    constexpr int TOK_TILE = ROUTER_TT(EP), NTHR = ROUTER_NTHR(EP);
    constexpr int EPT = ROUTER_EPT(EP);           // experts per thread
    constexpr int EL = EP / EPT;                  // threads across the experts
    constexpr int NT = TOK_TILE * EL / NTHR;      // tokens per thread
    constexpr int TPP = NTHR / EL;                // tokens per pass
    static_assert(NT >= 1 && NT * NTHR == TOK_TILE * EL, "every thread owns whole (token, expert) sums");
    constexpr int TPR = NTHR / TOK_TILE;          // staging threads per token row (8 or 16)
    static_assert(TPR * TOK_TILE == NTHR && KC % (8 * TPR) == 0, "whole staging vectors per thread");
    const int tid = threadIdx.x;
    const int e1 = tid % EL, tg = tid / EL;
    // staging: every thread carries 8 consecutive k of one token and of WCH gate rows from global memory to LDS;
    // the next chunk is fetched into registers while the current one is being summed
    constexpr int XCH = KC / (8 * TPR);
    constexpr int WCH = EP * (KC / 8) / NTHR;
    static_assert(EP * (KC / 8) % NTHR == 0, "every thread stages the same number of gate vectors");
    const int x_tt = tid / TPR, x_ks = (tid % TPR) * 8;
    // raw staging registers: 8 k of bf16 = one uint4, 8 k of fp32 = two; conversion happens when they are
    // written to LDS, so the global loads stay in flight during the sums of the current chunk
    uint4 xr[XCH][2], wr[WCH][2];
    auto load8 = [&](const void *base, int row, int rows, int k, uint4 *out) {
        out[0] = make_uint4(0, 0, 0, 0);
        out[1] = make_uint4(0, 0, 0, 0);
        if (FAST_IO) {
            const size_t off = (size_t)min(row, rows - 1) * d + k;
            if (XBF) {
                out[0] = *(const uint4 *)((const bf16_t *)base + off);
            } else {
                out[0] = *(const uint4 *)((const float *)base + off);
                out[1] = *(const uint4 *)((const float *)base + off + 4);
            }
        } else if (row < rows) {  // unaligned or ragged rows: element by element, packed into the same form
            const size_t row_off = (size_t)row * d;
            uint32_t u[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                u[q] = 0;
                if (k + q < d)
                    u[q] = XBF ? (uint32_t)((const bf16_t *)base)[row_off + k + q]
                               : __float_as_uint(((const float *)base)[row_off + k + q]);
            }
            if (XBF) {
                out[0] = make_uint4(u[0] | (u[1] << 16), u[2] | (u[3] << 16), u[4] | (u[5] << 16), u[6] | (u[7] << 16));
            } else {
                out[0] = make_uint4(u[0], u[1], u[2], u[3]);
                out[1] = make_uint4(u[4], u[5], u[6], u[7]);
            }
        }
    };
    auto widen = [&](const uint4 *in, float *dst) {  // 8 floats to LDS
        float4 lo, hi;
        if (XBF) {
            lo = make_float4(__uint_as_float(in[0].x << 16), __uint_as_float(in[0].x & 0xffff0000u),
                             __uint_as_float(in[0].y << 16), __uint_as_float(in[0].y & 0xffff0000u));
            hi = make_float4(__uint_as_float(in[0].z << 16), __uint_as_float(in[0].z & 0xffff0000u),
                             __uint_as_float(in[0].w << 16), __uint_as_float(in[0].w & 0xffff0000u));
        } else {
            lo = make_float4(__uint_as_float(in[0].x), __uint_as_float(in[0].y), __uint_as_float(in[0].z), __uint_as_float(in[0].w));
            hi = make_float4(__uint_as_float(in[1].x), __uint_as_float(in[1].y), __uint_as_float(in[1].z), __uint_as_float(in[1].w));
        }
        *(float4 *)dst = lo;
        *(float4 *)(dst + 4) = hi;
    };
    auto fetch = [&](int k0) {
#pragma unroll
        for (int c = 0; c < XCH; ++c) load8(x, t0 + x_tt, T, k0 + x_ks + 8 * TPR * c, xr[c]);
#pragma unroll
        for (int c = 0; c < WCH; ++c) {
            const int idx = tid + c * NTHR;
            load8(Wg, idx / (KC / 8), E, k0 + (idx % (KC / 8)) * 8, wr[c]);
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int c = 0; c < XCH; ++c) widen(xr[c], &xs[x_tt][x_ks + 8 * TPR * c]);
#pragma unroll
        for (int c = 0; c < WCH; ++c) {
            const int idx = tid + c * NTHR;
            widen(wr[c], &ws[idx / (KC / 8)][(idx % (KC / 8)) * 8]);
        }
    };

    // a wave whose lowest token is past the end of the batch has no sum to form (small batches, ragged last tile):
    // the sums are bound by LDS reads, which its silence leaves to the waves that have tokens
    const bool wave_live = t0 + (tid & ~63) / EL < T;
    fetch(0);
    for (int k0 = 0; k0 < d; k0 += KC) {
        const int kend = min(KC, d - k0);
        stash();
        __syncthreads();
        if (k0 + KC < d) fetch(k0 + KC);
        // the products are added one k at a time in index order: EXACT with a separate multiply and add,
        // FAST with a fused multiply-add (one rounding per step).  With bf16 operands the two are the same
        // arithmetic: a product of two 8-bit significands has 16 bits and is exact in fp32 (unless it falls below
        // 2^-134, far outside anything a layer holds), so the separate multiply rounds nothing and EXACT takes the
        // fused form too - bit for bit the sequential unfused sum, at one instruction per term.
#define ROUTER_K4(k4)                                                                  \
    do {                                                                               \
        float4 wv[EPT];                                                                \
        _Pragma("unroll") for (int x_ = 0; x_ < EPT; ++x_)                             \
            wv[x_] = *(const float4 *)&ws[e1 + x_ * EL][(k4) * 4];                     \
        _Pragma("unroll") for (int i = 0; i < NT; ++i)                                 \
        {                                                                              \
            const float4 xv = *(const float4 *)&xs[tg + i * TPP][(k4) * 4];            \
            _Pragma("unroll") for (int x_ = 0; x_ < EPT; ++x_)                         \
            {                                                                          \
                float &a_ = acc[x_ * NT + i];                                          \
                if (EXACT && !XBF) {                                                   \
                    float prod;                                                        \
                    prod = xv.x * wv[x_].x; a_ = a_ + prod;                            \
                    prod = xv.y * wv[x_].y; a_ = a_ + prod;                            \
                    prod = xv.z * wv[x_].z; a_ = a_ + prod;                            \
                    prod = xv.w * wv[x_].w; a_ = a_ + prod;                            \
                } else {                                                               \
                    a_ = fmaf(xv.x, wv[x_].x, a_);                                     \
                    a_ = fmaf(xv.y, wv[x_].y, a_);                                     \
                    a_ = fmaf(xv.z, wv[x_].z, a_);                                     \
                    a_ = fmaf(xv.w, wv[x_].w, a_);                                     \
                }                                                                      \
            }                                                                          \
        }                                                                              \
    } while (0)
        if (MFMA) {
            constexpr int UNITS = 2 * ((EP + 63) / 64), MU = ROUTER_MU(EP);
            const int lane = tid & 63, wave = tid >> 6;
            const float *xrow[MU], *wrow[MU];
#pragma unroll
            for (int j = 0; j < MU; ++j) {
                const int u = min(wave + 4 * j, UNITS - 1);  // (waves without a unit do not enter the loop below)
                xrow[j] = &xs[(u & 1) * 16 + (lane & 15)][0];
                wrow[j] = &ws[min((u >> 1) * 64 + lane, EP - 1)][0];
            }
            if (wave < UNITS) {  // uniform over the wave
#pragma unroll 4
                for (int k4 = 0; k4 < KC / 4; ++k4) {  // (beyond d the staged chunk is zero: a +0 term changes nothing)
#pragma unroll
                    for (int j = 0; j < MU; ++j) {
                        if (wave + 4 * j >= UNITS) continue;
                        const float4 xv = *(const float4 *)(xrow[j] + k4 * 4), wv = *(const float4 *)(wrow[j] + k4 * 4);
                        macc[j] = __builtin_amdgcn_mfma_f32_16x16x1f32(xv.x, wv.x, macc[j], 0, 0, 0);
                        macc[j] = __builtin_amdgcn_mfma_f32_16x16x1f32(xv.y, wv.y, macc[j], 0, 0, 0);
                        macc[j] = __builtin_amdgcn_mfma_f32_16x16x1f32(xv.z, wv.z, macc[j], 0, 0, 0);
                        macc[j] = __builtin_amdgcn_mfma_f32_16x16x1f32(xv.w, wv.w, macc[j], 0, 0, 0);
                    }
                }
            }
        } else if (!wave_live) {
            // every token of this wave lies beyond T: it only stages and keeps the barriers
        } else if (FAST_IO || kend == KC) {
            // whole chunk: no exit test inside, so the LDS reads of later steps are issued ahead of the sums
#pragma unroll(NT * EPT >= 8 ? 4 : 16)
            for (int k4 = 0; k4 < KC / 4; ++k4) ROUTER_K4(k4);
        } else {
            // last, partial chunk (zero-filled beyond d: a +0 product leaves every sum unchanged)
            for (int k4 = 0; k4 * 4 < kend; ++k4) ROUTER_K4(k4);
        }
#undef ROUTER_K4
        __syncthreads();
    }
}

// Phases 2 and 3 for the tokens of one workgroup, from the logits in lg (all threads; lg and hist are complete and
// visible on entry; lg is overwritten).  LPT = NTHR / TOK_TILE lanes (8 or 16) share a token; lane j of them owns the
// experts j, j + LPT, ...  Softmax in the reference's order (J/engine/gpu/SoftmaxKernel.cu:4-24): the row maximum
// (any order gives the same value), e = (float)exp((double)(z - max)) written back to LDS, then ONE lane per token adds
// the E values in expert order - the reference's thread-per-row loop, run for all tokens of the tile side by side - and
// every lane divides.  Top-k: K rounds; a lane scans its own experts in ascending order with a strict comparison, the
// LPT lanes combine by a butterfly on (value, index) with "greater value, or equal value and lower index", so ties go
// to the lowest expert; the winner is masked out.  RELAXED (the matrix-core FAST path, tolerance mode) takes the
// exponentials in single precision.
template <int EP, bool RELAXED = false, int TOK_TILE = 32, int NTHR = 256>
__device__ __forceinline__ void router_select(float (*lg)[EP], int *hist, int t0, int tile, int T, int E, int K, int renorm,
                                              int32_t *__restrict__ ids, float *__restrict__ wout,
                                              int32_t *__restrict__ tile_counts, float *__restrict__ probs_out)
{
    constexpr int LPT = NTHR / TOK_TILE;            // lanes per token
    constexpr int VPL = (EP + LPT - 1) / LPT;       // experts per lane
    constexpr int KPL = (64 + LPT - 1) / LPT;       // slots per lane (K <= 64)
    static_assert(LPT == 8 || LPT == 16, "a token's lanes lie in one wave");
    const int tid = threadIdx.x;
    const int tt = tid / LPT, sub = tid % LPT;
    const int t = t0 + tt;
    const bool live = t < T;  // uniform over the LPT lanes that exchange data
    float p[VPL];
    float mx = -INFINITY;
#pragma unroll
    for (int q = 0; q < VPL; ++q) {
        const int e = sub + q * LPT;
        p[q] = (e < E && e < EP) ? lg[tt][e] : -INFINITY;
        mx = fmaxf(mx, p[q]);
    }
#pragma unroll
    for (int m = LPT / 2; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, LPT));
#pragma unroll
    for (int q = 0; q < VPL; ++q) {
        const int e = sub + q * LPT;
        p[q] = (e < E && e < EP) ? (RELAXED ? __expf(p[q] - mx) : (float)exp((double)(p[q] - mx))) : 0.0f;
        if (e < EP) lg[tt][e] = p[q];
    }
    __syncthreads();
    float s = 0.0f;
    if (sub == 0 && live)
        for (int e = 0; e < E; ++e) s = s + lg[tt][e];
    s = __shfl(s, 0, LPT);
#pragma unroll
    for (int q = 0; q < VPL; ++q) {
        const int e = sub + q * LPT;
        p[q] = p[q] / s;
        if (probs_out != nullptr && live && e < E) probs_out[(size_t)t * E + e] = p[q];
        if (e >= E) p[q] = -1.0f;  // never selected: probabilities are >= 0
    }
    // lane `sub` keeps the winners of the rounds j = sub, sub + LPT, ...
    int myid[KPL];
    float myw[KPL];
#pragma unroll
    for (int u = 0; u < KPL; ++u) { myid[u] = 0; myw[u] = 0.0f; }
    float rs = 0.0f;  // sum of the selected weights in slot order, the same in all lanes of the token
    for (int j = 0; j < K; ++j) {
        float bv = p[0];
        int bi = sub;
#pragma unroll
        for (int q = 1; q < VPL; ++q)
            if (p[q] > bv) { bv = p[q]; bi = sub + q * LPT; }
#pragma unroll
        for (int m = LPT / 2; m >= 1; m >>= 1) {
            const float ov = __shfl_xor(bv, m, LPT);
            const int oi = __shfl_xor(bi, m, LPT);
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
        rs = rs + bv;
#pragma unroll
        for (int u = 0; u < KPL; ++u)
            if (j == sub + u * LPT) { myid[u] = bi; myw[u] = bv; }
#pragma unroll
        for (int q = 0; q < VPL; ++q)
            if (bi == sub + q * LPT) p[q] = -1.0f;
    }
#pragma unroll
    for (int u = 0; u < KPL; ++u) {
        const int j = sub + u * LPT;
        if (j < K && live) {
            ids[(size_t)t * K + j] = myid[u];
            wout[(size_t)t * K + j] = renorm ? myw[u] / rs : myw[u];
            atomicAdd(&hist[myid[u]], 1);
        }
    }
    __syncthreads();
    for (int e = tid; e < E; e += NTHR) tile_counts[(size_t)tile * E + e] = hist[e];
}

template <int EP, int KC, bool EXACT, bool MFMA = false>
__global__ __launch_bounds__(ROUTER_NTHR(EP)) void router_kernel(const void *__restrict__ x, int dtype, const void *__restrict__ Wg,
                                                     const float *__restrict__ bg, int T, int d, int E, int K,
                                                     int renorm, int32_t *__restrict__ ids,
                                                     float *__restrict__ wout, int32_t *__restrict__ tile_counts,
                                                     float *__restrict__ logits_out, float *__restrict__ probs_out)
{
    constexpr int TOK_TILE = ROUTER_TT(EP), NTHR = ROUTER_NTHR(EP);
    constexpr int EPT = ROUTER_EPT(EP), EL = EP / EPT;  // phase 1: experts per thread, threads across the experts
    constexpr int NT = TOK_TILE * EL / NTHR;            // tokens per thread in phase 1
    constexpr int TPP = NTHR / EL;                      // tokens per pass
    constexpr int LDW = KC + 4;  // LDS row stride in floats: rows stay 16-byte aligned and bank-staggered
    __shared__ __attribute__((aligned(16))) float xs[TOK_TILE][LDW];
    __shared__ __attribute__((aligned(16))) float ws[EP][LDW];
    // up to 64 experts the logits take the place of the staged gate rows once phase 1 is over (its last step is a
    // barrier); measured a fifth faster at 64 experts and slightly slower at 128, which keep an array of their own
    constexpr bool LG_ALIAS = EP <= 64;
    static_assert(LDW >= TOK_TILE, "the gate staging area holds the logits");
    __shared__ float lg_own[LG_ALIAS ? 1 : TOK_TILE][EP];
    float(*lg)[EP] = LG_ALIAS ? (float(*)[EP]) & ws[0][0] : lg_own;
    __shared__ int hist[EP];

    const int tid = threadIdx.x;
    const int tile = blockIdx.x;
    const int t0 = tile * TOK_TILE;
    const int e1 = tid % EL, tg = tid / EL;
    if (tid < EP) hist[tid] = 0;

    float acc[NT * EPT];
#pragma unroll
    for (int i = 0; i < NT * EPT; ++i) acc[i] = 0.0f;

    rt_f32x16 macc[ROUTER_MU(EP)];
#pragma unroll
    for (int j = 0; j < ROUTER_MU(EP); ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) macc[j][r] = 0.0f;

    const bool fast_io = (d % KC == 0) && (((uintptr_t)x | (uintptr_t)Wg) % 16 == 0);
    if (MFMA) {  // bf16 layers only (the launcher sees to it)
        if (fast_io) router_sums<EP, KC, EXACT, true, true, true>(x, Wg, T, d, E, t0, xs, ws, acc, macc);
        else router_sums<EP, KC, EXACT, true, false, true>(x, Wg, T, d, E, t0, xs, ws, acc, macc);
    } else if (dtype == OMEGA_DTYPE_BF16) {
        if (fast_io) router_sums<EP, KC, EXACT, true, true>(x, Wg, T, d, E, t0, xs, ws, acc, macc);
        else router_sums<EP, KC, EXACT, true, false>(x, Wg, T, d, E, t0, xs, ws, acc, macc);
    } else {
        if (fast_io) router_sums<EP, KC, EXACT, false, true>(x, Wg, T, d, E, t0, xs, ws, acc, macc);
        else router_sums<EP, KC, EXACT, false, false>(x, Wg, T, d, E, t0, xs, ws, acc, macc);
    }
    if (MFMA) {
        // unit u = (token half u % 2, expert group u / 2); lane: expert l % 16 of block b, register 4*b + r -> token 4*(l/16) + r
        constexpr int UNITS = 2 * ((EP + 63) / 64);
        const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
        for (int j = 0; j < ROUTER_MU(EP); ++j) {
            const int u = wave + 4 * j;
            if (u >= UNITS) continue;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int e = (u >> 1) * 64 + 16 * b + (lane & 15);
                if (e >= EP) continue;
                const float bias = (bg != nullptr && e < E) ? bg[e] : 0.0f;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int tt = (u & 1) * 16 + 4 * (lane >> 4) + r;
                    const float z = bg != nullptr ? macc[j][4 * b + r] + bias : macc[j][4 * b + r];
                    lg[tt][e] = z;
                    if (logits_out != nullptr && t0 + tt < T && e < E) logits_out[(size_t)(t0 + tt) * E + e] = z;
                }
            }
        }
    }
#pragma unroll
    for (int x_ = 0; x_ < (MFMA ? 0 : EPT); ++x_) {
        const int e = e1 + x_ * EL;
        const float b = (bg != nullptr && e < E) ? bg[e] : 0.0f;
#pragma unroll
        for (int i = 0; i < NT; ++i) {
            const float z = bg != nullptr ? acc[x_ * NT + i] + b : acc[x_ * NT + i];
            lg[tg + i * TPP][e] = z;
            const int t = t0 + tg + i * TPP;
            if (logits_out != nullptr && t < T && e < E) logits_out[(size_t)t * E + e] = z;
        }
    }
    __syncthreads();

    router_select<EP, false, TOK_TILE, NTHR>(lg, hist, t0, tile, T, E, K, renorm, ids, wout, tile_counts, probs_out);
}

// FAST mode of bf16 layers with 32 experts or more: the gate projection on the matrix cores.  x and Wg are bf16, so
// every product is exact in fp32 and only the order of the additions differs from the sequential sum (tolerance
// mode by definition).  One workgroup = 32 tokens x EP experts = EP/32 blocks of v_mfma_f32_32x32x16_bf16; its four
// waves split the k range (partial sums are added in a fixed order through LDS) or, from 128 experts on, the blocks.  Operand fragments come straight from memory (16 bytes per lane; the 64 bytes a lane pair
// needs of a row per 32 k are fetched by consecutive loads, so every line is read once): the kernel moves x once
// (Wg stays in the L2) and has almost no arithmetic, it lives on loads in flight.
template <int EP>
__global__ __launch_bounds__(256) void router_mfma_kernel(const bf16_t *__restrict__ x, const bf16_t *__restrict__ Wg,
                                                          const float *__restrict__ bg, int T, int d, int E, int K,
                                                          int renorm, int32_t *__restrict__ ids, float *__restrict__ wout,
                                                          int32_t *__restrict__ tile_counts, float *__restrict__ logits_out,
                                                          float *__restrict__ probs_out)
{
    constexpr int TOK_TILE = 32;                // only layers with more than 16 experts take this kernel
    constexpr int NB = EP / 32;                 // expert blocks
    // up to 64 experts every wave takes all blocks and a quarter of k; from 128 on the waves split the blocks (measured:
    // 64 experts 0.064 -> 0.058 ms with the k split at T = 8192, d = 2048; 128 experts 0.125 -> 0.157 ms at T = 16384)
    constexpr int KS = NB <= 2 ? 4 : 1;         // k splits
    constexpr int BPW = NB <= 2 ? NB : NB / 4;  // expert blocks per wave
    __shared__ float lg[TOK_TILE][EP];
    __shared__ float part[KS > 1 ? KS : 1][KS > 1 ? TOK_TILE : 1][KS > 1 ? EP : 1];
    __shared__ int hist[EP];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tile = blockIdx.x, t0 = tile * TOK_TILE;
    if (tid < EP) hist[tid] = 0;
    const int l32 = lane & 31, kh = lane >> 5;
    const int b0 = KS > 1 ? 0 : wave * BPW;           // first expert block of this wave
    const int ks = KS > 1 ? wave : 0;
    const int klen = d / KS, kbeg = ks * klen;        // d is a multiple of 256
    const bf16_t *xrow = x + (size_t)min(t0 + l32, T - 1) * d + kh * 8;
    const bf16_t *wrow[BPW];
#pragma unroll
    for (int b = 0; b < BPW; ++b) wrow[b] = Wg + (size_t)min((b0 + b) * 32 + l32, E - 1) * d + kh * 8;
    rt_f32x16 acc[BPW];
#pragma unroll
    for (int b = 0; b < BPW; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[b][r] = 0.0f;
    // 64 k per trip: 4 MFMA steps of 16 k; the fragments of the next trip are loaded while this one computes
    rt_bf16x8 xa[2][4], wb[2][BPW][4];
    auto fetch = [&](int buf, int k0) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            xa[buf][q] = *(const rt_bf16x8 *)(xrow + k0 + q * 16);
#pragma unroll
            for (int b = 0; b < BPW; ++b) wb[buf][b][q] = *(const rt_bf16x8 *)(wrow[b] + k0 + q * 16);
        }
    };
    auto compute = [&](int buf) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int b = 0; b < BPW; ++b)
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[buf][q], wb[buf][b][q], acc[b], 0, 0, 0);
    };
    const int kend = kbeg + klen;  // klen is a multiple of 64
    int k0 = kbeg;
    fetch(0, k0);
    for (; k0 + 128 <= kend; k0 += 128) {
        fetch(1, k0 + 64);
        compute(0);
        fetch(0, min(k0 + 128, kend - 64));  // (past the end: re-reads the last trip, never used)
        compute(1);
    }
    if (k0 < kend) compute(0);  // an odd number of trips: the last one sits in buffer 0
    // lane: expert column l32 of its block; register r -> token 8*(r/4) + 4*kh + r%4
#pragma unroll
    for (int b = 0; b < BPW; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int tt = 8 * (r >> 2) + 4 * kh + (r & 3), e = (b0 + b) * 32 + l32;
            if (KS > 1) part[ks][tt][e] = acc[b][r];
            else lg[tt][e] = acc[b][r];
        }
    __syncthreads();
    for (int i = tid; i < TOK_TILE * EP; i += 256) {
        const int tt = i / EP, e = i % EP;
        float z;
        if (KS > 1) {
            z = part[0][tt][e];
#pragma unroll
            for (int q = 1; q < KS; ++q) z = z + part[q][tt][e];
        } else {
            z = lg[tt][e];
        }
        if (bg != nullptr && e < E) z = z + bg[e];
        lg[tt][e] = z;
        if (logits_out != nullptr && t0 + tt < T && e < E) logits_out[(size_t)(t0 + tt) * E + e] = z;
    }
    __syncthreads();
    router_select<EP, true>(lg, hist, t0, tile, T, E, K, renorm, ids, wout, tile_counts, probs_out);
}

// Batches of at most one 16-token tile per compute unit, bf16, at most 16 experts, d a multiple of 512: the whole
// kernel is as long as ONE chain of d dependent multiply-adds (about 6 clocks a term on a SIMD that has no second wave
// to fill them), so everything else is taken out of the waves that run the chains.  The workgroup has two kinds of
// waves: 16*EP/64 sum waves, one lane per (token, expert), that only read LDS and add; and two staging waves that
// carry the NEXT 512-k chunk of x and Wg from memory to a second LDS buffer as fp32 while the current one is summed.
// One barrier per chunk, executed by every wave of both kinds (B_c: chunk c is staged, and chunk c-1 is summed - so
// its buffer may take chunk c+1).  The terms are the exact fp32 products of bf16 operands, added in k order by
// fused multiply-adds: the same bits as the separate multiply and add of the sequential sum, in either router mode.
#define RP_KC 512
#define RP_LDW (RP_KC + 4)
#define RP_STAGERS 128
template <int EP>
__global__ __launch_bounds__(16 * EP + RP_STAGERS) void router_pipe_kernel(
    const bf16_t *__restrict__ x, const bf16_t *__restrict__ Wg, const float *__restrict__ bg, int T, int d, int E, int K,
    int renorm, int32_t *__restrict__ ids, float *__restrict__ wout, int32_t *__restrict__ tile_counts,
    float *__restrict__ logits_out, float *__restrict__ probs_out)
{
    constexpr int TT = 16, CT = 16 * EP, ST = RP_STAGERS, KC = RP_KC, LDW = RP_LDW;
    extern __shared__ __attribute__((aligned(16))) float rp_smem[];
    float(*xs)[TT][LDW] = (float(*)[TT][LDW])rp_smem;                  // [2][TT][LDW]
    float(*ws)[EP][LDW] = (float(*)[EP][LDW])(rp_smem + 2 * TT * LDW);  // [2][EP][LDW]
    __shared__ float lg[TT][EP];
    __shared__ int hist[EP];
    const int tid = threadIdx.x, tile = blockIdx.x, t0 = tile * TT;
    if (tid < EP) hist[tid] = 0;
    const int nch = d / KC;
    if (tid >= CT) {
        // staging wave: thread st carries 8 consecutive k (16 bytes of bf16) of one row per load
        const int st = tid - CT;
        constexpr int XCH = TT * (KC / 8) / ST, WCH = EP * (KC / 8) / ST;
        static_assert(TT * (KC / 8) % ST == 0 && EP * (KC / 8) % ST == 0, "whole vectors per staging thread");
        // (a second chunk of loads in flight gained nothing: the sum waves, bound by their LDS reads, set the pace)
        uint4 xr[XCH], wr[WCH];
        auto fetch = [&](int k0) {
#pragma unroll
            for (int c = 0; c < XCH; ++c) {
                const int idx = st + c * ST;
                xr[c] = *(const uint4 *)(x + (size_t)min(t0 + idx / (KC / 8), T - 1) * d + k0 + (idx % (KC / 8)) * 8);
            }
#pragma unroll
            for (int c = 0; c < WCH; ++c) {
                const int idx = st + c * ST;
                wr[c] = *(const uint4 *)(Wg + (size_t)min(idx / (KC / 8), E - 1) * d + k0 + (idx % (KC / 8)) * 8);
            }
        };
        auto widen = [&](const uint4 &v, float *dst) {
            *(float4 *)dst = make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u),
                                         __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u));
            *(float4 *)(dst + 4) = make_float4(__uint_as_float(v.z << 16), __uint_as_float(v.z & 0xffff0000u),
                                               __uint_as_float(v.w << 16), __uint_as_float(v.w & 0xffff0000u));
        };
        fetch(0);
        for (int c = 0; c < nch; ++c) {
            const int b = c & 1;
#pragma unroll
            for (int q = 0; q < XCH; ++q) {
                const int idx = st + q * ST;
                widen(xr[q], &xs[b][idx / (KC / 8)][(idx % (KC / 8)) * 8]);
            }
#pragma unroll
            for (int q = 0; q < WCH; ++q) {
                const int idx = st + q * ST;
                widen(wr[q], &ws[b][idx / (KC / 8)][(idx % (KC / 8)) * 8]);
            }
            if (c + 1 < nch) fetch((c + 1) * KC);
            __syncthreads();  // B_c
        }
    } else {
        const int e1 = tid % EP, tg = tid / EP;
        // a wave whose lowest token is past the end of the batch forms no sum; it keeps the barriers
        const bool wave_live = t0 + (tid & ~63) / EP < T;
        float a_ = 0.0f;
        for (int c = 0; c < nch; ++c) {
            __syncthreads();  // B_c
            if (!wave_live) continue;
            const float4 *wp = (const float4 *)&ws[c & 1][e1][0], *xp = (const float4 *)&xs[c & 1][tg][0];
            float4 wa[8], xa[8], wb[8], xb[8];
#define ROUTER_LD(W, X, g)                                    \
    _Pragma("unroll") for (int j = 0; j < 8; ++j)             \
    {                                                         \
        W[j] = wp[(g) * 8 + j];                               \
        X[j] = xp[(g) * 8 + j];                               \
    }
#define ROUTER_FM(W, X)                                       \
    _Pragma("unroll") for (int j = 0; j < 8; ++j)             \
    {                                                         \
        a_ = fmaf(X[j].x, W[j].x, a_);                        \
        a_ = fmaf(X[j].y, W[j].y, a_);                        \
        a_ = fmaf(X[j].z, W[j].z, a_);                        \
        a_ = fmaf(X[j].w, W[j].w, a_);                        \
    }
            // the LDS reads of the next 32 k are in flight while the terms of the current 32 are added (the fences
            // keep the reads where they are written: ahead of the other set's terms)
            ROUTER_LD(wa, xa, 0)
            for (int g = 0; g < KC / 32; g += 2) {
                __builtin_amdgcn_sched_barrier(0);
                ROUTER_LD(wb, xb, g + 1)
                __builtin_amdgcn_sched_barrier(0);
                ROUTER_FM(wa, xa)
                __builtin_amdgcn_sched_barrier(0);
                if (g + 2 < KC / 32) {
                    ROUTER_LD(wa, xa, g + 2)
                }
                __builtin_amdgcn_sched_barrier(0);
                ROUTER_FM(wb, xb)
            }
#undef ROUTER_LD
#undef ROUTER_FM
        }
        const float z = (bg != nullptr && e1 < E) ? a_ + bg[e1] : a_;
        lg[tg][e1] = z;
        if (logits_out != nullptr && t0 + tg < T && e1 < E) logits_out[(size_t)(t0 + tg) * E + e1] = z;
    }
    __syncthreads();
    if (tid < CT) {
        router_select<EP, false, TT, CT>(lg, hist, t0, tile, T, E, K, renorm, ids, wout, tile_counts, probs_out);
    } else {
        __syncthreads();  // the staging waves keep the two barriers of the selection
        __syncthreads();
    }
}

int router_pipe_smem_bytes(int EP) { return 2 * (16 + EP) * RP_LDW * (int)sizeof(float); }

hipError_t router_init(void)
{
    hipError_t e = hipFuncSetAttribute((const void *)router_pipe_kernel<8>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       router_pipe_smem_bytes(8));
    if (e == hipSuccess)
        e = hipFuncSetAttribute((const void *)router_pipe_kernel<16>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                router_pipe_smem_bytes(16));
    return e;
}

hipError_t launch_router(const omega_moe *m, const void *x, int T, float *logits_out, float *probs_out, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const int tiles = ceil_div(T, router_tok_tile(c.E));
    const int exact = c.router_mode == OMEGA_ROUTER_EXACT;
    const float *bg = c.has_gate_bias ? m->bg : nullptr;
    if (!exact && c.dtype == OMEGA_DTYPE_BF16 && c.E > 16 && ((uintptr_t)x % 16) == 0) {
#define ROUTER_MFMA_LAUNCH(EPV)                                                                                          \
    hipLaunchKernelGGL(router_mfma_kernel<EPV>, dim3(tiles), dim3(256), 0, s, (const bf16_t *)x, (const bf16_t *)m->Wg, bg, T, \
                       c.d, c.E, c.K, c.renorm, m->ids, m->w, m->tile_counts, logits_out, probs_out)
        if (c.E <= 32) ROUTER_MFMA_LAUNCH(32);
        else if (c.E <= 64) ROUTER_MFMA_LAUNCH(64);
        else if (c.E <= 128) ROUTER_MFMA_LAUNCH(128);
        else ROUTER_MFMA_LAUNCH(256);
#undef ROUTER_MFMA_LAUNCH
        return hipGetLastError();
    }
    // at most 16 experts, bf16, at most one tile per compute unit: chains fed by staging waves (either mode: same bits)
    if (c.dtype == OMEGA_DTYPE_BF16 && c.E <= 16 && tiles <= m->ctx->num_cus && c.d % RP_KC == 0 &&
        (((uintptr_t)x | (uintptr_t)m->Wg) % 16) == 0) {
        if (c.E <= 8)
            hipLaunchKernelGGL(router_pipe_kernel<8>, dim3(tiles), dim3(16 * 8 + RP_STAGERS), router_pipe_smem_bytes(8), s,
                               (const bf16_t *)x, (const bf16_t *)m->Wg, bg, T, c.d, c.E, c.K, c.renorm, m->ids, m->w,
                               m->tile_counts, logits_out, probs_out);
        else
            hipLaunchKernelGGL(router_pipe_kernel<16>, dim3(tiles), dim3(16 * 16 + RP_STAGERS), router_pipe_smem_bytes(16), s,
                               (const bf16_t *)x, (const bf16_t *)m->Wg, bg, T, c.d, c.E, c.K, c.renorm, m->ids, m->w,
                               m->tile_counts, logits_out, probs_out);
        return hipGetLastError();
    }
    // exact sums of bf16 layers with more than 16 experts: on the matrix cores, one k per instruction
    const bool exact_mfma = exact && c.dtype == OMEGA_DTYPE_BF16 && c.E > 16;
#define ROUTER_LAUNCH(EPV, KCV)                                                                                    \
    do {                                                                                                           \
        if (exact_mfma)                                                                                            \
            hipLaunchKernelGGL((router_kernel<EPV, KCV, true, (EPV > 16)>), dim3(tiles), dim3(ROUTER_NTHR(EPV)), 0, s, x, c.dtype, m->Wg, bg, \
                               T, c.d, c.E, c.K, c.renorm, m->ids, m->w, m->tile_counts, logits_out, probs_out);   \
        else if (exact)                                                                                            \
            hipLaunchKernelGGL((router_kernel<EPV, KCV, true>), dim3(tiles), dim3(ROUTER_NTHR(EPV)), 0, s, x, c.dtype, m->Wg, bg, \
                               T, c.d, c.E, c.K, c.renorm, m->ids, m->w, m->tile_counts, logits_out, probs_out);   \
        else                                                                                                       \
            hipLaunchKernelGGL((router_kernel<EPV, KCV, false>), dim3(tiles), dim3(ROUTER_NTHR(EPV)), 0, s, x, c.dtype, m->Wg,    \
                               bg, T, c.d, c.E, c.K, c.renorm, m->ids, m->w, m->tile_counts, logits_out,           \
                               probs_out);                                                                         \
    } while (0)
    if (c.E <= 8) ROUTER_LAUNCH(8, ROUTER_KC_SMALL);
    else if (c.E <= 16) ROUTER_LAUNCH(16, ROUTER_KC_SMALL);
    else if (c.E <= 32) ROUTER_LAUNCH(32, 128);
    else if (c.E <= 64) ROUTER_LAUNCH(64, 64);
    else if (c.E <= 128) ROUTER_LAUNCH(128, 64);
    else ROUTER_LAUNCH(256, 64);
#undef ROUTER_LAUNCH
    return hipGetLastError();
}
