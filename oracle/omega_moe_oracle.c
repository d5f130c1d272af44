/*
 * CPU oracle for the mixture-of-experts forward path.  TEST INFRASTRUCTURE ONLY:
 * nothing in the shipped library links, loads or calls this file; it exists so that
 * tests, the smoke check and the benchmark's cpu_baseline leg can check the HIP path.
 *
 * Every function restates, in plain sequential C, the arithmetic of the reference
 * primitive it cites (paths relative to the reference checkout,
 * J/ = src/main/java/com/omega/).  The reference has no mixture-of-experts layer; the
 * routing steps that have no reference primitive (top-k, dispatch, combine) follow the
 * frozen composition described beside each function.
 *
 * Pinning status (what independent check covers each function; see tests/test_oracle_*.py):
 *   orc_fill_normal      NumPy twin bit-exact + moments / KS distance        (pinned)
 *   orc_gate             fp64 matmul cross-check, all-ones closed form        (pinned to tolerance;
 *                        the reference's cuBLAS sgemm summation order cannot be reproduced:
 *                        GEMM bits are "parity unpinned", tolerance only)
 *   orc_softmax          NumPy twin written from the kernel text, sum-to-one, shift invariance (pinned)
 *   orc_topk             stable argsort brute force, tie cases                (pinned)
 *   orc_dispatch         stable argsort brute force, bijection / stability invariants (pinned)
 *   orc_swiglu_rows      fp64 cross-check, SiLU closed forms                  (pinned to tolerance; GEMM bits unpinned as above)
 *   orc_combine / orc_moe_forward   dense-MoE identity in fp64                (pinned)
 *   orc_rmsnorm          NumPy twin written from the kernel text (bit-exact), closed forms (all-ones row,
 *                        scale invariance), fp64 formula to 1e-6 (pinned, except the order of the five
 *                        additions inside cooperative_groups::reduce, which is library code outside the
 *                        reference tree: taken as the xor butterfly, "parity unpinned" at the ulp level)
 *   orc_block_tokens / orc_block_forward   residual identity out - x == layer(rmsnorm(x)) (pinned by composition)
 *
 * Build: make -C oracle   (gcc -O2 -ffp-contract=off; no fast-math, so every float
 * operation below is a single IEEE-754 rounding in the order written).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "oracle_common.h"

/* ------------------------------------------------------------------------------------------
 * Seeded synthetic data: counter-based SplitMix64 + Box-Muller written with +,-,*,/,sqrt only,
 * so that C, NumPy and the device generator agree bit for bit.
 * element i of stream s under seed:  key = mix(seed ^ mix(s*GAMMA2 + 1));
 *   h1 = mix(key + GAMMA*(2i+1)), h2 = mix(key + GAMMA*(2i+2))
 *   u  = ((h1>>11)+1) * 2^-53  in (0,1];  r = sqrt(-2 ln u)
 *   th = ((h2>>8)&(2^53-1)) * 2^-53 * pi/4; trig = bit62(h2) ? sin th : cos th; sign = bit63(h2)
 *   value = (float)( (+-) r * trig * std )
 * ------------------------------------------------------------------------------------------ */
#define GAMMA  0x9E3779B97F4A7C15ULL
#define GAMMA2 0xD1342543DE82EF95ULL

static uint64_t mix64(uint64_t z)
{
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

uint64_t orc_stream_key(uint64_t seed, uint64_t stream)
{
    return mix64(seed ^ mix64(stream * GAMMA2 + 1ULL));
}

static const double INV_ODD[11] = {
    0x1.0000000000000p+0, 0x1.5555555555555p-2, 0x1.999999999999ap-3, 0x1.2492492492492p-3,
    0x1.c71c71c71c71cp-4, 0x1.745d1745d1746p-4, 0x1.3b13b13b13b14p-4, 0x1.1111111111111p-4,
    0x1.e1e1e1e1e1e1ep-5, 0x1.af286bca1af28p-5, 0x1.8618618618618p-5};
static const double INV_FACT[21] = {
    0x1.0000000000000p+0,  0x1.0000000000000p+0,  0x1.0000000000000p-1,  0x1.5555555555555p-3,
    0x1.5555555555555p-5,  0x1.1111111111111p-7,  0x1.6c16c16c16c17p-10, 0x1.a01a01a01a01ap-13,
    0x1.a01a01a01a01ap-16, 0x1.71de3a556c734p-19, 0x1.27e4fb7789f5cp-22, 0x1.ae64567f544e4p-26,
    0x1.1eed8eff8d898p-29, 0x1.6124613a86d09p-33, 0x1.93974a8c07c9dp-37, 0x1.ae7f3e733b81fp-41,
    0x1.ae7f3e733b81fp-45, 0x1.952c77030ad4ap-49, 0x1.6827863b97d97p-53, 0x1.2f49b46814157p-57,
    0x1.e542ba4020225p-62};
#define LN2_D   0x1.62e42fefa39efp-1
#define PI_4_D  0x1.921fb54442d18p-1
#define SQRT_HALF_D 0x1.6a09e667f3bcdp-1
#define TWO_M53 0x1.0p-53

/* ln(u) for u in (0,1]: u = m*2^e, m in [sqrt(1/2), sqrt(2)); ln m = 2 atanh((m-1)/(m+1)). */
static double det_log(double u)
{
    int e;
    double m = frexp(u, &e); /* exact: m in [0.5,1) */
    if (m < SQRT_HALF_D) { m = m * 2.0; e -= 1; }
    double s = (m - 1.0) / (m + 1.0);
    double s2 = s * s;
    double p = INV_ODD[10];
    for (int k = 9; k >= 0; --k) p = p * s2 + INV_ODD[k];
    return (double)e * LN2_D + 2.0 * s * p;
}

static void det_sincos(double th, double *sn, double *cs)
{
    double t2 = th * th;
    /* cos: sum_{k=0..9} (-1)^k t^(2k)/(2k)!  ; sin: t * sum_{k=0..9} (-1)^k t^(2k)/(2k+1)! */
    double c = INV_FACT[18];
    double s = INV_FACT[19];
    for (int k = 8; k >= 0; --k) {
        c = INV_FACT[2 * k] - t2 * c;
        s = INV_FACT[2 * k + 1] - t2 * s;
    }
    *cs = c;
    *sn = th * s;
}

static float normal_at(uint64_t key, uint64_t i, double std)
{
    uint64_t h1 = mix64(key + GAMMA * (2ULL * i + 1ULL));
    uint64_t h2 = mix64(key + GAMMA * (2ULL * i + 2ULL));
    double u = (double)((h1 >> 11) + 1ULL) * TWO_M53;
    double r = sqrt(-2.0 * det_log(u));
    double th = (double)((h2 >> 8) & ((1ULL << 53) - 1ULL)) * TWO_M53 * PI_4_D;
    double sn, cs;
    det_sincos(th, &sn, &cs);
    double z = r * (((h2 >> 62) & 1ULL) ? sn : cs);
    if ((h2 >> 63) & 1ULL) z = -z;
    return (float)(z * std);
}

/* out[j] = N(0,std) element (first+j) of stream `stream`. */
void orc_fill_normal(float *out, uint64_t n, uint64_t seed, uint64_t stream, double std, uint64_t first)
{
    uint64_t key = orc_stream_key(seed, stream);
    for (uint64_t j = 0; j < n; ++j) out[j] = normal_at(key, first + j, std);
}

void orc_round_bf16(float *buf, uint64_t n)
{
    for (uint64_t i = 0; i < n; ++i) buf[i] = bf16_round(buf[i]);
}

/* ------------------------------------------------------------------------------------------
 * S1 gate: logit[t,e] = sum_k x[t,k]*Wg[e,k] (+ bg[e]).
 * Layout W[out,in], y = x W^T + b: J/engine/nn/layer/FullyLayer.java:181,232-243.
 * Summation order: sequential k with separate multiply and add, as the reference's CPU dot
 * J/common/utils/MatrixOperation.java:1472-1478.
 * ------------------------------------------------------------------------------------------ */
void orc_gate(const float *x, const float *Wg, const float *bg, int T, int d, int E, float *logits)
{
    for (int t = 0; t < T; ++t)
        for (int e = 0; e < E; ++e) {
            float acc = 0.0f;
            const float *xr = x + (size_t)t * d, *wr = Wg + (size_t)e * d;
            for (int k = 0; k < d; ++k) {
                float prod = xr[k] * wr[k];
                acc = acc + prod;
            }
            if (bg) acc = acc + bg[e];
            logits[(size_t)t * E + e] = acc;
        }
}

/* S2 softmax: three sequential passes per row, max scanned with <=, exponent evaluated in
 * double and narrowed, sum in index order, then divide.
 * J/engine/gpu/SoftmaxKernel.cu:4-24 and its CPU twin J/engine/gpu/SoftmaxKernel.java:69-87. */
void orc_softmax(const float *logits, int T, int E, float *p)
{
    for (int t = 0; t < T; ++t) {
        const float *in = logits + (size_t)t * E;
        float *out = p + (size_t)t * E;
        float mx = -3.402823466e+38F, sum = 0.0f;
        for (int i = 0; i < E; ++i)
            if (mx <= in[i]) mx = in[i];
        for (int i = 0; i < E; ++i) {
            float e = (float)exp((double)(in[i] - mx));
            sum += e;
            out[i] = e;
        }
        for (int i = 0; i < E; ++i) out[i] /= sum;
    }
}

/* S3 + S4 top-k: K rounds of arg-max over the probabilities with a strict '>' scan from
 * expert 0 upward (ties go to the lowest expert index), chosen experts excluded from later
 * rounds; slot j holds the j-th selection.  Optional renormalisation divides each weight by
 * the slot-order sum.  No reference primitive exists for this step. */
void orc_topk(const float *p, int T, int E, int K, int renorm, int32_t *ids, float *w)
{
    unsigned char *taken = (unsigned char *)malloc((size_t)E);
    for (int t = 0; t < T; ++t) {
        const float *pr = p + (size_t)t * E;
        memset(taken, 0, (size_t)E);
        for (int j = 0; j < K; ++j) {
            int best = -1;
            float bv = 0.0f;
            for (int e = 0; e < E; ++e) {
                if (taken[e]) continue;
                if (best < 0 || pr[e] > bv) { best = e; bv = pr[e]; }
            }
            taken[best] = 1;
            ids[(size_t)t * K + j] = best;
            w[(size_t)t * K + j] = bv;
        }
        if (renorm) {
            float s = 0.0f;
            for (int j = 0; j < K; ++j) s += w[(size_t)t * K + j];
            for (int j = 0; j < K; ++j) w[(size_t)t * K + j] /= s;
        }
    }
    free(taken);
}

/* S5 dispatch: pair p = t*K+j; counts per expert, exclusive scan, stable destination
 * dst[p] = off[id_p] + #{q<p : id_q == id_p}; src_row[dst[p]] = t.
 * offsets has E+1 entries (offsets[E] = T*K). */
void orc_dispatch(const int32_t *ids, int T, int K, int E, int32_t *counts, int32_t *offsets,
                  int32_t *dst, int32_t *src_row)
{
    int P = T * K;
    memset(counts, 0, sizeof(int32_t) * (size_t)E);
    for (int p = 0; p < P; ++p) counts[ids[p]]++;
    offsets[0] = 0;
    for (int e = 0; e < E; ++e) offsets[e + 1] = offsets[e] + counts[e];
    int32_t *cur = (int32_t *)malloc(sizeof(int32_t) * (size_t)E);
    memcpy(cur, offsets, sizeof(int32_t) * (size_t)E);
    for (int p = 0; p < P; ++p) {
        int r = cur[ids[p]]++;
        dst[p] = r;
        src_row[r] = p / K;
    }
    free(cur);
}

/* Row gather xg[r,:] = x[src_row[r],:]; index semantics as img_token_drop,
 * J/engine/nn/layer/dit/kernel/TokenDropKernel.cu:147-160. */
void orc_gather(const float *x, const int32_t *src_row, int P, int d, float *xg)
{
    for (int r = 0; r < P; ++r) memcpy(xg + (size_t)r * d, x + (size_t)src_row[r] * d, sizeof(float) * (size_t)d);
}

/* S6 expert body for `rows` rows that all belong to one expert:
 * h1 = xg W1^T, h3 = xg W3^T, a = silu(h1)*h3, y = a W2^T
 * (J/engine/nn/layer/llama/LlamaMLPLayer.java:117-130; product J/engine/ad/op/gpu/OPKernel.cu:1103-1110).
 * W1,W3: [H,d]; W2: [d,H].  bf16_mode rounds `a` to bf16 before the second product.
 * scratch must hold H floats. */
void orc_swiglu_rows(const float *xg, int rows, const float *W1, const float *W3, const float *W2, int d,
                     int H, int bf16_mode, float *y, float *scratch)
{
    for (int r = 0; r < rows; ++r) {
        const float *xr = xg + (size_t)r * d;
        for (int h = 0; h < H; ++h) {
            const float *w1 = W1 + (size_t)h * d, *w3 = W3 + (size_t)h * d;
            float a1 = 0.0f, a3 = 0.0f;
            for (int k = 0; k < d; ++k) {
                float p1 = xr[k] * w1[k];
                a1 = a1 + p1;
                float p3 = xr[k] * w3[k];
                a3 = a3 + p3;
            }
            float a = silu_f(a1) * a3;
            scratch[h] = bf16_mode ? bf16_round(a) : a;
        }
        for (int c = 0; c < d; ++c) {
            const float *w2 = W2 + (size_t)c * H;
            float acc = 0.0f;
            for (int h = 0; h < H; ++h) {
                float pr = scratch[h] * w2[h];
                acc = acc + pr;
            }
            y[(size_t)r * d + c] = acc;
        }
    }
}

/* S7 combine: out[t,:] = sum_j w[t,j]*y[dst[t*K+j],:] in slot order (weighted sum shaped like
 * add_mul_kernel, J/engine/gpu/BaseKernel.cu:228-241), then + shared-expert rows
 * (add: J/engine/ad/op/gpu/OPKernel.cu:359-366).  yshared may be NULL; it is [Es,T,d]. */
void orc_combine_resid(const float *y, const int32_t *dst, const float *w, const float *yshared, const float *resid,
                       int T, int K, int d, int Es, int bf16_mode, float *out)
{
    for (int t = 0; t < T; ++t)
        for (int c = 0; c < d; ++c) {
            float acc = 0.0f;
            for (int j = 0; j < K; ++j) {
                float term = w[(size_t)t * K + j] * y[(size_t)dst[(size_t)t * K + j] * d + c];
                acc = acc + term;
            }
            for (int s = 0; s < Es; ++s) acc = acc + yshared[((size_t)s * T + t) * d + c];
            /* block form: the residual is added to the fp32 sum before the one rounding of the output
             * (Tensor_OP().add(mlp_out, tmp1, tmp2), J/engine/nn/layer/llama/LlamaTransformerBlock.java:136;
             * add_kernel, J/engine/ad/op/gpu/OPKernel.cu:359-366) */
            if (resid) acc = acc + resid[(size_t)t * d + c];
            out[(size_t)t * d + c] = bf16_mode ? bf16_round(acc) : acc;
        }
}

void orc_combine(const float *y, const int32_t *dst, const float *w, const float *yshared, int T, int K, int d,
                 int Es, int bf16_mode, float *out)
{
    orc_combine_resid(y, dst, w, yshared, NULL, T, K, d, Es, bf16_mode, out);
}

/* Pre-norm of the block: rmsnorm_forward_kernel2 (J/engine/nn/layer/normalization/gpu/RMSKernel.cu:185-223), the
 * kernel RMSLayer.output runs (J/engine/nn/layer/normalization/RMSLayer.java:230 -> RMSKernel.java:232-249).
 * One 32-lane group per row: lane l adds x[i]*x[i] for i = l, l+32, ... in index order (written
 * `sum_squares += x[i] * x[i]`, one fused multiply-add per step under nvcc's default contraction); the 32 partial
 * sums are combined by cooperative_groups::reduce(warp, ., plus), taken here as the xor butterfly with strides
 * 16, 8, 4, 2, 1; rms = sqrtf(sum / C + 1e-6f); out[c] = (x[c] / rms) * weight[c].
 * bf16 mode: the normalised row is rounded to bf16 (the activation storage type).  rms_o may be NULL. */
void orc_rmsnorm(const float *x, const float *gamma, int T, int d, int bf16_mode, float *h, float *rms_o)
{
    for (int t = 0; t < T; ++t) {
        const float *xr = x + (size_t)t * d;
        float part[32];
        for (int l = 0; l < 32; ++l) {
            float s = 0.0f;
            for (int i = l; i < d; i += 32) s = fmaf(xr[i], xr[i], s);
            part[l] = s;
        }
        for (int m = 16; m >= 1; m >>= 1) {
            float nxt[32];
            for (int l = 0; l < 32; ++l) nxt[l] = part[l] + part[l ^ m];
            memcpy(part, nxt, sizeof(part));
        }
        float rms = sqrtf(part[0] / (float)d + 1e-6f);
        if (rms_o) rms_o[t] = rms;
        for (int c = 0; c < d; ++c) {
            float n = xr[c] / rms;
            float v = n * gamma[c];
            h[(size_t)t * d + c] = bf16_mode ? bf16_round(v) : v;
        }
    }
}

/* Whole layer for a subset of tokens (tok_list, n_tok) of a T-token batch whose routing
 * (ids, w over all T tokens) is already known: used to check full-size runs on a sample.
 * W1,W3,W2 hold E+Es experts back to back.  out is [n_tok, d]. */
static void moe_tokens_impl(const float *x, const float *resid, const int32_t *ids, const float *w, const float *W1,
                            const float *W3, const float *W2, int d, int H, int E, int K, int Es, int bf16_mode,
                            const int32_t *tok_list, int n_tok, float *out)
{
    float *scratch = (float *)malloc(sizeof(float) * (size_t)H);
    float *yk = (float *)malloc(sizeof(float) * (size_t)d * (size_t)(K + Es));
    for (int i = 0; i < n_tok; ++i) {
        int t = tok_list[i];
        const float *xr = x + (size_t)t * d;
        for (int j = 0; j < K + Es; ++j) {
            int e = j < K ? ids[(size_t)t * K + j] : E + (j - K);
            orc_swiglu_rows(xr, 1, W1 + (size_t)e * H * d, W3 + (size_t)e * H * d, W2 + (size_t)e * d * H, d, H,
                            bf16_mode, yk + (size_t)j * d, scratch);
        }
        for (int c = 0; c < d; ++c) {
            float acc = 0.0f;
            for (int j = 0; j < K; ++j) {
                float term = w[(size_t)t * K + j] * yk[(size_t)j * d + c];
                acc = acc + term;
            }
            for (int s = 0; s < Es; ++s) acc = acc + yk[(size_t)(K + s) * d + c];
            if (resid) acc = acc + resid[(size_t)t * d + c];
            out[(size_t)i * d + c] = bf16_mode ? bf16_round(acc) : acc;
        }
    }
    free(scratch);
    free(yk);
}

void orc_moe_tokens(const float *x, const int32_t *ids, const float *w, const float *W1, const float *W3,
                    const float *W2, int d, int H, int E, int K, int Es, int bf16_mode, const int32_t *tok_list,
                    int n_tok, float *out)
{
    moe_tokens_impl(x, NULL, ids, w, W1, W3, W2, d, H, E, K, Es, bf16_mode, tok_list, n_tok, out);
}

/* Block form for a subset of tokens: the layer runs on h = rmsnorm(x) (rows of h for all T tokens, as the routing
 * ids/w were computed from them) and x is added back: out = x + layer(h)
 * (getNorm2().forward(tmp1); getMlp().forward(norm2 out); add(mlp out, tmp1), LlamaTransformerBlock.java:134-136). */
void orc_block_tokens(const float *x, const float *h, const int32_t *ids, const float *w, const float *W1,
                      const float *W3, const float *W2, int d, int H, int E, int K, int Es, int bf16_mode,
                      const int32_t *tok_list, int n_tok, float *out)
{
    moe_tokens_impl(h, x, ids, w, W1, W3, W2, d, H, E, K, Es, bf16_mode, tok_list, n_tok, out);
}

/* Whole layer, all tokens, through the materialised dispatch (S1..S7). Outputs every
 * intermediate the parity tests compare.  Any output pointer except `out` may be NULL. */
static void moe_forward_impl(const float *x, const float *resid, const float *Wg, const float *bg, const float *W1,
                             const float *W3, const float *W2, int T, int d, int E, int K, int H, int Es, int renorm,
                             int bf16_mode, float *logits_o, float *p_o, int32_t *ids_o, float *w_o,
                             int32_t *counts_o, int32_t *offsets_o, int32_t *dst_o, int32_t *src_row_o, float *out)
{
    int P = T * K;
    float *logits = (float *)malloc(sizeof(float) * (size_t)T * E);
    float *p = (float *)malloc(sizeof(float) * (size_t)T * E);
    int32_t *ids = (int32_t *)malloc(sizeof(int32_t) * (size_t)P);
    float *w = (float *)malloc(sizeof(float) * (size_t)P);
    int32_t *counts = (int32_t *)malloc(sizeof(int32_t) * (size_t)E);
    int32_t *offsets = (int32_t *)malloc(sizeof(int32_t) * (size_t)(E + 1));
    int32_t *dst = (int32_t *)malloc(sizeof(int32_t) * (size_t)P);
    int32_t *src_row = (int32_t *)malloc(sizeof(int32_t) * (size_t)P);
    float *xg = (float *)malloc(sizeof(float) * (size_t)P * d);
    float *y = (float *)malloc(sizeof(float) * (size_t)P * d);
    float *ysh = Es ? (float *)malloc(sizeof(float) * (size_t)Es * T * d) : NULL;
    float *scratch = (float *)malloc(sizeof(float) * (size_t)H);

    orc_gate(x, Wg, bg, T, d, E, logits);
    orc_softmax(logits, T, E, p);
    orc_topk(p, T, E, K, renorm, ids, w);
    orc_dispatch(ids, T, K, E, counts, offsets, dst, src_row);
    orc_gather(x, src_row, P, d, xg);
    for (int e = 0; e < E; ++e)
        orc_swiglu_rows(xg + (size_t)offsets[e] * d, counts[e], W1 + (size_t)e * H * d, W3 + (size_t)e * H * d,
                        W2 + (size_t)e * d * H, d, H, bf16_mode, y + (size_t)offsets[e] * d, scratch);
    for (int s = 0; s < Es; ++s)
        orc_swiglu_rows(x, T, W1 + (size_t)(E + s) * H * d, W3 + (size_t)(E + s) * H * d,
                        W2 + (size_t)(E + s) * d * H, d, H, bf16_mode, ysh + (size_t)s * T * d, scratch);
    orc_combine_resid(y, dst, w, ysh, resid, T, K, d, Es, bf16_mode, out);

    if (logits_o) memcpy(logits_o, logits, sizeof(float) * (size_t)T * E);
    if (p_o) memcpy(p_o, p, sizeof(float) * (size_t)T * E);
    if (ids_o) memcpy(ids_o, ids, sizeof(int32_t) * (size_t)P);
    if (w_o) memcpy(w_o, w, sizeof(float) * (size_t)P);
    if (counts_o) memcpy(counts_o, counts, sizeof(int32_t) * (size_t)E);
    if (offsets_o) memcpy(offsets_o, offsets, sizeof(int32_t) * (size_t)(E + 1));
    if (dst_o) memcpy(dst_o, dst, sizeof(int32_t) * (size_t)P);
    if (src_row_o) memcpy(src_row_o, src_row, sizeof(int32_t) * (size_t)P);
    free(logits); free(p); free(ids); free(w); free(counts); free(offsets); free(dst); free(src_row);
    free(xg); free(y); free(ysh); free(scratch);
}

void orc_moe_forward(const float *x, const float *Wg, const float *bg, const float *W1, const float *W3,
                     const float *W2, int T, int d, int E, int K, int H, int Es, int renorm, int bf16_mode,
                     float *logits_o, float *p_o, int32_t *ids_o, float *w_o, int32_t *counts_o,
                     int32_t *offsets_o, int32_t *dst_o, int32_t *src_row_o, float *out)
{
    moe_forward_impl(x, NULL, Wg, bg, W1, W3, W2, T, d, E, K, H, Es, renorm, bf16_mode, logits_o, p_o, ids_o, w_o,
                     counts_o, offsets_o, dst_o, src_row_o, out);
}

/* Block form, all tokens: h = rmsnorm(x) (returned in h_o, [T,d]; rms in rms_o, may be NULL), the layer on h,
 * out = x + layer(h)  (LlamaTransformerBlock.java:134-136). */
void orc_block_forward(const float *x, const float *gamma, const float *Wg, const float *bg, const float *W1,
                       const float *W3, const float *W2, int T, int d, int E, int K, int H, int Es, int renorm,
                       int bf16_mode, float *h_o, float *rms_o, float *logits_o, float *p_o, int32_t *ids_o,
                       float *w_o, int32_t *counts_o, int32_t *offsets_o, int32_t *dst_o, int32_t *src_row_o,
                       float *out)
{
    orc_rmsnorm(x, gamma, T, d, bf16_mode, h_o, rms_o);
    moe_forward_impl(h_o, x, Wg, bg, W1, W3, W2, T, d, E, K, H, Es, renorm, bf16_mode, logits_o, p_o, ids_o, w_o,
                     counts_o, offsets_o, dst_o, src_row_o, out);
}
