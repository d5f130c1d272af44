/*
 * CPU oracle for the backward pass of the mixture-of-experts layer.  TEST INFRASTRUCTURE ONLY (see
 * omega_moe_oracle.c): nothing in the shipped library links, loads or calls this file.
 *
 * The reference has no mixture-of-experts layer; the backward pass composes the backward steps of the primitives the
 * forward pass is built from (paths relative to the reference checkout, J/ = src/main/java/com/omega/):
 *   linear layer       diffW = delta^T . input (overwritten, beta = 0), diff = delta . W, diffB = column sums of delta
 *                      (FullyLayer.diff, J/engine/nn/layer/FullyLayer.java:292-334)
 *   SwiGLU wiring      w2 back; dh3 = d(a) * silu(h1); dh1 = silu'(h1) applied to d(a) * h3; input gradient =
 *                      w1's + w3's (LlamaMLPLayer.diff, J/engine/nn/layer/llama/LlamaMLPLayer.java:139-158)
 *   SiLU               diff = delta * s * (1 + x * (1 - s)), s = 1/(1+exp(-x))
 *                      (silu_backward, J/engine/nn/layer/active/gpu/activeFunction.cu:182-190)
 *   softmax            sum = sum_e out*delta; diff = (delta - sum) * out   (softmax_back, J/engine/gpu/SoftmaxKernel.cu:101-112)
 * The routing (expert ids, dispatch permutation) is piecewise constant and carries no gradient; the gate weights get
 * theirs through the combine weights: combine -> (renormalisation) -> selected probabilities -> softmax -> gate.
 *
 * bf16 mode (build-defined, the reference is fp32 only): x, dout and the weights arrive rounded; every sum is fp32;
 * the row gradients that feed a matrix product are rounded to bf16 first (dy = w*dout, dh1, dh3), `a` as in the
 * forward pass; dx is rounded once at the end; weight gradients stay fp32.
 *
 * Pinning status:
 *   orc_moe_backward   torch float64 autograd of the dense formulation with the routing held fixed, and central
 *                      finite differences of an independent float64 NumPy forward (pinned to tolerance; the
 *                      summation order of the reference's cuBLAS products cannot be reproduced: bits "parity unpinned")
 *   orc_moe_backward_routed   the same code path with the routing passed in: equals orc_moe_backward on the same tokens
 *                      when given its routing (pinned by that identity)
 *   orc_rmsnorm_backward / orc_block_backward   torch float64 autograd of x + layer(rmsnorm(x)) with the routing fixed,
 *                      closed forms (gamma = 1 and dh orthogonal to x: dx = dh/rms; dh = x: dgamma = sum x^2/rms)
 *                      (pinned to tolerance; the order of the atomicAdd accumulation of dweight over the rows is
 *                      undefined in the reference and the additions inside cooperative_groups::reduce are library
 *                      code: "parity unpinned" at the ulp level)
 */
#include <stdlib.h>

#include "oracle_common.h"

void orc_gate(const float *x, const float *Wg, const float *bg, int T, int d, int E, float *logits);
void orc_softmax(const float *logits, int T, int E, float *p);
void orc_topk(const float *p, int T, int E, int K, int renorm, int32_t *ids, float *w);
void orc_dispatch(const int32_t *ids, int T, int K, int E, int32_t *counts, int32_t *offsets, int32_t *dst,
                  int32_t *src_row);
void orc_rmsnorm(const float *x, const float *gamma, int T, int d, int bf16_mode, float *h, float *rms_o);

/* Backward of the SwiGLU expert g over `rows` rows.  xin: the rows' inputs (rows x d, row r at xin + r*d); dy: their
 * output gradients (rows x d).  Writes dxin (rows x d) and OVERWRITES dW1,dW3 [H,d], dW2 [d,H] (zero when rows == 0).
 * Scratch: 6*H floats. */
static void expert_backward(const float *xin, const float *dy, int rows, const float *W1, const float *W3,
                            const float *W2, int d, int H, int bf16_mode, float *dxin, float *dW1, float *dW3,
                            float *dW2, float *scratch)
{
    float *h1 = scratch, *h3 = scratch + H, *a = scratch + 2 * H, *dh1 = scratch + 3 * H, *dh3 = scratch + 4 * H;
    memset(dW1, 0, sizeof(float) * (size_t)H * d);
    memset(dW3, 0, sizeof(float) * (size_t)H * d);
    memset(dW2, 0, sizeof(float) * (size_t)H * d);
    for (int r = 0; r < rows; ++r) {
        const float *xr = xin + (size_t)r * d, *dyr = dy + (size_t)r * d;
        for (int h = 0; h < H; ++h) {
            const float *w1 = W1 + (size_t)h * d, *w3 = W3 + (size_t)h * d;
            float a1 = 0.0f, a3 = 0.0f;
            for (int k = 0; k < d; ++k) {
                float p1 = xr[k] * w1[k];
                a1 = a1 + p1;
                float p3 = xr[k] * w3[k];
                a3 = a3 + p3;
            }
            h1[h] = a1;
            h3[h] = a3;
            float av = silu_f(a1) * a3;
            a[h] = bf16_mode ? bf16_round(av) : av;
        }
        /* w2 back: da = dy . W2 ; dW2 += dy^T a */
        for (int h = 0; h < H; ++h) {
            float da = 0.0f;
            for (int c = 0; c < d; ++c) {
                float pr = dyr[c] * W2[(size_t)c * H + h];
                da = da + pr;
            }
            float sg = 1.0f / (1.0f + (float)exp(-(double)h1[h]));
            float g3 = da * silu_f(h1[h]);
            float tmp = da * h3[h];
            float g1 = tmp * sg * (1.0f + h1[h] * (1.0f - sg));
            dh3[h] = bf16_mode ? bf16_round(g3) : g3;
            dh1[h] = bf16_mode ? bf16_round(g1) : g1;
        }
        for (int c = 0; c < d; ++c)
            for (int h = 0; h < H; ++h) {
                float pr = dyr[c] * a[h];
                dW2[(size_t)c * H + h] = dW2[(size_t)c * H + h] + pr;
            }
        for (int h = 0; h < H; ++h)
            for (int k = 0; k < d; ++k) {
                float p1 = dh1[h] * xr[k];
                dW1[(size_t)h * d + k] = dW1[(size_t)h * d + k] + p1;
                float p3 = dh3[h] * xr[k];
                dW3[(size_t)h * d + k] = dW3[(size_t)h * d + k] + p3;
            }
        for (int k = 0; k < d; ++k) {
            float s1 = 0.0f, s3 = 0.0f;
            for (int h = 0; h < H; ++h) {
                float p1 = dh1[h] * W1[(size_t)h * d + k];
                s1 = s1 + p1;
                float p3 = dh3[h] * W3[(size_t)h * d + k];
                s3 = s3 + p3;
            }
            dxin[(size_t)r * d + k] = s1 + s3;
        }
    }
}

/* The pass for a given routing.  p [T,E]: softmax of the gate logits; ids [T,K]: selected experts as the gate numbers
 * them (0..E-1); wid [T,K]: the same experts as indices into W1/W3/W2, which hold Ew routed experts followed by Es
 * shared ones (wid == ids and Ew == E for a whole layer; a test that checks a few tokens of a large batch passes only
 * the experts those tokens use); w [T,K]: combine weights.  Outputs as orc_moe_backward (dWg, dbg sum over the T
 * tokens given). */
static void backward_core(const float *x, const float *dout, const float *Wg, const float *p, const int32_t *ids,
                          const int32_t *wid, const float *w, const float *W1, const float *W3, const float *W2, int T,
                          int d, int E, int Ew, int K, int H, int Es, int renorm, int bf16_mode, float *dx, float *dWg,
                          float *dbg, float *dW1, float *dW3, float *dW2, float *dw_o, float *dlogits_o)
{
    const int P = T * K;
    const size_t HD = (size_t)H * d;
    int32_t *counts = (int32_t *)malloc(sizeof(int32_t) * (size_t)Ew);
    int32_t *offsets = (int32_t *)malloc(sizeof(int32_t) * (size_t)(Ew + 1));
    int32_t *dst = (int32_t *)malloc(sizeof(int32_t) * (size_t)(P ? P : 1));
    int32_t *src_row = (int32_t *)malloc(sizeof(int32_t) * (size_t)(P ? P : 1));
    float *xg = (float *)malloc(sizeof(float) * (size_t)(P ? P : 1) * d);
    float *y = (float *)malloc(sizeof(float) * (size_t)(P ? P : 1) * d);
    float *dy = (float *)malloc(sizeof(float) * (size_t)(P ? P : 1) * d);
    float *dxg = (float *)malloc(sizeof(float) * (size_t)(P ? P : 1) * d);
    float *dxs = Es ? (float *)malloc(sizeof(float) * (size_t)Es * T * d) : NULL;
    float *dw = (float *)malloc(sizeof(float) * (size_t)(P ? P : 1));
    float *dlog = (float *)malloc(sizeof(float) * (size_t)T * E);
    float *scratch = (float *)malloc(sizeof(float) * (size_t)6 * H);
    float *g1 = (float *)malloc(sizeof(float) * HD), *g3 = (float *)malloc(sizeof(float) * HD),
          *g2 = (float *)malloc(sizeof(float) * HD);

    orc_dispatch(wid, T, K, Ew, counts, offsets, dst, src_row);
    for (int r = 0; r < P; ++r) memcpy(xg + (size_t)r * d, x + (size_t)src_row[r] * d, sizeof(float) * (size_t)d);
    {
        /* y of the routed rows (needed for the gradient of the combine weights) */
        float *a = scratch;
        for (int e = 0; e < Ew; ++e)
            for (int r = offsets[e]; r < offsets[e + 1]; ++r) {
                const float *xr = xg + (size_t)r * d;
                const float *w1b = W1 + (size_t)e * HD, *w3b = W3 + (size_t)e * HD, *w2b = W2 + (size_t)e * HD;
                for (int h = 0; h < H; ++h) {
                    float a1 = 0.0f, a3 = 0.0f;
                    for (int k = 0; k < d; ++k) {
                        float p1 = xr[k] * w1b[(size_t)h * d + k];
                        a1 = a1 + p1;
                        float p3 = xr[k] * w3b[(size_t)h * d + k];
                        a3 = a3 + p3;
                    }
                    float av = silu_f(a1) * a3;
                    a[h] = bf16_mode ? bf16_round(av) : av;
                }
                for (int c = 0; c < d; ++c) {
                    float acc = 0.0f;
                    for (int h = 0; h < H; ++h) {
                        float pr = a[h] * w2b[(size_t)c * H + h];
                        acc = acc + pr;
                    }
                    y[(size_t)r * d + c] = acc;
                }
            }
    }

    /* combine backward: dy[r,:] = w[t,j] * dout[t,:], dw[t,j] = dout[t,:] . y[r,:] */
    for (int t = 0; t < T; ++t)
        for (int j = 0; j < K; ++j) {
            const int r = dst[(size_t)t * K + j];
            const float wv = w[(size_t)t * K + j];
            float acc = 0.0f;
            for (int c = 0; c < d; ++c) {
                float g = wv * dout[(size_t)t * d + c];
                dy[(size_t)r * d + c] = bf16_mode ? bf16_round(g) : g;
                float pr = dout[(size_t)t * d + c] * y[(size_t)r * d + c];
                acc = acc + pr;
            }
            dw[(size_t)t * K + j] = acc;
        }

    /* experts */
    for (int e = 0; e < Ew; ++e) {
        expert_backward(xg + (size_t)offsets[e] * d, dy + (size_t)offsets[e] * d, counts[e], W1 + (size_t)e * HD,
                        W3 + (size_t)e * HD, W2 + (size_t)e * HD, d, H, bf16_mode, dxg + (size_t)offsets[e] * d, g1,
                        g3, g2, scratch);
        if (dW1) memcpy(dW1 + (size_t)e * HD, g1, sizeof(float) * HD);
        if (dW3) memcpy(dW3 + (size_t)e * HD, g3, sizeof(float) * HD);
        if (dW2) memcpy(dW2 + (size_t)e * HD, g2, sizeof(float) * HD);
    }
    for (int s = 0; s < Es; ++s) {
        const int g = Ew + s;
        expert_backward(x, dout, T, W1 + (size_t)g * HD, W3 + (size_t)g * HD, W2 + (size_t)g * HD, d, H, bf16_mode,
                        dxs + (size_t)s * T * d, g1, g3, g2, scratch);
        if (dW1) memcpy(dW1 + (size_t)g * HD, g1, sizeof(float) * HD);
        if (dW3) memcpy(dW3 + (size_t)g * HD, g3, sizeof(float) * HD);
        if (dW2) memcpy(dW2 + (size_t)g * HD, g2, sizeof(float) * HD);
    }

    /* router: renormalisation, scatter to the selected experts, softmax, gate */
    for (int t = 0; t < T; ++t) {
        float *dl = dlog + (size_t)t * E;
        const float *pr = p + (size_t)t * E;
        for (int e = 0; e < E; ++e) dl[e] = 0.0f; /* holds dp first */
        float S = 1.0f, dot = 0.0f;
        if (renorm) {
            S = 0.0f;
            for (int j = 0; j < K; ++j) S += pr[ids[(size_t)t * K + j]];
            for (int j = 0; j < K; ++j) {
                float term = dw[(size_t)t * K + j] * w[(size_t)t * K + j];
                dot = dot + term;
            }
        }
        for (int j = 0; j < K; ++j) {
            float g = dw[(size_t)t * K + j];
            if (renorm) g = (g - dot) / S;
            dl[ids[(size_t)t * K + j]] = g;
        }
        float sum = 0.0f;
        for (int e = 0; e < E; ++e) sum += pr[e] * dl[e];
        for (int e = 0; e < E; ++e) dl[e] = (dl[e] - sum) * pr[e];
    }
    if (dWg)
        for (int e = 0; e < E; ++e)
            for (int k = 0; k < d; ++k) {
                float acc = 0.0f;
                for (int t = 0; t < T; ++t) {
                    float term = dlog[(size_t)t * E + e] * x[(size_t)t * d + k];
                    acc = acc + term;
                }
                dWg[(size_t)e * d + k] = acc;
            }
    if (dbg)
        for (int e = 0; e < E; ++e) {
            float acc = 0.0f;
            for (int t = 0; t < T; ++t) acc = acc + dlog[(size_t)t * E + e];
            dbg[e] = acc;
        }

    /* input gradient: experts in slot order, shared experts, gate */
    for (int t = 0; t < T; ++t)
        for (int k = 0; k < d; ++k) {
            float acc = 0.0f;
            for (int j = 0; j < K; ++j) acc = acc + dxg[(size_t)dst[(size_t)t * K + j] * d + k];
            for (int s = 0; s < Es; ++s) acc = acc + dxs[((size_t)s * T + t) * d + k];
            float gsum = 0.0f;
            for (int e = 0; e < E; ++e) {
                float term = dlog[(size_t)t * E + e] * Wg[(size_t)e * d + k];
                gsum = gsum + term;
            }
            acc = acc + gsum;
            dx[(size_t)t * d + k] = bf16_mode ? bf16_round(acc) : acc;
        }

    if (dw_o) memcpy(dw_o, dw, sizeof(float) * (size_t)P);
    if (dlogits_o) memcpy(dlogits_o, dlog, sizeof(float) * (size_t)T * E);
    free(counts); free(offsets); free(dst); free(src_row);
    free(xg); free(y); free(dy); free(dxg); free(dxs); free(dw); free(dlog); free(scratch);
    free(g1); free(g3); free(g2);
}

/* Whole backward pass.  x, dout: [T,d]; weights as in orc_moe_forward (W1,W3: [E+Es,H,d], W2: [E+Es,d,H]).
 * The forward quantities it needs are recomputed here.  Outputs (any may be NULL except dx): dx [T,d], dWg [E,d],
 * dbg [E], dW1,dW3 [E+Es,H,d], dW2 [E+Es,d,H], dw [T,K] (gradient of the combine weights), dlogits [T,E]. */
void orc_moe_backward(const float *x, const float *dout, const float *Wg, const float *bg, const float *W1,
                      const float *W3, const float *W2, int T, int d, int E, int K, int H, int Es, int renorm,
                      int bf16_mode, float *dx, float *dWg, float *dbg, float *dW1, float *dW3, float *dW2,
                      float *dw_o, float *dlogits_o)
{
    const int P = T * K;
    float *logits = (float *)malloc(sizeof(float) * (size_t)T * E);
    float *p = (float *)malloc(sizeof(float) * (size_t)T * E);
    int32_t *ids = (int32_t *)malloc(sizeof(int32_t) * (size_t)(P ? P : 1));
    float *w = (float *)malloc(sizeof(float) * (size_t)(P ? P : 1));
    orc_gate(x, Wg, bg, T, d, E, logits);
    orc_softmax(logits, T, E, p);
    orc_topk(p, T, E, K, renorm, ids, w);
    backward_core(x, dout, Wg, p, ids, ids, w, W1, W3, W2, T, d, E, E, K, H, Es, renorm, bf16_mode, dx, dWg, dbg, dW1,
                  dW3, dW2, dw_o, dlogits_o);
    free(logits); free(p); free(ids); free(w);
}

/* The pass for a few tokens of a larger batch whose routing is known (see backward_core for p, ids, wid, w, Ew). */
void orc_moe_backward_routed(const float *x, const float *dout, const float *Wg, const float *p, const int32_t *ids,
                             const int32_t *wid, const float *w, const float *W1, const float *W3, const float *W2,
                             int T, int d, int E, int Ew, int K, int H, int Es, int renorm, int bf16_mode, float *dx,
                             float *dw_o, float *dlogits_o)
{
    backward_core(x, dout, Wg, p, ids, wid, w, W1, W3, W2, T, d, E, Ew, K, H, Es, renorm, bf16_mode, dx, NULL, NULL,
                  NULL, NULL, NULL, dw_o, dlogits_o);
}

/* Backward of the pre-norm of the block: rmsnorm_backward_kernel2 (J/engine/nn/layer/normalization/gpu/RMSKernel.cu:226-277,
 * the kernel RMSLayer.diff launches, J/engine/nn/layer/normalization/RMSLayer.java:292 -> RMSKernel.java:296-310).
 * Per row, one 32-lane group: rms as in the forward kernel (passed in); dweight[i] += (inp[i]/rms) * dout[i] (atomicAdd
 * over the rows in the reference: the order of those additions is not defined there; here rows in index order);
 * drms = sum_i inp[i]*dout[i]*weight[i], lane l adding i = l, l+32, ... in index order (the product inp*dout rounded,
 * then one fused multiply-add with weight, nvcc's default contraction), xor butterfly over the lanes, times
 * -1/(rms*rms*rms*C); dinp[i] = dout[i]*weight[i]/rms + drms*inp[i] (the last multiply-add fused).
 * resid != NULL: the gradient that reaches the block's input past the norm is added (Tensor_OP().add(norm2.diff, delta),
 * J/engine/nn/layer/llama/LlamaTransformerBlock.java:157-158) before the one rounding of bf16 mode. */
void orc_rmsnorm_backward(const float *x, const float *dh, const float *gamma, const float *rms, const float *resid, int T,
                          int d, int bf16_mode, float *dx, float *dgamma)
{
    for (int c = 0; c < d; ++c) dgamma[c] = 0.0f;
    for (int t = 0; t < T; ++t) {
        const float *xr = x + (size_t)t * d, *gr = dh + (size_t)t * d;
        const float r = rms[t];
        for (int c = 0; c < d; ++c) {
            float n = xr[c] / r;
            float pr = n * gr[c];
            dgamma[c] = dgamma[c] + pr;
        }
        float part[32];
        for (int l = 0; l < 32; ++l) {
            float s = 0.0f;
            for (int i = l; i < d; i += 32) {
                float pr = xr[i] * gr[i];
                s = fmaf(pr, gamma[i], s);
            }
            part[l] = s;
        }
        for (int m = 16; m >= 1; m >>= 1) {
            float nxt[32];
            for (int l = 0; l < 32; ++l) nxt[l] = part[l] + part[l ^ m];
            memcpy(part, nxt, sizeof(part));
        }
        float drms = part[0] * (-1.0f / (r * r * r * (float)d));
        for (int c = 0; c < d; ++c) {
            float a = gr[c] * gamma[c];
            float q = a / r;
            float v = fmaf(drms, xr[c], q);
            if (resid) v = v + resid[(size_t)t * d + c];
            dx[(size_t)t * d + c] = bf16_mode ? bf16_round(v) : v;
        }
    }
}

/* Backward of the block form out = x + layer(rmsnorm(x)):
 *   getMlp().back(delta); getNorm2().back(getMlp().diff); Tensor_OP().add(getNorm2().diff, delta, getNorm2().diff)
 * (J/engine/nn/layer/llama/LlamaTransformerBlock.java:156-158).  The layer's input gradient dh is its `diff` (rounded to
 * bf16 in bf16 mode, like every activation the layer hands out).  Outputs as orc_moe_backward plus dgamma [d]; dh_o [T,d]
 * may be NULL. */
void orc_block_backward(const float *x, const float *gamma, const float *dout, const float *Wg, const float *bg,
                        const float *W1, const float *W3, const float *W2, int T, int d, int E, int K, int H, int Es,
                        int renorm, int bf16_mode, float *dx, float *dgamma, float *dWg, float *dbg, float *dW1, float *dW3,
                        float *dW2, float *dh_o)
{
    float *h = (float *)malloc(sizeof(float) * (size_t)T * d);
    float *rms = (float *)malloc(sizeof(float) * (size_t)T);
    float *dh = (float *)malloc(sizeof(float) * (size_t)T * d);
    orc_rmsnorm(x, gamma, T, d, bf16_mode, h, rms);
    orc_moe_backward(h, dout, Wg, bg, W1, W3, W2, T, d, E, K, H, Es, renorm, bf16_mode, dh, dWg, dbg, dW1, dW3, dW2, NULL, NULL);
    orc_rmsnorm_backward(x, dh, gamma, rms, dout, T, d, bf16_mode, dx, dgamma);
    if (dh_o) memcpy(dh_o, dh, sizeof(float) * (size_t)T * d);
    free(h); free(rms); free(dh);
}
