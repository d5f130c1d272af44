/*
 * libomega_hip.so -- C ABI of the MI355X (gfx950) mixture-of-experts layer: forward, block form, backward, update.
 *
 * Plain C: opaque handles, raw device addresses, sizes and ints.  Every entry point returns an
 * omega_status (0 = OK) and never throws or aborts across the boundary; a human-readable message
 * for the last failure on a context is available from omega_hip_last_error().
 *
 * Each declaration names the reference interface it stands in for
 * (J/ = src/main/java/com/omega/ in the reference checkout).
 */
#ifndef OMEGA_HIP_H
#define OMEGA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct omega_ctx omega_ctx; /* one device + one stream; calls on a ctx are serialised */
typedef struct omega_moe omega_moe; /* one MoE layer: owns its weights and its workspace      */

typedef enum {
    OMEGA_OK = 0,
    OMEGA_ERR_INVALID_ARG = 1,
    OMEGA_ERR_OOM = 2,
    OMEGA_ERR_HIP = 3,
    OMEGA_ERR_UNSUPPORTED = 4
} omega_status;

typedef enum { OMEGA_DTYPE_F32 = 0, OMEGA_DTYPE_BF16 = 1 } omega_dtype;

/* EXACT: gate logits summed sequentially over k with separate multiply and add (the order of the
 * reference's CPU dot, J/common/utils/MatrixOperation.java:1472-1478), so expert ids are
 * reproducible bit for bit.  FAST: wave-parallel fp32 FMA reduction, tolerance only. */
typedef enum { OMEGA_ROUTER_EXACT = 0, OMEGA_ROUTER_FAST = 1 } omega_router_mode;

typedef enum {
    OMEGA_W_GATE = 0,      /* [E,d]            */
    OMEGA_W_GATE_BIAS = 1, /* [E] always fp32  */
    OMEGA_W_W1 = 2,        /* [H,d] per expert */
    OMEGA_W_W3 = 3,        /* [H,d] per expert */
    OMEGA_W_W2 = 4,        /* [d,H] per expert */
    OMEGA_W_NORM = 5       /* [d] always fp32: weight (gamma) of the RMSNorm in front of the layer, block form only
                              (RMSLayer.gamma, J/engine/nn/layer/normalization/RMSLayer.java) */
} omega_weight_kind;

/* Constructor arguments of the layer, in the house style of
 * LlamaMLPLayer(embedDim, nChannel, multiple_of, bias, network), J/engine/nn/layer/llama/LlamaMLPLayer.java:47-63. */
typedef struct {
    int32_t T_max;         /* workspace is sized for this many tokens; grows on demand            */
    int32_t d;             /* model width (embedDim)                                               */
    int32_t E;             /* routed experts                                                       */
    int32_t K;             /* experts per token                                                    */
    int32_t H;             /* expert hidden width                                                  */
    int32_t Es;            /* always-on shared experts (same SwiGLU shape), summed into the output */
    int32_t renorm;        /* 1: top-k weights divided by their sum                                */
    int32_t has_gate_bias; /* 1: logits += bg[e]                                                   */
    int32_t dtype;         /* omega_dtype of x, out and all weights                                */
    int32_t router_mode;   /* omega_router_mode                                                    */
} omega_moe_config;

/* Library version, major*10000 + minor*100 + patch. */
int omega_hip_version(void);

/* Per-device context.  Replaces new CUDAManager(rank) -> cuInit/cuCtxCreate
 * (J/engine/gpu/CUDAManager.java:111-116) and the per-rank pool J/engine/parallel/cuda/CUDAPool.java:12-22.
 * No module loading is needed: kernels are linked into the library
 * (replaces CUDAManager.getLocalFunctionByModule, J/engine/gpu/CUDAManager.java:125-159). */
int omega_hip_ctx_create(int device, omega_ctx **out);
int omega_hip_ctx_destroy(omega_ctx *ctx);
/* Message of the last failed call on ctx (or of the last failed ctx_create when ctx is NULL).
 * Mirrors checkCUDA's "Error code N:msg" RuntimeException, J/engine/gpu/CUDAMemoryManager.java:179-201. */
const char *omega_hip_last_error(omega_ctx *ctx);

/* Device memory.  Replaces CUDAMemoryManager.getPointer / free
 * (J/engine/gpu/CUDAMemoryManager.java:115-123,161-165). */
int omega_hip_malloc(omega_ctx *ctx, size_t bytes, void **dptr);
int omega_hip_free(omega_ctx *ctx, void *dptr);
/* Blocking copies, as Tensor.hostToDevice / Tensor.syncHost (J/engine/tensor/Tensor.java:559-579). */
int omega_hip_memcpy_h2d(omega_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes);
int omega_hip_memcpy_d2h(omega_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes);
/* Tensor.clearGPU (J/engine/tensor/Tensor.java:680-685). */
int omega_hip_memset(omega_ctx *ctx, void *dptr, int value, size_t bytes);
/* JCuda.cudaDeviceSynchronize() as used around timed regions (J/engine/nn/network/Llama3.java:140-156). */
int omega_hip_sync(omega_ctx *ctx);

/* java.util.Random on the host (no device involved), for initialising a layer with the numbers a Java run of the
 * reference draws: RandomUtils keeps one java.util.Random (RandomUtils.setSeed / getInstance,
 * J/common/utils/RandomUtils.java:18-28); omega_jrandom_normal is RandomUtils.normal_ (RandomUtils.java:697-703):
 * out[i] = (float)(std * nextGaussian() + mean).  The state is plain data owned by the caller. */
typedef struct {
    int64_t state;              /* 48-bit state of the linear congruential generator */
    double next_gaussian;       /* the second value of the last polar-method pair ... */
    int32_t have_next_gaussian; /* ... if it has not been handed out yet              */
} omega_jrandom;
void omega_jrandom_seed(omega_jrandom *r, int64_t seed);
int32_t omega_jrandom_next_int(omega_jrandom *r);
double omega_jrandom_next_double(omega_jrandom *r);
double omega_jrandom_next_gaussian(omega_jrandom *r);
void omega_jrandom_normal(omega_jrandom *r, float *out, size_t n, float mean, float std);

/* Seeded synthetic data on the device: element i of `stream` under `seed`, N(0,std), written as
 * `dtype`.  Counter-based, so any slice (first, n) of a stream can be produced independently.
 * Stands in for RandomUtils.normal_ (J/common/utils/RandomUtils.java:697-703) + Tensor upload. */
int omega_hip_fill_normal(omega_ctx *ctx, void *dptr, uint64_t n, uint64_t seed, uint64_t stream, double std,
                          uint64_t first, int dtype);
/* fp32 <-> bf16 conversion of device buffers (round to nearest even). */
int omega_hip_convert(omega_ctx *ctx, void *dst, int dst_dtype, const void *src, int src_dtype, uint64_t n);

/* Layer life cycle.  create = the layer constructor + initParam (weights allocated, zeroed);
 * the workspace plays the role of the lazily (re)allocated activation tensors of init()
 * (J/engine/nn/layer/llama/LlamaMLPLayer.java:98-104, J/engine/nn/layer/FullyLayer.java:159-175). */
int omega_moe_create(omega_ctx *ctx, const omega_moe_config *cfg, omega_moe **out);
int omega_moe_destroy(omega_moe *moe);

/* Load / read back one weight tensor in the reference's layout ([out,in] row-major,
 * J/engine/nn/layer/FullyLayer.java:181), elements of the layer dtype (gate bias: fp32), from / to host or
 * device memory.  expert: 0..E-1 routed, E..E+Es-1 shared; ignored for the gate.  The layer keeps bf16 expert
 * weights in its own tiled order; these two calls convert.  Stand in for FullyLayer.loadModel / saveModel and
 * the weight upload (J/engine/nn/layer/FullyLayer.java:854-866). */
int omega_moe_set_weights(omega_moe *moe, int which, int expert, const void *src, int is_device);
int omega_moe_get_weights(omega_moe *moe, int which, int expert, void *dst, int is_device);

/* forward(Tensor): x_dev [T,d] -> out_dev [T,d], both of the layer dtype, caller-owned device
 * buffers.  Asynchronous on the context's stream; omega_hip_sync / memcpy_d2h make it visible.
 * The drop-in for the FFN slot, J/engine/nn/layer/llama/LlamaTransformerBlock.java:135 ->
 * LlamaMLPLayer.forward(Tensor) (J/engine/nn/layer/llama/LlamaMLPLayer.java:200-217). */
int omega_moe_forward(omega_moe *moe, const void *x_dev, int T, void *out_dev);

/* Block form: out = x + layer(rmsnorm(x)), the second half of the transformer block,
 *   getNorm2().forward(tmp1); getMlp().forward(getNorm2().getOutput()); Tensor_OP().add(getMlp().getOutput(), tmp1, tmp2)
 * (J/engine/nn/layer/llama/LlamaTransformerBlock.java:134-136), in one call: one kernel writes the row statistics
 * and the normalised rows h (layer dtype) that the router and the gather then read, and the combine kernel adds the
 * row of x to its fp32 sum before the one rounding of the output, so the layer output never makes a round trip
 * through memory on its own.
 * rmsnorm = rmsnorm_forward_kernel2 (J/engine/nn/layer/normalization/gpu/RMSKernel.cu:185-223, the kernel
 * RMSLayer.output launches, RMSLayer.java:230): rms = sqrtf(mean(x^2) + 1e-6f), h = (x / rms) * gamma, with the
 * sum of squares taken lane by lane as that kernel takes it; bf16 layers round h to bf16 and round x + layer(h) once.
 * The norm weight must have been set (omega_moe_set_weights(moe, OMEGA_W_NORM, 0, gamma, is_device)). */
int omega_moe_forward_block(omega_moe *moe, const void *x_dev, int T, void *out_dev);
/* rms[t] of the last omega_moe_forward_block, T floats to host (blocking).  For tests; the normalised rows
 * themselves are visible as the gathered rows, omega_moe_get_workspace(moe, 0, ...). */
int omega_moe_get_norm(omega_moe *moe, int T, float *rms_host);

/* back(Tensor delta): gradients for the output gradient dout_dev [T,d] (layer dtype) of the omega_moe_forward call
 * that ran last on this layer with the same x_dev and T (its routing and its activation buffers are reused; h1 and
 * h3 are recomputed).  Writes the input gradient dx_dev [T,d] (layer dtype; Layer.diff) and OVERWRITES the layer's
 * parameter gradients (diffW / diffB of every child linear layer: beta = 0 in FullyLayer.diff,
 * J/engine/nn/layer/FullyLayer.java:292-334).  Composition: combine backward (gradient of the rows and of the
 * combine weights) -> SwiGLU backward per expert as LlamaMLPLayer.diff
 * (J/engine/nn/layer/llama/LlamaMLPLayer.java:139-158) with silu_backward
 * (J/engine/nn/layer/active/gpu/activeFunction.cu:182-190) -> un-dispatch; combine weights -> renormalisation ->
 * softmax_back (J/engine/gpu/SoftmaxKernel.cu:101-112) -> gate linear layer.  The expert ids and the permutation carry
 * no gradient.  Asynchronous on the context's stream. */
int omega_moe_backward(omega_moe *moe, const void *x_dev, const void *dout_dev, int T, void *dx_dev);
/* Backward of the block form, after omega_moe_forward_block of the same x_dev and T:
 *   getMlp().back(delta); getNorm2().back(getMlp().diff); Tensor_OP().add(getNorm2().diff, delta, getNorm2().diff)
 * (J/engine/nn/layer/llama/LlamaTransformerBlock.java:156-158), the norm backward being rmsnorm_backward_kernel2
 * (J/engine/nn/layer/normalization/gpu/RMSKernel.cu:226-277, launched by RMSLayer.diff, RMSLayer.java:292).  The layer's
 * input gradient stays inside the library; dx_dev receives dout + norm backward of it (one rounding in bf16 layers), and
 * the gradient of the norm weight becomes available as omega_moe_get_grad(moe, OMEGA_W_NORM, ...) (it is zero after a
 * plain omega_moe_backward).  The weight gradient is summed in a fixed order (the reference uses atomicAdd). */
int omega_moe_backward_block(omega_moe *moe, const void *x_dev, const void *dout_dev, int T, void *dx_dev);
/* Training mode (off at creation).  The reference's layers keep their outputs for back() (LlamaMLPLayer.diff reads
 * active.getOutput() and getLinear3().getOutput(), J/engine/nn/layer/llama/LlamaMLPLayer.java:148-152); with training
 * on, omega_moe_forward of a bf16 layer likewise stores h1 and h3 (fp32, from the accumulators of its up product) and
 * omega_moe_backward reads them instead of recomputing them.  Same results either way; the forward pass writes
 * 8*H bytes more per expert row.  fp32 layers ignore the switch. */
int omega_moe_set_training(omega_moe *moe, int on);
/* How the rows of x reach the experts of a bf16 layer.  The reference has no dispatch (its row gathers, e.g.
 * img_token_drop, J/engine/nn/layer/dit/kernel/TokenDropKernel.cu:147-160, always write the gathered copy).
 *   OMEGA_GATHER_AUTO (default): by shape - see below;
 *   OMEGA_GATHER_COPY: the dispatch stage writes every token row into its K places of an expert-contiguous buffer;
 *   OMEGA_GATHER_ON_LOAD: no copy - the loads of the up product fetch each row of a tile from x through the
 *     row -> token table of the dispatch stage.  Same results bit for bit.  The loads then read 64-byte pieces of
 *     rows instead of whole lines, which costs the product 1-8 %, and K row copies per token are saved: AUTO takes
 *     this form while H/128 <= 2 K (a row tile is read H/128 times).
 * Training mode and fp32 layers always copy.  x must stay unchanged until the forward pass has finished either way;
 * with ON_LOAD, omega_moe_get_workspace(moe, 0, ...) and a backward pass gather the rows when they are asked for,
 * from the x of the last dispatch, which must still hold that batch. */
#define OMEGA_GATHER_AUTO 0
#define OMEGA_GATHER_COPY 1
#define OMEGA_GATHER_ON_LOAD 2
int omega_moe_set_gather_mode(omega_moe *moe, int mode);
/* 1 if the last dispatch stage left the rows to the up product's loads, 0 if it wrote the gathered copy (what AUTO
 * chose for the shape; no counterpart in the reference). */
int omega_moe_gather_on_load(omega_moe *moe);
/* One parameter gradient of the last omega_moe_backward, always fp32, in the layout of the weight it belongs to
 * (which / expert as for omega_moe_set_weights).  Stands in for reading layer.diffW / diffB
 * (LlamaMLPLayer.putParamterGrads, J/engine/nn/layer/llama/LlamaMLPLayer.java:285-295). */
int omega_moe_get_grad(omega_moe *moe, int which, int expert, void *dst, int is_device);
/* accGrad(scale): the first call after an update copies the gradients into the accumulators, later calls add
 * scale * gradient (FullyLayer.accGrad, J/engine/nn/layer/FullyLayer.java:593-607). */
int omega_moe_acc_grad(omega_moe *moe, float scale);
/* The layer's share of Network.clipGradNorm (J/engine/nn/network/Network.java:379-432).  grad_sumsq: the sum of the
 * squares of all parameter gradients of the layer - of the accumulators when accGrad has run since the last update, as
 * getAccGradNorm / getGradNorm choose (Network.java:325-378) - copied to the host (blocking); what the reference adds
 * up over its layers as c.syncHost()[0] (Network.java:388-393).  Summed in a fixed order (the reference's
 * vectorL2NormKernel, J/engine/gpu/GlobalNormKernel.cu:3-30, uses atomicAdd).  scale_grad: the same tensors times
 * coef, rounded once per element (tensorOP.mul(diffW, clip_coef, diffW), Network.java:401-431).  The caller forms
 * clip_coef = min(1, gradClip / (sqrt(total) + 1e-6)) from the totals of all its layers. */
int omega_moe_grad_sumsq(omega_moe *moe, float *sumsq_host);
int omega_moe_scale_grad(omega_moe *moe, float coef);
/* update() of a layer without an updater: the accumulated gradients, if any, replace the gradients, then
 * w -= lr * diffW, b -= lr * diffB, and the accumulators are cleared (FullyLayer.update,
 * J/engine/nn/layer/FullyLayer.java:569-590).  The optimisers behind Updater are not part of this library.
 * bf16 layers take the step on fp32 master copies of their weights (made from the weights at the first update after
 * they were set, kept across updates) and re-round the weights from them.  The forward pass must run again before the
 * next backward pass. */
int omega_moe_update(omega_moe *moe, float lr);
/* update() of a layer whose network uses the AdamW updater (FullyLayer.update -> updater.update(this),
 * J/engine/nn/layer/FullyLayer.java:569-590; AdamW.update, J/engine/updater/AdamW.java:69-92): every parameter tensor
 * of the layer - gate weight and bias, expert weights, and the norm weight of the block form, which the reference
 * steps through updateForBN with the same kernel - takes one step of adamw_kernel
 * (J/engine/updater/gpu/updater.cu:31-52) with eps = 1e-8 and the bias corrections (float)(1 - pow(beta, train_time))
 * formed on the host as AdamWKernel.updateW does (J/engine/updater/gpu/AdamWKernel.java:177-195); weight_decay
 * applies to all of them, as there.  train_time is the network's step counter, starting at 1.  The moments live in
 * the handle (zero at the first call, kept across set_weights).  Accumulated gradients, bf16 master copies and the
 * need for a new forward pass are as for omega_moe_update.  Defaults of the reference: beta1 0.9, beta2 0.95
 * (AdamWKernel.java:25-26), weight_decay 1e-4 (AdamW.java:27). */
int omega_moe_update_adamw(omega_moe *moe, float lr, float beta1, float beta2, float weight_decay, int train_time);

/* The four stages of forward, callable one at a time (per-stage timing and tests); they use the
 * same kernels and workspace as omega_moe_forward and must be called in this order for one T:
 *   router   x -> ids, weights, per-tile expert histogram      (gate: FullyLayer.output, FullyLayer.java:218-243;
 *                                                               softmax: J/engine/gpu/SoftmaxKernel.cu:4-24)
 *   dispatch histogram -> counts, offsets, dst, src_row, tile list; gather x rows into the
 *            expert-contiguous buffer                           (gather as img_token_drop,
 *                                                               J/engine/nn/layer/dit/kernel/TokenDropKernel.cu:147-160)
 *   experts  grouped SwiGLU: a = silu(xg W1^T) * (xg W3^T); y = a W2^T
 *                                                              (LlamaMLPLayer.output, LlamaMLPLayer.java:117-130)
 *   combine  out[t] = sum_j w[t,j] * y[dst[t*K+j]] (+ shared)   (weighted sum as add_mul_kernel,
 *                                                               J/engine/gpu/BaseKernel.cu:228-241) */
int omega_moe_router(omega_moe *moe, const void *x_dev, int T);
int omega_moe_dispatch(omega_moe *moe, const void *x_dev, int T);
int omega_moe_experts(omega_moe *moe, const void *x_dev, int T);
int omega_moe_combine(omega_moe *moe, int T, void *out_dev);
/* The two products of the experts stage separately (profiling). */
int omega_moe_experts_up(omega_moe *moe, const void *x_dev, int T);
int omega_moe_experts_down(omega_moe *moe, int T);

/* Routing of the last forward/router+dispatch call, copied to host (blocking).  Any pointer may
 * be NULL.  ids,w: [T,K]; counts: [E]; offsets: [E+1]; dst, src_row: [T*K]
 * (dst[p] = row of pair p=t*K+j in the expert-contiguous buffer; src_row[r] = token of row r). */
int omega_moe_get_routing(omega_moe *moe, int T, int32_t *ids, float *w, int32_t *counts, int32_t *offsets,
                          int32_t *dst, int32_t *src_row);
/* Router intermediates, for tests: runs the router on x_dev and copies logits and probabilities
 * [T,E] to host (blocking).  Overwrites the routing state like omega_moe_router. */
int omega_moe_get_router_probs(omega_moe *moe, const void *x_dev, int T, float *logits, float *probs);
/* omega_moe_get_router_probs for callers that cannot allocate device memory (tight serving loops, harnesses that
 * forbid hipMalloc).  It has no counterpart in the reference.  Same result and same effect on the routing state, and
 * like it a blocking call (it waits for the stream and copies to pageable host memory, so it cannot itself be
 * captured into a HIP graph), but it calls no hipMalloc / hipFree: logits and probabilities are staged in a
 * static device array of the library (2 x 4 MiB per device, held until the process ends) and the layer's workspace is
 * never grown.  Refused with a message: T above the workspace the layer already holds (create it with T_max >= T), and
 * T*E above 1048576.  All calls on one device share the array: calls that overlap on one device (two contexts, two
 * threads) race on it. */
int omega_moe_get_router_probs_noalloc(omega_moe *moe, const void *x_dev, int T, float *logits, float *probs);
/* Host copy (blocking) of a workspace buffer of the last call, rows in logical order (row dst[p] of pair p,
 * then T rows per shared expert), row-major: which = 0 xg [T*K,d] (layer dtype), 1 a [T*K+Es*T,H] (layer
 * dtype), 2 y [T*K+Es*T,d] fp32; after omega_moe_backward of a bf16 layer also 3 dh1|dh3 [T*K+Es*T,2H] bf16, and for
 * any layer 4 dlogits [T,E] fp32.  For tests. */
int omega_moe_get_workspace(omega_moe *moe, int which, int T, void *host_dst);
/* Fills a whole workspace buffer, padding rows included, with one byte value (which = 1 a, 2 y; Tensor.clearGPU /
 * Tensor.fill on a layer-owned tensor, J/engine/tensor/Tensor.java:680-685).  For tests: with 0xFF every element reads
 * as NaN, so a row that a forward pass should have written and did not cannot go unnoticed. */
int omega_moe_fill_workspace(omega_moe *moe, int which, int byte_value);

/* Average duration in milliseconds of the launches of one stage, measured with events on the
 * context's stream: runs `iters` back-to-back repetitions of the stage (0 router, 1 dispatch,
 * 2 experts_up, 3 experts_down, 4 combine, 5 whole forward, 6 dispatch index kernels only, 7 dispatch
 * row gather only, 8 whole forward_block, 9 the pre-norm kernel of the block form only) after `warmup` untimed ones.
 * x_dev/out_dev as for forward; the stages before `stage` must have been run for this T. */
int omega_moe_time_stage(omega_moe *moe, int stage, const void *x_dev, int T, void *out_dev, int warmup, int iters,
                         float *ms_avg);

/* Average duration in milliseconds of omega_moe_backward, measured like omega_moe_time_stage; the forward pass for
 * x_dev and T must have run. */
int omega_moe_time_backward(omega_moe *moe, const void *x_dev, const void *dout_dev, int T, void *dx_dev, int warmup,
                            int iters, float *ms_avg);

/* Per-stage timing of omega_moe_forward itself: while profiling is on, every forward records events
 * on the context's stream around its five stages (router, dispatch, experts_up, experts_down,
 * combine).  get_profile waits for the stream, returns the summed duration of each stage in
 * milliseconds over the forwards since profiling was switched on (or since the last get_profile)
 * and their number, and starts a new accumulation.  Replaces the hand-placed
 * cudaDeviceSynchronize + System.nanoTime prints of J/engine/nn/network/Llama3.java:140-156. */
int omega_moe_set_profiling(omega_moe *moe, int on);
int omega_moe_get_profile(omega_moe *moe, float stage_ms_sum[5], int *n_calls);

#ifdef __cplusplus
}
#endif
#endif /* OMEGA_HIP_H */
