/*
 * CPU baseline in the reference's own CPU style.  TEST/BENCH INFRASTRUCTURE ONLY (see the
 * header of omega_moe_oracle.c): it is timed next to the GPU path, never shipped.
 *
 * The reference has no composed CPU path for a mixture-of-experts layer; what it has are CPU
 * primitives, and this file composes them in their own loop orders:
 *   GEMM     J/engine/cpu/SimplePerfCpuBlasBatchSgemmJdk8.java:37-79,84-131 : column-major
 *            batched sgemm, loops j (8 wide) -> p -> i, unfused C += (A*alpha)*B, a fixed
 *            pool of threads, one task per batch item (here: one task per expert).
 *   softmax  J/engine/gpu/SoftmaxKernel.java:69-87
 *   silu, *  J/engine/nn/layer/active/gpu/activeFunction.cu:172-179,
 *            J/common/utils/MatrixOperation.java:985-991 (single-thread elementwise loops)
 * It is a C restatement (no JDK is available), labelled as such wherever it is reported.
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

void orc_gate(const float *, const float *, const float *, int, int, int, float *);
void orc_softmax(const float *, int, int, float *);
void orc_topk(const float *, int, int, int, int, int32_t *, float *);
void orc_dispatch(const int32_t *, int, int, int, int32_t *, int32_t *, int32_t *, int32_t *);
void orc_gather(const float *, const int32_t *, int, int, float *);
void orc_combine(const float *, const int32_t *, const float *, const float *, int, int, int, int, int, float *);

#define SIMD_WIDTH 8

/* Column-major C[m x n] += alpha * op(A) * B with op(A)=A^T (A stored [k x m], lda) and B [k x n]:
 * the only operand form the layer needs (row-major Y[T,H] = X W^T is column-major Y^T = W . X^T,
 * i.e. A = W buffer transposed, B = X buffer).  Loop order and the unfused update follow
 * tiledSgemm, SimplePerfCpuBlasBatchSgemmJdk8.java:104-130. */
static void tiled_sgemm_tn(int m, int n, int k, float alpha, const float *A, int lda, const float *B, int ldb,
                           float beta, float *C, int ldc)
{
    if (beta != 1.0f)
        for (int j = 0; j < n; ++j)
            for (int i = 0; i < m; ++i) C[i + (size_t)j * ldc] *= beta;
    for (int j = 0; j < n; j += SIMD_WIDTH) {
        int jend = j + SIMD_WIDTH < n ? j + SIMD_WIDTH : n;
        for (int p = 0; p < k; ++p) {
            float bcol[SIMD_WIDTH] = {0};
            for (int jj = j; jj < jend; ++jj) bcol[jj - j] = B[p + (size_t)jj * ldb];
            for (int i = 0; i < m; ++i) {
                float aval = A[p + (size_t)i * lda] * alpha;
                for (int jj = j; jj < jend; ++jj) C[i + (size_t)jj * ldc] += aval * bcol[jj - j];
            }
        }
    }
}

typedef struct {
    int m, n, k;
    const float *A, *B;
    float *C;
    int lda, ldb, ldc;
} gemm_task;

typedef struct {
    gemm_task *tasks;
    int n_tasks;
    int next;
    pthread_mutex_t mu;
} task_queue;

static void *worker(void *arg)
{
    task_queue *q = (task_queue *)arg;
    for (;;) {
        pthread_mutex_lock(&q->mu);
        int i = q->next < q->n_tasks ? q->next++ : -1;
        pthread_mutex_unlock(&q->mu);
        if (i < 0) break;
        gemm_task *t = &q->tasks[i];
        if (t->n > 0) tiled_sgemm_tn(t->m, t->n, t->k, 1.0f, t->A, t->lda, t->B, t->ldb, 0.0f, t->C, t->ldc);
    }
    return NULL;
}

/* batchSgemm: a fixed pool of n_threads workers, one task per batch item
 * (SimplePerfCpuBlasBatchSgemmJdk8.java:37-79). */
static void batch_sgemm(gemm_task *tasks, int n_tasks, int n_threads)
{
    task_queue q = {tasks, n_tasks, 0, PTHREAD_MUTEX_INITIALIZER};
    pthread_t th[256];
    if (n_threads > 256) n_threads = 256;
    for (int i = 0; i < n_threads; ++i) pthread_create(&th[i], NULL, worker, &q);
    for (int i = 0; i < n_threads; ++i) pthread_join(th[i], NULL);
}

static double now_s(void)
{
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

/* One forward pass over T tokens in the reference's CPU style; returns seconds.
 * Weights [E+Es] experts back to back, fp32 values (already bf16-rounded when emulating bf16). */
double orc_cpu_baseline_forward(const float *x, const float *Wg, const float *bg, const float *W1,
                                const float *W3, const float *W2, int T, int d, int E, int K, int H, int Es,
                                int renorm, int n_threads, float *out)
{
    int P = T * K, G = E + Es;
    size_t rows_total = (size_t)P + (size_t)Es * T;
    /* the product outputs are zero-initialised, as Java's new float[n] is: the beta == 0 update C *= beta of the
     * restated sgemm would turn stale NaN patterns of a recycled heap block into NaN results */
    float *logits = (float *)calloc((size_t)T * E, sizeof(float));
    float *p = (float *)malloc(sizeof(float) * (size_t)T * E);
    int32_t *ids = (int32_t *)malloc(sizeof(int32_t) * (size_t)P);
    float *w = (float *)malloc(sizeof(float) * (size_t)P);
    int32_t *counts = (int32_t *)malloc(sizeof(int32_t) * (size_t)E);
    int32_t *offsets = (int32_t *)malloc(sizeof(int32_t) * (size_t)(E + 1));
    int32_t *dst = (int32_t *)malloc(sizeof(int32_t) * (size_t)P);
    int32_t *src_row = (int32_t *)malloc(sizeof(int32_t) * (size_t)P);
    float *xg = (float *)malloc(sizeof(float) * (size_t)P * d);
    float *h1 = (float *)calloc(rows_total * H, sizeof(float));
    float *h3 = (float *)calloc(rows_total * H, sizeof(float));
    float *y = (float *)calloc(rows_total * d, sizeof(float));
    gemm_task *tasks = (gemm_task *)malloc(sizeof(gemm_task) * (size_t)G);

    double t0 = now_s();
    /* gate: one sgemm task (batch of 1), then bias */
    gemm_task gt = {E, T, d, Wg, x, logits, d, d, E};
    batch_sgemm(&gt, 1, n_threads);
    if (bg)
        for (int t = 0; t < T; ++t)
            for (int e = 0; e < E; ++e) logits[(size_t)t * E + e] += bg[e];
    orc_softmax(logits, T, E, p);
    orc_topk(p, T, E, K, renorm, ids, w);
    orc_dispatch(ids, T, K, E, counts, offsets, dst, src_row);
    orc_gather(x, src_row, P, d, xg);
    for (int pass = 0; pass < 2; ++pass) {
        const float *W = pass == 0 ? W1 : W3;
        float *h = pass == 0 ? h1 : h3;
        for (int g = 0; g < G; ++g) {
            int rows = g < E ? counts[g] : T;
            size_t r0 = g < E ? (size_t)offsets[g] : (size_t)P + (size_t)(g - E) * T;
            const float *B = g < E ? xg + r0 * d : x;
            gemm_task tk = {H, rows, d, W + (size_t)g * H * d, B, h + r0 * H, d, d, H};
            tasks[g] = tk;
        }
        batch_sgemm(tasks, G, n_threads);
    }
    for (size_t i = 0; i < rows_total * (size_t)H; ++i) h1[i] = h1[i] / (1.0f + (float)exp(-(double)h1[i]));
    for (size_t i = 0; i < rows_total * (size_t)H; ++i) h1[i] = h1[i] * h3[i];
    for (int g = 0; g < G; ++g) {
        int rows = g < E ? counts[g] : T;
        size_t r0 = g < E ? (size_t)offsets[g] : (size_t)P + (size_t)(g - E) * T;
        gemm_task tk = {d, rows, H, W2 + (size_t)g * d * H, h1 + r0 * H, y + r0 * d, H, H, d};
        tasks[g] = tk;
    }
    batch_sgemm(tasks, G, n_threads);
    orc_combine(y, dst, w, Es ? y + (size_t)P * d : NULL, T, K, d, Es, 0, out);
    double t1 = now_s();

    free(logits); free(p); free(ids); free(w); free(counts); free(offsets); free(dst); free(src_row);
    free(xg); free(h1); free(h3); free(y); free(tasks);
    return t1 - t0;
}

/* Known-answer hook for the GEMM restatement: C = op(A) B on caller data. */
void orc_cpu_sgemm_tn(int m, int n, int k, const float *A, int lda, const float *B, int ldb, float *C, int ldc,
                      int n_threads)
{
    gemm_task t = {m, n, k, A, B, C, lda, ldb, ldc};
    batch_sgemm(&t, 1, n_threads);
}
