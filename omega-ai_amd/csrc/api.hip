// C ABI of libomega_hip.so: contexts, device memory, the MoE layer handle, its forward stages, its backward pass and update.
#include <stdio.h>
#include <string.h>

#include <new>

#include "common.h"
#include <algorithm>

#define OMEGA_VERSION 100  // 0.1.0

static thread_local std::string g_create_error;

// Staging area of omega_moe_get_router_probs_noalloc: logits in the first half, probabilities in the second.  Every
// device the library runs on holds its own copy of the array for the life of the process; host code never uses the
// array's name as an address - omega_hip_ctx_create asks the runtime for the device's copy (hipGetSymbolAddress) and
// keeps it per device.
#define OMEGA_NOALLOC_MAX_FLOATS (1u << 20)  // T * E may not exceed this: 2 x 4 MiB per device
static __device__ __align__(256) float scratch[2 * (size_t)OMEGA_NOALLOC_MAX_FLOATS];
#define OMEGA_MAX_DEVICES 64
static float *g_scratch_ptr[OMEGA_MAX_DEVICES];  // by device ordinal; written under g_scratch_mu
static std::mutex g_scratch_mu;

int omega_set_error(omega_ctx *ctx, int status, const char *what, hipError_t herr, const char *file, int line)
{
    char buf[512];
    const char *base = strrchr(file, '/');
    if (herr != hipSuccess)
        snprintf(buf, sizeof buf, "Error code %d:%s (%s at %s:%d)", (int)herr, hipGetErrorString(herr), what,
                 base ? base + 1 : file, line);
    else
        snprintf(buf, sizeof buf, "Error code %d:%s (%s:%d)", status, what, base ? base + 1 : file, line);
    if (ctx) ctx->last_error = buf; else g_create_error = buf;
    return status;
}

extern "C" {

int omega_hip_version(void) { return OMEGA_VERSION; }

const char *omega_hip_last_error(omega_ctx *ctx) { return ctx ? ctx->last_error.c_str() : g_create_error.c_str(); }

int omega_hip_ctx_create(int device, omega_ctx **out)
{
    if (!out) OMEGA_FAIL(nullptr, OMEGA_ERR_INVALID_ARG, "ctx_create: out is NULL");
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0)
        return omega_set_error(nullptr, OMEGA_ERR_HIP, "ctx_create: no HIP device available", e, __FILE__, __LINE__);
    if (device < 0 || device >= n) OMEGA_FAIL(nullptr, OMEGA_ERR_INVALID_ARG, "ctx_create: device index out of range");
    OMEGA_HIP_CHECK(nullptr, hipSetDevice(device));
    hipDeviceProp_t prop;
    OMEGA_HIP_CHECK(nullptr, hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        OMEGA_FAIL(nullptr, OMEGA_ERR_UNSUPPORTED, "ctx_create: device is not gfx950 (MI355X)");
    if (device >= OMEGA_MAX_DEVICES) OMEGA_FAIL(nullptr, OMEGA_ERR_UNSUPPORTED, "ctx_create: device ordinal above 63");
    float *scratch_dev = nullptr;
    {
        // once per device, with that device current: the address of its copy of the static scratch array
        std::lock_guard<std::mutex> lk(g_scratch_mu);
        if (!g_scratch_ptr[device]) {
            void *p = nullptr;
            OMEGA_HIP_CHECK(nullptr, hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
            g_scratch_ptr[device] = (float *)p;
        }
        scratch_dev = g_scratch_ptr[device];
    }
    omega_ctx *c = new (std::nothrow) omega_ctx();
    if (!c) OMEGA_FAIL(nullptr, OMEGA_ERR_OOM, "ctx_create: host allocation failed");
    c->device = device;
    c->noalloc_scratch = scratch_dev;
    c->num_cus = prop.multiProcessorCount;
    e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = experts_bf16_init();
    if (e == hipSuccess) e = router_init();
    if (e != hipSuccess) {
        delete c;
        return omega_set_error(nullptr, OMEGA_ERR_HIP, "ctx_create: stream / kernel attribute setup", e, __FILE__, __LINE__);
    }
    *out = c;
    return OMEGA_OK;
}

int omega_hip_ctx_destroy(omega_ctx *ctx)
{
    if (!ctx) return OMEGA_OK;
    hipSetDevice(ctx->device);
    hipStreamSynchronize(ctx->stream);
    hipStreamDestroy(ctx->stream);
    delete ctx;
    return OMEGA_OK;
}

#define CTX_ENTER(ctx)                                                                      \
    if (!(ctx)) OMEGA_FAIL(nullptr, OMEGA_ERR_INVALID_ARG, "NULL context");                \
    std::lock_guard<std::mutex> _lk((ctx)->mu);                                             \
    OMEGA_HIP_CHECK((ctx), hipSetDevice((ctx)->device))

int omega_hip_malloc(omega_ctx *ctx, size_t bytes, void **dptr)
{
    CTX_ENTER(ctx);
    if (!dptr) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "malloc: dptr is NULL");
    *dptr = nullptr;
    if (bytes == 0) return OMEGA_OK;
    OMEGA_HIP_CHECK(ctx, hipMalloc(dptr, bytes));
    return OMEGA_OK;
}

int omega_hip_free(omega_ctx *ctx, void *dptr)
{
    CTX_ENTER(ctx);
    if (!dptr) return OMEGA_OK;
    OMEGA_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    OMEGA_HIP_CHECK(ctx, hipFree(dptr));
    return OMEGA_OK;
}

int omega_hip_memcpy_h2d(omega_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes)
{
    CTX_ENTER(ctx);
    if (bytes == 0) return OMEGA_OK;
    if (!dst_dev || !src_host) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "memcpy_h2d: NULL pointer");
    OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
    OMEGA_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    return OMEGA_OK;
}

int omega_hip_memcpy_d2h(omega_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes)
{
    CTX_ENTER(ctx);
    if (bytes == 0) return OMEGA_OK;
    if (!dst_host || !src_dev) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "memcpy_d2h: NULL pointer");
    OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    OMEGA_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    return OMEGA_OK;
}

int omega_hip_memset(omega_ctx *ctx, void *dptr, int value, size_t bytes)
{
    CTX_ENTER(ctx);
    if (bytes == 0) return OMEGA_OK;
    if (!dptr) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "memset: NULL pointer");
    OMEGA_HIP_CHECK(ctx, hipMemsetAsync(dptr, value, bytes, ctx->stream));
    return OMEGA_OK;
}

int omega_hip_sync(omega_ctx *ctx)
{
    CTX_ENTER(ctx);
    OMEGA_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    return OMEGA_OK;
}

static bool dtype_ok(int dt) { return dt == OMEGA_DTYPE_F32 || dt == OMEGA_DTYPE_BF16; }

int omega_hip_fill_normal(omega_ctx *ctx, void *dptr, uint64_t n, uint64_t seed, uint64_t stream, double std,
                          uint64_t first, int dtype)
{
    CTX_ENTER(ctx);
    if (n == 0) return OMEGA_OK;
    if (!dptr || !dtype_ok(dtype)) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "fill_normal: bad pointer or dtype");
    OMEGA_HIP_CHECK(ctx, launch_fill_normal(dptr, n, seed, stream, std, first, dtype, ctx->stream));
    return OMEGA_OK;
}

int omega_hip_convert(omega_ctx *ctx, void *dst, int dst_dtype, const void *src, int src_dtype, uint64_t n)
{
    CTX_ENTER(ctx);
    if (n == 0) return OMEGA_OK;
    if (!dst || !src || !dtype_ok(dst_dtype) || !dtype_ok(src_dtype))
        OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "convert: bad pointer or dtype");
    OMEGA_HIP_CHECK(ctx, launch_convert(dst, dst_dtype, src, src_dtype, n, ctx->stream));
    return OMEGA_OK;
}

// ------------------------------------------------------------------------------------------ layer

static void moe_free_backward_workspace(omega_moe *m)
{
    void **bw[] = {(void **)&m->bw_probs, (void **)&m->bw_dw, (void **)&m->bw_dlogits, (void **)&m->bw_gpart, (void **)&m->bw_dy, (void **)&m->bw_h1,
                   (void **)&m->bw_h3, (void **)&m->bw_dxg, &m->bw_dhx, &m->bw_dy16, &m->bw_dys16, &m->bw_dh16, &m->bw_dyT, &m->bw_aT,
                   &m->bw_xgT, &m->bw_dhT, (void **)&m->bw_kt0, (void **)&m->desc_da, (void **)&m->wq_da,
                   (void **)&m->desc_w2, (void **)&m->wq_w2, (void **)&m->desc_w13, (void **)&m->wq_w13};
    for (void **p : bw) {
        if (*p) hipFree(*p);
        *p = nullptr;
    }
    m->bw_T_cap = 0;
    m->bw_rows_cap = 0;
    m->bw_ksteps_cap = 0;
}

static void moe_free_workspace(omega_moe *m)
{
    void *ptrs[] = {m->ids, m->w, m->tile_counts, m->dst, m->dstp, m->src_row, m->tiles, m->xg, m->xs, m->a, m->y,
                    m->desc_up, m->desc_down, m->wq_up, m->wq_down, m->rms, m->hbuf, m->tokp};
    for (void *p : ptrs)
        if (p) hipFree(p);
    m->ids = nullptr; m->w = nullptr; m->tile_counts = nullptr; m->dst = nullptr; m->dstp = nullptr; m->src_row = nullptr; m->xs = nullptr; m->desc_up = nullptr; m->desc_down = nullptr; m->wq_up = nullptr; m->wq_down = nullptr; m->rms = nullptr; m->hbuf = nullptr;
    m->tiles = nullptr; m->xg = nullptr; m->a = nullptr; m->y = nullptr; m->tokp = nullptr;
    m->xg_valid = false;
    m->T_cap = 0;
    moe_free_backward_workspace(m);
    m->fwd_T = -1;
    m->routed_T = m->dispatched_T = -1;
}

static size_t grad_block_floats(const omega_moe *m)
{
    const omega_moe_config &c = m->cfg;
    // dWg, dbg and dgamma (each rounded up to whole 16-byte units, so the expert gradients stay 16-byte aligned), dW13, dW2
    return (size_t)c.E * c.d + (size_t)((c.E + 3) & ~3) + (size_t)((c.d + 3) & ~3) + 3 * (size_t)m->G * c.H * c.d;
}

// Gradient buffers (once) and the workspace of the backward pass for the current forward workspace.
static int moe_reserve_backward(omega_moe *m, int T)
{
    omega_ctx *ctx = m->ctx;
    const omega_moe_config &c = m->cfg;
    const bool bf = c.dtype == OMEGA_DTYPE_BF16;
    const size_t HD = (size_t)c.H * c.d;
    if (!m->dWg) {
        float *blk = nullptr;
        OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&blk, grad_block_floats(m) * 4));
        OMEGA_HIP_CHECK(ctx, hipMemsetAsync(blk, 0, grad_block_floats(m) * 4, ctx->stream));
        m->dWg = blk;
        m->dbg = m->dWg + (size_t)c.E * c.d;
        m->dgamma = m->dbg + ((c.E + 3) & ~3);
        m->dW13 = m->dgamma + ((c.d + 3) & ~3);
        m->dW2 = m->dW13 + 2 * (size_t)m->G * HD;
        OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->bw_zero_state, (size_t)2 * m->G * 4));
        OMEGA_HIP_CHECK(ctx, hipMemsetAsync(m->bw_zero_state, 0, (size_t)2 * m->G * 4, ctx->stream));
        m->bw_zero_valid = false;
    }
    if (bf && !m->W2T) {
        // one row group of slack behind W2T: the last 256-column tile of a width H = 128 mod 256 reads it (and drops it)
        OMEGA_HIP_CHECK(ctx, hipMalloc(&m->W2T, ((size_t)m->G * HD + (size_t)128 * c.d) * 2));
        OMEGA_HIP_CHECK(ctx, hipMemsetAsync(m->W2T, 0, ((size_t)m->G * HD + (size_t)128 * c.d) * 2, ctx->stream));
        OMEGA_HIP_CHECK(ctx, hipMalloc(&m->W13T, (size_t)m->G * 2 * HD * 2));
        m->wT_valid = false;
    }
    if (bf && !m->wT_valid) {
        // W2[g] [d,H] -> W2T[g] [H,d];  W1[g], W3[g] [H,d] -> W13T[g] [d, H | H]
        OMEGA_HIP_CHECK(ctx, launch_transpose_images(m->W2, c.d, c.H, m->W2T, c.d / 32, 0, m->G, HD * 2, HD * 2, ctx->stream));
        OMEGA_HIP_CHECK(ctx, launch_transpose_images(m->W1, c.H, c.d, m->W13T, 2 * c.H / 32, 0, m->G, HD * 2, 2 * HD * 2, ctx->stream));
        OMEGA_HIP_CHECK(ctx, launch_transpose_images(m->W3, c.H, c.d, m->W13T, 2 * c.H / 32, c.H / 32, m->G, HD * 2, 2 * HD * 2, ctx->stream));
        m->wT_valid = true;
    }
    if (m->bw_T_cap >= T && m->bw_rows_cap >= m->rows_cap) return OMEGA_OK;
    OMEGA_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    moe_free_backward_workspace(m);
    const int Tc = m->T_cap;
    const size_t rc = m->rows_cap;
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->bw_probs, (size_t)Tc * c.E * 4));
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->bw_dw, (size_t)Tc * c.K * 4));
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->bw_dlogits, (size_t)Tc * c.E * 4));
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->bw_gpart, (size_t)32 * c.E * c.d * 4));
    OMEGA_HIP_CHECK(ctx, hipMalloc(&m->bw_dhx, (size_t)Tc * c.d * m->esize));
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->bw_h1, rc * c.H * 4));
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->bw_h3, rc * c.H * 4));
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->bw_dxg, rc * c.d * 4));
    if (!bf) {
        OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->bw_dy, rc * c.d * 4));
    } else {
        const int bm = m->bm ? m->bm : 256;
        auto alloc0 = [&](void **p, size_t bytes) -> hipError_t {
            hipError_t e = hipMalloc(p, bytes);
            return e != hipSuccess ? e : hipMemsetAsync(*p, 0, bytes, ctx->stream);
        };
        // row images: padding rows are read by the products (results dropped): keep them finite
        OMEGA_HIP_CHECK(ctx, alloc0(&m->bw_dy16, rc * c.d * 2));
        OMEGA_HIP_CHECK(ctx, alloc0(&m->bw_dh16, rc * 2 * c.H * 2));
        if (c.Es > 0) OMEGA_HIP_CHECK(ctx, alloc0(&m->bw_dys16, (size_t)ceil_div(Tc, bm) * bm * c.d * 2));
        // transposed images over k space (see bw_tables_kernel): at most 8 k steps of rounding per group; one row
        // group of slack behind aT for the last column tile of a width H = 128 mod 256
        m->bw_ksteps_cap = (int)(rc / 32) + 8 * m->G;
        const size_t kb = (size_t)m->bw_ksteps_cap * 64;  // bytes of one image row
        OMEGA_HIP_CHECK(ctx, alloc0(&m->bw_dyT, (size_t)c.d * kb));
        OMEGA_HIP_CHECK(ctx, alloc0(&m->bw_aT, (size_t)(c.H + 128) * kb));
        OMEGA_HIP_CHECK(ctx, alloc0(&m->bw_xgT, (size_t)c.d * kb));
        OMEGA_HIP_CHECK(ctx, alloc0(&m->bw_dhT, (size_t)2 * c.H * kb));
        OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->bw_kt0, (size_t)(m->G + 1) * 4));
        const int nH = ceil_div(c.H, 256);
        const size_t n_da = (size_t)m->tiles_cap * nH + OMEGA_TAIL_EXTRA;
        const size_t n_w2 = (size_t)m->G * (c.d / 256) * nH, n_w13 = (size_t)m->G * (2 * c.H / 256) * (c.d / 256);
        OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->desc_da, n_da * sizeof(omega_tile_desc)));
        OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->desc_w2, n_w2 * sizeof(omega_tile_desc)));
        OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->desc_w13, n_w13 * sizeof(omega_tile_desc)));
        OMEGA_HIP_CHECK(ctx, alloc0((void **)&m->wq_da, (n_da / m->n_wg + 2) * m->n_wg * sizeof(omega_tile_desc)));
        OMEGA_HIP_CHECK(ctx, alloc0((void **)&m->wq_w2, (n_w2 / m->n_wg + 2) * m->n_wg * sizeof(omega_tile_desc)));
        OMEGA_HIP_CHECK(ctx, alloc0((void **)&m->wq_w13, (n_w13 / m->n_wg + 2) * m->n_wg * sizeof(omega_tile_desc)));
    }
    m->bw_T_cap = Tc;
    m->bw_rows_cap = rc;
    return OMEGA_OK;
}

static int moe_tile_m(const omega_moe *m, int T)
{
    return m->cfg.dtype == OMEGA_DTYPE_BF16 ? experts_bf16_tile_m(m, T) : experts_f32_tile_m();
}

static int moe_max_m_tiles(const omega_moe *m, int T, int bm)
{
    const omega_moe_config &c = m->cfg;
    return (T * c.K) / bm + c.E + c.Es * ceil_div(T, bm);
}

// Sizes the workspace for T tokens (grow-only, like the named caches of
// J/engine/gpu/CUDAMemoryManager.java:34-55).
static int moe_reserve(omega_moe *m, int T)
{
    omega_ctx *ctx = m->ctx;
    if (T <= m->T_cap) return OMEGA_OK;
    OMEGA_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    moe_free_workspace(m);
    const omega_moe_config &c = m->cfg;
    const size_t P = (size_t)T * c.K;
    const int n_tok_tiles = ceil_div(T, router_tok_tile(c.E));
    const int bm = moe_tile_m(m, T);
    // every expert's rows start on a row-tile boundary: the buffers hold whole tiles
    m->tiles_cap = moe_max_m_tiles(m, T, bm);
    m->rows_cap = (size_t)m->tiles_cap * bm;
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->ids, P * 4));
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->w, P * 4));
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->rms, (size_t)T * 4));
    OMEGA_HIP_CHECK(ctx, hipMalloc(&m->hbuf, (size_t)T * c.d * m->esize));
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->tile_counts, (size_t)n_tok_tiles * c.E * 4));
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->dst, P * 4));
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->dstp, P * 4));
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->src_row, P * 4));
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->tokp, m->rows_cap * 4));
    OMEGA_HIP_CHECK(ctx, hipMemsetAsync(m->tokp, 0, m->rows_cap * 4, ctx->stream));
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->tiles, (size_t)m->tiles_cap * sizeof(omega_tile)));
    OMEGA_HIP_CHECK(ctx, hipMalloc(&m->xg, m->rows_cap * c.d * m->esize));
    OMEGA_HIP_CHECK(ctx, hipMalloc(&m->a, m->rows_cap * c.H * m->esize));
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->y, m->rows_cap * c.d * 4));
    // padding rows of xg / a are read by the product kernels (their results are discarded): keep them finite
    OMEGA_HIP_CHECK(ctx, hipMemsetAsync(m->xg, 0, m->rows_cap * c.d * m->esize, ctx->stream));
    OMEGA_HIP_CHECK(ctx, hipMemsetAsync(m->a, 0, m->rows_cap * c.H * m->esize, ctx->stream));
    if (c.dtype == OMEGA_DTYPE_BF16) {
        OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->desc_up, ((size_t)m->tiles_cap * (c.H / 128) + OMEGA_TAIL_EXTRA) * sizeof(omega_tile_desc)));
        m->n_wg = std::min(256, ctx->num_cus / 8 * 8);
        // (room for the half-width items of small batches: at most n_wg of them)
        OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->desc_down, (std::max((size_t)m->tiles_cap * (c.d / 256), (size_t)m->n_wg) + OMEGA_TAIL_EXTRA) * sizeof(omega_tile_desc)));
        const size_t q_up = ((size_t)m->tiles_cap * (c.H / 128) + OMEGA_TAIL_EXTRA) / m->n_wg + 2;
        const size_t q_down = (std::max((size_t)m->tiles_cap * (c.d / 256), (size_t)m->n_wg) + OMEGA_TAIL_EXTRA) / m->n_wg + 2;
        OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->wq_up, q_up * m->n_wg * sizeof(omega_tile_desc)));
        OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->wq_down, q_down * m->n_wg * sizeof(omega_tile_desc)));
        // partial results of k-sliced items of the down product: sliced entries never exceed 256, each a tile of 256 x 256
        if (!m->y_slabs) OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->y_slabs, (size_t)256 * 256 * 256 * 4));
        // an all-zero queue is an empty one: the product kernels return at once if no dispatch has run yet
        OMEGA_HIP_CHECK(ctx, hipMemsetAsync(m->wq_up, 0, q_up * m->n_wg * sizeof(omega_tile_desc), ctx->stream));
        OMEGA_HIP_CHECK(ctx, hipMemsetAsync(m->wq_down, 0, q_down * m->n_wg * sizeof(omega_tile_desc), ctx->stream));
    }
    if (c.dtype == OMEGA_DTYPE_BF16 && c.Es > 0) {
        const size_t xs_rows = (size_t)ceil_div(T, bm) * bm;
        OMEGA_HIP_CHECK(ctx, hipMalloc(&m->xs, xs_rows * c.d * m->esize));
        OMEGA_HIP_CHECK(ctx, hipMemsetAsync(m->xs, 0, xs_rows * c.d * m->esize, ctx->stream));
    }
    m->T_cap = T;
    return OMEGA_OK;
}

int omega_moe_create(omega_ctx *ctx, const omega_moe_config *cfg, omega_moe **out)
{
    CTX_ENTER(ctx);
    if (!cfg || !out) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "moe_create: NULL argument");
    *out = nullptr;
    const omega_moe_config &c = *cfg;
    if (c.T_max < 0 || c.d <= 0 || c.E <= 0 || c.K <= 0 || c.H <= 0 || c.Es < 0)
        OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "moe_create: dimensions must be positive");
    if (c.K > c.E) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "moe_create: K must not exceed E");
    if (!dtype_ok(c.dtype)) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "moe_create: unknown dtype");
    if (c.router_mode != OMEGA_ROUTER_EXACT && c.router_mode != OMEGA_ROUTER_FAST)
        OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "moe_create: unknown router mode");
    if (c.E > 256) OMEGA_FAIL(ctx, OMEGA_ERR_UNSUPPORTED, "moe_create: more than 256 routed experts");
    if (c.Es > 64) OMEGA_FAIL(ctx, OMEGA_ERR_UNSUPPORTED, "moe_create: more than 64 shared experts");
    if (c.K > 64 || (c.E <= 8 && c.K > 8)) OMEGA_FAIL(ctx, OMEGA_ERR_UNSUPPORTED, "moe_create: K above 64");
    if (c.dtype == OMEGA_DTYPE_BF16 && (c.d % 256 != 0 || c.H % 128 != 0 || c.H < 256))
        OMEGA_FAIL(ctx, OMEGA_ERR_UNSUPPORTED, "moe_create: bf16 layers need d % 256 == 0, H % 128 == 0 and H >= 256");
    if ((double)c.T_max * c.K * (double)(c.d > c.H ? c.d : c.H) > 2.0e9)
        OMEGA_FAIL(ctx, OMEGA_ERR_UNSUPPORTED, "moe_create: T_max*K*max(d,H) exceeds 2e9 elements");

    omega_moe *m = new (std::nothrow) omega_moe();
    if (!m) OMEGA_FAIL(ctx, OMEGA_ERR_OOM, "moe_create: host allocation failed");
    m->ctx = ctx;
    m->cfg = c;
    m->G = c.E + c.Es;
    m->esize = c.dtype == OMEGA_DTYPE_BF16 ? 2 : 4;
    const size_t wsz = (size_t)m->G * c.H * c.d * m->esize;
    hipError_t e = hipSuccess;
    auto alloc0 = [&](void **p, size_t bytes) {
        if (e != hipSuccess) return;
        e = hipMalloc(p, bytes);
        if (e == hipSuccess) e = hipMemsetAsync(*p, 0, bytes, ctx->stream);
    };
    alloc0(&m->Wg, (size_t)c.E * c.d * m->esize);
    alloc0((void **)&m->bg, (size_t)c.E * 4);
    alloc0((void **)&m->gamma, (size_t)c.d * 4);
    alloc0(&m->W1, wsz);
    alloc0(&m->W3, wsz);
    alloc0(&m->W2, wsz);
    alloc0((void **)&m->counts, (size_t)c.E * 4);
    alloc0((void **)&m->offsets, (size_t)(c.E + 1) * 4);
    alloc0((void **)&m->tile_meta, (size_t)(m->G + 10) * 4);
    if (e == hipSuccess) e = hipEventCreate(&m->ev0);
    if (e == hipSuccess) e = hipEventCreate(&m->ev1);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        omega_set_error(ctx, e == hipErrorOutOfMemory ? OMEGA_ERR_OOM : OMEGA_ERR_HIP, "moe_create: allocation", e,
                        __FILE__, __LINE__);
        // release whatever was allocated
        void *ptrs[] = {m->Wg, m->bg, m->W1, m->W3, m->W2, m->counts, m->offsets, m->tile_meta, m->gamma};
        for (void *p : ptrs)
            if (p) hipFree(p);
        if (m->ev0) hipEventDestroy(m->ev0);
        if (m->ev1) hipEventDestroy(m->ev1);
        delete m;
        return e == hipErrorOutOfMemory ? OMEGA_ERR_OOM : OMEGA_ERR_HIP;
    }
    if (c.T_max > 0) {
        int st = moe_reserve(m, c.T_max);
        if (st != OMEGA_OK) {
            moe_free_workspace(m);
            void *ptrs[] = {m->Wg, m->bg, m->W1, m->W3, m->W2, m->counts, m->offsets, m->tile_meta, m->gamma};
            for (void *p : ptrs)
                if (p) hipFree(p);
            hipEventDestroy(m->ev0);
            hipEventDestroy(m->ev1);
            delete m;
            return st;
        }
    }
    *out = m;
    return OMEGA_OK;
}

int omega_moe_destroy(omega_moe *m)
{
    if (!m) return OMEGA_OK;
    omega_ctx *ctx = m->ctx;
    CTX_ENTER(ctx);
    hipStreamSynchronize(ctx->stream);
    moe_free_workspace(m);
    void *ptrs[] = {m->Wg, m->bg, m->W1, m->W3, m->W2, m->counts, m->offsets, m->tile_meta, m->gamma};
    for (void *p : ptrs)
        if (p) hipFree(p);
    if (m->dWg) hipFree(m->dWg);
    if (m->acc_grad) hipFree(m->acc_grad);
    if (m->sumsq_part) hipFree(m->sumsq_part);
    if (m->bw_zero_state) hipFree(m->bw_zero_state);
    if (m->y_slabs) hipFree(m->y_slabs);
    if (m->adam_m) hipFree(m->adam_m);
    if (m->adam_v) hipFree(m->adam_v);
    if (m->master) hipFree(m->master);
    if (m->W2T) hipFree(m->W2T);
    if (m->W13T) hipFree(m->W13T);
    hipEventDestroy(m->ev0);
    hipEventDestroy(m->ev1);
    for (hipEvent_t ev : m->prof_events) hipEventDestroy(ev);
    delete m;
    return OMEGA_OK;
}

static int weight_slot(omega_moe *m, int which, int expert, void **ptr, size_t *bytes)
{
    const omega_moe_config &c = m->cfg;
    const size_t per = (size_t)c.H * c.d * m->esize;
    switch (which) {
        case OMEGA_W_GATE: *ptr = m->Wg; *bytes = (size_t)c.E * c.d * m->esize; return OMEGA_OK;
        case OMEGA_W_GATE_BIAS: *ptr = m->bg; *bytes = (size_t)c.E * 4; return OMEGA_OK;
        case OMEGA_W_NORM: *ptr = m->gamma; *bytes = (size_t)c.d * 4; return OMEGA_OK;
        case OMEGA_W_W1: case OMEGA_W_W3: case OMEGA_W_W2: {
            if (expert < 0 || expert >= m->G) return OMEGA_ERR_INVALID_ARG;
            unsigned char *base = (unsigned char *)(which == OMEGA_W_W1 ? m->W1 : which == OMEGA_W_W3 ? m->W3 : m->W2);
            *ptr = base + per * (size_t)expert;
            *bytes = per;
            return OMEGA_OK;
        }
        default: return OMEGA_ERR_INVALID_ARG;
    }
}

static bool weight_is_packed(const omega_moe *m, int which)
{
    return m->cfg.dtype == OMEGA_DTYPE_BF16 && (which == OMEGA_W_W1 || which == OMEGA_W_W3 || which == OMEGA_W_W2);
}

// bf16 expert weights are stored as the packed tile image the product kernels load (pack.h); the caller
// always sees the [out,in] row-major layout of J/engine/nn/layer/FullyLayer.java:181.
int omega_moe_set_weights(omega_moe *m, int which, int expert, const void *src, int is_device)
{
    if (!m) OMEGA_FAIL(nullptr, OMEGA_ERR_INVALID_ARG, "NULL layer");
    omega_ctx *ctx = m->ctx;
    CTX_ENTER(ctx);
    void *p; size_t bytes;
    if (!src || weight_slot(m, which, expert, &p, &bytes) != OMEGA_OK)
        OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "set_weights: bad kind, expert index or source");
    m->master_valid = false;  // fp32 master copies of a bf16 layer are remade from the weights at the next update
    // the activations (and, in training mode, the h1 / h3 records) of the last forward belong to the old weights: a
    // backward pass needs a new forward first
    m->fwd_T = -1;
    m->fwd_block = false;
    m->rec_valid = false;
    if (!weight_is_packed(m, which)) {
        OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(p, src, bytes, is_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice, ctx->stream));
        OMEGA_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
        if (which == OMEGA_W_NORM) m->gamma_set = true;
        return OMEGA_OK;
    }
    const int R = which == OMEGA_W_W2 ? m->cfg.d : m->cfg.H, Kd = which == OMEGA_W_W2 ? m->cfg.H : m->cfg.d;
    m->wT_valid = false;  // the transposed copies of the backward pass are rebuilt by the next backward
    void *stage = nullptr;
    if (!is_device) {
        OMEGA_HIP_CHECK(ctx, hipMalloc(&stage, bytes));
        hipError_t e = hipMemcpyAsync(stage, src, bytes, hipMemcpyHostToDevice, ctx->stream);
        if (e != hipSuccess) { hipFree(stage); OMEGA_HIP_CHECK(ctx, e); }
    }
    hipError_t e = launch_pack_rows(p, is_device ? src : stage, R, Kd, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (stage) hipFree(stage);
    OMEGA_HIP_CHECK(ctx, e);
    return OMEGA_OK;
}

int omega_moe_get_weights(omega_moe *m, int which, int expert, void *dst, int is_device)
{
    if (!m) OMEGA_FAIL(nullptr, OMEGA_ERR_INVALID_ARG, "NULL layer");
    omega_ctx *ctx = m->ctx;
    CTX_ENTER(ctx);
    void *p; size_t bytes;
    if (!dst || weight_slot(m, which, expert, &p, &bytes) != OMEGA_OK)
        OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "get_weights: bad kind, expert index or destination");
    if (!weight_is_packed(m, which)) {
        OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(dst, p, bytes, is_device ? hipMemcpyDeviceToDevice : hipMemcpyDeviceToHost, ctx->stream));
        OMEGA_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
        return OMEGA_OK;
    }
    const int R = which == OMEGA_W_W2 ? m->cfg.d : m->cfg.H, Kd = which == OMEGA_W_W2 ? m->cfg.H : m->cfg.d;
    void *stage = nullptr;
    if (!is_device) OMEGA_HIP_CHECK(ctx, hipMalloc(&stage, bytes));
    hipError_t e = launch_unpack_rows(is_device ? dst : stage, p, R, Kd, ctx->stream);
    if (e == hipSuccess && !is_device) e = hipMemcpyAsync(dst, stage, bytes, hipMemcpyDeviceToHost, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (stage) hipFree(stage);
    OMEGA_HIP_CHECK(ctx, e);
    return OMEGA_OK;
}

// ---- stages (caller holds the context lock) ----
// Whether the up product should fetch the rows of x itself instead of reading a gathered copy: its A loads then read
// 64-byte pieces of rows (half a line each), which costs the product 1-8 %, and the gather (K row copies per token) is
// saved.  Every row tile is read once per column tile, H/128 times; the gather writes K rows per token: worth it while
// H/128 <= 2 K.  Measured (forward pass): 16384 tokens, 128 experts, K = 8, H = 768: 1.63 -> 1.49 ms; 8192 tokens, 64
// experts, K = 6, H = 1408: 1.244 -> 1.234 ms; 4096 tokens, 8 experts, K = 2, H = 14336: 2.32 -> 2.35 ms (not taken).
static bool gather_on_load_wanted(const omega_moe *m)
{
    if (m->gather_mode != OMEGA_GATHER_AUTO) return m->gather_mode == OMEGA_GATHER_ON_LOAD;
    return m->cfg.H / 128 <= 2 * m->cfg.K;
}
static int check_T(omega_moe *m, const void *x, int T, bool need_x)
{
    omega_ctx *ctx = m->ctx;
    if (T < 0) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "forward: negative token count");
    if (need_x && T > 0 && !x) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "forward: x is NULL");
    if ((double)T * m->cfg.K * (double)(m->cfg.d > m->cfg.H ? m->cfg.d : m->cfg.H) > 2.0e9)
        OMEGA_FAIL(ctx, OMEGA_ERR_UNSUPPORTED, "forward: T*K*max(d,H) exceeds 2e9 elements");
    return OMEGA_OK;
}

// a stage run on its own rewrites part of what a backward pass would read: the last forward no longer counts
static void stage_invalidates(omega_moe *m)
{
    m->fwd_T = -1;
    m->fwd_block = false;
    m->rec_valid = false;
}

static int stage_router(omega_moe *m, const void *x, int T)
{
    // training mode (bf16 layers, backward workspace in place): the probabilities are kept for the backward pass
    float *probs = (m->training && m->cfg.dtype == OMEGA_DTYPE_BF16 && m->bw_T_cap >= T) ? m->bw_probs : nullptr;
    m->routed_T = m->dispatched_T = -1;
    OMEGA_HIP_CHECK(m->ctx, launch_router(m, x, T, nullptr, probs, m->ctx->stream));
    m->routed_T = T;
    return OMEGA_OK;
}
static int stage_dispatch(omega_moe *m, const void *x, int T)
{
    if (m->routed_T != T) OMEGA_FAIL(m->ctx, OMEGA_ERR_INVALID_ARG, "dispatch: the router has not run for this T");
    m->dispatched_T = -1;
    const int bm = moe_tile_m(m, T);
    m->bm = bm;
    m->max_m_tiles = moe_max_m_tiles(m, T, bm);
    if (m->cfg.dtype == OMEGA_DTYPE_BF16) {
        // A batch whose down product has output tiles for at most half of the compute units is bound by the weight
        // bytes each workgroup keeps in flight.  With H >= 512 the table builder then cuts every tile's k range into
        // up to 8 slices (as many as fill the compute units; it knows how many experts have rows), which write partial
        // results that a small kernel adds up; narrower layers get 128-column items instead.
        // (The host knows only bounds of the number of row tiles: slicing is switched on when the fewest tiles this
        //  batch can have would qualify, and the table builder decides by the tiles there are.)
        const omega_moe_config &c = m->cfg;
        const int min_tiles = ceil_div(T * c.K, bm) + c.Es * ceil_div(T, bm);
        const bool small = m->max_m_tiles * (c.d / 256) <= m->n_wg / 2;
        m->down_ks_max = min_tiles * (c.d / 256) <= m->n_wg / 2 && c.H >= 512 ? 8 : 1;
        m->down_cols = small && m->down_ks_max == 1 ? 128 : 256;
        // A large batch whose last round of output tiles would occupy at most half of the compute units: those tiles
        // are cut into up to 4 k slices (rather than row slices, which stream the whole weight tile for a quarter of
        // the rows and are bound by that stream), if a slice keeps at least 64 k steps.
        m->down_tail_ks = (m->down_ks_max == 1 && !small && c.H >= 2 * 64 * 32) ? 4 : 1;
    }
    if (m->max_m_tiles > m->tiles_cap) OMEGA_FAIL(m->ctx, OMEGA_ERR_INVALID_ARG, "dispatch: workspace too small for this T");
    // bf16 layers outside training: the up product fetches the rows of x through the row -> token table itself, so the
    // gathered copy xg (and the packed copy xs for shared experts) is neither written nor read; it is made on demand
    // for what still wants it (a backward pass, omega_moe_get_workspace).  A lane's offset into x is 32 bits wide.
    m->gather_on_load = m->cfg.dtype == OMEGA_DTYPE_BF16 && !m->training && gather_on_load_wanted(m) &&
                        (double)T * m->cfg.d * 2.0 < 4.0e9;
    m->xg_valid = false;
    m->last_x = x;
    // (bf16 layers: the index launch copies the rows as well; fp32 layers gather in a launch of its own)
    const bool bf = m->cfg.dtype == OMEGA_DTYPE_BF16;
    OMEGA_HIP_CHECK(m->ctx, launch_dispatch_index(m, T, bm, m->ctx->stream, bf && !m->gather_on_load ? x : nullptr));
    if (!bf) OMEGA_HIP_CHECK(m->ctx, launch_dispatch_gather(m, x, T, m->ctx->stream));
    m->xg_valid = !m->gather_on_load;
    m->dispatched_T = T;
    return OMEGA_OK;
}
// the gathered rows xg / xs of the batch the dispatch stage last ran for, if the forward pass went without them
static int ensure_gathered(omega_moe *m, const void *x, int T)
{
    if (m->xg_valid) return OMEGA_OK;
    if (!x) OMEGA_FAIL(m->ctx, OMEGA_ERR_INVALID_ARG, "the gathered rows need the layer input of the last dispatch");
    OMEGA_HIP_CHECK(m->ctx, launch_dispatch_gather(m, x, T, m->ctx->stream));
    m->xg_valid = true;
    return OMEGA_OK;
}
// x: the rows the shared experts read in fp32 layers (bf16 layers read the packed copy the gather left in xs)
static int stage_experts(omega_moe *m, const void *x, int T, int which)
{
    if (m->dispatched_T != T || m->bm != moe_tile_m(m, T))
        OMEGA_FAIL(m->ctx, OMEGA_ERR_INVALID_ARG, "experts: dispatch has not run for this T");
    if (which == 0 && m->gather_on_load && !x) OMEGA_FAIL(m->ctx, OMEGA_ERR_INVALID_ARG, "experts: x is NULL");
    if (which == 1 && !m->a_valid) OMEGA_FAIL(m->ctx, OMEGA_ERR_INVALID_ARG, "experts_down: the up product has not run since `a` was overwritten");
    if (m->cfg.dtype == OMEGA_DTYPE_BF16) OMEGA_HIP_CHECK(m->ctx, launch_experts_bf16(m, x, T, which, m->ctx->stream));
    else OMEGA_HIP_CHECK(m->ctx, launch_experts_f32(m, x, T, which, m->ctx->stream));
    if (which == 0) m->a_valid = true;
    else m->y_valid = true;
    return OMEGA_OK;
}
static int stage_combine(omega_moe *m, int T, void *out, const void *resid)
{
    if (m->dispatched_T != T) OMEGA_FAIL(m->ctx, OMEGA_ERR_INVALID_ARG, "combine: dispatch has not run for this T");
    if (!m->y_valid) OMEGA_FAIL(m->ctx, OMEGA_ERR_INVALID_ARG, "combine: the down product has not run since `y` was overwritten");
    OMEGA_HIP_CHECK(m->ctx, launch_combine(m, T, out, resid, m->ctx->stream));
    return OMEGA_OK;
}

#define MOE_ENTER(m)                                                          \
    if (!(m)) OMEGA_FAIL(nullptr, OMEGA_ERR_INVALID_ARG, "NULL layer");      \
    omega_ctx *ctx = (m)->ctx;                                                \
    CTX_ENTER(ctx)

#define RUN(expr)                         \
    do {                                  \
        int _st = (expr);                 \
        if (_st != OMEGA_OK) return _st;  \
    } while (0)

static int forward_impl(omega_moe *m, const void *x, int T, void *out, int block)
{
    omega_ctx *ctx = m->ctx;
    RUN(check_T(m, x, T, true));
    if (T == 0) return OMEGA_OK;
    if (!out) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "forward: out is NULL");
    if (block && !m->gamma_set) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "forward_block: the norm weight (OMEGA_W_NORM) has not been set");
    RUN(moe_reserve(m, T));
    // block form: the layer runs on the normalised rows h (one small kernel writes them and rms), the combine adds x back
    const void *resid = block ? x : nullptr;
    const void *xin = block ? m->hbuf : x;
    m->fwd_T = T;
    m->fwd_block = block != 0;
    // training mode (bf16 layers): the up product also leaves h1 / h3 for the backward pass
    const bool keep = m->training && m->cfg.dtype == OMEGA_DTYPE_BF16;
    if (keep) {
        m->bm = moe_tile_m(m, T);
        RUN(moe_reserve_backward(m, T));
    }
    m->rec_valid = false;
    if (m->profiling) {
        // six events bracket the five stages; durations are read back by omega_moe_get_profile
        if (m->prof_used + 6 > m->prof_events.size()) {
            for (int i = 0; i < 6; ++i) {
                hipEvent_t ev;
                OMEGA_HIP_CHECK(ctx, hipEventCreate(&ev));
                m->prof_events.push_back(ev);
            }
        }
        hipEvent_t *ev = &m->prof_events[m->prof_used];
        OMEGA_HIP_CHECK(ctx, hipEventRecord(ev[0], ctx->stream));
        if (block) OMEGA_HIP_CHECK(ctx, launch_rmsnorm(m, x, T, m->hbuf, ctx->stream));
        RUN(stage_router(m, xin, T));
        OMEGA_HIP_CHECK(ctx, hipEventRecord(ev[1], ctx->stream));
        RUN(stage_dispatch(m, xin, T));
        OMEGA_HIP_CHECK(ctx, hipEventRecord(ev[2], ctx->stream));
        RUN(stage_experts(m, xin, T, 0));
        OMEGA_HIP_CHECK(ctx, hipEventRecord(ev[3], ctx->stream));
        RUN(stage_experts(m, xin, T, 1));
        OMEGA_HIP_CHECK(ctx, hipEventRecord(ev[4], ctx->stream));
        RUN(stage_combine(m, T, out, resid));
        OMEGA_HIP_CHECK(ctx, hipEventRecord(ev[5], ctx->stream));
        m->prof_used += 6;
        m->rec_valid = keep;
        return OMEGA_OK;
    }
    if (block) OMEGA_HIP_CHECK(ctx, launch_rmsnorm(m, x, T, m->hbuf, ctx->stream));
    RUN(stage_router(m, xin, T));
    RUN(stage_dispatch(m, xin, T));
    RUN(stage_experts(m, xin, T, 0));
    RUN(stage_experts(m, xin, T, 1));
    RUN(stage_combine(m, T, out, resid));
    m->rec_valid = keep;
    return OMEGA_OK;
}

int omega_moe_set_training(omega_moe *m, int on)
{
    MOE_ENTER(m);
    if (m->training != (on != 0)) m->dispatched_T = -1;  // the dispatch stage prepares different things for the two modes
    m->training = on != 0;
    m->rec_valid = false;
    return OMEGA_OK;
}

int omega_moe_set_gather_mode(omega_moe *m, int mode)
{
    MOE_ENTER(m);
    if (mode != OMEGA_GATHER_AUTO && mode != OMEGA_GATHER_COPY && mode != OMEGA_GATHER_ON_LOAD)
        OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "set_gather_mode: unknown mode");
    if (m->gather_mode != mode) m->dispatched_T = -1;  // the dispatch stage prepares different things for the two forms
    m->gather_mode = mode;
    return OMEGA_OK;
}

int omega_moe_gather_on_load(omega_moe *m) { return m != nullptr && m->gather_on_load ? 1 : 0; }

int omega_moe_forward(omega_moe *m, const void *x, int T, void *out)
{
    MOE_ENTER(m);
    return forward_impl(m, x, T, out, 0);
}

int omega_moe_forward_block(omega_moe *m, const void *x, int T, void *out)
{
    MOE_ENTER(m);
    return forward_impl(m, x, T, out, 1);
}

static int backward_impl(omega_moe *m, const void *x, const void *dout, int T, void *dx, bool block)
{
    omega_ctx *ctx = m->ctx;
    RUN(check_T(m, x, T, true));
    if (T == 0) return OMEGA_OK;  // an empty batch: nothing to do, as in forward
    if (T != m->fwd_T || block != m->fwd_block)
        OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, block ? "backward_block: no omega_moe_forward_block has run for this T"
                                                     : "backward: no omega_moe_forward has run for this T");
    if (!dout || !dx) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "backward: dout or dx is NULL");
    RUN(moe_reserve_backward(m, T));
    const bool bf = m->cfg.dtype == OMEGA_DTYPE_BF16;
    // block form: the layer ran on the normalised rows it still holds; its input gradient then passes the norm backwards
    // and meets the gradient of the residual branch
    const void *xin = block ? m->hbuf : x;
    void *dxl = block ? m->bw_dhx : dx;
    if (bf) RUN(ensure_gathered(m, xin, T));
    OMEGA_HIP_CHECK(ctx, bf ? launch_backward_bf16(m, xin, dout, T, dxl, ctx->stream) : launch_backward_f32(m, xin, dout, T, dxl, ctx->stream));
    if (bf) {  // the pass wrote the states of the weight-gradient blocks into the other copy
        m->bw_zero_phase ^= 1;
        m->bw_zero_valid = true;
    }
    if (block) OMEGA_HIP_CHECK(ctx, launch_rmsnorm_backward(m, x, m->bw_dhx, dout, T, dx, ctx->stream));
    else OMEGA_HIP_CHECK(ctx, launch_zero_f32(m->dgamma, (size_t)m->cfg.d, ctx->stream));  // the norm took no part
    return OMEGA_OK;
}

int omega_moe_backward(omega_moe *m, const void *x, const void *dout, int T, void *dx)
{
    MOE_ENTER(m);
    return backward_impl(m, x, dout, T, dx, false);
}

int omega_moe_backward_block(omega_moe *m, const void *x, const void *dout, int T, void *dx)
{
    MOE_ENTER(m);
    return backward_impl(m, x, dout, T, dx, true);
}

int omega_moe_time_backward(omega_moe *m, const void *x, const void *dout, int T, void *dx, int warmup, int iters, float *ms_avg)
{
    MOE_ENTER(m);
    RUN(check_T(m, x, T, true));
    if (T <= 0 || T != m->fwd_T || m->fwd_block) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "time_backward: no omega_moe_forward has run for this T");
    if (!dout || !dx || !ms_avg || iters <= 0 || warmup < 0) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "time_backward: bad argument");
    RUN(moe_reserve_backward(m, T));
    const bool bf = m->cfg.dtype == OMEGA_DTYPE_BF16;
    if (bf) RUN(ensure_gathered(m, x, T));
    for (int i = 0; i < warmup + iters; ++i) {
        if (i == warmup) OMEGA_HIP_CHECK(ctx, hipEventRecord(m->ev0, ctx->stream));
        OMEGA_HIP_CHECK(ctx, bf ? launch_backward_bf16(m, x, dout, T, dx, ctx->stream) : launch_backward_f32(m, x, dout, T, dx, ctx->stream));
        if (bf) {
            m->bw_zero_phase ^= 1;
            m->bw_zero_valid = true;
        }
    }
    OMEGA_HIP_CHECK(ctx, hipEventRecord(m->ev1, ctx->stream));
    OMEGA_HIP_CHECK(ctx, hipEventSynchronize(m->ev1));
    float ms = 0.0f;
    OMEGA_HIP_CHECK(ctx, hipEventElapsedTime(&ms, m->ev0, m->ev1));
    *ms_avg = ms / (float)iters;
    return OMEGA_OK;
}

static int grad_slot(omega_moe *m, int which, int expert, float **ptr, size_t *floats)
{
    const omega_moe_config &c = m->cfg;
    const size_t per = (size_t)c.H * c.d;
    switch (which) {
        case OMEGA_W_GATE: *ptr = m->dWg; *floats = (size_t)c.E * c.d; return OMEGA_OK;
        case OMEGA_W_GATE_BIAS: *ptr = m->dbg; *floats = (size_t)c.E; return OMEGA_OK;
        case OMEGA_W_NORM: *ptr = m->dgamma; *floats = (size_t)c.d; return OMEGA_OK;
        case OMEGA_W_W1: case OMEGA_W_W3: case OMEGA_W_W2:
            if (expert < 0 || expert >= m->G) return OMEGA_ERR_INVALID_ARG;
            *ptr = which == OMEGA_W_W2 ? m->dW2 + per * (size_t)expert
                                       : m->dW13 + per * (2 * (size_t)expert + (which == OMEGA_W_W3 ? 1 : 0));
            *floats = per;
            return OMEGA_OK;
        default: return OMEGA_ERR_INVALID_ARG;
    }
}

int omega_moe_get_grad(omega_moe *m, int which, int expert, void *dst, int is_device)
{
    MOE_ENTER(m);
    if (!m->dWg) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "get_grad: no backward has run");
    float *p; size_t n;
    if (!dst || grad_slot(m, which, expert, &p, &n) != OMEGA_OK)
        OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "get_grad: bad kind, expert index or destination");
    OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(dst, p, n * 4, is_device ? hipMemcpyDeviceToDevice : hipMemcpyDeviceToHost, ctx->stream));
    OMEGA_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    return OMEGA_OK;
}

int omega_moe_acc_grad(omega_moe *m, float scale)
{
    MOE_ENTER(m);
    if (!m->dWg) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "acc_grad: no backward has run");
    const size_t n = grad_block_floats(m);
    if (!m->acc_grad) OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->acc_grad, n * 4));
    if (!m->acc_valid) {
        OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(m->acc_grad, m->dWg, n * 4, hipMemcpyDeviceToDevice, ctx->stream));
        m->acc_valid = true;
    } else {
        OMEGA_HIP_CHECK(ctx, launch_axpy_f32(m->acc_grad, m->dWg, scale, n, ctx->stream));
    }
    return OMEGA_OK;
}

int omega_moe_grad_sumsq(omega_moe *m, float *sumsq_host)
{
    MOE_ENTER(m);
    if (!m->dWg) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "grad_sumsq: no backward has run");
    if (!sumsq_host) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "grad_sumsq: destination is NULL");
    if (!m->sumsq_part) OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->sumsq_part, OMEGA_SUMSQ_SLOTS * sizeof(double)));
    // the gradients lie in one block whose padding is zero, so one pass covers every tensor
    OMEGA_HIP_CHECK(ctx, launch_sumsq_f32(m->acc_valid ? m->acc_grad : m->dWg, grad_block_floats(m), m->sumsq_part, ctx->stream));
    double total = 0.0;
    OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(&total, m->sumsq_part + OMEGA_SUMSQ_SLOTS - 1, sizeof(double), hipMemcpyDeviceToHost, ctx->stream));
    OMEGA_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    *sumsq_host = (float)total;
    return OMEGA_OK;
}

int omega_moe_scale_grad(omega_moe *m, float coef)
{
    MOE_ENTER(m);
    if (!m->dWg) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "scale_grad: no backward has run");
    OMEGA_HIP_CHECK(ctx, launch_scale_f32(m->acc_valid ? m->acc_grad : m->dWg, coef, grad_block_floats(m), ctx->stream));
    return OMEGA_OK;
}

int omega_moe_update(omega_moe *m, float lr)
{
    MOE_ENTER(m);
    if (!m->dWg) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "update: no backward has run");
    const omega_moe_config &c = m->cfg;
    if (m->acc_valid) {
        OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(m->dWg, m->acc_grad, grad_block_floats(m) * 4, hipMemcpyDeviceToDevice, ctx->stream));
        m->acc_valid = false;
        m->bw_zero_valid = false;  // the gradient block now holds the accumulators
    }
    if (c.dtype == OMEGA_DTYPE_BF16) {
        // the step is taken on fp32 master copies (made from the weights at the first update after they were set); the
        // layer's bf16 weights are the masters re-rounded, and the transposed copies of the backward pass follow
        if (!m->master) OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->master, grad_block_floats(m) * 4));
        if (!m->master_valid) {
            OMEGA_HIP_CHECK(ctx, launch_update_bf16(m, m->master, 0.0f, 1, ctx->stream));
            m->master_valid = true;
        }
        OMEGA_HIP_CHECK(ctx, launch_update_bf16(m, m->master, lr, 0, ctx->stream));
        if (c.has_gate_bias) OMEGA_HIP_CHECK(ctx, launch_axpy_f32(m->bg, m->dbg, -lr, (size_t)c.E, ctx->stream));
        if (m->gamma_set) OMEGA_HIP_CHECK(ctx, launch_axpy_f32(m->gamma, m->dgamma, -lr, (size_t)c.d, ctx->stream));
        m->wT_valid = false;
        stage_invalidates(m);
        return OMEGA_OK;
    }
    const size_t per = (size_t)c.H * c.d;
    OMEGA_HIP_CHECK(ctx, launch_axpy_f32((float *)m->Wg, m->dWg, -lr, (size_t)c.E * c.d, ctx->stream));
    if (c.has_gate_bias) OMEGA_HIP_CHECK(ctx, launch_axpy_f32(m->bg, m->dbg, -lr, (size_t)c.E, ctx->stream));
    if (m->gamma_set) OMEGA_HIP_CHECK(ctx, launch_axpy_f32(m->gamma, m->dgamma, -lr, (size_t)c.d, ctx->stream));
    for (int g = 0; g < m->G; ++g) {
        OMEGA_HIP_CHECK(ctx, launch_axpy_f32((float *)m->W1 + per * g, m->dW13 + per * 2 * g, -lr, per, ctx->stream));
        OMEGA_HIP_CHECK(ctx, launch_axpy_f32((float *)m->W3 + per * g, m->dW13 + per * (2 * g + 1), -lr, per, ctx->stream));
    }
    OMEGA_HIP_CHECK(ctx, launch_axpy_f32((float *)m->W2, m->dW2, -lr, per * m->G, ctx->stream));
    stage_invalidates(m);  // the weights changed: a backward pass needs a new forward
    return OMEGA_OK;
}

int omega_moe_update_adamw(omega_moe *m, float lr, float beta1, float beta2, float weight_decay, int train_time)
{
    MOE_ENTER(m);
    if (!m->dWg) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "update_adamw: no backward has run");
    if (train_time < 1 || !(beta1 >= 0.0f && beta1 < 1.0f) || !(beta2 >= 0.0f && beta2 < 1.0f))
        OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "update_adamw: train_time starts at 1 and the betas lie in [0, 1)");
    const omega_moe_config &c = m->cfg;
    const size_t n = grad_block_floats(m);
    if (m->acc_valid) {
        OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(m->dWg, m->acc_grad, n * 4, hipMemcpyDeviceToDevice, ctx->stream));
        m->acc_valid = false;
        m->bw_zero_valid = false;  // the gradient block now holds the accumulators
    }
    if (!m->adam_m) {
        OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->adam_m, n * 4));
        if (hipMalloc((void **)&m->adam_v, n * 4) != hipSuccess) {
            hipFree(m->adam_m);
            m->adam_m = nullptr;
            OMEGA_FAIL(ctx, OMEGA_ERR_OOM, "update_adamw: out of device memory for the moments");
        }
        OMEGA_HIP_CHECK(ctx, launch_zero_f32(m->adam_m, n, ctx->stream));
        OMEGA_HIP_CHECK(ctx, launch_zero_f32(m->adam_v, n, ctx->stream));
    }
    // the corrections as the reference forms them on the host: (float)(1.0f - Math.pow(beta, train_time))
    const omega_adamw p = {lr, beta1, beta2, (float)(1.0 - pow((double)beta1, (double)train_time)),
                           (float)(1.0 - pow((double)beta2, (double)train_time)), 1e-8f, weight_decay};
    if (c.dtype == OMEGA_DTYPE_BF16) {
        if (!m->master) OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&m->master, n * 4));
        if (!m->master_valid) {
            OMEGA_HIP_CHECK(ctx, launch_update_bf16(m, m->master, 0.0f, 1, ctx->stream));
            m->master_valid = true;
        }
        m->wT_valid = false;
    }
    OMEGA_HIP_CHECK(ctx, launch_update_adamw(m, m->master, m->adam_m, m->adam_v, p, ctx->stream));
    stage_invalidates(m);  // the weights changed: a backward pass needs a new forward
    return OMEGA_OK;
}

int omega_moe_get_norm(omega_moe *m, int T, float *rms_host)
{
    MOE_ENTER(m);
    if (!rms_host || T < 0 || T > m->T_cap) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "get_norm: bad argument or no forward_block has run for this T");
    OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(rms_host, m->rms, (size_t)T * 4, hipMemcpyDeviceToHost, ctx->stream));
    OMEGA_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    return OMEGA_OK;
}

int omega_moe_set_profiling(omega_moe *m, int on)
{
    MOE_ENTER(m);
    m->profiling = on != 0;
    m->prof_used = 0;
    return OMEGA_OK;
}

int omega_moe_get_profile(omega_moe *m, float *stage_ms_sum, int *n_calls)
{
    MOE_ENTER(m);
    if (!stage_ms_sum || !n_calls) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "get_profile: NULL argument");
    OMEGA_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    for (int i = 0; i < 5; ++i) stage_ms_sum[i] = 0.0f;
    const size_t calls = m->prof_used / 6;
    for (size_t c = 0; c < calls; ++c)
        for (int i = 0; i < 5; ++i) {
            float ms = 0.0f;
            OMEGA_HIP_CHECK(ctx, hipEventElapsedTime(&ms, m->prof_events[c * 6 + i], m->prof_events[c * 6 + i + 1]));
            stage_ms_sum[i] += ms;
        }
    *n_calls = (int)calls;
    m->prof_used = 0;
    return OMEGA_OK;
}

int omega_moe_router(omega_moe *m, const void *x, int T)
{
    MOE_ENTER(m);
    stage_invalidates(m);
    RUN(check_T(m, x, T, true));
    if (T == 0) return OMEGA_OK;
    RUN(moe_reserve(m, T));
    return stage_router(m, x, T);
}

int omega_moe_dispatch(omega_moe *m, const void *x, int T)
{
    MOE_ENTER(m);
    stage_invalidates(m);
    RUN(check_T(m, x, T, true));
    if (T == 0) return OMEGA_OK;
    if (T > m->T_cap) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "dispatch: router has not run for this T");
    return stage_dispatch(m, x, T);
}

int omega_moe_experts_up(omega_moe *m, const void *x, int T)
{
    MOE_ENTER(m);
    stage_invalidates(m);
    RUN(check_T(m, x, T, m->cfg.Es > 0 || m->gather_on_load));
    if (T == 0) return OMEGA_OK;
    if (T > m->T_cap) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "experts: router has not run for this T");
    return stage_experts(m, x, T, 0);
}

int omega_moe_experts_down(omega_moe *m, int T)
{
    MOE_ENTER(m);
    stage_invalidates(m);
    RUN(check_T(m, nullptr, T, false));
    if (T == 0) return OMEGA_OK;
    if (T > m->T_cap) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "experts: router has not run for this T");
    return stage_experts(m, nullptr, T, 1);
}

int omega_moe_experts(omega_moe *m, const void *x, int T)
{
    int st = omega_moe_experts_up(m, x, T);
    return st != OMEGA_OK ? st : omega_moe_experts_down(m, T);
}

int omega_moe_combine(omega_moe *m, int T, void *out)
{
    MOE_ENTER(m);
    RUN(check_T(m, nullptr, T, false));
    if (T == 0) return OMEGA_OK;
    if (!out) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "combine: out is NULL");
    if (T > m->T_cap) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "combine: router has not run for this T");
    return stage_combine(m, T, out, nullptr);
}

int omega_moe_get_routing(omega_moe *m, int T, int32_t *ids, float *w, int32_t *counts, int32_t *offsets, int32_t *dst,
                          int32_t *src_row)
{
    MOE_ENTER(m);
    if (T < 0 || T > m->T_cap) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "get_routing: T exceeds the last forward");
    const size_t P = (size_t)T * m->cfg.K;
    hipStream_t s = ctx->stream;
    if (ids && P) OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(ids, m->ids, P * 4, hipMemcpyDeviceToHost, s));
    if (w && P) OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(w, m->w, P * 4, hipMemcpyDeviceToHost, s));
    if (counts) OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(counts, m->counts, (size_t)m->cfg.E * 4, hipMemcpyDeviceToHost, s));
    if (offsets) OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(offsets, m->offsets, (size_t)(m->cfg.E + 1) * 4, hipMemcpyDeviceToHost, s));
    if (dst && P) OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(dst, m->dst, P * 4, hipMemcpyDeviceToHost, s));
    if (src_row && P) OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(src_row, m->src_row, P * 4, hipMemcpyDeviceToHost, s));
    OMEGA_HIP_CHECK(ctx, hipStreamSynchronize(s));
    return OMEGA_OK;
}

int omega_moe_get_router_probs(omega_moe *m, const void *x, int T, float *logits, float *probs)
{
    MOE_ENTER(m);
    stage_invalidates(m);
    RUN(check_T(m, x, T, true));
    if (T == 0) return OMEGA_OK;
    RUN(moe_reserve(m, T));
    const size_t n = (size_t)T * m->cfg.E;
    float *dl = nullptr, *dp = nullptr;
    OMEGA_HIP_CHECK(ctx, hipMalloc((void **)&dl, n * 4));
    hipError_t e = hipMalloc((void **)&dp, n * 4);
    m->routed_T = m->dispatched_T = -1;
    if (e == hipSuccess) e = launch_router(m, x, T, dl, dp, ctx->stream);
    if (e == hipSuccess) m->routed_T = T;
    if (e == hipSuccess && logits) e = hipMemcpyAsync(logits, dl, n * 4, hipMemcpyDeviceToHost, ctx->stream);
    if (e == hipSuccess && probs) e = hipMemcpyAsync(probs, dp, n * 4, hipMemcpyDeviceToHost, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    hipFree(dl);
    if (dp) hipFree(dp);
    OMEGA_HIP_CHECK(ctx, e);
    return OMEGA_OK;
}

// omega_moe_get_router_probs without any allocation: the device-side staging of logits and probabilities is the static
// scratch array (this device's copy, through the pointer kept at ctx_create), and the workspace is never grown.
// The router kernel writes every element of [T,E] that is copied out, so nothing needs clearing between calls.
int omega_moe_get_router_probs_noalloc(omega_moe *m, const void *x, int T, float *logits, float *probs)
{
    MOE_ENTER(m);
    stage_invalidates(m);
    RUN(check_T(m, x, T, true));
    if (T == 0) return OMEGA_OK;
    if (T > m->T_cap)
        OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "get_router_probs_noalloc: T exceeds the workspace the layer holds (create it with T_max >= T); this entry point never allocates");
    const size_t n = (size_t)T * m->cfg.E;
    if (n > OMEGA_NOALLOC_MAX_FLOATS)
        OMEGA_FAIL(ctx, OMEGA_ERR_UNSUPPORTED, "get_router_probs_noalloc: T*E exceeds the static scratch of 1048576 values");
    if (!ctx->noalloc_scratch) OMEGA_FAIL(ctx, OMEGA_ERR_HIP, "get_router_probs_noalloc: no scratch address for this device");
    float *dl = ctx->noalloc_scratch, *dp = ctx->noalloc_scratch + OMEGA_NOALLOC_MAX_FLOATS;
    m->routed_T = m->dispatched_T = -1;
    OMEGA_HIP_CHECK(ctx, launch_router(m, x, T, dl, dp, ctx->stream));
    m->routed_T = T;
    if (logits) OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(logits, dl, n * 4, hipMemcpyDeviceToHost, ctx->stream));
    if (probs) OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(probs, dp, n * 4, hipMemcpyDeviceToHost, ctx->stream));
    OMEGA_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    return OMEGA_OK;
}

// Host copy of a workspace buffer in logical row order (row r of expert e = offsets[e] + rank), row-major:
// the padding between experts and the packed tile image of bf16 layers are undone here.
int omega_moe_get_workspace(omega_moe *m, int which, int T, void *host_dst)
{
    MOE_ENTER(m);
    if (!host_dst || which < 0 || which > 4 || T <= 0 || T > m->T_cap || m->bm == 0)
        OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "get_workspace: bad selector, T, or no dispatch has run");
    const omega_moe_config &c = m->cfg;
    if (which >= 3 && (T > m->bw_T_cap || (which == 3 && !m->bw_dh16)))
        OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "get_workspace: no backward has run (selector 3: of a bf16 layer)");
    if (which == 4) {
        OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(host_dst, m->bw_dlogits, (size_t)T * c.E * 4, hipMemcpyDeviceToHost, ctx->stream));
        OMEGA_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
        return OMEGA_OK;
    }
    const int G = c.E + c.Es, bm = m->bm;
    const int cols = which == 1 ? c.H : which == 3 ? 2 * c.H : c.d;
    const size_t es = which == 2 ? 4 : m->esize;
    const bool packed = c.dtype == OMEGA_DTYPE_BF16 && which != 2;
    if (which == 0 && c.dtype == OMEGA_DTYPE_BF16) {
        if (m->dispatched_T != T) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "get_workspace: dispatch has not run for this T");
        RUN(ensure_gathered(m, m->last_x, T));
    }
    const void *src = which == 0 ? m->xg : which == 1 ? m->a : which == 3 ? m->bw_dh16 : (const void *)m->y;
    const size_t bytes = m->rows_cap * cols * es;
    std::vector<int32_t> meta(G + 2), off(c.E + 1);
    OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(meta.data(), m->tile_meta, meta.size() * 4, hipMemcpyDeviceToHost, ctx->stream));
    OMEGA_HIP_CHECK(ctx, hipMemcpyAsync(off.data(), m->offsets, off.size() * 4, hipMemcpyDeviceToHost, ctx->stream));
    void *stage = nullptr;
    if (packed) {
        OMEGA_HIP_CHECK(ctx, hipMalloc(&stage, bytes));
        hipError_t e = launch_unpack_rows(stage, src, (int)m->rows_cap, cols, ctx->stream);
        if (e != hipSuccess) { hipFree(stage); OMEGA_HIP_CHECK(ctx, e); }
        src = stage;
    }
    std::vector<unsigned char> raw(bytes);
    hipError_t e = hipMemcpyAsync(raw.data(), src, bytes, hipMemcpyDeviceToHost, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (stage) hipFree(stage);
    OMEGA_HIP_CHECK(ctx, e);
    const size_t rb = (size_t)cols * es, P = (size_t)T * c.K;
    unsigned char *out = (unsigned char *)host_dst;
    const int groups = which == 0 ? c.E : G;  // xg holds routed rows only
    for (int g = 0; g < groups; ++g) {
        const size_t rows = g < c.E ? (size_t)(off[g + 1] - off[g]) : (size_t)T;
        const size_t l0 = g < c.E ? (size_t)off[g] : P + (size_t)(g - c.E) * T;
        memcpy(out + l0 * rb, raw.data() + (size_t)meta[1 + g] * bm * rb, rows * rb);
    }
    return OMEGA_OK;
}

int omega_moe_fill_workspace(omega_moe *m, int which, int byte_value)
{
    MOE_ENTER(m);
    if ((which != 1 && which != 2) || m->rows_cap == 0)
        OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "fill_workspace: selector must be 1 (a) or 2 (y) and the workspace must exist");
    void *p = which == 1 ? m->a : (void *)m->y;
    const size_t bytes = which == 1 ? m->rows_cap * m->cfg.H * m->esize : m->rows_cap * m->cfg.d * 4;
    // what the last forward left in the buffer is gone: a backward pass needs a new forward, and the stages that read
    // the buffer (down product, combine) a new run of the stage that writes it.  (The routing and the dispatch tables
    // are untouched: omega_moe_experts_up / _down may follow.)
    stage_invalidates(m);
    if (which == 1) m->a_valid = false;
    m->y_valid = false;
    OMEGA_HIP_CHECK(ctx, hipMemsetAsync(p, byte_value, bytes, ctx->stream));
    return OMEGA_OK;
}

int omega_moe_time_stage(omega_moe *m, int stage, const void *x, int T, void *out, int warmup, int iters, float *ms_avg)
{
    MOE_ENTER(m);
    stage_invalidates(m);
    RUN(check_T(m, x, T, stage == 0 || stage == 1 || stage == 5 || stage == 7 || stage == 8 || stage == 9));
    if ((stage == 6 || stage == 7) && m->bm == 0) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "time_stage: dispatch has not run");
    if (!ms_avg || iters <= 0 || warmup < 0 || stage < 0 || stage > 9 || T <= 0)
        OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "time_stage: bad argument");
    if ((stage == 4 || stage == 5 || stage == 8) && !out) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "time_stage: out is NULL");
    if (stage == 0 || stage == 5 || stage == 8 || stage == 9) RUN(moe_reserve(m, T));
    else if (T > m->T_cap) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "time_stage: earlier stages have not run for this T");
    auto once = [&]() -> int {
        switch (stage) {
            case 0: return stage_router(m, x, T);
            case 1: return stage_dispatch(m, x, T);
            case 2: return stage_experts(m, x, T, 0);
            case 3: return stage_experts(m, x, T, 1);
            case 4: return stage_combine(m, T, out, nullptr);
            case 6:
            case 7:
                // parts of a dispatch that has already run for this T (same buffers, same result)
                if (m->dispatched_T != T) OMEGA_FAIL(ctx, OMEGA_ERR_INVALID_ARG, "time_stage: dispatch has not run for this T");
                if (stage == 6) OMEGA_HIP_CHECK(ctx, launch_dispatch_index(m, T, m->bm, ctx->stream));
                else OMEGA_HIP_CHECK(ctx, launch_dispatch_gather(m, x, T, ctx->stream));
                return OMEGA_OK;
            case 8: return forward_impl(m, x, T, out, 1);
            case 9:
                OMEGA_HIP_CHECK(ctx, launch_rmsnorm(m, x, T, m->hbuf, ctx->stream));
                return OMEGA_OK;
            default:
                RUN(stage_router(m, x, T));
                RUN(stage_dispatch(m, x, T));
                RUN(stage_experts(m, x, T, 0));
                RUN(stage_experts(m, x, T, 1));
                return stage_combine(m, T, out, nullptr);
        }
    };
    for (int i = 0; i < warmup; ++i) RUN(once());
    OMEGA_HIP_CHECK(ctx, hipEventRecord(m->ev0, ctx->stream));
    for (int i = 0; i < iters; ++i) RUN(once());
    OMEGA_HIP_CHECK(ctx, hipEventRecord(m->ev1, ctx->stream));
    OMEGA_HIP_CHECK(ctx, hipEventSynchronize(m->ev1));
    float ms = 0.0f;
    OMEGA_HIP_CHECK(ctx, hipEventElapsedTime(&ms, m->ev0, m->ev1));
    *ms_avg = ms / (float)iters;
    return OMEGA_OK;
}

}  // extern "C"
