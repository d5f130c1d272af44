// Internal declarations shared by the translation units of libomega_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>
#include <string>
#include <vector>

#include "omega_hip.h"

typedef uint16_t bf16_t;  // raw bf16 bit pattern in device buffers

struct omega_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    std::mutex mu;
    std::string last_error;
    int num_cus = 256;
    float *noalloc_scratch = nullptr;  // this device's copy of the static scratch array of the allocation-free entry point
};

// One entry per row tile of the grouped products: written on the device by the scan kernel.
// Rows of the expert-contiguous buffers xg / a / y are "physical" rows: expert g owns the row tiles
// first_tile[g] .. first_tile[g+1]-1, each bm rows high, so every expert starts on a tile boundary and the
// row tile with list index i covers physical rows i*bm .. i*bm+rows-1 (the rest of the tile is padding that
// is never computed).  The logical row of a pair (offsets[e] + rank, what get_routing reports) and its
// physical row (first_tile[e]*bm + rank) differ only by that padding.
struct __attribute__((aligned(16))) omega_tile {
    int32_t g;      // weight index: 0..E-1 routed, E..E+Es-1 shared
    int32_t row0;   // first physical row (= list index * bm)
    int32_t rows;   // valid rows in this tile (1..bm)
    int32_t xrow0;  // -1: routed expert; >=0: shared expert, first token of this tile (A operand = x rows)
};

// One entry per work item of a grouped product, in launch order (expert, column tile, row tile - row tiles
// fastest): everything a workgroup needs to start, in one 32-byte load.  A work item is an output tile or, for the
// last tiles of a launch that would leave most compute units idle, a slice of 64 or 128 rows of one (row0 is then
// not a multiple of the tile height).  The table can hold OMEGA_TAIL_EXTRA entries more than there are tiles.
#define OMEGA_TAIL_EXTRA 192
struct __attribute__((aligned(32))) omega_tile_desc {
    int32_t g, row0, rows, xrow0;  // as omega_tile
    int32_t n0;                    // first output column of the tile
    // weight-gradient items: row groups (128 rows) of the two operand tiles in their transposed images and the first
    // k step of the expert's rows there; xrow0 then holds the item's number of k steps.  Other items: zero, except
    // b_rg = 1 in an item of the down product that covers 128 columns instead of 256
    int32_t a_rg, b_rg, kt0;
};

struct omega_moe {
    omega_ctx *ctx = nullptr;
    omega_moe_config cfg{};
    int G = 0;            // E + Es
    size_t esize = 4;     // bytes per element of the layer dtype
    int T_cap = 0;        // tokens the workspace is sized for
    int bm = 0;           // row-tile height the tile list was built for
    // weights (layer dtype except bg)
    void *Wg = nullptr;   // [E,d]
    float *bg = nullptr;  // [E]
    void *W1 = nullptr;   // [G,H,d]
    void *W3 = nullptr;   // [G,H,d]
    void *W2 = nullptr;   // [G,d,H]
    float *gamma = nullptr;  // [d] weight of the RMSNorm in front of the layer (block form), fp32
    bool gamma_set = false;
    // workspace
    float *rms = nullptr;            // [T] row statistics of the pre-norm (block form)
    void *hbuf = nullptr;            // [T,d] normalised rows (block form), layer dtype
    int32_t *ids = nullptr;          // [T,K]
    float *w = nullptr;              // [T,K]
    int32_t *tile_counts = nullptr;  // [n_tok_tiles,E] histogram per token tile (router)
    int32_t *counts = nullptr;       // [E]
    int32_t *offsets = nullptr;      // [E+1]
    int32_t *dst = nullptr;          // [T*K] logical row of each pair
    int32_t *dstp = nullptr;         // [T*K] physical row of each pair
    int32_t *src_row = nullptr;      // [T*K]
    int32_t *tokp = nullptr;         // [rows_cap] token of every physical row of a routed expert (padding rows: stale or 0)
    // bf16 layers: the up product of this batch fetches the rows of x through tokp itself and no gathered copy exists
    // (xg / xs hold an earlier batch) until something that needs one asks for it
    bool gather_on_load = false;
    int gather_mode = OMEGA_GATHER_AUTO;  // omega_moe_set_gather_mode
    bool xg_valid = false;
    const void *last_x = nullptr;    // input of the last dispatch (the caller's buffer, or hbuf in the block form)
    omega_tile *tiles = nullptr;     // [max_m_tiles]
    int32_t *tile_meta = nullptr;    // [0] = number of row tiles; [1+g] = first row tile of group g (G+1 entries);
                                     // [G+2], [G+3] = entries of desc_up, desc_down; [G+4..G+6] = entries of the
                                     // backward tables desc_da, desc_w2, desc_w13; [G+7] = k slices per tile of a
                                     // small batch; [G+8], [G+9] = first k-sliced entry of desc_down and their number
    omega_tile_desc *desc_up = nullptr;    // bf16: [tiles_cap * H/128] output tiles of the up product
    omega_tile_desc *desc_down = nullptr;  // bf16: [tiles_cap * d/256] output tiles of the down product
    // bf16: the same work items as one queue per workgroup of the (persistent) product kernels, entry q of workgroup w
    // at [q * n_wg + w]; a queue ends with an entry of 0 rows
    omega_tile_desc *wq_up = nullptr, *wq_down = nullptr;
    int n_wg = 0;                          // workgroups of a product launch: one per compute unit, a multiple of 8
    // columns of a work item of the down product: 256, or 128 when 256-column tiles would leave at least half of the
    // compute units without an item (a few tokens: the product is bound by streaming W2, which every unit must share)
    int down_cols = 256;
    int down_ks_max = 1;             // > 1: the down table of this batch may hold k slices of every tile (small batches)
    int down_tail_ks = 1;            // > 1: the last tiles of the down table may be cut into up to this many k slices
    float *y_slabs = nullptr;        // partial results of the k slices: 256 tiles of 256 x 256 floats, one per sliced entry
    void *xg = nullptr;              // [rows_cap,d]  gathered tokens (bf16: packed tile image, see pack.h)
    void *xs = nullptr;              // bf16 with shared experts: packed copy of x, [ceil(T/bm)*bm,d]
    void *a = nullptr;               // [rows_cap,H]  (bf16: packed tile image)
    float *y = nullptr;              // [rows_cap,d]  row-major fp32
    size_t rows_cap = 0;             // physical rows the buffers hold: tile capacity * bm
    int tiles_cap = 0;               // entries of `tiles`
    int max_m_tiles = 0;
    // backward pass (allocated by the first omega_moe_backward): parameter gradients, always fp32, in the layout of
    // their weights, the accumulators of accGrad, and the workspace of the pass, indexed by physical rows like xg / a / y
    // (dW13: [G][2][H,d], the gradients of W1 and W3 of an expert back to back)
    float *dWg = nullptr, *dbg = nullptr, *dgamma = nullptr, *dW13 = nullptr, *dW2 = nullptr;
    float *acc_grad = nullptr;       // accumulators, one block in the order dWg, dbg, dgamma, dW13, dW2
    bool acc_valid = false;          // accGrad has run since the last update
    int32_t *bw_zero_state = nullptr;  // [2][G]: which groups' weight-gradient blocks are known to be zero (two copies, used in turn)
    int bw_zero_phase = 0;           // which copy the next backward pass reads
    bool bw_zero_valid = false;      // false: the gradient block was written from outside the backward pass
    double *sumsq_part = nullptr;    // scratch of the gradient-norm reduction
    float *adam_m = nullptr;         // AdamW moments, each laid out like the gradient block (allocated by the first AdamW update)
    float *adam_v = nullptr;
    float *master = nullptr;         // bf16 layers: fp32 master copies of Wg, W1|W3, W2 (layout of the gradient block)
    bool master_valid = false;       // ... and whether they match the weights (set_weights invalidates)
    float *bw_probs = nullptr;       // [T,E] softmax of the gate logits
    float *bw_dw = nullptr;          // [T,K] gradient of the combine weights
    float *bw_dlogits = nullptr;     // [T,E]
    float *bw_gpart = nullptr;       // [32][E,d] partial sums of the gate weight gradient over token slices
    float *bw_dy = nullptr;          // [rows_cap,d] gradient of the expert outputs
    float *bw_h1 = nullptr;          // [rows_cap,H] h1, then dh1
    float *bw_h3 = nullptr;          // [rows_cap,H] h3, then dh3
    float *bw_dxg = nullptr;         // [rows_cap,d] gradient of the expert inputs
    // bf16 layers: the products of the pass run on the matrix-core kernel of the forward pass (see experts_bf16.hip)
    void *bw_dy16 = nullptr;         // [rows_cap,d] packed bf16: dy
    void *bw_dys16 = nullptr;        // [ceil(T/bm)*bm,d] packed bf16 copy of dout (rows of the shared experts)
    void *bw_dh16 = nullptr;         // [rows_cap,2H] packed bf16: dh1 | dh3  (bw_h1 / bw_h3 hold the h1 / h3 block records)
    void *bw_dyT = nullptr, *bw_aT = nullptr, *bw_xgT = nullptr, *bw_dhT = nullptr;  // transposed packed images over k space
    int32_t *bw_kt0 = nullptr;       // [G+1] first k step of each group in k space
    int bw_ksteps_cap = 0;           // k steps the transposed images are laid out for
    omega_tile_desc *desc_da = nullptr, *wq_da = nullptr;    // d(a) product: 256-column tiles over H
    omega_tile_desc *desc_w2 = nullptr, *wq_w2 = nullptr;    // dW2 = dy^T a
    omega_tile_desc *desc_w13 = nullptr, *wq_w13 = nullptr;  // dW1 | dW3 = dh^T xg
    void *W2T = nullptr;             // [G][H,d] packed: transposed W2 (+ one row group of slack)
    void *W13T = nullptr;            // [G][d,2H] packed: W1^T | W3^T
    bool wT_valid = false;           // the transposed copies match the weights
    int bw_T_cap = 0;
    size_t bw_rows_cap = 0;
    int fwd_T = -1;                  // tokens of the last forward (what a backward pass may follow), -1: none
    // which batch the index buffers describe: ids / w / tile_counts hold the router's result for routed_T tokens, and
    // dst / dstp / src_row, the tile list and the work queues the dispatch stage's for dispatched_T (-1: none yet, or
    // the buffers were reallocated).  A stage is refused unless the stage before it ran for the same T, because the
    // index buffers are what the next stage's addresses are formed from.
    int routed_T = -1, dispatched_T = -1;
    bool a_valid = true, y_valid = true;  // false once omega_moe_fill_workspace has overwritten the buffer
    bool fwd_block = false;          // ... and whether it was the block form
    void *bw_dhx = nullptr;          // [T,d] layer dtype: input gradient of the layer inside the block form
    bool training = false;           // forward keeps h1 / h3 (bf16 layers: as block records in bw_h1 / bw_h3)
    bool rec_valid = false;          // bw_h1 / bw_h3 hold h1 / h3 of the last forward
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    // per-stage event profiling of forward calls (6 events per call), off by default
    bool profiling = false;
    std::vector<hipEvent_t> prof_events;
    size_t prof_used = 0;
};

// Tokens per router workgroup = per row of tile_counts and per workgroup of the dispatch kernel: 16 for layers
// with at most 16 experts, else 32 (router.hip).
int router_tok_tile(int E);
#define ROUTER_TOK_TILE_MAX 32

// Size of the last-level (memory-side) cache of the device: streams larger than this are written / read around it.
#define OMEGA_LLC_BYTES ((size_t)256 << 20)

__host__ __device__ static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

int omega_set_error(omega_ctx *ctx, int status, const char *what, hipError_t herr, const char *file, int line);

#define OMEGA_FAIL(ctx, status, what) return omega_set_error((ctx), (status), (what), hipSuccess, __FILE__, __LINE__)
#define OMEGA_HIP_CHECK(ctx, expr)                                                             \
    do {                                                                                       \
        hipError_t _e = (expr);                                                                \
        if (_e != hipSuccess)                                                                  \
            return omega_set_error((ctx), _e == hipErrorOutOfMemory ? OMEGA_ERR_OOM : OMEGA_ERR_HIP, #expr, _e, \
                                   __FILE__, __LINE__);                                        \
    } while (0)

// ---- launchers (one per .hip file); all asynchronous on `s`, returning the launch status ----
hipError_t launch_fill_normal(void *dptr, uint64_t n, uint64_t seed, uint64_t stream_id, double std, uint64_t first,
                              int dtype, hipStream_t s);
hipError_t launch_convert(void *dst, int dst_dtype, const void *src, int src_dtype, uint64_t n, hipStream_t s);

// h[t,:] = (x[t,:] / rms[t]) * gamma in the layer's storage type, rms[t] into m->rms; h == nullptr: statistics only
hipError_t launch_rmsnorm(const omega_moe *m, const void *x, int T, void *h, hipStream_t s);
hipError_t launch_rmsnorm_backward(const omega_moe *m, const void *x, const void *dh, const void *resid, int T, void *dx,
                                   hipStream_t s);
hipError_t launch_router(const omega_moe *m, const void *x, int T, float *logits_out, float *probs_out, hipStream_t s);
hipError_t launch_dispatch_index(const omega_moe *m, int T, int bm, hipStream_t s, const void *x_rows = nullptr);
hipError_t launch_dispatch_gather(const omega_moe *m, const void *x, int T, hipStream_t s);
hipError_t launch_experts_f32(const omega_moe *m, const void *x, int T, int which, hipStream_t s);
hipError_t launch_experts_bf16(const omega_moe *m, const void *x, int T, int which, hipStream_t s);
// resid != nullptr: out = resid + layer output (one rounding of the fp32 sum)
hipError_t launch_combine(const omega_moe *m, int T, void *out, const void *resid, hipStream_t s);
hipError_t launch_backward_f32(const omega_moe *m, const void *x, const void *dout, int T, void *dx, hipStream_t s);
hipError_t launch_backward_bf16(const omega_moe *m, const void *x, const void *dout, int T, void *dx, hipStream_t s);
hipError_t launch_backward_tables(const omega_moe *m, int T, hipStream_t s);
hipError_t launch_transpose_groups(const omega_moe *m, const void *src, const void *src_alt, int cols, void *dst, int T,
                                   hipStream_t s);
hipError_t launch_transpose_images(const void *src, int R, int cols, void *dst, int KTd, int k0, int n, size_t src_stride,
                                   size_t dst_stride, hipStream_t s);
// products of the matrix-core kernel (experts_bf16.hip describes each)
enum { MODE_UP = 0, MODE_DOWN = 1, MODE_UPRAW = 2, MODE_DA = 3, MODE_WGRAD = 4, MODE_UPREC = 5 };
hipError_t launch_product_bf16(const omega_moe *m, int mode, const void *A, const void *Aalt, const void *Wa, const void *Wb,
                               void *Cout, void *Aux1, void *Aux2, const omega_tile_desc *wq, int N, int Kd, hipStream_t s);
hipError_t launch_update_bf16(const omega_moe *m, float *master, float lr, int init, hipStream_t s);
hipError_t launch_zero_f32(float *dst, size_t n, hipStream_t s);
hipError_t launch_axpy_f32(float *dst, const float *src, float scale, size_t n, hipStream_t s);
#define OMEGA_SUMSQ_SLOTS 2049  // doubles of scratch launch_sumsq_f32 needs; the result is the last one
hipError_t launch_sumsq_f32(const float *src, size_t n, double *part, hipStream_t s);
hipError_t launch_scale_f32(float *dst, float coef, size_t n, hipStream_t s);
struct omega_adamw {
    float lr, beta1, beta2, b1c, b2c, eps, wd;  // b1c, b2c: 1 - beta^t, formed on the host
};
hipError_t launch_update_adamw(const omega_moe *m, float *master, float *mw, float *vw, const omega_adamw &p, hipStream_t s);
hipError_t launch_pack_rows(void *dst_packed, const void *src_rowmajor, int R, int Kd, hipStream_t s);
hipError_t launch_unpack_rows(void *dst_rowmajor, const void *src_packed, int R, int Kd, hipStream_t s);
int experts_bf16_tile_m(const omega_moe *m, int T);
int experts_f32_tile_m(void);
hipError_t experts_bf16_init(void);
hipError_t launch_down_slab_reduce(const omega_moe *m, float *y, hipStream_t s);  // y += partial results of k-sliced items
hipError_t router_init(void);  // kernel attributes of the router (LDS beyond 64 KiB), once per device

// ---- device helpers ----
#ifdef __HIPCC__
__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }
__device__ __forceinline__ bf16_t f32_to_bf16(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}
// One element of the pre-norm: (x / rms) * weight with two roundings, as rmsnorm_forward_kernel2 writes it
// (J/engine/nn/layer/normalization/gpu/RMSKernel.cu:218-222); bf16 layers store the result as bf16.
template <bool XBF>
__device__ __forceinline__ float norm_apply(float v, float rms, float g)
{
    const float n = v / rms;
    const float h = n * g;
    return XBF ? bf16_to_f32(f32_to_bf16(h)) : h;
}
#endif
