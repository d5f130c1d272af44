// Grouped expert SwiGLU products in bf16 on the CDNA4 matrix cores (v_mfma_f32_32x32x16_bf16, fp32 accumulate).
//   up    a[r,h] = silu(xg[r,:].W1g[h,:]) * (xg[r,:].W3g[h,:])   -> bf16      (one pass over xg for both weights)
//   down  y[r,c] = a[r,:].W2g[c,:]                                -> fp32
// (J/engine/nn/layer/llama/LlamaMLPLayer.java:117-130; y = x W^T with W [out,in], J/engine/nn/layer/FullyLayer.java:181,235.)
//
// Both operands are K-contiguous ("NT" product), so a lane's 8 consecutive k values are one 16-byte LDS read.
// Workgroup = 4 waves (2x2), tile 256 rows x 256 MFMA columns x 64 k, each wave 128x128 = 4x4 MFMA blocks.
// For the up product the 256 MFMA columns are 128 columns of W1 and the same 128 columns of W3, arranged so
// that a wave holds h1 and h3 of the same output element and applies silu(h1)*h3 in registers.
// LDS: two stages of (A 256x64 + B 256x64) bf16 = 128 KiB, 16-byte chunks XOR-swizzled by row.
// Scheduling: the dispatch stage leaves a list of row tiles (never straddling two experts; empty experts
// have none) and the first row tile of every expert; workgroup -> (expert, column tile, row tile) is
// derived from those on the device, row tiles fastest so that the workgroups resident on one XCD share
// weight tiles in its L2.  Consecutive workgroup ids go round-robin over the 8 XCDs, so the id is first
// remapped to give each XCD a contiguous run of tiles.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

#define BM 256
#define BNT 256  // MFMA columns per tile
#define BK 64
#define STAGE_BYTES (BM * BK * 2)
#define SMEM_BYTES (4 * STAGE_BYTES)
#define NUM_XCD 8

int experts_bf16_tile_m(const omega_moe *, int) { return BM; }

__device__ __forceinline__ int swz(int row) { return (row >> 1) & 7; }
__device__ __forceinline__ int lds_off(int row, int kc) { return row * (BK * 2) + ((kc ^ swz(row)) << 4); }

template <bool FUSED>
__global__ __launch_bounds__(256, 1) void experts_bf16_kernel(const bf16_t *__restrict__ Axg, const bf16_t *__restrict__ Ax,
                                                              const bf16_t *__restrict__ Wa, const bf16_t *__restrict__ Wb,
                                                              void *__restrict__ Cout, const omega_tile *__restrict__ tiles,
                                                              const int32_t *__restrict__ tile_meta, int G, int N, int Kd)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    constexpr int NCOLS = FUSED ? 128 : 256;  // output columns per tile
    const int NT = N / NCOLS;
    // ---- workgroup -> tile ----
    const int total = tile_meta[0] * NT;
    const int chunk = (total + NUM_XCD - 1) / NUM_XCD;
    const int pid = blockIdx.x;
    const int slot = pid / NUM_XCD;
    const int L = (pid % NUM_XCD) * chunk + slot;
    if (slot >= chunk || L >= total) return;
    int lo = 0, hi = G;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (tile_meta[1 + mid] * NT <= L) lo = mid; else hi = mid;
    }
    const int mt0 = tile_meta[1 + lo], Mg = tile_meta[2 + lo] - mt0;
    const int l = L - mt0 * NT;
    const int nt = l / Mg;
    const omega_tile tl = tiles[mt0 + (l % Mg)];
    const int n0 = nt * NCOLS;

    const bf16_t *A = (FUSED && tl.xrow0 >= 0) ? Ax + (size_t)tl.xrow0 * Kd : Axg + (size_t)tl.row0 * Kd;
    const bf16_t *B0 = Wa + ((size_t)tl.g * N + n0) * Kd;
    const bf16_t *B1 = FUSED ? Wb + ((size_t)tl.g * N + n0) * Kd : B0 + (size_t)128 * Kd;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lrow = tid >> 3, lkc = tid & 7;

    int aoff[8], boff[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int r = lrow + 32 * i;
        aoff[i] = min(r, tl.rows - 1) * Kd + lkc * 8;
        boff[i] = (r & 127) * Kd + lkc * 8;
    }
    uint4 ra[8], rb[8];
    auto gload = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            ra[i] = *(const uint4 *)(A + aoff[i] + k0);
            rb[i] = *(const uint4 *)((i < 4 ? B0 : B1) + boff[i] + k0);
        }
    };
    auto lstore = [&](int buf) {
        unsigned char *as = smem + buf * STAGE_BYTES;
        unsigned char *bs = smem + 2 * STAGE_BYTES + buf * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int r = lrow + 32 * i;
            *(uint4 *)(as + lds_off(r, lkc)) = ra[i];
            *(uint4 *)(bs + lds_off(r, lkc)) = rb[i];
        }
    };

    f32x16_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    const int l32 = lane & 31, lhi = lane >> 5;
    int arow[4], brow[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        arow[i] = wm * 128 + i * 32 + l32;
        brow[i] = FUSED ? ((i >> 1) * 128 + wn * 64 + (i & 1) * 32 + l32) : (wn * 128 + i * 32 + l32);
    }

    const int KT = Kd / BK;
    gload(0);
    lstore(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < KT) gload((kt + 1) * BK);
        const unsigned char *as = smem + cur * STAGE_BYTES;
        const unsigned char *bs = smem + 2 * STAGE_BYTES + cur * STAGE_BYTES;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            bf16x8_t af[4], bfr[4];
            const int kc = ks * 2 + lhi;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                af[i] = *(const bf16x8_t *)(as + lds_off(arow[i], kc));
                bfr[i] = *(const bf16x8_t *)(bs + lds_off(brow[i], kc));
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < KT) lstore(cur ^ 1);
        __syncthreads();
    }

    // ---- epilogue: lane holds column l32 of each 32x32 block; register r -> row 8*(r/4) + 4*lhi + r%4 ----
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = wm * 128 + i * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
            if (row >= tl.rows) continue;
            if (FUSED) {
                bf16_t *out = (bf16_t *)Cout + (size_t)(tl.row0 + row) * N + n0 + wn * 64 + l32;
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const float h1 = acc[i][j][r], h3 = acc[i][j + 2][r];
                    out[j * 32] = f32_to_bf16((h1 / (1.0f + __expf(-h1))) * h3);
                }
            } else {
                float *out = (float *)Cout + (size_t)(tl.row0 + row) * N + n0 + wn * 128 + l32;
#pragma unroll
                for (int j = 0; j < 4; ++j) out[j * 32] = acc[i][j][r];
            }
        }
    }
}

hipError_t experts_bf16_init(void)
{
    hipError_t e = hipFuncSetAttribute((const void *)experts_bf16_kernel<true>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES);
    if (e != hipSuccess) return e;
    return hipFuncSetAttribute((const void *)experts_bf16_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                               SMEM_BYTES);
}

hipError_t launch_experts_bf16(const omega_moe *m, const void *x, int T, int which, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    (void)T;
    const int G = c.E + c.Es;
    if (which == 0) {
        int grid = m->max_m_tiles * (c.H / 128);
        grid = (grid + NUM_XCD - 1) / NUM_XCD * NUM_XCD;
        hipLaunchKernelGGL(experts_bf16_kernel<true>, dim3(grid), dim3(256), SMEM_BYTES, s, (const bf16_t *)m->xg,
                           (const bf16_t *)x, (const bf16_t *)m->W1, (const bf16_t *)m->W3, m->a, m->tiles, m->tile_meta,
                           G, c.H, c.d);
    } else {
        int grid = m->max_m_tiles * (c.d / 256);
        grid = (grid + NUM_XCD - 1) / NUM_XCD * NUM_XCD;
        hipLaunchKernelGGL(experts_bf16_kernel<false>, dim3(grid), dim3(256), SMEM_BYTES, s, (const bf16_t *)m->a,
                           (const bf16_t *)nullptr, (const bf16_t *)m->W2, (const bf16_t *)nullptr, (void *)m->y, m->tiles,
                           m->tile_meta, G, c.d, c.H);
    }
    return hipGetLastError();
}
