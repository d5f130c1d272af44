// Grouped expert SwiGLU products in bf16 on the CDNA4 matrix cores (v_mfma_f32_32x32x16_bf16, fp32 accumulate).
//   up    a[r,h] = silu(xg[r,:].W1g[h,:]) * (xg[r,:].W3g[h,:])   -> bf16      (one pass over xg for both weights)
//   down  y[r,c] = a[r,:].W2g[c,:]                                -> fp32
// (J/engine/nn/layer/llama/LlamaMLPLayer.java:117-130; y = x W^T with W [out,in], J/engine/nn/layer/FullyLayer.java:181,235.)
//
// Both operands are K-contiguous ("NT" product), so a lane's 8 consecutive k values are one 16-byte LDS read.
// Workgroup = 8 waves (2 row halves x 4 column quarters, two waves per SIMD so that one computes while the
// other waits on LDS, on the address unit or at the barrier); tile = 256 rows x 256 MFMA columns, each wave
// 4x2 MFMA blocks (the 32-row blocks of the tile alternate between the row halves, so a ragged tile splits evenly) with its 128 accumulators in AGPRs.  For the up product the 256 MFMA columns are
// 128 columns of W1 and the same 128 columns of W3, arranged so that a wave holds h1 and h3 of the same
// output element and applies silu(h1)*h3 in registers.
//
// Data movement: global -> LDS directly (global_load_lds_dwordx4, no staging registers) into a ring of five
// stages of (A 256x32 + B 256x32) bf16 = 160 KiB, i.e. all of a CU's LDS.  A wave-wide direct load fills 1 KiB
// of LDS in lane order = 16 rows of four 16-byte chunks.  All three operands (weights, xg, a) are kept in
// memory as that very image (pack.h: 1 KiB blocks of 16 rows x 32 k with the chunk index XOR-swizzled so the
// MFMA operand reads are free of bank conflicts), so every direct load reads 1 KiB of contiguous memory.
// The weights are packed once when they are set, xg by the gather kernel, a by the up product's epilogue.
// Pipeline per 32-k step and wave: two phases of 8 MFMAs; the fragments of the next phase are read from LDS
// while the current one computes; one barrier per step, after which the stage just read is refilled with the
// step five ahead.  The direct loads are issued one at a time between MFMAs because the address unit is
// shared by all waves of the CU and a burst of loads stalls the issuing wave.
//
// Scheduling: the dispatch stage leaves a table of output tiles (one 32-byte descriptor each; row tiles never
// straddle two experts, empty experts have none) ordered (expert, column tile, row tile) with row tiles
// fastest, so that the workgroups resident on one XCD share weight tiles in its L2.
#include "common.h"
#include "pack.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

#define BM 256
#define BK 32
#define TILE_BYTES (BM * BK * 2)           // one operand tile: 16 KiB
#define STAGE_BYTES (2 * TILE_BYTES)       // A + B
#define NSTAGE 5
#define SMEM_BYTES (NSTAGE * STAGE_BYTES)  // 160 KiB: all of a CU's LDS
#define NWAVES 8
#define LOADS_PER_STEP 4                   // direct loads a wave issues per 32-k step (2 per operand)
#define NUM_XCD 8

int experts_bf16_tile_m(const omega_moe *, int) { return BM; }

__device__ __forceinline__ int swz(int row) { return pk_swz(row); }

// two floats -> two bf16 (round to nearest even) in one instruction, v_cvt_pk_bf16_f32; lo in bits 0..15
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi)
{
    const f32x2_t v = {lo, hi};
    const bf16x2_t r = __builtin_convertvector(v, bf16x2_t);
    return *(const uint32_t *)&r;
}

// 16 bytes per lane from global memory straight into LDS: lane l lands at lds_base + 16*l.
__device__ __forceinline__ void dma16(const void *sbase, uint32_t voff, uint32_t lds_base)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0" ::"s"(sbase), "v"(voff), "s"(lds_base)
                 : "memory");
}

// One output tile.  NBLK = number of 32-row blocks of this wave that hold valid rows (the others are never
// computed: a ragged last row tile of an expert costs only the blocks it fills).  NBLK == 0: the wave only
// takes part in the loads and barriers.
// A: packed row group of the tile's first row; B0/B1: packed row groups of the two 128-row halves of the B tile.
template <bool FUSED, int NBLK>
__device__ __forceinline__ void run_tile(unsigned char *smem, const unsigned char *A, const unsigned char *B0,
                                         const unsigned char *B1, void *Cout, const omega_tile tl, int n0, int N, int Kd,
                                         int wave, int lane)
{
    constexpr int NB = NBLK > 0 ? NBLK : 1;
    const int wm = wave >> 2, wn = wave & 3;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;

    const int KT = Kd / BK;
    // ---- direct-load addressing: wave-load q (0..15) of an operand tile is the packed block q % 8 of row
    //      group q / 8; this wave issues q = wave and q = wave + 8 of both operands.  Consecutive k steps of
    //      a row group are 8 KiB apart. ----
    const uint32_t blk_off = (uint32_t)wave * 1024u + (uint32_t)lane * 16u;
    // A blocks that hold no valid row (ragged last tile of an expert) are never used by an MFMA whose result is
    // kept: their loads are pointed at block 0 of the tile, which another wave loads in the same step anyway,
    // so they cost no extra L2 traffic while every wave still issues the same number of loads per step
    // (A points at the row group of the whole tile; a slice starts blk0 16-row blocks into it)
    const int blk0 = (tl.row0 & (BM - 1)) >> 4;
    const int qa0 = blk0 + (16 * wave < tl.rows ? wave : 0), qa1 = blk0 + (16 * (wave + 8) < tl.rows ? wave + 8 : 0);
    const uint32_t a_off0 = (uint32_t)(qa0 >> 3) * (uint32_t)KT * 8192u + (uint32_t)(qa0 & 7) * 1024u + (uint32_t)lane * 16u;
    const uint32_t a_off1 = (uint32_t)(qa1 >> 3) * (uint32_t)KT * 8192u + (uint32_t)(qa1 & 7) * 1024u + (uint32_t)lane * 16u;
// direct load n (0..3) of one 32-k step: n -> (operand, row group) = (n & 1 ? B : A, n >> 1)
#define ISSUE_LOAD1(stage, kstep, n)                                                                       \
    do {                                                                                                   \
        const uint32_t sb = lds0 + (stage) * STAGE_BYTES + wave * 1024;                                     \
        const uint32_t kb = (uint32_t)(kstep) * 8192u;                                                      \
        if (((n) & 1) == 0) dma16(A, kb + (((n) >> 1) ? a_off1 : a_off0), sb + ((n) >> 1) * 8192);          \
        else dma16(((n) >> 1) == 0 ? B0 : B1, kb + blk_off, sb + TILE_BYTES + ((n) >> 1) * 8192);            \
    } while (0)

    // ---- MFMA operand addressing ----
    const int l32 = lane & 31, lhi = lane >> 5;
    uint32_t a_rb[NB], b_rb[2];
    int a_sw[NB], b_sw[2];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        const int ar = (2 * i + wm) * 32 + l32;
        a_rb[i] = ar * (BK * 2);
        a_sw[i] = swz(ar);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        // up product: block 0 = 32 columns of W1, block 1 = the same 32 columns of W3
        const int br = FUSED ? (j * 128 + wn * 32 + l32) : (wn * 64 + j * 32 + l32);
        b_rb[j] = TILE_BYTES + br * (BK * 2);
        b_sw[j] = swz(br);
    }
#define READ_FRAGS(AF, BF, stage, ks)                                                                       \
    do {                                                                                                    \
        if (NBLK > 0) {                                                                                     \
            const unsigned char *sp = smem + (stage) * STAGE_BYTES;                                          \
            const int c = (ks) * 2 + lhi;                                                                    \
            _Pragma("unroll") for (int i = 0; i < NB; ++i)                                                   \
                AF[i] = *(const bf16x8_t *)(sp + a_rb[i] + ((c ^ a_sw[i]) << 4));                            \
            _Pragma("unroll") for (int j = 0; j < 2; ++j)                                                    \
                BF[j] = *(const bf16x8_t *)(sp + b_rb[j] + ((c ^ b_sw[j]) << 4));                            \
        }                                                                                                   \
    } while (0)
// the two MFMAs of row block i.  The up product feeds the weights as the first operand, so that a lane ends
// up with 4 consecutive output columns of one row (8 bytes of the packed `a`), the down product the rows, so
// that 32 lanes hold 32 consecutive columns of one row of y.
#define MFMA2(AF, BF, i)                                                                                     \
    do {                                                                                                    \
        if ((i) < NBLK) {                                                                                   \
            _Pragma("unroll") for (int j = 0; j < 2; ++j)                                                    \
                acc[i][j] = FUSED ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(BF[j], AF[i], acc[i][j], 0, 0, 0) \
                                  : __builtin_amdgcn_mfma_f32_32x32x16_bf16(AF[i], BF[j], acc[i][j], 0, 0, 0); \
        }                                                                                                   \
    } while (0)

    f32x16_t acc[NB][2];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    bf16x8_t af0[NB], bf0[2], af1[NB], bf1[2];

    // prologue: stages 0..NSTAGE-1 <- steps 0..NSTAGE-1; wait for step 0 only when all were issued
    for (int st = 0; st < NSTAGE && st < KT; ++st) {
#pragma unroll
        for (int n = 0; n < LOADS_PER_STEP; ++n) ISSUE_LOAD1(st, st, n);
    }
    if (KT >= NSTAGE) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");  // LOADS_PER_STEP * (NSTAGE - 1)
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    READ_FRAGS(af0, bf0, 0, 0);

// One 32-k step on stage `cur`.  The 4 direct loads a wave owes per step are issued one per pair of row blocks:
//   LOADS_B: first half of the loads of step kt+NSTAGE, into the stage this step releases at its barrier
//   LOADS_A: second half of the loads of step kt-1+NSTAGE, into the stage the previous step released
// STEADY: all loads up to step kt-1+NSTAGE exist, so exactly NSTAGE-2 younger steps (12 loads) may stay in
// flight at the barrier; otherwise (tail) everything must have landed.
#define K_STEP(kt, LOADS_A, LOADS_B, STEADY, NEXT)                                                  \
    do {                                                                                            \
        const int nxt = cur + 1 == NSTAGE ? 0 : cur + 1;                                            \
        const int prv = cur == 0 ? NSTAGE - 1 : cur - 1;                                            \
        __builtin_amdgcn_sched_barrier(0);                                                          \
        READ_FRAGS(af1, bf1, cur, 1);                                                               \
        _Pragma("unroll") for (int i = 0; i < 4; ++i)                                               \
        {                                                                                           \
            if (LOADS_A && (i & 1) == 0) ISSUE_LOAD1(prv, (kt) - 1 + NSTAGE, 2 + (i >> 1));     \
            MFMA2(af0, bf0, i);                                                                     \
        }                                                                                           \
        __builtin_amdgcn_sched_barrier(0);                                                          \
        /* every wave has taken its last fragments of this stage; the next stage must have landed */ \
        if (STEADY) asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)" ::: "memory");                    \
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");                            \
        __syncthreads();                                                                            \
        if (NEXT) READ_FRAGS(af0, bf0, nxt, 0);                                                     \
        _Pragma("unroll") for (int i = 0; i < 4; ++i)                                               \
        {                                                                                           \
            if (LOADS_B && (i & 1) == 0) ISSUE_LOAD1(cur, (kt) + NSTAGE, i >> 1);               \
            MFMA2(af1, bf1, i);                                                                     \
        }                                                                                           \
        cur = nxt;                                                                                  \
    } while (0)

    int kt = 0, cur = 0;
    if (KT > NSTAGE) {
        K_STEP(kt, false, true, true, true);
        for (kt = 1; kt + NSTAGE < KT; ++kt) K_STEP(kt, true, true, true, true);
        K_STEP(kt, true, false, true, true);  // kt == KT - NSTAGE: last step of the steady wait count
        ++kt;
    }
    for (; kt + 1 < KT; ++kt) K_STEP(kt, false, false, false, true);
    K_STEP(kt, false, false, false, false);
#undef K_STEP

    // ---- epilogue ----
    if (FUSED) {
        // lane: row l32 of block i; register r -> column 8*(r/4) + 4*lhi + r%4 of the wave's 32 columns, which are
        // one k step of the packed `a` (K dimension = N): chunk r/4, bytes lhi*8 .. lhi*8+7
        const int KTa = N / BK;
        const int kba = (n0 >> 5) + wn;
#pragma unroll
        for (int i = 0; i < NBLK; ++i) {
            const int row = (2 * i + wm) * 32 + l32;
            if (row < tl.rows) {
                const int prow = tl.row0 + row;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    uint32_t pk[2];
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        float v[2];
#pragma unroll
                        for (int u = 0; u < 2; ++u) {
                            const float h1 = acc[i][0][t * 4 + h * 2 + u], h3 = acc[i][1][t * 4 + h * 2 + u];
                            v[u] = h1 * __builtin_amdgcn_rcpf(1.0f + __expf(-h1)) * h3;  // v_exp_f32, v_rcp_f32: 1 ulp each
                        }
                        pk[h] = pack_bf16x2(v[0], v[1]);
                    }
                    uint2 o = {pk[0], pk[1]};
                    *(uint2 *)((unsigned char *)Cout + pk_chunk_off(prow, kba, t, KTa) + lhi * 8) = o;
                }
            }
        }
    } else {
        // lane: column l32 of each 32x32 block; register r -> row 8*(r/4) + 4*lhi + r%4
#pragma unroll
        for (int i = 0; i < NBLK; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = (2 * i + wm) * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
                if (row >= tl.rows) continue;
                float *out = (float *)Cout + (size_t)(tl.row0 + row) * N + n0 + wn * 64 + l32;
#pragma unroll
                for (int j = 0; j < 2; ++j) out[j * 32] = acc[i][j][r];
            }
        }
    }
#undef ISSUE_LOAD1
#undef READ_FRAGS
#undef MFMA2
}

template <bool FUSED>
__global__ __launch_bounds__(NWAVES * 64) void experts_bf16_kernel(const bf16_t *__restrict__ Axg, const bf16_t *__restrict__ Ax,
                                                                   const bf16_t *__restrict__ Wa, const bf16_t *__restrict__ Wb,
                                                                   void *__restrict__ Cout, const omega_tile_desc *__restrict__ desc,
                                                                   const int32_t *__restrict__ tile_meta, int total_slot, int N, int Kd)
{
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    constexpr int NCOLS = FUSED ? 128 : 256;  // output columns per tile
    const int NT = N / NCOLS;
    // ---- workgroup -> tile ----
    // Consecutive workgroup ids go round-robin over the 8 XCDs, and an XCD (32 compute units, one workgroup each)
    // starts its workgroups in id order.  The table is cut into rounds of 256 consecutive entries; within a round
    // XCD x takes a contiguous eighth - of what is left, in the last round, so that a short tail (or a launch of
    // fewer than 256 tiles) still spreads over all eight L2s.
    const int total = tile_meta[total_slot];
    const int pid = blockIdx.x;
    const int q = pid / NUM_XCD, base = (q >> 5) * 256;
    const int left = min(256, total - base);
    if (left <= 0) return;
    const int per = (left + NUM_XCD - 1) / NUM_XCD;
    const int L = base + (pid % NUM_XCD) * per + (q & 31);
    if ((q & 31) >= per || L >= base + left) return;
    const omega_tile_desc dsc = desc[L];
    const omega_tile tl = {dsc.g, dsc.row0, dsc.rows, dsc.xrow0};
    if (tl.rows <= 0) return;  // empty slice of a ragged tile
    const int n0 = dsc.n0;

    // packed operands: a row group (128 rows) occupies KT * 8 KiB
    const size_t rg_bytes = (size_t)(Kd / BK) * 8192;
    const unsigned char *A = (FUSED && tl.xrow0 >= 0) ? (const unsigned char *)Ax + (size_t)(tl.xrow0 / BM * 2) * rg_bytes
                                                      : (const unsigned char *)Axg + (size_t)(tl.row0 / BM * 2) * rg_bytes;
    const size_t wrg = (size_t)tl.g * (N >> 7) + (n0 >> 7);  // row group of the weight tile
    const unsigned char *B0 = (const unsigned char *)Wa + wrg * rg_bytes;
    const unsigned char *B1 = FUSED ? (const unsigned char *)Wb + wrg * rg_bytes : B0 + rg_bytes;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // 32-row blocks alternate between the two row halves of the workgroup: block b belongs to waves with wm = b % 2
    const int nblk = max(0, min(4, (((tl.rows + 31) >> 5) + 1 - (wave >> 2)) >> 1));
    switch (nblk) {
        case 4: run_tile<FUSED, 4>(smem, A, B0, B1, Cout, tl, n0, N, Kd, wave, lane); break;
        case 3: run_tile<FUSED, 3>(smem, A, B0, B1, Cout, tl, n0, N, Kd, wave, lane); break;
        case 2: run_tile<FUSED, 2>(smem, A, B0, B1, Cout, tl, n0, N, Kd, wave, lane); break;
        case 1: run_tile<FUSED, 1>(smem, A, B0, B1, Cout, tl, n0, N, Kd, wave, lane); break;
        default: run_tile<FUSED, 0>(smem, A, B0, B1, Cout, tl, n0, N, Kd, wave, lane); break;
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
    if (which == 0) {
        int grid = m->max_m_tiles * (c.H / 128) + OMEGA_TAIL_EXTRA;
        grid = (grid + 255) / 256 * 256;
        hipLaunchKernelGGL(experts_bf16_kernel<true>, dim3(grid), dim3(NWAVES * 64), SMEM_BYTES, s, (const bf16_t *)m->xg,
                           (const bf16_t *)m->xs, (const bf16_t *)m->W1, (const bf16_t *)m->W3, m->a, m->desc_up, m->tile_meta,
                           c.E + c.Es + 2, c.H, c.d);
    } else {
        int grid = m->max_m_tiles * (c.d / 256) + OMEGA_TAIL_EXTRA;
        grid = (grid + 255) / 256 * 256;
        hipLaunchKernelGGL(experts_bf16_kernel<false>, dim3(grid), dim3(NWAVES * 64), SMEM_BYTES, s, (const bf16_t *)m->a,
                           (const bf16_t *)nullptr, (const bf16_t *)m->W2, (const bf16_t *)nullptr, (void *)m->y, m->desc_down,
                           m->tile_meta, c.E + c.Es + 3, c.d, c.H);
    }
    return hipGetLastError();
}
