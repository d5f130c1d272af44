// Grouped expert SwiGLU products in bf16 on the CDNA4 matrix cores (v_mfma_f32_16x16x32_bf16, fp32 accumulate; four of
// them per 32x32 block and 32-k step: measured 3.5 % faster than one v_mfma_f32_32x32x16_bf16 pair at the same LDS traffic).
//   up    a[r,h] = silu(xg[r,:].W1g[h,:]) * (xg[r,:].W3g[h,:])   -> bf16      (one pass over xg for both weights)
//   down  y[r,c] = a[r,:].W2g[c,:]                                -> fp32
// (J/engine/nn/layer/llama/LlamaMLPLayer.java:117-130; y = x W^T with W [out,in], J/engine/nn/layer/FullyLayer.java:181,235.)
//
// Both operands are K-contiguous ("NT" product), so a lane's 8 consecutive k values are one 16-byte LDS read.
// Tile = 256 rows x 256 MFMA columns; for the up product the 256 MFMA columns are 128 columns of W1 and the same 128
// columns of W3, arranged so that a wave holds h1 and h3 of the same output element and applies silu(h1)*h3 in
// registers.  Two kernels share everything below except the shape of a workgroup:
//   experts_up4_kernel   four waves of 128 x 128, one per SIMD, 256 accumulator registers each (AGPRs), 16 fragment
//                        reads per 64 MFMAs, the instruction order of a k step pinned (a lone wave issues one instruction
//                        every four cycles, an MFMA occupies the matrix core for sixteen).  The forward pass's up
//                        product (it can fetch its rows from x through the row -> token table), the down product with
//                        256-column items and the backward pass's input-gradient product: 2-3 % faster than eight waves.
//   experts_bf16_kernel  eight waves (2 row halves x 4 column quarters, two per SIMD, 128 accumulator registers each;
//                        the 32-row blocks of the tile alternate between the row halves, so a ragged tile splits
//                        evenly): the products that keep or read h1 / h3 records, the weight gradients, and down
//                        products with 128-column items.
//
// Data movement: global -> LDS directly (global_load_lds_dwordx4, no staging registers) into a ring of five
// stages of (A 256x32 + B 256x32) bf16 = 160 KiB, i.e. all of a CU's LDS.  A wave-wide direct load fills 1 KiB
// of LDS in lane order = 16 rows of four 16-byte chunks.  All three operands (weights, xg, a) are kept in
// memory as that very image (pack.h: 1 KiB blocks of 16 rows x 32 k with the chunk index XOR-swizzled so the
// MFMA operand reads are free of bank conflicts), so every direct load reads 1 KiB of contiguous memory.
// The weights are packed once when they are set, xg by the dispatch launch, a by the up product's epilogue.
// Pipeline per 32-k step and wave (eight waves): two phases of 16 MFMAs; the fragments of the next phase are read from LDS
// while the current one computes; one barrier per step, after which the stage just read is refilled with the
// step five ahead; four direct loads per wave and step.  Every step of every item is the same code (the addresses the
// loads read from next sit in scalar registers and are switched to the next item when its turn comes), and the bulk of
// an item runs five steps at a time from ring position 0 with every LDS address a constant: under the power cap the
// launch time follows the work per MFMA, instructions included (68-71 per step and wave, 32 of them MFMAs).
//
// Scheduling: persistent, one workgroup per compute unit.  The dispatch stage leaves every workgroup a queue of
// work items (32-byte descriptors: an output tile, or a slice of the rows of one for the last tiles of a launch;
// row tiles never straddle two experts, empty experts have none), dealt so that the workgroups of an XCD work on
// neighbouring tiles - (expert, column tile, row tile) with row tiles fastest - at the same time and share weight
// tiles in its L2, and so that all queues hold the same amount of work.  The ring of LDS stages runs on from one
// item to the next: the last steps of an item already fetch the first steps of the next, so a workgroup pays
// the load latency once per launch, not once per tile.
//
// The backward pass of bf16 layers runs on the same kernel (MODE below): every product of it is brought into the
// "both operands K-contiguous" form by keeping transposed packed copies of the weights and by transposing the
// activations for the weight gradients, so the matrix-core pipeline is the one above and only the epilogues differ.
#include "common.h"
#include "pack.h"

// What one instantiation of the product kernel computes (tile shape, operand order, epilogue):
//   UP     tile 256 x (128 of Wa + 128 of Wb), silu(h1)*h3 -> packed bf16 a
//   DOWN   tile 256 x 256, fp32 row-major output; an item may be a k slice of a tile (see make_ctx)
//   UPRAW  as UP, but h1 and h3 are stored as they sit in the accumulators (Cout = h1, Aux1 = h3): one 4 KiB record
//          per 32x32 MFMA block, [row block][column block][register 0..15][lane 0..63]
//   UPREC  UP and UPRAW in one: the forward pass of a layer in training mode (a -> Cout, h1 -> Aux1, h3 -> Aux2)
//   DA     tile 256 x 256 of d(a) = dy . W2 (B = packed W2^T); the epilogue reads the h1/h3 records of its blocks
//          (Aux1, Aux2), applies the SwiGLU backward and writes dh1 | dh3 as one packed bf16 image with 2N columns
//   WGRAD  tile 256 x 256 of dW = A^T . B over the rows of one expert: both operands are transposed packed images
//          whose K axis is the experts' rows; the item names its operand row groups, first k step and k steps
//          (a_rg, b_rg, kt0, xrow0); fp32 row-major output, row0 = expert * M + first row
#define FUSED_TILE(M) ((M) == MODE_UP || (M) == MODE_UPRAW || (M) == MODE_UPREC)
#define PLAIN_DOWN(M) ((M) == MODE_DOWN)
#define SWAPPED(M) (!PLAIN_DOWN(M) && (M) != MODE_WGRAD)
#define ITEM_K(M) ((M) == MODE_WGRAD || PLAIN_DOWN(M))  // the k range belongs to the item, not to the launch

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

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

// 16 bytes per lane from global memory straight into LDS: lane l lands at lds_base + LDS_OFF + 16*l (the sum is formed
// in m0 by the instruction that sets it: a constant offset costs nothing).
template <int LDS_OFF>
__device__ __forceinline__ void dma16(const void *sbase, uint32_t voff, uint32_t lds_base)
{
    asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0" ::"s"(sbase), "v"(voff), "s"(lds_base), "n"(LDS_OFF)
                 : "memory", "scc");
}

// Non-temporal form, for weight tiles that no other item will read again (small batches: the weights are streamed
// once, and letting them pass the last-level cache by is worth 9 % of the stream: 5.9 -> 6.5 TB/s at 64 tokens)
template <int LDS_OFF>
__device__ __forceinline__ void dma16_nt(const void *sbase, uint32_t voff, uint32_t lds_base)
{
    asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0 nt" ::"s"(sbase), "v"(voff), "s"(lds_base), "n"(LDS_OFF)
                 : "memory", "scc");
}

// The same with only the lanes of `mask` taking part: a wave whose 16-row block of the A tile holds no valid row keeps
// its place in the load sequence (the waits count instructions) but moves 16 bytes instead of 1 KiB.  `active` = the
// lanes that are active at the call (read once per work item, read_active_lanes) and are active again afterwards;
// `mask` must be a subset of them.
template <int LDS_OFF>
__device__ __forceinline__ void dma16_masked(const void *sbase, uint32_t voff, uint32_t lds_base, uint64_t mask, uint64_t active)
{
    asm volatile("s_add_u32 m0, %2, %5\n\ts_mov_b64 exec, %3\n\tglobal_load_lds_dwordx4 %1, %0\n\ts_mov_b64 exec, %4"
                 :
                 : "s"(sbase), "v"(voff), "s"(lds_base), "s"(mask), "s"(active), "n"(LDS_OFF)
                 : "memory", "scc");
}
__device__ __forceinline__ uint64_t read_active_lanes() { return __builtin_amdgcn_read_exec(); }

// Everything the loads of one work item need, uniform over the wave: lane l adds 16 l to every address.
// A0/A1: k step 0 of this wave's two 16-row blocks of the A tile (packed row groups of the tile's first row and of the
// one 128 rows on); B0/B1: the same of the two 128-row halves of the B tile.
struct TileCtx {
    const unsigned char *A0, *A1, *B0, *B1;
    uint64_t a_mask0, a_mask1;  // lanes that take part in the two A loads: all, or lane 0 alone for a block without valid rows
    int row0, rows, n0;
    int kt;                   // k steps of the item
    int half;                 // plain 256-column products: the item covers the first 128 columns only
    int slab;                 // down products: 0 = the item writes the output, > 0 = partial result `slab` of those behind Aux1
    int rec0;                 // products that write or read h1 / h3 block records: record of the item's first 32-row block
};

__device__ __forceinline__ const unsigned char *uniform_ptr(const unsigned char *p)
{
    const uint64_t v = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const unsigned char *)(((uint64_t)hi << 32) | lo);
}

__device__ __forceinline__ uint64_t uniform_u64(uint64_t v)
{
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return ((uint64_t)hi << 32) | lo;
}

// slices: the launch has room for partial results (Aux1), so items that are k slices run as such
template <int MODE>
__device__ __forceinline__ TileCtx make_ctx(const omega_tile_desc &d, const bf16_t *Axg, const bf16_t *Ax, const bf16_t *Wa,
                                            const bf16_t *Wb, int N, int Kd, int wave, int lane, bool slices)
{
    constexpr bool FUSED = FUSED_TILE(MODE);
    TileCtx c;
    const int KT = Kd / BK;
    const size_t rg_bytes = (size_t)KT * 8192;  // a packed row group (128 rows) occupies KT * 8 KiB
    c.row0 = d.row0;
    c.rows = d.rows;
    c.n0 = d.n0;
    if (MODE == MODE_WGRAD) {
        const size_t k0 = (size_t)d.kt0 * 8192;
        c.kt = d.xrow0;
        c.half = 0;
        c.slab = 0;
        c.rec0 = 0;
        c.A0 = uniform_ptr((const unsigned char *)Axg + (size_t)d.a_rg * rg_bytes + k0 + (size_t)wave * 1024u);
        c.A1 = uniform_ptr(c.A0 + rg_bytes);
        c.B0 = uniform_ptr((const unsigned char *)Wa + (size_t)d.b_rg * rg_bytes + k0 + (size_t)wave * 1024u);
        c.B1 = uniform_ptr(c.B0 + rg_bytes);
        c.a_mask0 = c.a_mask1 = ~0ull;
        return c;
    }
    c.kt = KT;
    c.slab = 0;
    c.rec0 = d.kt0;
    c.half = FUSED ? 0 : d.b_rg;
    // k slices of a down product (items with a_rg = KS > 1, kt0 = ks, xrow0 = number of the partial result: every tile of
    // a small batch, or the last tiles of a launch that would leave most compute units idle): slice ks runs over its own
    // part of the k range; slice 0 writes the output, the others partial results that down_slab_reduce_kernel adds to
    // it.  A launch without room for partial results computes the whole range in the item of slice 0 and only keeps
    // the other slices' workgroups in step (no rows: loads and barriers, no results).
    size_t k0 = 0;
    if (PLAIN_DOWN(MODE) && d.a_rg > 1) {
        if (slices) {
            const int first = (d.kt0 * KT) / d.a_rg;  // even parts: every slice has at least KT / KS >= 8 steps
            c.kt = ((d.kt0 + 1) * KT) / d.a_rg - first;
            c.slab = d.kt0 > 0 ? d.xrow0 : 0;
            k0 = (size_t)first * 8192;
        } else if (d.kt0 > 0) {
            c.rows = 0;
        }
    }
    const unsigned char *A = ((!PLAIN_DOWN(MODE) && Ax != nullptr && d.xrow0 >= 0)
                                  ? (const unsigned char *)Ax + (size_t)(d.xrow0 / BM * 2) * rg_bytes
                                  : (const unsigned char *)Axg + (size_t)(d.row0 / BM * 2) * rg_bytes) + k0;
    const size_t wrg = (size_t)d.g * (N >> 7) + (d.n0 >> 7);  // row group of the weight tile
    c.B0 = uniform_ptr((const unsigned char *)Wa + wrg * rg_bytes + k0 + (size_t)wave * 1024u);
    // (a half-width item loads its 128 weight rows twice - the second copy comes out of the L2 - and drops the results
    //  of the duplicate: the products it is used for are bound by streaming the weights from memory, not by the MFMAs)
    c.B1 = uniform_ptr(FUSED ? (const unsigned char *)Wb + wrg * rg_bytes + k0 + (size_t)wave * 1024u : c.half ? c.B0 : c.B0 + rg_bytes);
    // Wave-load q (0..15) of an operand tile is the packed block q % 8 of row group q / 8; this wave issues q = wave
    // and q = wave + 8 of both operands.  A points at the row group of the whole row tile; a slice starts blk0
    // 16-row blocks into it.  A blocks that hold no valid row (ragged tile) are never used by an MFMA whose result
    // is kept: their loads are pointed at the first block, which another wave loads in the same step anyway, so
    // they cost no extra L2 traffic while every wave still issues the same number of loads per step.
    c.a_mask0 = 16 * wave < c.rows ? ~0ull : 1ull;
    c.a_mask1 = 16 * (wave + 8) < c.rows ? ~0ull : 1ull;
    const int blk0 = (d.row0 & (BM - 1)) >> 4;
    const int qa0 = blk0 + (16 * wave < d.rows ? wave : 0), qa1 = blk0 + (16 * (wave + 8) < d.rows ? wave + 8 : 0);
    c.A0 = uniform_ptr(A + (size_t)(qa0 >> 3) * rg_bytes + (size_t)(qa0 & 7) * 1024u);
    c.A1 = uniform_ptr(A + (size_t)(qa1 >> 3) * rg_bytes + (size_t)(qa1 & 7) * 1024u);
    return c;
}

// direct load n (0..3) of k step `kstep` of a work item into ring stage `stage`: n -> (operand, row group) =
// (n & 1 ? B : A, n >> 1)
// A blocks without valid rows move 16 bytes (a_mask0 / a_mask1).
template <bool WNT = false>
__device__ __forceinline__ void issue_load(const TileCtx &c, uint32_t lds_wave, uint32_t lane_off, int stage, int kstep, int n,
                                           uint64_t active)
{
    const uint32_t sb = lds_wave + stage * STAGE_BYTES;
    const size_t kb = (size_t)kstep * 8192u;
    if ((n & 1) == 0)
        dma16_masked<0>(((n >> 1) ? c.A1 : c.A0) + kb, lane_off, sb + (n >> 1) * 8192, ((n >> 1) ? c.a_mask1 : c.a_mask0) & active, active);
    else if (WNT) dma16_nt<0>(((n >> 1) == 0 ? c.B0 : c.B1) + kb, lane_off, sb + TILE_BYTES + (n >> 1) * 8192);
    else dma16<0>(((n >> 1) == 0 ? c.B0 : c.B1) + kb, lane_off, sb + TILE_BYTES + (n >> 1) * 8192);
}

// Where the four loads a wave owes per k step read next: the pointers move on by one k step (8 KiB of the packed image)
// with every load and are pointed at the next work item when this one's last step has been asked for.  Loads 0 and 1
// (first row group of A and of B) run one step ahead of loads 2 and 3.
struct LoadCursor {
    const unsigned char *a0, *a1, *b0, *b1;
    uint64_t m0, m1;
};

// One work item.  NBLK = number of 32-row blocks of this wave that hold valid rows (the others are never
// computed: a ragged last row tile of an expert costs only the blocks it fills).  NBLK == 0: the wave only
// takes part in the loads and barriers.
// The ring of stages runs on across work items: on entry, stage `cur` holds (or is about to receive) k step 0 of this
// item, k steps 0..NSTAGE-2 and the first half of step NSTAGE-1 are in flight, and the barrier that makes step 0
// visible has been passed.  The last NSTAGE steps issue the first loads of the next item (dn) instead of their own,
// so the matrix cores of the next item start on data that travelled during this item's epilogue; behind the last item
// of a queue they fetch this item's first steps once more (lane 0 only for A), so that every step of every item
// issues the same four loads and waits the same way.
template <int MODE, int NBLK, bool WNT>
__device__ __forceinline__ void run_tile(unsigned char *smem, const TileCtx ctx_in, TileCtx &nx, const omega_tile_desc &dn,
                                         const bf16_t *Axg, const bf16_t *Ax, const bf16_t *Wa, const bf16_t *Wb, int &cur_io,
                                         void *Cout, void *Aux1, void *Aux2, int N, int Kd, int wave, int lane)
{
    constexpr bool FUSED = FUSED_TILE(MODE), SWAP = SWAPPED(MODE);
    constexpr int NB = NBLK > 0 ? NBLK : 1;
    // the item's uniform fields and the ring position live in scalar registers for the whole item (the direct loads
    // take their base address and LDS address from scalar operands)
    TileCtx ctx = ctx_in;
    ctx.A0 = uniform_ptr(ctx_in.A0);
    ctx.A1 = uniform_ptr(ctx_in.A1);
    ctx.B0 = uniform_ptr(ctx_in.B0);
    ctx.B1 = uniform_ptr(ctx_in.B1);
    ctx.row0 = __builtin_amdgcn_readfirstlane(ctx_in.row0);
    ctx.rows = __builtin_amdgcn_readfirstlane(ctx_in.rows);
    ctx.n0 = __builtin_amdgcn_readfirstlane(ctx_in.n0);
    ctx.half = __builtin_amdgcn_readfirstlane(ctx_in.half);
    ctx.slab = __builtin_amdgcn_readfirstlane(ctx_in.slab);
    ctx.rec0 = __builtin_amdgcn_readfirstlane(ctx_in.rec0);
    ctx.a_mask0 = uniform_u64(ctx_in.a_mask0);
    ctx.a_mask1 = uniform_u64(ctx_in.a_mask1);
    int cur = __builtin_amdgcn_readfirstlane(cur_io);
    const int wm = wave >> 2, wn = wave & 3;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    const uint32_t lds_wave = lds0 + wave * 1024;
    const uint32_t lane_off = (uint32_t)lane * 16u;
    const int KT = ITEM_K(MODE) ? __builtin_amdgcn_readfirstlane(ctx_in.kt) : Kd / BK;
    const bool has_next = dn.rows > 0;
    LoadCursor lc;
    lc.a0 = ctx.A0 + (size_t)NSTAGE * 8192;
    lc.b0 = ctx.B0 + (size_t)NSTAGE * 8192;
    lc.a1 = ctx.A1 + (size_t)(NSTAGE - 1) * 8192;
    lc.b1 = ctx.B1 + (size_t)(NSTAGE - 1) * 8192;
    // (the masked A loads switch lanes off and on again: the lanes active here, and the masks as subsets of them)
    const uint64_t active = uniform_u64(read_active_lanes());
    lc.m0 = ctx.a_mask0 & active;
    lc.m1 = ctx.a_mask1 & active;
#define LOAD_B(ptr, voff, lds, off) do { if (WNT) dma16_nt<off>(ptr, voff, lds); else dma16<off>(ptr, voff, lds); } while (0)

    // ---- MFMA operand addressing ----
    // Row (2i + wm)*32 + 16 rh + l16 of A, row j*128 + wn*32 + 16 ch + l16 (up: block 0 = 32 columns of W1, block 1 = the
    // same 32 columns of W3) or wn*64 + j*32 + 16 ch + l16 (down) of B.  The chunk swizzle depends on the row through
    // l16 and bit 4 only (rows differ by multiples of 32 otherwise), so one swizzled offset per half serves every block
    // and the blocks are constant byte offsets.  (An item may start 16 rows into a 32-row unit of the packed image: the
    // swizzle of the A rows follows the physical row, i.e. bit 4 flipped.)
    // Fragments of v_mfma_f32_16x16x32_bf16: 16 rows x 32 k = one 1 KiB block of the tile image; lane l supplies row
    // l % 16, chunk l / 16.  rh / ch = which 16-row half of a 32-row block of A / 32-column block of B.
    const int l16 = lane & 15, lq = lane >> 4;
    uint32_t pa[2], pb[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int par_a = MODE == MODE_WGRAD ? h : (h ^ ((ctx.row0 >> 4) & 1));  // bit 4 of the physical row
        pa[h] = (uint32_t)(wm * 32 + 16 * h + l16) * (BK * 2) + ((uint32_t)(lq ^ swz(l16 | (par_a << 4))) << 4);
        pb[h] = TILE_BYTES + (uint32_t)((FUSED ? wn * 32 : wn * 64) + 16 * h + l16) * (BK * 2) +
                ((uint32_t)(lq ^ swz(l16 | (h << 4))) << 4);
    }
    constexpr uint32_t A_BLK = 64 * BK * 2, B_BLK = (FUSED ? 128 : 32) * BK * 2;
// the rh-th 16-row halves of this wave's row blocks
#define READ_A(AF, stage, rh)                                                                               \
    do {                                                                                                    \
        if (NBLK > 0) {                                                                                     \
            const unsigned char *sp = smem + (stage) * STAGE_BYTES;                                          \
            _Pragma("unroll") for (int i = 0; i < NB; ++i)                                                   \
                AF[i] = *(const bf16x8_t *)(sp + pa[rh] + i * A_BLK);                                        \
        }                                                                                                   \
    } while (0)
// the four 16-column pieces of this wave's two column blocks: BF[2 * j + ch]
#define READ_B(BF, stage)                                                                                   \
    do {                                                                                                    \
        if (NBLK > 0) {                                                                                     \
            const unsigned char *sp = smem + (stage) * STAGE_BYTES;                                          \
            _Pragma("unroll") for (int q = 0; q < 4; ++q)                                                    \
                BF[q] = *(const bf16x8_t *)(sp + pb[q & 1] + (q >> 1) * B_BLK);                              \
        }                                                                                                   \
    } while (0)
// the four MFMAs of half rh of row block i.  The up product feeds the weights as the first operand, so that a lane
// ends up with 4 consecutive output columns of one row (8 bytes of the packed `a`), the down product the rows, so
// that 16 lanes hold 16 consecutive columns of one row of y.
#define MFMA4(AF, BF, i, rh, Z)                                                                              \
    do {                                                                                                    \
        if ((i) < NBLK) {                                                                                   \
            _Pragma("unroll") for (int q = 0; q < 4; ++q)                                                    \
                acc[i][q >> 1][rh][q & 1] =                                                                  \
                    SWAP ? __builtin_amdgcn_mfma_f32_16x16x32_bf16(BF[q], AF[i], (Z) ? zero4 : acc[i][q >> 1][rh][q & 1], 0, 0, 0) \
                         : __builtin_amdgcn_mfma_f32_16x16x32_bf16(AF[i], BF[q], (Z) ? zero4 : acc[i][q >> 1][rh][q & 1], 0, 0, 0); \
        }                                                                                                   \
    } while (0)

    // acc[i][j][rh][ch]: 16 x 16 piece (rh, ch) of the 32 x 32 block (row block i, column block j)
    f32x4_t acc[NB][2][2][2];
    const f32x4_t zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
    // The products with the weights as first operand start their accumulators from zero operands in a first step of its
    // own instead of clearing 128 registers per wave and item: up product 1.1-1.7 % faster at 128-step items.  (The down
    // product measured 0.8-1.3 % slower next to it even where its code is the very same: the part runs at its power cap,
    // and what one product gains the next one pays back in clock; the forward pass as a whole gains 0.4 %.)  The other
    // products clear the registers: with the zero-operand step they were slower.
    constexpr bool ZFIRST = SWAP;
    if (!ZFIRST) {
#pragma unroll
        for (int i = 0; i < NB; ++i)
#pragma unroll
            for (int q = 0; q < 8; ++q) acc[i][q >> 2][(q >> 1) & 1][q & 1] = zero4;
    }

    bf16x8_t af0[NB], af1[NB], bq[4], bn[4];
    READ_A(af0, cur, 0);
    READ_B(bq, cur);

    // One 32-k step on stage `cur`.  The 4 direct loads a wave owes per step are issued one per pair of row blocks:
    //   before the barrier: loads 2 and 3 of step kt-1+NSTAGE, into the stage the previous step released
    //   after the barrier:  loads 0 and 1 of step kt+NSTAGE, into the stage this step releases
    // Every step of every item issues its four loads (see LoadCursor), so exactly NSTAGE-2 younger steps (12 loads) may
    // stay in flight at the barrier, and every step reads the fragments of the one behind it (the last step of an item
    // those of the next item's first, which run_tile reads again on entry).
// BP + IP / BC + IC: LDS address of this wave's first load into the previous / the current stage (scalar register +
// constant); VOFF: the lane's offset from the load pointers, which then move on by ADV bytes
#define K_STEP_BODY(cur, BP, IP, BC, IC, VOFF, ADV, Z)                                                                \
    do {                                                                                                    \
        const int nxt = (cur) + 1 == NSTAGE ? 0 : (cur) + 1;                                                \
        __builtin_amdgcn_sched_barrier(0);                                                                  \
        READ_A(af1, cur, 1);                                                                                \
        _Pragma("unroll") for (int i = 0; i < 4; ++i)                                                       \
        {                                                                                                   \
            if (i == 0) dma16_masked<(IP) + 8192>(lc.a1, VOFF, BP, lc.m1, active);                                  \
            if (i == 2) LOAD_B(lc.b1, VOFF, BP, (IP) + TILE_BYTES + 8192);                                  \
            MFMA4(af0, bq, i, 0, Z);                                                                         \
        }                                                                                                   \
        lc.a1 += (ADV);                                                                                     \
        lc.b1 += (ADV);                                                                                     \
        __builtin_amdgcn_sched_barrier(0);                                                                  \
        /* every wave has taken its last fragments of this stage; the next stage must have landed */        \
        asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)" ::: "memory");                                        \
        __syncthreads();                                                                                    \
        READ_A(af0, nxt, 0);                                                                                \
        READ_B(bn, nxt);                                                                                    \
        _Pragma("unroll") for (int i = 0; i < 4; ++i)                                                       \
        {                                                                                                   \
            if (i == 0) dma16_masked<(IC)>(lc.a0, VOFF, BC, lc.m0, active);                                     \
            if (i == 2) LOAD_B(lc.b0, VOFF, BC, (IC) + TILE_BYTES);                                         \
            MFMA4(af1, bq, i, 1, Z);                                                                         \
        }                                                                                                   \
        lc.a0 += (ADV);                                                                                     \
        lc.b0 += (ADV);                                                                                     \
        _Pragma("unroll") for (int q = 0; q < 4; ++q) bq[q] = bn[q];                                        \
    } while (0)
// the step at a ring position known at compile time
// (one of five in a row from position 0: the lane offsets carry the k step, the pointers move once per five)
#define K_STEP_AT(c, Z) \
    K_STEP_BODY(c, lds_wave, ((c) == 0 ? NSTAGE - 1 : (c)-1) * STAGE_BYTES, lds_wave, (c)*STAGE_BYTES, lane_off + (c)*8192u, 0, Z)
// the step at the ring's position, whatever it is
#define K_STEP(Z)                                                                                             \
    do {                                                                                                    \
        const uint32_t sb_prv = lds_wave + (cur == 0 ? NSTAGE - 1 : cur - 1) * STAGE_BYTES;                 \
        const uint32_t sb_cur = lds_wave + cur * STAGE_BYTES;                                               \
        K_STEP_BODY(cur, sb_prv, 0, sb_cur, 0, lane_off, 8192, Z);                                                       \
        cur = cur + 1 == NSTAGE ? 0 : cur + 1;                                                              \
    } while (0)

    // (every item has at least NSTAGE + 1 steps: widths are multiples of 256, a k slice has 8 steps or more, an item of
    //  the weight-gradient products 6)
    int kt = 0;
    if (ZFIRST) {
        K_STEP(true);
        ++kt;
    }
    // The steps whose loads are all this item's own run five at a time from ring position 0, one copy of the step per
    // position, so that every LDS address in them is a constant (no address arithmetic per step: 79 instead of 96
    // instructions); single steps bring the ring to position 0 first, and what is left over runs with the item's last
    // steps below.  (Every wave of a workgroup runs the same form: with the five-step form in the waves of full row
    // blocks only, ragged tiles were 2-4 % slower than without it.)
    static_assert(NSTAGE == 5, "one copy of the step per stage");
    int left = KT - NSTAGE - kt;
    for (; left > 0 && cur != 0; --left) K_STEP(false);
    for (; left >= NSTAGE; left -= NSTAGE) {
        K_STEP_AT(0, false);
        K_STEP_AT(1, false);
        K_STEP_AT(2, false);
        K_STEP_AT(3, false);
        K_STEP_AT(4, false);
        lc.a0 += NSTAGE * 8192;
        lc.b0 += NSTAGE * 8192;
        lc.a1 += NSTAGE * 8192;
        lc.b1 += NSTAGE * 8192;
    }
    // the remaining steps; in the last NSTAGE of them the loads belong to the next item, loads 2 and 3 one step later
    nx = make_ctx<MODE>(dn, Axg, Ax, Wa, Wb, N, Kd, wave, lane, PLAIN_DOWN(MODE) && Aux1 != nullptr);
#pragma unroll 1
    for (int s = -left; s < NSTAGE; ++s) {
        if (s == 0) {
            lc.a0 = has_next ? nx.A0 : ctx.A0;
            lc.b0 = has_next ? nx.B0 : ctx.B0;
            lc.m0 = (has_next ? nx.a_mask0 : 1ull) & active;
        }
        if (s == 1) {
            lc.a1 = has_next ? nx.A1 : ctx.A1;
            lc.b1 = has_next ? nx.B1 : ctx.B1;
            lc.m1 = (has_next ? nx.a_mask1 : 1ull) & active;
        }
        K_STEP(false);
    }
#undef K_STEP
#undef K_STEP_AT
#undef K_STEP_BODY
#undef LOAD_B
    cur_io = cur;

    // ---- epilogue ----
    if (MODE == MODE_UP || MODE == MODE_UPREC) {
        // lane: row 16 rh + l16 of block i; piece (rh, ch), register r -> column 16 ch + 4 lq + r of the wave's 32
        // columns, which are one k step of the packed `a` (K dimension = N): chunk 2 ch + lq / 2, bytes (lq % 2) * 8 ..
        const int KTa = N / BK;
        const int kba = (ctx.n0 >> 5) + wn;
#pragma unroll
        for (int i = 0; i < NBLK; ++i) {
#pragma unroll
            for (int rh = 0; rh < 2; ++rh) {
                const int row = (2 * i + wm) * 32 + 16 * rh + l16;
                if (row < ctx.rows) {
                    const int prow = ctx.row0 + row;
#pragma unroll
                    for (int ch = 0; ch < 2; ++ch) {
                        float v[4];
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const float h1 = acc[i][0][rh][ch][r], h3 = acc[i][1][rh][ch][r];
                            v[r] = h1 * __builtin_amdgcn_rcpf(1.0f + __expf(-h1)) * h3;  // v_exp_f32, v_rcp_f32: 1 ulp each
                        }
                        const uint2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
                        *(uint2 *)((unsigned char *)Cout + pk_chunk_off(prow, kba, 2 * ch + (lq >> 1), KTa) + (lq & 1) * 8) = o;
                    }
                }
            }
        }
    }
    if (MODE == MODE_UPRAW || MODE == MODE_UPREC) {
        // the accumulators as they are, one record per 32x32 block (whole blocks: rows past the item's last are
        // never read back as valid)
        const size_t cb = (size_t)(ctx.n0 >> 5) + wn, ncb = (size_t)(N >> 5);
        float *r1 = (float *)(MODE == MODE_UPRAW ? Cout : Aux1), *r3 = (float *)(MODE == MODE_UPRAW ? Aux1 : Aux2);
#pragma unroll
        for (int i = 0; i < NBLK; ++i) {
            const size_t rb = (size_t)ctx.rec0 + 2 * i + wm;
            float *o1 = r1 + (rb * ncb + cb) * 1024 + lane, *o3 = r3 + (rb * ncb + cb) * 1024 + lane;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                o1[r * 64] = acc[i][0][(r >> 3) & 1][(r >> 2) & 1][r & 3];
                o3[r * 64] = acc[i][1][(r >> 3) & 1][(r >> 2) & 1][r & 3];
            }
        }
    } else if (MODE == MODE_DA) {
        // acc = d(a) of (row 16 rh + l16 of block i, columns 16 ch + 4 lq + r of column block j); h1, h3 of the same
        // elements come from their records.  dh3 = da * silu(h1); dh1 = da*h3 * s*(1 + h1*(1-s)), s = sigmoid(h1)
        // (silu_backward, J/engine/nn/layer/active/gpu/activeFunction.cu:182-190).  Output: packed image with 2N
        // columns, dh1 in k steps 0..N/32-1, dh3 behind them.
        const int ncb = N >> 5, KTa = 2 * ncb;
#pragma unroll
        for (int i = 0; i < NBLK; ++i) {
            const size_t rb = (size_t)ctx.rec0 + 2 * i + wm;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int cb = (ctx.n0 >> 5) + wn * 2 + j;
                if (cb >= ncb) continue;  // last column tile of a width that is not a multiple of 256
                const float *p1 = (const float *)Aux1 + (rb * ncb + cb) * 1024 + lane;
                const float *p3 = (const float *)Aux2 + (rb * ncb + cb) * 1024 + lane;
#pragma unroll
                for (int rh = 0; rh < 2; ++rh) {
                    const int row = (2 * i + wm) * 32 + 16 * rh + l16;
                    const int prow = ctx.row0 + row;
#pragma unroll
                    for (int ch = 0; ch < 2; ++ch) {
                        float g1[4], g3[4];
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const int rr = (rh * 2 + ch) * 4 + r;
                            const float h1 = p1[rr * 64], h3 = p3[rr * 64], da = acc[i][j][rh][ch][r];
                            const float sg = __builtin_amdgcn_rcpf(1.0f + __expf(-h1));
                            g3[r] = da * (h1 * sg);
                            g1[r] = (da * h3) * sg * (1.0f + h1 * (1.0f - sg));
                        }
                        if (row < ctx.rows) {
                            const uint2 o1 = {pack_bf16x2(g1[0], g1[1]), pack_bf16x2(g1[2], g1[3])};
                            const uint2 o3 = {pack_bf16x2(g3[0], g3[1]), pack_bf16x2(g3[2], g3[3])};
                            const int t = 2 * ch + (lq >> 1);
                            *(uint2 *)((unsigned char *)Cout + pk_chunk_off(prow, cb, t, KTa) + (lq & 1) * 8) = o1;
                            *(uint2 *)((unsigned char *)Cout + pk_chunk_off(prow, ncb + cb, t, KTa) + (lq & 1) * 8) = o3;
                        }
                    }
                }
            }
        }
    } else if ((PLAIN_DOWN(MODE) || MODE == MODE_WGRAD) && !(ctx.half && wn >= 2)) {
        // a k slice other than the first writes partial result ctx.slab of those behind Aux1: a tile of BM x 256 of its own
        float *Cbase = PLAIN_DOWN(MODE) ? (float *)Cout + (size_t)ctx.row0 * N + ctx.n0 : (float *)Cout;
        int ld = N;
        if (PLAIN_DOWN(MODE) && ctx.slab > 0) {
            Cbase = (float *)Aux1 + (size_t)ctx.slab * (BM * 256);
            ld = 256;
        }
        // lane: column 16 ch + l16 of each 32x32 block; piece (rh, ch), register r -> row 16 rh + 4 lq + r
#pragma unroll
        for (int i = 0; i < NBLK; ++i) {
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int rh = q >> 2, r = q & 3;
                const int row = (2 * i + wm) * 32 + 16 * rh + 4 * lq + r;
                if (row >= ctx.rows) continue;
                // (16 lanes x 4 bytes = half a 128-byte line per row and store)
                float *out = PLAIN_DOWN(MODE) ? Cbase + (size_t)row * ld + wn * 64 + l16
                                              : Cbase + (size_t)(ctx.row0 + row) * N + ctx.n0 + wn * 64 + l16;
#pragma unroll
                for (int j = 0; j < 2; ++j)  // (non-temporal stores of the weight gradients were 10 % slower)
#pragma unroll
                    for (int ch = 0; ch < 2; ++ch)
                        if (PLAIN_DOWN(MODE) || ctx.n0 + wn * 64 + j * 32 + ch * 16 < N) out[j * 32 + ch * 16] = acc[i][j][rh][ch][r];
            }
        }
    }
#undef READ_A
#undef READ_B
#undef MFMA4
}

// Persistent: one workgroup per compute unit walks its queue of work items (built by the dispatch stage).
// WNT: weight tiles are loaded around the last-level cache (see dma16_nt)
template <int MODE, bool WNT = false>
__global__ __launch_bounds__(NWAVES * 64) void experts_bf16_kernel(const bf16_t *__restrict__ Axg, const bf16_t *__restrict__ Ax,
                                                                   const bf16_t *__restrict__ Wa, const bf16_t *__restrict__ Wb,
                                                                   void *__restrict__ Cout, void *Aux1, void *Aux2,
                                                                   const omega_tile_desc *__restrict__ wq, int N, int Kd)
{
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n_wg = gridDim.x, wg = blockIdx.x;

    omega_tile_desc d = wq[wg];
    if (d.rows <= 0) return;
    TileCtx cur_ctx = make_ctx<MODE>(d, Axg, Ax, Wa, Wb, N, Kd, wave, lane, PLAIN_DOWN(MODE) && Aux1 != nullptr);
    {
        // first item: k steps 0..NSTAGE-2 and the first half of step NSTAGE-1 into stages 0..NSTAGE-1
        const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
        const uint32_t lds_wave = lds0 + wave * 1024;
        const uint32_t lane_off = (uint32_t)lane * 16u;
        const uint64_t active = read_active_lanes();
        for (int st = 0; st < NSTAGE - 1; ++st) {
#pragma unroll
            for (int n = 0; n < LOADS_PER_STEP; ++n) issue_load<WNT>(cur_ctx, lds_wave, lane_off, st, st, n, active);
        }
        issue_load<WNT>(cur_ctx, lds_wave, lane_off, NSTAGE - 1, NSTAGE - 1, 0, active);
        issue_load<WNT>(cur_ctx, lds_wave, lane_off, NSTAGE - 1, NSTAGE - 1, 1, active);
        asm volatile("s_waitcnt vmcnt(14)" ::: "memory");  // all but steps 1.. : LOADS_PER_STEP * (NSTAGE - 2) + 2
        __syncthreads();
    }
    int stage = 0;
    TileCtx nx = cur_ctx;
    for (int q = 1;; ++q) {
        const omega_tile_desc dn = wq[(size_t)q * n_wg + wg];
        // 32-row blocks alternate between the two row halves of the workgroup: block b belongs to waves with wm = b % 2
        const int nblk = max(0, min(4, (((cur_ctx.rows + 31) >> 5) + 1 - (wave >> 2)) >> 1));
#define RUN_TILE(NBLK) \
    run_tile<MODE, NBLK, WNT>(smem, cur_ctx, nx, dn, Axg, Ax, Wa, Wb, stage, Cout, Aux1, Aux2, N, Kd, wave, lane)
        switch (nblk) {
            case 4: RUN_TILE(4); break;
            case 3: RUN_TILE(3); break;
            case 2: RUN_TILE(2); break;
            case 1: RUN_TILE(1); break;
            default: RUN_TILE(0); break;
        }
#undef RUN_TILE
        if (dn.rows <= 0) break;
        cur_ctx = nx;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (the loads behind the last item land in LDS that nobody reads)
}

// =====================================================================================================================
// Up product with one wave per SIMD (forward pass outside training): four waves of 128 rows x 128 MFMA columns, the 256
// accumulators of a wave in the AGPRs.  Same 256 x 256 tile, LDS ring, packed operands, work items and queues as the
// kernel above; what changes is the fragment traffic - a wave reads 8 A and 8 B fragments per 64 MFMAs (16 KiB) where
// two waves of 128 x 64 read 24 KiB - and that one barrier per k step joins four waves instead of eight.
// 16-row units of the tile alternate between the two row halves of the workgroup (unit u belongs to the waves with
// wm = u % 2), so a ragged tile leaves both halves the same work; units without valid rows issue no MFMAs.
// Every k step is the same code: the MFMAs run on one set of fragments while the other set is read for the next step
// and the wave's 8 direct loads of the step five ahead go out; when the loads reach the end of an item they turn to
// the next one of the queue.  Items start on rows that are multiples of 32 (item_desc), so a wave's fragment addresses
// never change and the fragments read during an item's last step are the next item's first.
// =====================================================================================================================
#define U4_WAVES 4
#define U4_LOADS 8  // direct loads per wave and k step

struct Up4Item {                // uniform over the wave unless said otherwise
    const unsigned char *A;    // k step 0 of the tile's rows (packed image), or x (GATHER)
    const unsigned char *B0, *B1;  // k step 0 of the 128 rows of W1 / of W3
    uint32_t va[4];             // per lane: what the lane adds to A for the wave's A loads (16-row blocks wave + 4 n)
    int row0, rows, n0;
    int kt;                     // k steps of the item (even, at least 8)
    int slab;                   // down product: 0 = the item writes the output, > 0 = partial result `slab`
};

// GATHER: token of tile row 16 * (wave + 4 n) + lane / 4, or 0 behind the item's rows
struct Up4Tok {
    int t[4];
};

// DOWN: the plain product y = a . W2^T: 256 columns of W2 (W1 = W2, W3 unused), A = the packed a; an item may be a k
// slice of a tile (a_rg slices, slice kt0, partial result xrow0: see make_ctx) - slices start on even k steps here
template <bool GATHER, bool DOWN = false>
__device__ __forceinline__ Up4Item up4_item(const omega_tile_desc &d, const bf16_t *Axg, const bf16_t *Ax, const bf16_t *W1,
                                            const bf16_t *W3, int N, int Kd, int wave, int lane, const Up4Tok &tk, bool slices = false)
{
    Up4Item c;
    const int KT = Kd / BK;
    const size_t rg_bytes = (size_t)KT * 8192;
    c.row0 = d.row0;
    c.rows = d.rows;
    c.n0 = d.n0;
    c.kt = KT;
    c.slab = 0;
    const size_t wrg = (size_t)d.g * (N >> 7) + (d.n0 >> 7);
    if (DOWN) {
        size_t k0 = 0;
        if (d.a_rg > 1) {
            if (slices) {
                const int first = ((d.kt0 * KT) / d.a_rg) & ~1;
                c.kt = (d.kt0 + 1 == d.a_rg ? KT : (((d.kt0 + 1) * KT) / d.a_rg) & ~1) - first;
                c.slab = d.kt0 > 0 ? d.xrow0 : 0;
                k0 = (size_t)first * 8192;
            } else if (d.kt0 > 0) {
                c.rows = 0;  // a launch without room for partial results: slice 0 computes the whole range
            }
        }
        c.B0 = uniform_ptr((const unsigned char *)W1 + wrg * rg_bytes + k0);
        c.B1 = uniform_ptr(c.B0 + rg_bytes);
        c.A = uniform_ptr((const unsigned char *)Axg + (size_t)(d.row0 / BM * 2) * rg_bytes + k0);
        const int blk0 = (d.row0 & (BM - 1)) >> 4;
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            const int q = wave + 4 * n;
            const bool valid = 16 * q < c.rows;
            const int qa = blk0 + (valid ? q : 0);
            c.va[n] = (uint32_t)(qa >> 3) * (uint32_t)rg_bytes + (uint32_t)(qa & 7) * 1024u + (valid ? (uint32_t)lane * 16u : 0u);
        }
        return c;
    }
    c.B0 = uniform_ptr((const unsigned char *)W1 + wrg * rg_bytes);
    c.B1 = uniform_ptr((const unsigned char *)W3 + wrg * rg_bytes);
    if (GATHER) {
        c.A = uniform_ptr((const unsigned char *)Axg);
        const int pr = d.row0 + 16 * wave + (lane >> 2);  // (rows 64 n further on have the same swizzle)
        const uint32_t ch = (uint32_t)(((lane & 3) ^ swz(pr)) << 4);
#pragma unroll
        for (int n = 0; n < 4; ++n) c.va[n] = (uint32_t)tk.t[n] * (uint32_t)(Kd * 2) + ch;
        return c;
    }
    c.A = uniform_ptr((Ax != nullptr && d.xrow0 >= 0) ? (const unsigned char *)Ax + (size_t)(d.xrow0 / BM * 2) * rg_bytes
                                                      : (const unsigned char *)Axg + (size_t)(d.row0 / BM * 2) * rg_bytes);
    const int blk0 = (d.row0 & (BM - 1)) >> 4;
#pragma unroll
    for (int n = 0; n < 4; ++n) {
        // a block without valid rows is never used by an MFMA whose result is kept: all its lanes read the same 16 bytes of
        // the item's first block (one request instead of sixteen lines), and every step still issues the same loads
        const int q = wave + 4 * n;
        const bool valid = 16 * q < d.rows;
        const int qa = blk0 + (valid ? q : 0);
        c.va[n] = (uint32_t)(qa >> 3) * (uint32_t)rg_bytes + (uint32_t)(qa & 7) * 1024u + (valid ? (uint32_t)lane * 16u : 0u);
    }
    return c;
}

__device__ __forceinline__ Up4Tok up4_tokens(const omega_tile_desc &d, const int32_t *__restrict__ tokp, int wave, int lane)
{
    Up4Tok k;
#pragma unroll
    for (int n = 0; n < 4; ++n) {
        const int r = 16 * (wave + 4 * n) + (lane >> 2);
        k.t[n] = r < d.rows ? (d.xrow0 >= 0 ? d.xrow0 + r : tokp[d.row0 + r]) : 0;
    }
    return k;
}

// What the waves of the kernel carry from one item to the next: the ring position, the fragments read during the
// step before, and where the loads have got to.
struct Up4State {
    int cur;
    bf16x8_t fa0[8], fb0[8], fa1[8], fb1[8];
    const unsigned char *lA, *lB0, *lB1;
    uint32_t va[4];
};

// One work item for a wave with NU units of valid rows (units beyond them issue no MFMAs; the accumulators live for
// one item, so every NU is its own straight-line code with NU * 32 accumulator registers).
template <int NU, bool WNT, bool GATHER, bool DOWN>
__device__ __forceinline__ void up4_run_item(unsigned char *smem, Up4State &st, const Up4Item &it, Up4Item &nxt_it,
                                             const omega_tile_desc &dn, const bf16_t *Axg, const bf16_t *Ax, const bf16_t *W1,
                                             const bf16_t *W3, void *Cout, void *slabs, int N, int Kd, int wave, int lane,
                                             const int32_t *__restrict__ tokp)
{
    constexpr int A_STEP = GATHER ? BK * 2 : 8192;
    constexpr int NA = NU > 0 ? NU : 1;
    const int wm = wave >> 1, wn = wave & 1;
    const int KT = DOWN ? __builtin_amdgcn_readfirstlane(it.kt) : Kd / BK;
    const int l16 = lane & 15, lq = lane >> 4;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    const uint32_t lds_wave = lds0 + wave * 1024;
    const uint32_t vb0 = (uint32_t)wave * 1024u + (uint32_t)lane * 16u, vb1 = vb0 + 4096u;
    const bool has_next = dn.rows > 0;
    // fragment addresses within a stage.  A fragment iu: rows of unit 2 iu + wm = block 2 iu + wm of the A tile; B fragment
    // c (16 MFMA columns): block (c / 4) * 8 + wn * 4 + c % 4 of the B tile, i.e. columns wn * 64 + 16 (c % 4) of the W1 half
    // (c < 4) or of the W3 half, so that acc[.][c] and acc[.][c + 4] are h1 and h3 of the same elements (DOWN: block
    // wn * 8 + c, columns wn * 128 + 16 c of the tile's 256).  Lane l supplies row l % 16, chunk l / 16; the chunk swizzle
    // depends on the row through l % 16 and the block's parity.
    const uint32_t pa = (uint32_t)(wm * 16 + l16) * (BK * 2) + ((uint32_t)(lq ^ swz(l16 | (wm << 4))) << 4);
    uint32_t pb[2];
#pragma unroll
    for (int h = 0; h < 2; ++h)
        pb[h] = TILE_BYTES + (uint32_t)(wn * (DOWN ? 128 : 64) + 16 * h + l16) * (BK * 2) + ((uint32_t)(lq ^ swz(l16 | (h << 4))) << 4);
    int cur = __builtin_amdgcn_readfirstlane(st.cur);
    const unsigned char *lA = uniform_ptr(st.lA), *lB0 = uniform_ptr(st.lB0), *lB1 = uniform_ptr(st.lB1);

    // GATHER: the tokens of the next item's rows are asked for now and used when the loads turn to that item, several
    // steps later: every step waits until at most 24 younger loads are in flight, so they have landed by then (the
    // compiler does not see these loads and must not be left to wait for them: its wait would drain the load ring)
    Up4Tok ntk = {{0, 0, 0, 0}};
    if (GATHER && has_next && dn.xrow0 < 0) {
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            const int r = 16 * (wave + 4 * n) + (lane >> 2);
            const uint32_t o = (uint32_t)(dn.row0 + (r < dn.rows ? r : 0)) * 4u;
            asm volatile("global_load_dword %0, %1, %2" : "=&v"(ntk.t[n]) : "v"(o), "s"(tokp) : "memory");
        }
    }
    if (!GATHER && has_next) nxt_it = up4_item<false, DOWN>(dn, Axg, Ax, W1, W3, N, Kd, wave, lane, Up4Tok{}, slabs != nullptr);

// fragment read r (0..7: B fragment r, 8..15: A fragment r - 8) of the stage whose read addresses are ra / rb0 / rb1
#define U4_READ(FA, FB, r)                                                                                              \
    do {                                                                                                                \
        if ((r) < 8) FB[(r) & 7] = *(const bf16x8_t *)(((r) & 1 ? rb1 : rb0) + (DOWN ? (((r) & 7) >> 1) * 2048u : (((r) & 3) >> 1) * 2048u + (((r) & 7) >> 2) * 8192u)); \
        else FA[((r) - 8) & 7] = *(const bf16x8_t *)(ra + (((r) - 8) & 7) * 2048u);                                     \
    } while (0)
// the wave's direct load l (0..7) of a k step into the stage at LDS address sb: A blocks wave + 4 n, then the B blocks
#define U4_LOAD(l, sb)                                                                                                  \
    do {                                                                                                                \
        if ((l) < 4) dma16<((l) & 3) * 4096>(lA, st.va[(l) & 3], sb);                                                   \
        else if (WNT) dma16_nt<TILE_BYTES + (((l) - 4) >> 1) * 8192 + ((l) & 1) * 4096>((l) < 6 ? lB0 : lB1, (l) & 1 ? vb1 : vb0, sb); \
        else dma16<TILE_BYTES + (((l) - 4) >> 1) * 8192 + ((l) & 1) * 4096>((l) < 6 ? lB0 : lB1, (l) & 1 ? vb1 : vb0, sb); \
    } while (0)
// One k step on the fragments PA / PB (taken from stage `cur` during the step before): group g of 4 MFMAs = unit g / 2,
// B fragments 4 (g % 2) ..; with the first 8 groups two fragment reads of the next step (stage cur + 1, into QA / QB), with
// every other group one direct load of the step five ahead into stage `cur`, which every wave has left.  At the barrier
// that ends the step the loads of the step after next must have landed: three younger steps (24 loads) may be in flight.
// Z: the accumulators start from zero operands (an item's first step).
// (the group index is spelled out: the LDS offsets of the loads are immediate operands)
#define U4_MFMA(PA, PB, Z, iu, c)                                                                                       \
    do {                                                                                                                \
        if ((iu) < NU)                                                                                                  \
            acc[(iu) % NA][c] = DOWN ? __builtin_amdgcn_mfma_f32_16x16x32_bf16(PA[iu], PB[c], (Z) ? zero4 : acc[(iu) % NA][c], 0, 0, 0) \
                                     : __builtin_amdgcn_mfma_f32_16x16x32_bf16(PB[c], PA[iu], (Z) ? zero4 : acc[(iu) % NA][c], 0, 0, 0); \
    } while (0)
// A wave issues one instruction every four cycles and an MFMA of this shape occupies the matrix core for sixteen: up
// to three other instructions fit behind each MFMA without delaying the next one.  The order is pinned so: an MFMA,
// then the two fragment reads or the direct load (three instructions with its m0 set-up) that go with it.
#define U4_GROUP(PA, PB, QA, QB, Z, g)                                                                                  \
    do {                                                                                                                \
        U4_MFMA(PA, PB, Z, (g) >> 1, 4 * ((g) & 1));                                                                    \
        if ((g) < 8) {                                                                                                  \
            U4_READ(QA, QB, 2 * (g));                                                                                   \
            U4_READ(QA, QB, 2 * (g) + 1);                                                                               \
        }                                                                                                               \
        __builtin_amdgcn_sched_barrier(0);                                                                              \
        U4_MFMA(PA, PB, Z, (g) >> 1, 4 * ((g) & 1) + 1);                                                                \
        if ((g) & 1) U4_LOAD((g) >> 1, sb);                                                                             \
        __builtin_amdgcn_sched_barrier(0);                                                                              \
        U4_MFMA(PA, PB, Z, (g) >> 1, 4 * ((g) & 1) + 2);                                                                \
        __builtin_amdgcn_sched_barrier(0);                                                                              \
        U4_MFMA(PA, PB, Z, (g) >> 1, 4 * ((g) & 1) + 3);                                                                \
        __builtin_amdgcn_sched_barrier(0);                                                                              \
    } while (0)
// (the last group of a step also moves the ring on - the stage the next step's loads go to, the addresses its
//  fragment reads come from, the load pointers - behind its MFMAs, so that the step after the barrier starts with work)
#define U4_STEP(PA, PB, QA, QB, Z)                                                                                      \
    do {                                                                                                                \
        U4_GROUP(PA, PB, QA, QB, Z, 0); U4_GROUP(PA, PB, QA, QB, Z, 1); U4_GROUP(PA, PB, QA, QB, Z, 2);                 \
        U4_GROUP(PA, PB, QA, QB, Z, 3); U4_GROUP(PA, PB, QA, QB, Z, 4); U4_GROUP(PA, PB, QA, QB, Z, 5);                 \
        U4_GROUP(PA, PB, QA, QB, Z, 6); U4_GROUP(PA, PB, QA, QB, Z, 7); U4_GROUP(PA, PB, QA, QB, Z, 8);                 \
        U4_GROUP(PA, PB, QA, QB, Z, 9); U4_GROUP(PA, PB, QA, QB, Z, 10); U4_GROUP(PA, PB, QA, QB, Z, 11);               \
        U4_GROUP(PA, PB, QA, QB, Z, 12); U4_GROUP(PA, PB, QA, QB, Z, 13); U4_GROUP(PA, PB, QA, QB, Z, 14);              \
        U4_MFMA(PA, PB, Z, 7, 4);                                                                                       \
        __builtin_amdgcn_sched_barrier(0);                                                                              \
        U4_MFMA(PA, PB, Z, 7, 5);                                                                                       \
        U4_LOAD(7, sb);                                                                                                 \
        __builtin_amdgcn_sched_barrier(0);                                                                              \
        U4_MFMA(PA, PB, Z, 7, 6);                                                                                       \
        cur = cur + 1 == NSTAGE ? 0 : cur + 1;                                                                          \
        sb = lds_wave + cur * STAGE_BYTES;                                                                              \
        lA += A_STEP;                                                                                                   \
        lB0 += 8192;                                                                                                    \
        lB1 += 8192;                                                                                                    \
        __builtin_amdgcn_sched_barrier(0);                                                                              \
        U4_MFMA(PA, PB, Z, 7, 7);                                                                                       \
        {                                                                                                               \
            const unsigned char *sn = smem + (cur + 1 == NSTAGE ? 0 : cur + 1) * STAGE_BYTES;                           \
            ra = sn + pa;                                                                                               \
            rb0 = sn + pb[0];                                                                                           \
            rb1 = sn + pb[1];                                                                                           \
        }                                                                                                               \
        __builtin_amdgcn_sched_barrier(0);                                                                              \
        asm volatile("s_waitcnt vmcnt(24) lgkmcnt(0)" ::: "memory");                                                    \
        __syncthreads();                                                                                                \
    } while (0)

    // the stage this step's loads go to and the addresses the fragments of the next step are read from
    uint32_t sb = lds_wave + cur * STAGE_BYTES;
    const unsigned char *ra, *rb0, *rb1;
    {
        const unsigned char *sn = smem + (cur + 1 == NSTAGE ? 0 : cur + 1) * STAGE_BYTES;
        ra = sn + pa;
        rb0 = sn + pb[0];
        rb1 = sn + pb[1];
    }
    f32x4_t acc[NA][8];  // acc[iu][c]: 16 x 16 piece (rows of unit 2 iu + wm, columns of B fragment c), weights as first operand
    const f32x4_t zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
    // KT steps (even, at least 8), two at a time.  The loads issued during steps 0 .. KT - 6 are the item's own (its steps
    // 5 .. KT - 1), those of the last five steps the next item's first five (behind the last item of a queue this item's
    // once more: nobody reads them).
    U4_STEP(st.fa0, st.fb0, st.fa1, st.fb1, true);
    U4_STEP(st.fa1, st.fb1, st.fa0, st.fb0, false);
    for (int k = 2; k < KT - 6; k += 2) {
        U4_STEP(st.fa0, st.fb0, st.fa1, st.fb1, false);
        U4_STEP(st.fa1, st.fb1, st.fa0, st.fb0, false);
    }
    U4_STEP(st.fa0, st.fb0, st.fa1, st.fb1, false);
    if (GATHER && has_next) {
        // three steps or more have passed since the token loads were issued: they have landed
        asm volatile("; token loads done" : "+v"(ntk.t[0]), "+v"(ntk.t[1]), "+v"(ntk.t[2]), "+v"(ntk.t[3])::"memory");
        if (dn.xrow0 >= 0) ntk = up4_tokens(dn, tokp, wave, lane);
        nxt_it = up4_item<true, false>(dn, Axg, Ax, W1, W3, N, Kd, wave, lane, ntk);
    }
    lA = uniform_ptr(nxt_it.A);
    lB0 = uniform_ptr(nxt_it.B0);
    lB1 = uniform_ptr(nxt_it.B1);
#pragma unroll
    for (int n = 0; n < 4; ++n) st.va[n] = nxt_it.va[n];
    U4_STEP(st.fa1, st.fb1, st.fa0, st.fb0, false);
    for (int k = 0; k < 2; ++k) {
        U4_STEP(st.fa0, st.fb0, st.fa1, st.fb1, false);
        U4_STEP(st.fa1, st.fb1, st.fa0, st.fb0, false);
    }
#undef U4_STEP
#undef U4_GROUP
#undef U4_LOAD
#undef U4_READ
    st.cur = cur;
    st.lA = lA;
    st.lB0 = lB0;
    st.lB1 = lB1;

    if (DOWN) {
        // ---- epilogue of the plain product: fp32 rows (a k slice other than the first: partial result it.slab, a tile of
        // BM x 256 of its own).  The rows were the MFMAs' first operand: lane l holds column l % 16 of the 16 of fragment c,
        // register r row 4 (l / 16) + r of the unit, so 16 lanes store 64 consecutive bytes of a row
        float *Cbase = (float *)Cout + (size_t)it.row0 * N + it.n0;
        int ld = N;
        if (it.slab > 0) {
            Cbase = (float *)slabs + (size_t)it.slab * (BM * 256);
            ld = 256;
        }
#pragma unroll
        for (int iu = 0; iu < NU; ++iu) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = 16 * (2 * iu + wm) + 4 * lq + r;
                if (row < it.rows) {
                    float *out = Cbase + (size_t)row * ld + wn * 128 + l16;
#pragma unroll
                    for (int c = 0; c < 8; ++c) out[16 * c] = acc[iu][c][r];
                }
            }
        }
        return;
    }
    // ---- epilogue: a = silu(h1) * h3 as packed bf16 ----
    // lane: row l16 of unit 2 iu + wm; registers r of acc[iu][c] and acc[iu][c + 4]: h1 and h3 of column
    // wn * 64 + 16 c + 4 lq + r of the tile's 128, i.e. k step n0 / 32 + 2 wn + c / 2 of the packed a, chunk 2 (c % 2) + lq / 2
    const int KTa = N / BK;
#pragma unroll
    for (int iu = 0; iu < NU; ++iu) {
        const int row = 16 * (2 * iu + wm) + l16;
        if (row < it.rows) {
            const int prow = it.row0 + row;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float h1 = acc[iu][c][r], h3 = acc[iu][c + 4][r];
                    v[r] = h1 * __builtin_amdgcn_rcpf(1.0f + __expf(-h1)) * h3;  // v_exp_f32, v_rcp_f32: 1 ulp each
                }
                const uint2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
                *(uint2 *)((unsigned char *)Cout + pk_chunk_off(prow, (it.n0 >> 5) + 2 * wn + (c >> 1), 2 * (c & 1) + (lq >> 1), KTa) +
                           (lq & 1) * 8) = o;
            }
        }
    }
}

// DOWN: the plain down product on the same kernel (W1 = W2, slabs = room for the partial results of k slices or null)
template <bool WNT, bool GATHER, bool DOWN = false>
__global__ __launch_bounds__(U4_WAVES * 64) void experts_up4_kernel(const bf16_t *__restrict__ Axg, const bf16_t *__restrict__ Ax,
                                                                    const bf16_t *__restrict__ W1, const bf16_t *__restrict__ W3,
                                                                    void *__restrict__ Cout, const omega_tile_desc *__restrict__ wq,
                                                                    int N, int Kd, const int32_t *__restrict__ tokp,
                                                                    void *slabs = nullptr)
{
    constexpr int A_STEP = GATHER ? BK * 2 : 8192;
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int n_wg = gridDim.x, wg = blockIdx.x;
    const int l16 = lane & 15, lq = lane >> 4;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;
    const uint32_t lds_wave = lds0 + wave * 1024;
    const uint32_t vb0 = (uint32_t)wave * 1024u + (uint32_t)lane * 16u, vb1 = vb0 + 4096u;

    omega_tile_desc d = wq[wg];
    if (d.rows <= 0) return;
    Up4Item it = up4_item<GATHER, DOWN>(d, Axg, Ax, W1, W3, N, Kd, wave, lane, GATHER ? up4_tokens(d, tokp, wave, lane) : Up4Tok{},
                                        slabs != nullptr);
    Up4State st;
    st.lA = it.A;
    st.lB0 = it.B0;
    st.lB1 = it.B1;
#pragma unroll
    for (int n = 0; n < 4; ++n) st.va[n] = it.va[n];
    // first item: k steps 0..4 into stages 0..4
    for (int s5 = 0; s5 < NSTAGE; ++s5) {
        const uint32_t sb = lds_wave + s5 * STAGE_BYTES;
        dma16<0>(st.lA, st.va[0], sb);
        dma16<4096>(st.lA, st.va[1], sb);
        dma16<8192>(st.lA, st.va[2], sb);
        dma16<12288>(st.lA, st.va[3], sb);
        if (WNT) {
            dma16_nt<TILE_BYTES>(st.lB0, vb0, sb);
            dma16_nt<TILE_BYTES + 4096>(st.lB0, vb1, sb);
            dma16_nt<TILE_BYTES + 8192>(st.lB1, vb0, sb);
            dma16_nt<TILE_BYTES + 12288>(st.lB1, vb1, sb);
        } else {
            dma16<TILE_BYTES>(st.lB0, vb0, sb);
            dma16<TILE_BYTES + 4096>(st.lB0, vb1, sb);
            dma16<TILE_BYTES + 8192>(st.lB1, vb0, sb);
            dma16<TILE_BYTES + 12288>(st.lB1, vb1, sb);
        }
        st.lA += A_STEP;
        st.lB0 += 8192;
        st.lB1 += 8192;
    }
    asm volatile("s_waitcnt vmcnt(32)" ::: "memory");  // step 0 has landed: U4_LOADS * (NSTAGE - 1) younger loads
    __syncthreads();
    {
        const uint32_t pa = (uint32_t)(wm * 16 + l16) * (BK * 2) + ((uint32_t)(lq ^ swz(l16 | (wm << 4))) << 4);
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const uint32_t pbr = TILE_BYTES + (uint32_t)(wn * (DOWN ? 128 : 64) + 16 * (r & 1) + l16) * (BK * 2) + ((uint32_t)(lq ^ swz(l16 | ((r & 1) << 4))) << 4);
            st.fb0[r] = *(const bf16x8_t *)(smem + pbr + (DOWN ? (r >> 1) * 2048u : ((r & 3) >> 1) * 2048u + (r >> 2) * 8192u));
            st.fa0[r] = *(const bf16x8_t *)(smem + pa + r * 2048u);
        }
    }
    // every wave has taken step 0 out of stage 0 before anyone refills it
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __syncthreads();
    st.cur = 0;

    for (int q = 1;; ++q) {
        const omega_tile_desc dn = wq[(size_t)q * n_wg + wg];
        // units of this wave that hold valid rows: unit u = 2 iu + wm is valid if 16 u < rows
        const int units = (it.rows + 15) >> 4;
        const int nu = __builtin_amdgcn_readfirstlane(max(0, min(8, (units + 1 - wm) >> 1)));
        Up4Item nxt_it = it;
#define U4_RUN(NU) up4_run_item<NU, WNT, GATHER, DOWN>(smem, st, it, nxt_it, dn, Axg, Ax, W1, W3, Cout, slabs, N, Kd, wave, lane, tokp)
        switch (nu) {
            case 8: U4_RUN(8); break;
            case 7: U4_RUN(7); break;
            case 6: U4_RUN(6); break;
            case 5: U4_RUN(5); break;
            case 4: U4_RUN(4); break;
            case 3: U4_RUN(3); break;
            case 2: U4_RUN(2); break;
            case 1: U4_RUN(1); break;
            default: U4_RUN(0); break;
        }
#undef U4_RUN
        if (dn.rows <= 0) break;
        it = nxt_it;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (the loads behind the last item land in LDS that nobody reads)
}

// y += the partial results of the k-sliced items of a down product, in slice order.  The sliced items are the
// tile_meta[meta_slot + 1] table entries from entry tile_meta[meta_slot] on (slices of a tile adjacent, slice 0 first);
// partial result i belongs to the i-th of them and is a tile of BM x 256 floats.  Workgroup (i, j): rows 32 j .. of the
// tile whose slice 0 is sliced entry i (one workgroup per tile moved 1.3 MB alone and took 40 us for 64 tiles).
__global__ __launch_bounds__(256) void down_slab_reduce_kernel(float *__restrict__ y, const float *__restrict__ slabs,
                                                               const omega_tile_desc *__restrict__ desc,
                                                               const int32_t *__restrict__ tile_meta, int meta_slot, int d)
{
    const int first = tile_meta[meta_slot], n = tile_meta[meta_slot + 1], i = blockIdx.x;
    if (i >= n) return;
    const omega_tile_desc e = desc[first + i];
    if (e.a_rg <= 1 || e.kt0 != 0) return;
    const int c = (threadIdx.x & 63) * 4;
    const int rend = min(e.rows, (int)(blockIdx.y + 1) * 32);
    for (int r0 = blockIdx.y * 32 + (threadIdx.x >> 6); r0 < rend; r0 += 8) {
        // two rows per trip: up to 8 independent 16-byte loads in flight per thread
        const int r1 = r0 + 4;
        const bool two = r1 < rend;
        float *o0 = y + (size_t)(e.row0 + r0) * d + e.n0 + c, *o1 = y + (size_t)(e.row0 + (two ? r1 : r0)) * d + e.n0 + c;
        float4 v0 = *(const float4 *)o0, v1 = *(const float4 *)o1;
        float4 u0[3], u1[3];
#pragma unroll
        for (int s = 1; s < 4; ++s) {
            const int ss = min(s, e.a_rg - 1);
            u0[s - 1] = *(const float4 *)(slabs + (size_t)(i + ss) * (BM * 256) + r0 * 256 + c);
            u1[s - 1] = *(const float4 *)(slabs + (size_t)(i + ss) * (BM * 256) + (two ? r1 : r0) * 256 + c);
        }
#pragma unroll
        for (int s = 1; s < 4; ++s) {
            if (s < e.a_rg) {
                v0.x += u0[s - 1].x; v0.y += u0[s - 1].y; v0.z += u0[s - 1].z; v0.w += u0[s - 1].w;
                v1.x += u1[s - 1].x; v1.y += u1[s - 1].y; v1.z += u1[s - 1].z; v1.w += u1[s - 1].w;
            }
        }
        for (int s = 4; s < e.a_rg; ++s) {  // (small batches: up to 8 slices)
            const float4 w0 = *(const float4 *)(slabs + (size_t)(i + s) * (BM * 256) + r0 * 256 + c);
            const float4 w1 = *(const float4 *)(slabs + (size_t)(i + s) * (BM * 256) + (two ? r1 : r0) * 256 + c);
            v0.x += w0.x; v0.y += w0.y; v0.z += w0.z; v0.w += w0.w;
            v1.x += w1.x; v1.y += w1.y; v1.z += w1.z; v1.w += w1.w;
        }
        *(float4 *)o0 = v0;
        if (two) *(float4 *)o1 = v1;
    }
}

hipError_t launch_down_slab_reduce(const omega_moe *m, float *y, hipStream_t s)
{
    hipLaunchKernelGGL(down_slab_reduce_kernel, dim3(256, BM / 32), dim3(256), 0, s, y, (const float *)m->y_slabs, m->desc_down, m->tile_meta,
                       m->G + 8, m->cfg.d);
    return hipGetLastError();
}

hipError_t experts_bf16_init(void)
{
    // (the plain up product runs on experts_up4_kernel only: the eight-wave kernel is not instantiated for it)
    const void *fns[] = {(const void *)experts_bf16_kernel<MODE_DOWN>,
                         (const void *)experts_bf16_kernel<MODE_UPRAW>, (const void *)experts_bf16_kernel<MODE_DA>,
                         (const void *)experts_bf16_kernel<MODE_WGRAD>, (const void *)experts_bf16_kernel<MODE_UPREC>,
                         (const void *)experts_bf16_kernel<MODE_DOWN, true>,
                         (const void *)experts_up4_kernel<false, false>, (const void *)experts_up4_kernel<true, false>,
                         (const void *)experts_up4_kernel<false, true>, (const void *)experts_up4_kernel<true, true>,
                         (const void *)experts_up4_kernel<false, false, true>, (const void *)experts_up4_kernel<true, false, true>};
    for (const void *f : fns) {
        hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

hipError_t launch_experts_bf16(const omega_moe *m, const void *x, int T, int which, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    // the ring must be shorter than an item: K >= (NSTAGE + 1) * BK (guaranteed at creation: d, H >= 256)
    if ((which == 0 ? c.d : c.H) < (NSTAGE + 1) * BK) return hipErrorInvalidValue;
    // A batch with at most 64 rows per routed expert on average streams every weight tile once (one row tile per
    // expert): nothing is gained by keeping them in the last-level cache.  Measured at d = 4096, H = 14336, E = 8, K = 2:
    // 16 / 64 tokens 9 % faster, 256 tokens equal, 512 tokens 5 % slower; at d = 2048, H = 1408, E = 64, K = 6: 64 and
    // 512 tokens 4-6 % faster, 2048 tokens 2 % slower.
    const bool wnt = (long long)T * c.K <= 64LL * c.E;
    if (which == 0 && m->training && m->bw_h1 != nullptr) {
        // training mode: h1 and h3 are kept for the backward pass, as the reference's layers keep their outputs
        hipLaunchKernelGGL(experts_bf16_kernel<MODE_UPREC>, dim3(m->n_wg), dim3(NWAVES * 64), SMEM_BYTES, s,
                           (const bf16_t *)m->xg, (const bf16_t *)m->xs, (const bf16_t *)m->W1, (const bf16_t *)m->W3, m->a,
                           (void *)m->bw_h1, (void *)m->bw_h3, m->wq_up, c.H, c.d);
    } else if (which == 0) {
        // the forward pass outside training: one wave per SIMD (experts_up4_kernel)
        const bf16_t *A = (const bf16_t *)(m->gather_on_load ? x : m->xg), *As = (const bf16_t *)(m->gather_on_load ? x : m->xs);
#define UP4_LAUNCH(WNTV, GV)                                                                                            \
    hipLaunchKernelGGL((experts_up4_kernel<WNTV, GV>), dim3(m->n_wg), dim3(U4_WAVES * 64), SMEM_BYTES, s, A, As, (const bf16_t *)m->W1, \
                       (const bf16_t *)m->W3, m->a, m->wq_up, c.H, c.d, m->tokp)
        if (m->gather_on_load) {
            if (wnt) UP4_LAUNCH(true, true);
            else UP4_LAUNCH(false, true);
        } else {
            if (wnt) UP4_LAUNCH(true, false);
            else UP4_LAUNCH(false, false);
        }
#undef UP4_LAUNCH
    } else {
        // the table may hold k slices (every tile of a small batch, or the last tiles of a large one): their partial
        // results go to y_slabs and are added into y right behind the product
        void *slabs = (m->down_ks_max > 1 || m->down_tail_ks > 1) ? (void *)m->y_slabs : nullptr;
        if (m->down_cols == 256) {
            // full-width items: one wave per SIMD (experts_up4_kernel, DOWN)
            if (wnt)
                hipLaunchKernelGGL((experts_up4_kernel<true, false, true>), dim3(m->n_wg), dim3(U4_WAVES * 64), SMEM_BYTES, s, (const bf16_t *)m->a,
                                   (const bf16_t *)nullptr, (const bf16_t *)m->W2, (const bf16_t *)nullptr, (void *)m->y, m->wq_down, c.d,
                                   c.H, (const int32_t *)nullptr, slabs);
            else
                hipLaunchKernelGGL((experts_up4_kernel<false, false, true>), dim3(m->n_wg), dim3(U4_WAVES * 64), SMEM_BYTES, s, (const bf16_t *)m->a,
                                   (const bf16_t *)nullptr, (const bf16_t *)m->W2, (const bf16_t *)nullptr, (void *)m->y, m->wq_down, c.d,
                                   c.H, (const int32_t *)nullptr, slabs);
        } else if (wnt)
            hipLaunchKernelGGL((experts_bf16_kernel<MODE_DOWN, true>), dim3(m->n_wg), dim3(NWAVES * 64), SMEM_BYTES, s, (const bf16_t *)m->a,
                               (const bf16_t *)nullptr, (const bf16_t *)m->W2, (const bf16_t *)nullptr, (void *)m->y,
                               slabs, (void *)nullptr, m->wq_down, c.d, c.H);
        else
            hipLaunchKernelGGL(experts_bf16_kernel<MODE_DOWN>, dim3(m->n_wg), dim3(NWAVES * 64), SMEM_BYTES, s, (const bf16_t *)m->a,
                               (const bf16_t *)nullptr, (const bf16_t *)m->W2, (const bf16_t *)nullptr, (void *)m->y,
                               slabs, (void *)nullptr, m->wq_down, c.d, c.H);
        if (slabs != nullptr) {
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return e;
            return launch_down_slab_reduce(m, m->y, s);
        }
    }
    return hipGetLastError();
}

// One product of the backward pass on the same kernel; `mode` as the enum above, operands and outputs as its comment says.
hipError_t launch_product_bf16(const omega_moe *m, int mode, const void *A, const void *Aalt, const void *Wa, const void *Wb,
                               void *Cout, void *Aux1, void *Aux2, const omega_tile_desc *wq, int N, int Kd, hipStream_t s)
{
    if (Kd < (NSTAGE + 1) * BK) return hipErrorInvalidValue;
    if (mode == MODE_DOWN && m->down_cols == 256 && Kd % 64 == 0 && Kd >= 8 * BK) {
        // plain full-width products (the input gradient of the experts): one wave per SIMD
        hipLaunchKernelGGL((experts_up4_kernel<false, false, true>), dim3(m->n_wg), dim3(U4_WAVES * 64), SMEM_BYTES, s, (const bf16_t *)A,
                           (const bf16_t *)nullptr, (const bf16_t *)Wa, (const bf16_t *)nullptr, Cout, wq, N, Kd, (const int32_t *)nullptr,
                           Aux1);
        return hipGetLastError();
    }
#define LAUNCH(MODE)                                                                                                   \
    hipLaunchKernelGGL(experts_bf16_kernel<MODE>, dim3(m->n_wg), dim3(NWAVES * 64), SMEM_BYTES, s, (const bf16_t *)A,      \
                       (const bf16_t *)Aalt, (const bf16_t *)Wa, (const bf16_t *)Wb, Cout, Aux1, Aux2, wq, N, Kd)
    switch (mode) {
        case MODE_DOWN: LAUNCH(MODE_DOWN); break;
        case MODE_UPRAW: LAUNCH(MODE_UPRAW); break;
        case MODE_DA: LAUNCH(MODE_DA); break;
        case MODE_WGRAD: LAUNCH(MODE_WGRAD); break;
        case MODE_UPREC: LAUNCH(MODE_UPREC); break;
        default: return hipErrorInvalidValue;
    }
#undef LAUNCH
    return hipGetLastError();
}
