// Dispatch: per-expert counts, prefix scan, stable permutation, row-tile list, coalesced row gather.
//
// Pair p = t*K+j goes to logical row dst[p] = offsets[id_p] + #{q<p : id_q == id_p} of the expert-contiguous
// order (a stable counting sort of the pair list by expert id); src_row[dst[p]] = t.  In the buffers the
// experts' segments start on row-tile boundaries (physical row dstp[p] = first_tile[id_p]*bm + rank).
// The router left one histogram row per token tile (16 or 32 tokens, router_tok_tile) in tile_counts[tile][e].  Two
// launches - three when the histogram is large:
//   scan    (histograms above 16384 cells only) one workgroup per 8 experts: exclusive prefix over the tiles of each
//           expert (tile_base) and the per-expert totals -> counts[e]
//   rank    one workgroup per token tile: the prefix of its tile and the totals (summed from the histogram rows in the
//           same pass unless a scan launch left them); offsets = exclusive scan of counts, first_tile = exclusive scan
//           of ceil(counts/bm); rank of each pair among the earlier pairs of its tile with the same expert (ballots
//           within 64-pair chunks, per-chunk counts across them); dst/dstp/src_row; workgroup g (mod grid) writes the
//           row tiles and the work items of group g, workgroup 0 publishes counts, offsets and the totals
//   gather  one wave per token: the row of x is read once with 16-byte accesses and written to its K
//           destination rows (gather semantics as img_token_drop,
//           J/engine/nn/layer/dit/kernel/TokenDropKernel.cu:147-160); fp32 layers keep rows contiguous,
//           bf16 layers write the packed tile image the product kernels load (pack.h)
// No global atomics anywhere, so counts, offsets and the permutation are deterministic.
#include "common.h"
#include "pack.h"

#define TOK_TILE_MAX ROUTER_TOK_TILE_MAX
#define SCAN_EC 8     // experts per scan workgroup
#define SCAN_SEG 32   // tile segments per expert

__global__ __launch_bounds__(256) void dispatch_scan_kernel(const int32_t *__restrict__ tile_counts,
                                                            int32_t *__restrict__ tile_base, int n_tiles, int E,
                                                            int32_t *__restrict__ counts)
{
    __shared__ int segsum[SCAN_SEG][SCAN_EC];
    const int el = threadIdx.x % SCAN_EC, seg = threadIdx.x / SCAN_EC;
    const int e = blockIdx.x * SCAN_EC + el;
    const int per = ceil_div(n_tiles, SCAN_SEG);
    const int b = min(seg * per, n_tiles), en = min(b + per, n_tiles);
    int sum = 0;
    if (e < E)
        for (int t = b; t < en; ++t) sum += tile_counts[(size_t)t * E + e];
    segsum[seg][el] = sum;
    __syncthreads();
    int base = 0, total = 0;
    for (int s2 = 0; s2 < SCAN_SEG; ++s2) {
        const int v = segsum[s2][el];
        if (s2 < seg) base += v;
        total += v;
    }
    if (e < E) {
        if (seg == 0) counts[e] = total;
        for (int t = b; t < en; ++t) {
            const int c = tile_counts[(size_t)t * E + e];
            tile_base[(size_t)t * E + e] = base;
            base += c;
        }
    }
}

// The work items of group g in one product's table (see the comment in dispatch_rank_kernel): NT column tiles of
// ncols columns, Mg row tiles starting at row tile mt0; the launch has total_mt row tiles in all.  All 256 threads.
// K slices of a table (small batches of the down product, see write_group_items): Nt output tiles that would leave
// at least half of the 256 compute units idle are each cut into KS <= ks_max slices of the k range, at least 8 k steps
// long; 1 = no slicing.
__device__ __forceinline__ int table_k_slices(int Nt, int ks_max, int KT)
{
    if (ks_max <= 1 || Nt <= 0 || Nt > 128) return 1;
    return max(1, min(min(ks_max, 256 / Nt), KT / 8));
}

// K slices of the last r tiles of a large launch (r = Nt mod 256 <= 128: they would leave at least half of the compute
// units idle): as many as fill the units, at most tail_ks, each at least 64 k steps long; 1 = none (row slices instead).
// Row slices stream the whole weight tile for a quarter of the rows and are bound by that stream; k slices are not, but
// their partial results have to be added up behind the product.  4096 tokens, 8 experts, k = 14336 (448 steps, 64 of 576
// tiles in 4 slices): product 0.834 -> 0.784 ms, adding up 0.020 ms; k = 1408 (44 steps, 2 slices): 0.369 -> 0.386 ms,
// hence the minimum length.
__device__ __forceinline__ int table_tail_k_slices(int Nt, int tail_ks, int KT)
{
    const int r = Nt % 256;
    if (tail_ks <= 1 || r == 0 || r > 128) return 1;
    return max(1, min(min(tail_ks, 256 / r), KT / 64));
}

// Row tiles of one group that run side by side on an XCD (see dispatch_rank_kernel): a group with more row tiles than
// this is cut into row blocks of about equal size, each of which walks all column tiles.
#define OMEGA_ROW_BLOCK_MAX 8

__device__ __forceinline__ void write_group_items(omega_tile_desc *__restrict__ desc, int NT, int ncols, int g, int rows,
                                                  int Mg, int mt0, int total_mt, int bm, bool shared, int ks_max = 1,
                                                  int KT = 0, int tail_ks = 1)
{
    if (desc == nullptr) return;
    const int Nt = total_mt * NT, r = Nt % 256;
    const int KS = table_k_slices(Nt, ks_max, KT);
    const int TKS = KS > 1 ? 1 : table_tail_k_slices(Nt, tail_ks, KT);
    const int S = (r == 0 || r > 128 || KS > 1 || TKS > 1) ? 1 : min(4, 256 / r);
    // the group's rows are dealt evenly, in blocks of 32, to its Mg row tiles (instead of full tiles and a ragged last
    // one): the same number of tiles and of MFMA blocks, but tiles of nearly one cost.  (Equal tiles in units of 16 rows -
    // every tile the same number of MFMA blocks, the last one of each half empty - cut the L2 miss traffic of the up
    // product by a fifth when every expert has 1040 rows, and still lost 4 % of time to the extra blocks.)
    const int nblk = (rows + 31) >> 5;
    const int qblk = nblk / Mg, nhi = nblk % Mg;  // the first nhi row tiles hold qblk + 1 blocks, the others qblk
    // order within the group: row blocks of RB row tiles; inside a row block column tile after column tile, the row
    // tiles of the block fastest.  (Walking the column tiles twice, first with the taller row tiles and then with the
    // others, makes most rounds of 32 entries cost the same, so that the queue builder has nothing to deal: dispatch
    // 50 -> 39 us at the Mixtral shape, but its up product 1.529 -> 1.544 ms - each weight tile is then fetched twice.)
    const int NB = (Mg + OMEGA_ROW_BLOCK_MAX - 1) / OMEGA_ROW_BLOCK_MAX;
    for (int l = threadIdx.x; l < Mg * NT; l += 256) {
        // row block b holds row tiles [b*Mg/NB, (b+1)*Mg/NB); the entries before it number (first tile) * NT
        int b = min(NB - 1, (l / NT) * NB / Mg);
        while ((b * Mg) / NB * NT > l) --b;
        while (b + 1 < NB && ((b + 1) * Mg) / NB * NT <= l) ++b;
        const int f = (b * Mg) / NB, RB = ((b + 1) * Mg) / NB - f;
        const int li = l - f * NT;
        const int mt = f + li % RB, n = li / RB;
        const int at = mt0 * NT + l;
        const int tfirst = 32 * (mt * qblk + min(mt, nhi));
        const int trows = min(32 * ((mt + 1) * qblk + min(mt + 1, nhi)), rows) - tfirst;
        omega_tile_desc dsc;
        dsc.g = g;
        dsc.n0 = n * ncols;
        dsc.a_rg = 0;
        dsc.b_rg = ncols == 128 ? 1 : 0;  // read by the plain 256-column products only: a half-width item
        // (items without k slices: kt0 = first 32 x 32 block record of the item - 8 records per row-tile slot - for the
        //  products that keep or read h1 / h3 block records)
        dsc.kt0 = (mt0 + mt) * 8;
        if (KS > 1) {
            // slice ks of KS (a_rg = KS, kt0 = ks, xrow0 = number of the sliced entry = of its partial result) runs over
            // its part of the k range; adjacent entries, so the slices of a tile run on one XCD and share its rows
            dsc.row0 = mt0 * bm + tfirst;
            dsc.rows = trows;
            dsc.a_rg = KS;
            for (int ks = 0; ks < KS; ++ks) {
                dsc.kt0 = ks;
                dsc.xrow0 = at * KS + ks;
                desc[at * KS + ks] = dsc;
            }
        } else if (at < Nt - r) {
            dsc.row0 = mt0 * bm + tfirst;
            dsc.rows = trows;
            dsc.xrow0 = shared ? tfirst : -1;
            desc[at] = dsc;
        } else if (TKS > 1) {
            // one of the last r tiles of a large launch, as TKS k slices (fields as above)
            const int ti = at - (Nt - r);
            dsc.row0 = mt0 * bm + tfirst;
            dsc.rows = trows;
            dsc.a_rg = TKS;
            for (int ks = 0; ks < TKS; ++ks) {
                dsc.kt0 = ks;
                dsc.xrow0 = ti * TKS + ks;
                desc[Nt - r + ti * TKS + ks] = dsc;
            }
        } else {
            const int tb = (trows + 31) >> 5;  // the tile's 32-row blocks, dealt evenly to the S slices
            const int rec0 = dsc.kt0;
            for (int sl = 0; sl < S; ++sl) {
                const int sfirst = 32 * ((sl * tb) / S);
                dsc.row0 = mt0 * bm + tfirst + sfirst;
                dsc.rows = max(0, min(32 * (((sl + 1) * tb) / S), trows) - sfirst);  // 0: nothing to do
                dsc.xrow0 = shared ? tfirst + sfirst : -1;
                dsc.kt0 = rec0 + (sfirst >> 5);
                desc[Nt - r + (at - (Nt - r)) * S + sl] = dsc;
            }
        }
    }
}

// entries of a table whose launch has total_mt row tiles and NT column tiles (with the last tiles sliced)
__device__ __forceinline__ int table_entries(int total_mt, int NT, int ks_max = 1, int KT = 0, int tail_ks = 1)
{
    const int Nt = total_mt * NT, r = Nt % 256;
    const int KS = table_k_slices(Nt, ks_max, KT);
    if (KS > 1) return Nt * KS;
    const int TKS = table_tail_k_slices(Nt, tail_ks, KT);
    if (TKS > 1) return Nt - r + r * TKS;
    const int S = (r == 0 || r > 128) ? 1 : min(4, 256 / r);
    return Nt - r + r * S;
}

// MAXE: experts are limited to 256 per layer by the router kernels.
#define MAXE 256
#define RANK_CHUNKS (TOK_TILE_MAX * 64 / 64)  // 64-pair chunks of the largest token tile (K <= 64)
// FUSED: the workgroup forms the prefix of its token tile over the tiles before it, and the per-expert totals, from
// the router's histogram rows itself (a single pass: no scan launch in front; used while the histogram is small enough
// for every workgroup to read all of it); else tile_base / counts come from dispatch_scan_kernel.
template <bool FUSED>
__global__ __launch_bounds__(256) void dispatch_rank_kernel(const int32_t *__restrict__ ids,
                                                            const int32_t *__restrict__ tile_counts,
                                                            const int32_t *__restrict__ tile_base,
                                                            int32_t *__restrict__ counts, int n_tiles, int T, int tok_tile,
                                                            int K, int E, int Es, int bm, int32_t *__restrict__ offsets,
                                                            int32_t *__restrict__ dst, int32_t *__restrict__ dstp,
                                                            int32_t *__restrict__ src_row,
                                                            omega_tile *__restrict__ tiles,
                                                            int32_t *__restrict__ tile_meta,
                                                            omega_tile_desc *__restrict__ desc_up, int nt_up, int ncols_up,
                                                            omega_tile_desc *__restrict__ desc_down, int nt_down,
                                                            int ncols_down, int ks_max_down, int kt_down, int tail_ks_down)
{
    __shared__ int off_s[MAXE + 1];        // logical first row of each expert
    __shared__ int mt_s[MAXE + 64 + 1];    // first row tile of each group (routed, then shared)
    __shared__ int id_s[TOK_TILE_MAX * 64];    // K <= 64
    __shared__ int base_s[MAXE];           // pairs of each expert in the token tiles before this one
    __shared__ int tot_s[MAXE];            // pairs of each expert in the whole batch
    __shared__ int part_s[2][256];
    __shared__ int ccount[RANK_CHUNKS][MAXE];  // pairs of each expert in each 64-pair chunk of this tile
    const int tid = threadIdx.x, tile = blockIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t0 = tile * tok_tile;
    const int npairs = min(tok_tile, T - t0) * K;
    const int nchunks = (npairs + 63) >> 6;

    for (int i = tid; i < npairs; i += 256) id_s[i] = ids[(size_t)t0 * K + i];
    for (int i = tid; i < nchunks * E; i += 256) ccount[i / E][i % E] = 0;
    if (FUSED) {
        // thread (segment s of the tiles, expert e): pairs of e in its tiles, and in those of them before this tile
        int ES = 1;
        while (ES < E) ES <<= 1;
        const int segs = 256 / ES, sg = tid / ES, e = tid % ES;
        const int per = (n_tiles + segs - 1) / segs;
        const int b = min(sg * per, n_tiles), en = min(b + per, n_tiles);
        int before = 0, all = 0;
        if (e < E) {
            int t = b;
            for (; t + 4 <= en; t += 4) {  // four independent loads in flight
                int c[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) c[u] = tile_counts[(size_t)(t + u) * E + e];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    all += c[u];
                    before += t + u < tile ? c[u] : 0;
                }
            }
            for (; t < en; ++t) {
                const int c = tile_counts[(size_t)t * E + e];
                all += c;
                before += t < tile ? c : 0;
            }
        }
        part_s[0][tid] = before;
        part_s[1][tid] = all;
        __syncthreads();
        if (tid < E) {
            int bsum = 0, asum = 0;
            for (int q = 0; q < segs; ++q) {
                bsum += part_s[0][q * ES + tid];
                asum += part_s[1][q * ES + tid];
            }
            base_s[tid] = bsum;
            tot_s[tid] = asum;
            if (tile == 0) counts[tid] = asum;
        }
    } else if (tid < E) {
        base_s[tid] = tile_base[(size_t)tile * E + tid];
        tot_s[tid] = counts[tid];
    }
    __syncthreads();

    // exclusive scans of the E counts and of their tile counts: one wave, 4 experts per lane
    if (tid < 64) {
        int c[4], run = 0, runt = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid * 4 + i;
            c[i] = e < E ? tot_s[e] : 0;
            run += c[i];
            runt += (c[i] + bm - 1) / bm;
        }
        int incl = run, inclt = runt;
#pragma unroll
        for (int m = 1; m < 64; m <<= 1) {
            const int o = __shfl_up(incl, m, 64);
            const int ot = __shfl_up(inclt, m, 64);
            if (tid >= m) { incl += o; inclt += ot; }
        }
        int ex = incl - run, ext = inclt - runt;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid * 4 + i;
            if (e < E) { off_s[e] = ex; mt_s[e] = ext; }
            ex += c[i];
            ext += (c[i] + bm - 1) / bm;
        }
        if (tid == 63) {  // counts beyond E are zero, so lane 63 holds the grand totals
            off_s[E] = incl;
            const int per_shared = (T + bm - 1) / bm;
            for (int s = 0; s <= Es; ++s) mt_s[E + s] = inclt + s * per_shared;
        }
    }

    // Stable rank of every pair among the pairs of its expert.  Within a 64-pair chunk (one wave): the lanes with one
    // expert find each other by ballot, a lane's rank is the number of them below it; across chunks: per-chunk counts
    // in LDS.  Each wave takes every fourth chunk.
    int my_rank[RANK_CHUNKS / 4], my_e[RANK_CHUNKS / 4];
#pragma unroll
    for (int cq = 0; cq < RANK_CHUNKS / 4; ++cq) {
        const int ch = wave + 4 * cq;
        my_rank[cq] = 0;
        my_e[cq] = -1;
        if (ch >= nchunks) continue;  // uniform over the wave
        const int i = ch * 64 + lane;
        const bool valid = i < npairs;
        const int e = valid ? id_s[i] : -1;
        unsigned long long todo = __ballot(valid), mine = 0;
        while (todo) {
            const int leader = __ffsll((long long)todo) - 1;
            const int le = __builtin_amdgcn_readlane(e, leader);
            const unsigned long long m = __ballot(e == le);
            if (e == le) mine = m;
            todo &= ~m;
        }
        if (valid) {
            const unsigned long long below = mine & ((1ull << lane) - 1ull);
            my_rank[cq] = __popcll(below);
            my_e[cq] = e;
            if (below == 0) ccount[ch][e] = __popcll(mine);  // the lowest lane of each expert of the chunk
        }
    }
    __syncthreads();
#pragma unroll
    for (int cq = 0; cq < RANK_CHUNKS / 4; ++cq) {
        const int ch = wave + 4 * cq, e = my_e[cq];
        if (ch >= nchunks || e < 0) continue;
        const int i = ch * 64 + lane;
        int rank = base_s[e] + my_rank[cq];
        for (int c2 = 0; c2 < ch; ++c2) rank += ccount[c2][e];
        const int r = off_s[e] + rank;
        dst[(size_t)t0 * K + i] = r;
        dstp[(size_t)t0 * K + i] = mt_s[e] * bm + rank;
        src_row[r] = t0 + i / K;
    }

    const int G = E + Es;
    if (tile == 0) {
        for (int e = tid; e <= E; e += 256) offsets[e] = off_s[e];
        if (tid == 0) tile_meta[0] = mt_s[G];
        for (int g = tid; g <= G; g += 256) tile_meta[1 + g] = mt_s[g];
    }
    // row-tile list: group g is written by workgroup g (mod grid), like the work-item tables below
    for (int g = tile; g < G; g += gridDim.x) {
        const int rows = g < E ? off_s[g + 1] - off_s[g] : T;
        const int nm = mt_s[g + 1] - mt_s[g];
        for (int mt = tid; mt < nm; mt += 256) {
            omega_tile tl;
            tl.g = g;
            tl.row0 = (mt_s[g] + mt) * bm;
            tl.rows = min(bm, rows - mt * bm);
            tl.xrow0 = g < E ? -1 : mt * bm;
            tiles[mt_s[g] + mt] = tl;
        }
    }

    // ---- work-item tables of the two grouped products (bf16 layers) ----
    // Tile number first_tile[g]*NT + n*Mg + m = (expert g, column tile n, row tile m): row tiles fastest, so that
    // tiles that run at the same time share weight tiles.  A group with more than OMEGA_ROW_BLOCK_MAX row tiles is cut
    // into row blocks of at most that many row tiles, each walking all column tiles (row tiles of the block fastest):
    // the 32 consecutive entries an XCD works on at a time then form a block of about 8 row tiles x 4 column tiles that
    // fetches each of its operand tiles once, where one column tile x 32 row tiles would fetch the rows again for every
    // column tile (down product: 8192 tokens, 64 experts + 2 shared, 0.390 -> 0.368 ms; 16384 tokens, 128 skewed
    // experts, 0.502 -> 0.486 ms).
    // The rows of a group are dealt evenly (in blocks of 32) to
    // its row tiles, instead of full tiles and a ragged last one: the same number of tiles and of MFMA blocks, but
    // tiles of one cost, so that the workgroups of an XCD, which share operand tiles through its L2, stay in step.
    // The compute units take 256 tiles at a time; when the
    // last r = Nt mod 256 tiles would occupy at most half of them, each of those tiles is cut into S = 256/r (2..4)
    // slices of its 32-row blocks (adjacent entries, so that the slices of a tile run side by side on one XCD and share
    // the weight tile in its L2).  Group g is written by workgroup g (mod grid).
    if (desc_up != nullptr || desc_down != nullptr) {
        if (tile == 0 && tid == 0) {
            tile_meta[G + 2] = table_entries(mt_s[G], nt_up);
            tile_meta[G + 3] = table_entries(mt_s[G], nt_down, ks_max_down, kt_down, tail_ks_down);
            const int Nt = mt_s[G] * nt_down, KS = table_k_slices(Nt, ks_max_down, kt_down);
            const int TKS = KS > 1 ? 1 : table_tail_k_slices(Nt, tail_ks_down, kt_down);
            tile_meta[G + 7] = KS;
            // the k-sliced entries of the down table (their partial results are added up behind the product)
            tile_meta[G + 8] = KS > 1 ? 0 : Nt - Nt % 256;
            tile_meta[G + 9] = KS > 1 ? Nt * KS : TKS > 1 ? (Nt % 256) * TKS : 0;
        }
        for (int g = tile; g < G; g += gridDim.x) {
            const int rows = g < E ? off_s[g + 1] - off_s[g] : T;
            const int Mg = mt_s[g + 1] - mt_s[g];
            write_group_items(desc_up, nt_up, ncols_up, g, rows, Mg, mt_s[g], mt_s[G], bm, g >= E);
            write_group_items(desc_down, nt_down, ncols_down, g, rows, Mg, mt_s[g], mt_s[G], bm, g >= E, ks_max_down, kt_down, tail_ks_down);
        }
    }
}

// Per-workgroup queues of the persistent product kernels.  A product launch has n_wg workgroups, one per compute
// unit; workgroup w runs on XCD w % 8.  The table is consumed in rounds of n_wg consecutive entries, XCD x taking a
// contiguous eighth of each round (of what is left, in the last one), so the tiles in flight on one XCD are
// neighbours in the table and share operand tiles in its L2.  Within a round the entries of an XCD are dealt to its
// workgroups cheapest entry to the workgroup with the most work so far (ragged row tiles cost less than full ones),
// which keeps the queues' total work level without any run-time arbitration.
// One workgroup of 256 threads per (product, XCD); it runs as one of the first workgroups of the gather launch, which
// needs nothing from it, so its time is hidden.  Three steps per chunk of SCHED_RC rounds: all threads fetch the
// costs; wave 0 deals the rounds one after the other (lane j < n_wg/8 stands for workgroup j*8 + x); all threads
// copy the descriptors to their queue slots.
#define SCHED_RC 256  // rounds per chunk (LDS: 32 bytes of cost + 64 bytes of placement per round)
#define SCHED_WGS 16  // 2 products x 8 XCDs

__device__ __forceinline__ int work_item_cost(int rows)
{
    if (rows <= 0) return 0;
    const int nb = (rows + 31) >> 5;  // 32-row MFMA blocks of the item (the two waves of a SIMD share them)
    return 2 + (14 * nb) / 8;         // sixteenths of a full tile; the loads and the fixed part do not shrink
}

// up to three tables per launch: table p is scheduled by workgroups 8p .. 8p+7
struct sched_args {
    const omega_tile_desc *desc[3];
    omega_tile_desc *wq[3];
    int total_slot[3];  // index in tile_meta of the table's number of entries
    int kcost[3];       // 0: an item costs by its rows; 1: by its k steps (weight-gradient items, all 256 rows high)
    const int32_t *tile_meta;
    int n_wg;
};

__device__ __forceinline__ void schedule_queues(const sched_args &a, int which)
{
    __shared__ unsigned char cost_s[SCHED_RC * 32];
    __shared__ unsigned short place_s[SCHED_RC * 32];  // [round][workgroup j] = 0x8000 | (queue slot - len0) << 5 | source lane
    __shared__ int len0_s[32];
    const int pass = which >> 3, x = which & 7, tid = threadIdx.x, lane = tid & 63;
    const omega_tile_desc *desc = pass == 0 ? a.desc[0] : pass == 1 ? a.desc[1] : a.desc[2];
    omega_tile_desc *wq = pass == 0 ? a.wq[0] : pass == 1 ? a.wq[1] : a.wq[2];
    const int kcost = pass == 0 ? a.kcost[0] : pass == 1 ? a.kcost[1] : a.kcost[2];
    const int n_wg = a.n_wg, wpx = n_wg >> 3;
    const int total = a.tile_meta[pass == 0 ? a.total_slot[0] : pass == 1 ? a.total_slot[1] : a.total_slot[2]];
    const int rounds = (total + n_wg - 1) / n_wg;
    // entry of (round r, place i of this XCD), or -1
    auto entry = [&](int r, int i) {
        const int base = r * n_wg, left = min(n_wg, total - base);
        const int per = (left + 7) >> 3;
        const int L = base + x * per + i;
        return (i < per && L < base + left) ? L : -1;
    };
    int work = 0, len = 0;  // wave 0, lane j: total cost and length of the queue of workgroup j*8 + x
    for (int r0 = 0; r0 < rounds; r0 += SCHED_RC) {
        const int nr = min(SCHED_RC, rounds - r0);
        for (int i0 = 0; i0 < nr * 32; i0 += 4 * 256) {  // four independent loads in flight per thread
            int rows[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int idx = i0 + u * 256 + tid;
                const int L = idx < nr * 32 ? entry(r0 + (idx >> 5), idx & 31) : -1;
                rows[u] = L >= 0 ? (kcost ? -desc[L].xrow0 : desc[L].rows) : 0;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int idx = i0 + u * 256 + tid;
                if (idx < nr * 32) cost_s[idx] = (unsigned char)(rows[u] < 0 ? min(255, 2 + (-rows[u]) / 8) : work_item_cost(rows[u]));
            }
        }
        if (tid < 32) len0_s[tid] = len;
        __syncthreads();
        if (tid < 64) {
            int c_next = lane < 32 ? cost_s[lane] : 0;
            for (int r = 0; r < nr; ++r) {
                const int c = c_next;
                c_next = (lane < 32 && r + 1 < nr) ? cost_s[(r + 1) * 32 + lane] : 0;
                int ce, src;
                // a round whose entries all cost the same (the common case: tiles of one expert after the even split)
                // needs no dealing - it adds the same work to every queue: each workgroup takes the entry of its place
                const unsigned long long act = __ballot(lane < wpx);
                const int c0 = __builtin_amdgcn_readfirstlane(c);
                if (__ballot(lane < wpx && c == c0) == act) {
                    ce = c;
                    src = lane;
                } else {
                    // place of the lane's entry by rising cost and of its workgroup by falling work; lanes that stand
                    // for no workgroup keep their own place
                    // keys are unique (ties go to the lower lane), so a place is a count of larger keys; lane o's key is
                    // broadcast through a scalar register
                    const int key = lane < wpx ? (work << 6) | (63 - lane) : -1;
                    int rank_w = 0;
#pragma unroll
                    for (int o = 0; o < 32; ++o) rank_w += __builtin_amdgcn_readlane(key, o) > key ? 1 : 0;
                    const int ckey = lane < wpx ? (c << 6) | lane : 0x7fffffff;
                    int rank_c = 0;
#pragma unroll
                    for (int o = 0; o < 32; ++o) rank_c += __builtin_amdgcn_readlane(ckey, o) < ckey ? 1 : 0;
                    if (lane >= wpx) { rank_c = lane; rank_w = lane; }
                    // lane p receives the entry whose cost has place p, then every workgroup fetches the entry of its place
                    const int sorted = __builtin_amdgcn_ds_permute(rank_c << 2, (c << 8) | lane);
                    const int mine = __builtin_amdgcn_ds_bpermute(rank_w << 2, sorted);
                    ce = mine >> 8;
                    src = mine & 31;
                }
                if (lane < 32) {
                    unsigned short pl = 0;
                    if (lane < wpx && ce > 0) {
                        pl = (unsigned short)(0x8000 | ((len - len0_s[lane]) << 5) | src);
                        work += ce;
                        ++len;
                    }
                    place_s[r * 32 + lane] = pl;
                }
            }
        }
        __syncthreads();
        for (int i0 = 0; i0 < nr * 32; i0 += 2 * 256) {  // two independent copies in flight per thread
            const int idx0 = i0 + tid, idx1 = i0 + 256 + tid;
            const unsigned short pl0 = idx0 < nr * 32 ? place_s[idx0] : 0, pl1 = idx1 < nr * 32 ? place_s[idx1] : 0;
            const uint4 *sp0 = (const uint4 *)(desc + (pl0 ? entry(r0 + (idx0 >> 5), pl0 & 31) : 0));
            const uint4 *sp1 = (const uint4 *)(desc + (pl1 ? entry(r0 + (idx1 >> 5), pl1 & 31) : 0));
            const uint4 lo0 = sp0[0], hi0 = sp0[1], lo1 = sp1[0], hi1 = sp1[1];
            if (pl0) {
                uint4 *dp = (uint4 *)(wq + (size_t)(len0_s[idx0 & 31] + ((pl0 >> 5) & 0x3ff)) * n_wg + (idx0 & 31) * 8 + x);
                dp[0] = lo0;
                dp[1] = hi0;
            }
            if (pl1) {
                uint4 *dp = (uint4 *)(wq + (size_t)(len0_s[idx1 & 31] + ((pl1 >> 5) & 0x3ff)) * n_wg + (idx1 & 31) * 8 + x);
                dp[0] = lo1;
                dp[1] = hi1;
            }
        }
        __syncthreads();
    }
    if (tid < wpx) {
        omega_tile_desc z = {};
        wq[(size_t)len * n_wg + tid * 8 + x] = z;
    }
}

// One wave per token; 16-byte chunks; up to 8 chunks in flight per lane.  PACKED: destination rows are in the
// packed tile image (chunk index = 4*kstep + c); when xs != nullptr, the token is also copied to row t of xs.
// The first n_sched workgroups build the product kernels' queues instead (see schedule_queues).
// NT: the rows are written with non-temporal stores, from half the last-level cache (256 MiB) of gathered rows on.
// 16384 tokens x 8 slots x 2048 (512 MiB): launch 0.204 -> 0.158 ms and the products that follow gain 2 %;
// 8192 x 6 x 2048 (192 MiB): launch 0.090 -> 0.073 ms, forward pass 1.332 -> 1.321 ms; 4096 x 2 x 4096 (64 MiB): launch
// -2.5 us, up product +3 us, the forward pass the same - left to the cache.
template <bool PACKED, bool NT>
__global__ __launch_bounds__(256) void dispatch_gather_kernel(const uint4 *__restrict__ x, const int32_t *__restrict__ dstp,
                                                              int T, int K, int chunks_per_row,
                                                              unsigned char *__restrict__ xg, unsigned char *__restrict__ xs,
                                                              int n_sched, sched_args sa)
{
    if (PACKED && (int)blockIdx.x < n_sched) {
        schedule_queues(sa, blockIdx.x);
        return;
    }
    const int lane = threadIdx.x & 63;
    const int t = ((int)blockIdx.x - n_sched) * 4 + (threadIdx.x >> 6);
    if (t >= T) return;
    const uint4 *src = x + (size_t)t * chunks_per_row;
    const int KT = chunks_per_row >> 2;
    for (int c0 = 0; c0 < chunks_per_row; c0 += 64 * 8) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int c = c0 + u * 64 + lane;
            v[u] = c < chunks_per_row ? src[c] : uint4{0u, 0u, 0u, 0u};  // always assigned: the array stays in registers
        }
        const int nd = K + (xs != nullptr ? 1 : 0);
        for (int j = 0; j < nd; ++j) {
            const int prow = j < K ? dstp[(size_t)t * K + j] : t;
            unsigned char *base = j < K ? xg : xs;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int c = c0 + u * 64 + lane;
                if (c < chunks_per_row) {
                    if (PACKED && NT) {
                        typedef unsigned v4u __attribute__((ext_vector_type(4)));
                        const v4u t4 = {v[u].x, v[u].y, v[u].z, v[u].w};
                        __builtin_nontemporal_store(t4, (v4u *)(base + pk_chunk_off(prow, c >> 2, c & 3, KT)));
                    } else if (PACKED) {
                        *(uint4 *)(base + pk_chunk_off(prow, c >> 2, c & 3, KT)) = v[u];
                    }
                    if (!PACKED) *(uint4 *)(base + ((size_t)prow * chunks_per_row + c) * 16) = v[u];
                }
            }
        }
    }
}

// Fallback for fp32 rows that are not a multiple of 16 bytes: element-wise copy.
__global__ __launch_bounds__(256) void dispatch_gather_bytes_kernel(const unsigned char *__restrict__ x,
                                                                    const int32_t *__restrict__ dstp, int T, int K,
                                                                    size_t row_bytes, unsigned char *__restrict__ xg)
{
    const int t = blockIdx.x;
    for (int j = 0; j < K; ++j) {
        unsigned char *out = xg + (size_t)dstp[(size_t)t * K + j] * row_bytes;
        for (size_t b = threadIdx.x; b < row_bytes; b += 256) out[b] = x[(size_t)t * row_bytes + b];
    }
}

// Largest histogram (token tiles x experts) for which every rank workgroup sums all of it itself instead of reading
// the prefix a scan launch left: 64 KiB per workgroup out of the L2.
#define RANK_FUSED_MAX_CELLS 16384

hipError_t launch_dispatch_index(const omega_moe *m, int T, int bm, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const int tok_tile = router_tok_tile(c.E);
    const int n_tiles = ceil_div(T, tok_tile);
    const bool fused = (size_t)n_tiles * c.E <= RANK_FUSED_MAX_CELLS;
    if (!fused) {
        hipLaunchKernelGGL(dispatch_scan_kernel, dim3(ceil_div(c.E, SCAN_EC)), dim3(256), 0, s, m->tile_counts,
                           m->tile_base, n_tiles, c.E, m->counts);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
#define RANK_LAUNCH(F)                                                                                                      \
    hipLaunchKernelGGL(dispatch_rank_kernel<F>, dim3(n_tiles), dim3(256), 0, s, m->ids, m->tile_counts, m->tile_base, m->counts, \
                       n_tiles, T, tok_tile, c.K, c.E, c.Es, bm, m->offsets, m->dst, m->dstp, m->src_row, m->tiles,          \
                       m->tile_meta, m->desc_up, c.H / 128, 128, m->desc_down, c.d / m->down_cols, m->down_cols,             \
                       m->down_ks_max, c.H / 32, m->down_tail_ks)
    if (fused) RANK_LAUNCH(true);
    else RANK_LAUNCH(false);
#undef RANK_LAUNCH
    return hipGetLastError();
}

hipError_t launch_dispatch_gather(const omega_moe *m, const void *x, int T, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const size_t row_bytes = (size_t)c.d * m->esize;
    if (c.dtype == OMEGA_DTYPE_BF16) {  // d % 256 == 0 is guaranteed at creation: rows are whole 64-byte k steps
        const int G = c.E + c.Es;
        sched_args sa = {{m->desc_up, m->desc_down, nullptr}, {m->wq_up, m->wq_down, nullptr}, {G + 2, G + 3, 0}, {0, 0, 0},
                         m->tile_meta, m->n_wg};
        if ((size_t)T * c.K * row_bytes > OMEGA_LLC_BYTES / 2)
            hipLaunchKernelGGL((dispatch_gather_kernel<true, true>), dim3(ceil_div(T, 4) + SCHED_WGS), dim3(256), 0, s, (const uint4 *)x,
                               m->dstp, T, c.K, (int)(row_bytes / 16), (unsigned char *)m->xg, (unsigned char *)m->xs, SCHED_WGS, sa);
        else
            hipLaunchKernelGGL((dispatch_gather_kernel<true, false>), dim3(ceil_div(T, 4) + SCHED_WGS), dim3(256), 0, s, (const uint4 *)x,
                               m->dstp, T, c.K, (int)(row_bytes / 16), (unsigned char *)m->xg, (unsigned char *)m->xs, SCHED_WGS, sa);
    } else if (row_bytes % 16 == 0 && ((uintptr_t)x % 16) == 0) {
        hipLaunchKernelGGL((dispatch_gather_kernel<false, false>), dim3(ceil_div(T, 4)), dim3(256), 0, s, (const uint4 *)x,
                           m->dstp, T, c.K, (int)(row_bytes / 16), (unsigned char *)m->xg, (unsigned char *)nullptr, 0,
                           sched_args{});
    } else {
        hipLaunchKernelGGL(dispatch_gather_bytes_kernel, dim3(T), dim3(256), 0, s, (const unsigned char *)x, m->dstp, T,
                           c.K, row_bytes, (unsigned char *)m->xg);
    }
    return hipGetLastError();
}

// ---- row-major <-> packed tile image (weights at load time, workspace inspection) ----
__global__ __launch_bounds__(256) void pack_rows_kernel(unsigned char *__restrict__ packed, uint4 *__restrict__ rowmajor,
                                                        int R, int chunks_per_row, int to_packed)
{
    const int KT = chunks_per_row >> 2;
    const size_t n = (size_t)R * chunks_per_row;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const int r = (int)(i / chunks_per_row), c = (int)(i % chunks_per_row);
        uint4 *pk = (uint4 *)(packed + pk_chunk_off(r, c >> 2, c & 3, KT));
        if (to_packed) *pk = rowmajor[i];
        else rowmajor[i] = *pk;
    }
}

hipError_t launch_pack_rows(void *dst_packed, const void *src_rowmajor, int R, int Kd, hipStream_t s)
{
    const size_t n = (size_t)R * (Kd / 8);
    const unsigned grid = (unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
    hipLaunchKernelGGL(pack_rows_kernel, dim3(grid), dim3(256), 0, s, (unsigned char *)dst_packed, (uint4 *)src_rowmajor, R,
                       Kd / 8, 1);
    return hipGetLastError();
}

hipError_t launch_unpack_rows(void *dst_rowmajor, const void *src_packed, int R, int Kd, hipStream_t s)
{
    const size_t n = (size_t)R * (Kd / 8);
    const unsigned grid = (unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
    hipLaunchKernelGGL(pack_rows_kernel, dim3(grid), dim3(256), 0, s, (unsigned char *)src_packed, (uint4 *)dst_rowmajor, R,
                       Kd / 8, 0);
    return hipGetLastError();
}


// ---- work-item tables of the backward products (bf16 layers) ----
// k space of the weight gradients: the experts' rows, expert after expert, each expert's share rounded up to 64 rows
// and to at least 192 (a product item must be longer than the load ring of the product kernel); kt0[g] = first k step
// (32 rows) of group g, kt0[G] = all of them.  Empty groups take no space and get no items.
__device__ __forceinline__ int kspace_steps(int rows) { return rows > 0 ? max((rows + 63) / 64 * 2, 6) : 0; }

// One workgroup per group g: the items of the d(a) product (256-column tiles over H, table as the forward ones), the
// group's place in k space, and its items of the two weight-gradient products (all 256 x 256 tiles of dW_g;
// descriptor: row0 = g*M + first row, xrow0 = k steps, a_rg / b_rg = operand row groups).
__global__ __launch_bounds__(256) void bw_tables_kernel(int32_t *__restrict__ tile_meta, const int32_t *__restrict__ counts,
                                                        int E, int Es, int T, int bm, omega_tile_desc *__restrict__ desc_da,
                                                        int nt_da, int32_t *__restrict__ kt0,
                                                        omega_tile_desc *__restrict__ desc_w2, int M2, int NT2,
                                                        omega_tile_desc *__restrict__ desc_w13, int M13, int NT13)
{
    __shared__ int red_k[4], red_n[4];
    const int G = E + Es, g = blockIdx.x, tid = threadIdx.x;
    const int rows = g < E ? counts[g] : T;
    const int mt0 = tile_meta[1 + g], Mg = tile_meta[2 + g] - mt0, total_mt = tile_meta[1 + G];
    write_group_items(desc_da, nt_da, 256, g, rows, Mg, mt0, total_mt, bm, g >= E);
    if (g == 0 && tid == 0) tile_meta[G + 4] = table_entries(total_mt, nt_da);
    // k steps and non-empty groups before g
    int ks = 0, ne = 0;
    for (int q = tid; q < g; q += 256) {
        const int r = q < E ? counts[q] : T;
        ks += kspace_steps(r);
        ne += r > 0 ? 1 : 0;
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        ks += __shfl_xor(ks, m, 64);
        ne += __shfl_xor(ne, m, 64);
    }
    if ((tid & 63) == 0) { red_k[tid >> 6] = ks; red_n[tid >> 6] = ne; }
    __syncthreads();
    ks = red_k[0] + red_k[1] + red_k[2] + red_k[3];
    ne = red_n[0] + red_n[1] + red_n[2] + red_n[3];
    const int my_ks = kspace_steps(rows);
    if (tid == 0) {
        kt0[g] = ks;
        if (g == G - 1) {
            kt0[G] = ks + my_ks;
            const int ne_all = ne + (rows > 0 ? 1 : 0);
            tile_meta[G + 5] = ne_all * (M2 / 256) * NT2;
            tile_meta[G + 6] = ne_all * (M13 / 256) * NT13;
        }
    }
    if (rows <= 0) return;
    for (int pass = 0; pass < 2; ++pass) {
        omega_tile_desc *desc = pass == 0 ? desc_w2 : desc_w13;
        const int M = pass == 0 ? M2 : M13, MT = M / 256, NT = pass == 0 ? NT2 : NT13;
        // the tile index with fewer values runs fastest, so that the 32 consecutive items an XCD works on at a time
        // form a block of row tiles x column tiles that is as square as possible and share operand tiles in its L2
        const bool m_fast = MT <= NT;
        for (int l = tid; l < MT * NT; l += 256) {
            const int mi = m_fast ? l % MT : l / NT, n = m_fast ? l / MT : l % NT;
            omega_tile_desc dsc;
            dsc.g = g;
            dsc.row0 = g * M + mi * 256;
            dsc.rows = 256;
            dsc.xrow0 = my_ks;
            dsc.n0 = n * 256;
            dsc.a_rg = mi * 2;
            dsc.b_rg = n * 2;
            dsc.kt0 = ks;
            desc[(size_t)ne * MT * NT + l] = dsc;
        }
    }
}

__global__ __launch_bounds__(256) void bw_sched_kernel(sched_args sa) { schedule_queues(sa, blockIdx.x); }

hipError_t launch_backward_tables(const omega_moe *m, int T, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const int G = c.E + c.Es;
    hipLaunchKernelGGL(bw_tables_kernel, dim3(G), dim3(256), 0, s, m->tile_meta, m->counts, c.E, c.Es, T, m->bm, m->desc_da,
                       ceil_div(c.H, 256), m->bw_kt0, m->desc_w2, c.d, ceil_div(c.H, 256), m->desc_w13, 2 * c.H, c.d / 256);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    sched_args sa = {{m->desc_da, m->desc_w2, m->desc_w13}, {m->wq_da, m->wq_w2, m->wq_w13}, {G + 4, G + 5, G + 6}, {0, 1, 1},
                     m->tile_meta, m->n_wg};
    hipLaunchKernelGGL(bw_sched_kernel, dim3(24), dim3(256), 0, s, sa);
    return hipGetLastError();
}

// ---- transposed packed images ----
// dst[c][32*k0 + (r - r0)] = src[r][c] for the rows r0 .. r0+nr-1 of a source image (KTs k steps wide, all its
// 32*KTs columns), zero for the next rows up to the end of the range's 32*ksteps places.  One workgroup moves
// 64 rows x 64 columns through LDS (grid.x: rows / k space, grid.y: columns).  by_group != 0: the row ranges are the experts' (the
// workgroup looks its group up in kt0; r0 = first physical row of the group, or row 0 of src_alt for a shared expert
// when src_alt is given); by_group == 0: one range (r0 = 0, nr rows, k0) per z, images src + z*src_stride ->
// dst + z*dst_stride.
__global__ __launch_bounds__(256) void transpose_packed_kernel(const unsigned char *__restrict__ src,
                                                               const unsigned char *__restrict__ src_alt, int KTs,
                                                               unsigned char *__restrict__ dst, int KTd, int by_group,
                                                               const int32_t *__restrict__ kt0,
                                                               const int32_t *__restrict__ tile_meta,
                                                               const int32_t *__restrict__ counts, int E, int G, int T, int bm,
                                                               int nr_single, int k0_single, size_t src_stride, size_t dst_stride)
{
    __shared__ uint16_t tile[64][64 + 8];
    const int tid = threadIdx.x;
    const int c0 = blockIdx.y * 64;  // source columns = destination rows
    int r0, nr, kd0, rb;             // rb: first row of this workgroup within the range
    const unsigned char *sp = src;
    if (by_group) {
        const int kb = blockIdx.x * 2;  // first k step of this workgroup
        if (kb >= kt0[G]) return;
        int lo = 0, hi = G;             // last group with kt0[g] <= kb (empty groups share their successor's kt0)
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (kt0[mid] <= kb) lo = mid; else hi = mid;
        }
        int g = lo;
        while (g + 1 < G && kt0[g + 1] <= kb) ++g;
        nr = g < E ? counts[g] : T;
        r0 = tile_meta[1 + g] * bm;
        if (g >= E && src_alt != nullptr) { sp = src_alt; r0 = 0; }
        kd0 = kb;
        rb = (kb - kt0[g]) * 32;
    } else {
        sp = src + blockIdx.z * src_stride;
        dst += blockIdx.z * dst_stride;
        r0 = 0;
        nr = nr_single;
        rb = blockIdx.x * 64;
        if (rb >= nr) return;
        kd0 = k0_single + blockIdx.x * 2;
    }
    // load: 64 rows x 8 chunks of 8 columns
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int idx = tid + u * 256;
        const int rr = idx >> 3, ch = idx & 7;
        uint4 v = {0u, 0u, 0u, 0u};
        if (rb + rr < nr) {
            const int c = c0 + ch * 8;
            v = *(const uint4 *)(sp + pk_chunk_off(r0 + rb + rr, c >> 5, (c & 31) >> 3, KTs));
        }
        *(uint4 *)&tile[rr][ch * 8] = v;
    }
    __syncthreads();
    // store: 64 destination rows x 8 chunks of 8 k places
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int idx = tid + u * 256;
        const int cc = idx & 63, kc = idx >> 6;  // destination row c0 + cc, k places kc*8 .. kc*8+7 of the 64
        uint16_t e[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) e[q] = tile[kc * 8 + q][cc];
        uint4 v;
        v.x = e[0] | ((uint32_t)e[1] << 16);
        v.y = e[2] | ((uint32_t)e[3] << 16);
        v.z = e[4] | ((uint32_t)e[5] << 16);
        v.w = e[6] | ((uint32_t)e[7] << 16);
        *(uint4 *)(dst + pk_chunk_off(c0 + cc, kd0 + (kc >> 2), kc & 3, KTd)) = v;
    }
}

// activations: rows of the experts -> k space (ksteps_cap = k steps the destination image is laid out for)
hipError_t launch_transpose_groups(const omega_moe *m, const void *src, const void *src_alt, int cols, void *dst, int T,
                                   hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    hipLaunchKernelGGL(transpose_packed_kernel, dim3(m->bw_ksteps_cap / 2, cols / 64), dim3(256), 0, s,
                       (const unsigned char *)src, (const unsigned char *)src_alt, cols / 32, (unsigned char *)dst,
                       m->bw_ksteps_cap, 1, m->bw_kt0, m->tile_meta, m->counts, c.E, c.E + c.Es, T, m->bm, 0, 0, (size_t)0,
                       (size_t)0);
    return hipGetLastError();
}

// weights: n images of R rows x cols columns -> images of cols rows, written at k step k0 of KTd
hipError_t launch_transpose_images(const void *src, int R, int cols, void *dst, int KTd, int k0, int n, size_t src_stride,
                                   size_t dst_stride, hipStream_t s)
{
    hipLaunchKernelGGL(transpose_packed_kernel, dim3(R / 64, cols / 64, n), dim3(256), 0, s, (const unsigned char *)src,
                       (const unsigned char *)nullptr, cols / 32, (unsigned char *)dst, KTd, 0, (const int32_t *)nullptr,
                       (const int32_t *)nullptr, (const int32_t *)nullptr, 0, 0, 0, 0, R, k0, src_stride, dst_stride);
    return hipGetLastError();
}
