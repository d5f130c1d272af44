// Dispatch: per-expert counts, prefix scan, stable permutation, row-tile list, coalesced row gather.
//
// Pair p = t*K+j goes to logical row dst[p] = offsets[id_p] + #{q<p : id_q == id_p} of the expert-contiguous
// order (a stable counting sort of the pair list by expert id); src_row[dst[p]] = t.  In the buffers the
// experts' segments start on row-tile boundaries (physical row dstp[p] = first_tile[id_p]*bm + rank).
// The router left one histogram row per token tile (16 or 32 tokens, router_tok_tile) in tile_counts[tile][e].  One launch (fp32 layers: two):
//   rank    one workgroup per token tile: the prefix of its tile and the experts' totals, summed from the histogram
//           rows in the same pass (a single-pass scan: no workgroup waits for another); offsets = exclusive scan of the
//           totals, first_tile = exclusive scan of ceil(totals/bm); rank of each pair among the earlier pairs of its
//           tile with the same expert (ballots within 64-pair chunks, per-chunk counts across them); dst / dstp /
//           src_row / tokp; the row-tile list and the work-item tables; workgroup 0 publishes counts, offsets and the
//           totals.  bf16 layers: the workgroup then copies the rows of its own tile into the packed image of the
//           gathered rows (copy_tile_rows) - unless the up product fetches them itself (tokp) -, and the launch's
//           first workgroups build the product kernels' per-workgroup queues from the same totals (schedule_queues)
//   gather  (fp32 layers, and bf16 rows asked for after the fact) one wave per token: the row of x is read once with
//           16-byte accesses and written to its K destination rows (gather semantics as img_token_drop,
//           J/engine/nn/layer/dit/kernel/TokenDropKernel.cu:147-160)
// No floating-point or order-dependent atomics anywhere: counts, offsets and the permutation are deterministic.
#include "common.h"
#include "pack.h"

#define TOK_TILE_MAX ROUTER_TOK_TILE_MAX

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

// a / b for 0 <= a < 2^22, 0 < b < 2^22 through the float reciprocal (a quarter of the instructions of the integer
// division the compiler emits); exact: the estimate is off by at most one, and is corrected
__device__ __forceinline__ int small_div(int a, int b)
{
    int q = (int)((float)a * __builtin_amdgcn_rcpf((float)b));
    const int r = a - q * b;
    q += r >= b ? 1 : 0;
    q -= r < 0 ? 1 : 0;
    return q;
}

// What a product's table is made for: NT column tiles of ncols columns; k slices as table_k_slices / table_tail_k_slices
struct table_params {
    int NT, ncols, ks_max, KT, tail_ks;
};

// How the tiles of a launch with total_mt row tiles map to table entries: the first Nt - r tiles are one entry each;
// when the last r = Nt mod 256 tiles would occupy at most half of the compute units, each of them is `per` adjacent
// entries - k slices (down product, long k) or S = 256/r (2..4) slices of its 32-row blocks -, so that the slices of a
// tile run side by side on one XCD and share operand tiles in its L2; a small batch has every tile in KS k slices.
struct table_shape {
    int Nt, r, KS, TKS, S;
    __device__ __forceinline__ table_shape(const table_params &tp, int total_mt)
    {
        Nt = total_mt * tp.NT;
        r = Nt % 256;
        KS = table_k_slices(Nt, tp.ks_max, tp.KT);
        TKS = KS > 1 ? 1 : table_tail_k_slices(Nt, tp.tail_ks, tp.KT);
        S = (r == 0 || r > 128 || KS > 1 || TKS > 1) ? 1 : min(4, 256 / r);
    }
    __device__ __forceinline__ int per(int at) const { return KS > 1 ? KS : at < Nt - r ? 1 : TKS > 1 ? TKS : S; }
    __device__ __forceinline__ int first(int at) const { return KS > 1 ? at * KS : at < Nt - r ? at : Nt - r + (at - (Nt - r)) * per(at); }
    __device__ __forceinline__ int entries() const { return KS > 1 ? Nt * KS : Nt - r + r * (TKS > 1 ? TKS : S); }
    // tile and slice of entry `ent`
    __device__ __forceinline__ void locate(int ent, int &at, int &sub) const
    {
        at = ent;
        sub = 0;
        if (KS > 1) {
            at = small_div(ent, KS);
            sub = ent - at * KS;
        } else if (ent >= Nt - r) {
            const int p = TKS > 1 ? TKS : S, ti = small_div(ent - (Nt - r), p);
            at = Nt - r + ti;
            sub = ent - (Nt - r) - ti * p;
        }
    }
};

// Slice `sub` of tile `at` of a table, a tile of group g (rows rows in Mg row tiles from row tile mt0 on).
// Order within a group: row blocks of at most OMEGA_ROW_BLOCK_MAX row tiles; inside a row block column tile after
// column tile, the row tiles of the block fastest.  (Walking the column tiles twice, first with the taller row tiles
// and then with the others, makes most rounds of 32 entries cost the same, so that the queue builder has nothing to
// deal: dispatch 50 -> 39 us at the Mixtral shape, but its up product 1.529 -> 1.544 ms - each weight tile is then
// fetched twice.)
// The group's rows are dealt evenly, in blocks of 32, to its Mg row tiles (instead of full tiles and a ragged last
// one): the same number of tiles and of MFMA blocks, but tiles of nearly one cost.  (Equal tiles in units of 16 rows -
// every tile the same number of MFMA blocks, the last one of each half empty - cut the L2 miss traffic of the up
// product by a fifth when every expert has 1040 rows, and still lost 4 % of time to the extra blocks.)
__device__ __forceinline__ omega_tile_desc group_item(const table_params &tp, const table_shape &ts, int at, int sub, int g,
                                                      int rows, int Mg, int mt0, int bm, bool shared)
{
    const int NT = tp.NT, l = at - mt0 * NT;
    const int nblk = (rows + 31) >> 5;
    const int qblk = small_div(nblk, Mg), nhi = nblk - qblk * Mg;  // the first nhi row tiles hold qblk + 1 blocks, the others qblk
    const int NB = (Mg + OMEGA_ROW_BLOCK_MAX - 1) / OMEGA_ROW_BLOCK_MAX;
    int f = 0, RB = Mg;
    if (NB > 1) {
        // row block b holds row tiles [b*Mg/NB, (b+1)*Mg/NB); the entries before it number (first tile) * NT
        int b = min(NB - 1, small_div(small_div(l, NT) * NB, Mg));
        while (small_div(b * Mg, NB) * NT > l) --b;
        while (b + 1 < NB && small_div((b + 1) * Mg, NB) * NT <= l) ++b;
        f = small_div(b * Mg, NB);
        RB = small_div((b + 1) * Mg, NB) - f;
    }
    const int li = l - f * NT;
    const int n = small_div(li, RB), mt = f + li - n * RB;
    const int tfirst = 32 * (mt * qblk + min(mt, nhi));
    const int trows = min(32 * ((mt + 1) * qblk + min(mt + 1, nhi)), rows) - tfirst;
    const int ent = ts.first(at) + sub;
    omega_tile_desc dsc;
    dsc.g = g;
    dsc.n0 = n * tp.ncols;
    dsc.a_rg = 0;
    dsc.b_rg = tp.ncols == 128 ? 1 : 0;  // read by the plain 256-column products only: a half-width item
    // (items without k slices: kt0 = first 32 x 32 block record of the item - 8 records per row-tile slot - for the
    //  products that keep or read h1 / h3 block records)
    dsc.kt0 = (mt0 + mt) * 8;
    dsc.row0 = mt0 * bm + tfirst;
    dsc.rows = trows;
    dsc.xrow0 = shared ? tfirst : -1;
    if (ts.KS > 1 || (at >= ts.Nt - ts.r && ts.TKS > 1)) {
        // slice `sub` of a_rg slices of the k range (kt0 = slice, xrow0 = number of the sliced entry = of its partial
        // result)
        dsc.a_rg = ts.KS > 1 ? ts.KS : ts.TKS;
        dsc.kt0 = sub;
        dsc.xrow0 = ts.KS > 1 ? ent : ent - (ts.Nt - ts.r);
    } else if (at >= ts.Nt - ts.r && ts.S > 1) {
        const int tb = (trows + 31) >> 5;  // the tile's 32-row blocks, dealt evenly to the S slices
        const int sfirst = 32 * small_div(sub * tb, ts.S);
        dsc.row0 += sfirst;
        dsc.rows = max(0, min(32 * small_div((sub + 1) * tb, ts.S), trows) - sfirst);  // 0: nothing to do
        dsc.xrow0 = shared ? tfirst + sfirst : -1;
        dsc.kt0 += sfirst >> 5;
    }
    return dsc;
}

// The work item at place `ent` of a table, from the groups' row counts alone (mt_s[g] = first row tile of group g,
// mt_s[G] = all row tiles; off_s[e] = first logical row of expert e; a shared expert holds T rows): whoever needs an
// entry - the table writers, the queue builders - forms it without waiting for anybody else.
__device__ __forceinline__ omega_tile_desc item_desc(int ent, const table_params &tp, const table_shape &ts, const int *mt_s,
                                                     const int *off_s, int E, int G, int T, int bm)
{
    int at, sub;
    ts.locate(ent, at, sub);
    // the group of tile `at`: the last g with first_tile[g]*NT <= at (groups without rows have no tiles and are passed over)
    int lo = 0, hi = G;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (mt_s[mid] * tp.NT <= at) lo = mid;
        else hi = mid;
    }
    const int g = lo;
    return group_item(tp, ts, at, sub, g, g < E ? off_s[g + 1] - off_s[g] : T, mt_s[g + 1] - mt_s[g], mt_s[g], bm, g >= E);
}

// The table entries of group g, written by the 256 threads of a workgroup.
__device__ __forceinline__ void write_group_items(omega_tile_desc *__restrict__ desc, int NT, int ncols, int g, int rows,
                                                  int Mg, int mt0, int total_mt, int bm, bool shared, int ks_max = 1,
                                                  int KT = 0, int tail_ks = 1)
{
    if (desc == nullptr) return;
    const table_params tp = {NT, ncols, ks_max, KT, tail_ks};
    const table_shape ts(tp, total_mt);
    for (int l = threadIdx.x; l < Mg * NT; l += 256) {
        const int at = mt0 * NT + l, per = ts.per(at), first = ts.first(at);
        for (int q = 0; q < per; ++q) desc[first + q] = group_item(tp, ts, at, q, g, rows, Mg, mt0, bm, shared);
    }
}

// entries of a table whose launch has total_mt row tiles and NT column tiles (with the last tiles sliced)
__device__ __forceinline__ int table_entries(int total_mt, int NT, int ks_max = 1, int KT = 0, int tail_ks = 1)
{
    const table_params tp = {NT, 0, ks_max, KT, tail_ks};
    return table_shape(tp, total_mt).entries();
}

// Per-workgroup queues of the persistent product kernels.  A product launch has n_wg workgroups, one per compute
// unit; workgroup w runs on XCD w % 8.  The table is consumed in rounds of n_wg consecutive entries, XCD x taking a
// contiguous eighth of each round (of what is left, in the last one), so the tiles in flight on one XCD are
// neighbours in the table and share operand tiles in its L2.  Within a round the entries of an XCD are dealt to its
// workgroups cheapest entry to the workgroup with the most work so far (ragged row tiles cost less than full ones),
// which keeps the queues' total work level without any run-time arbitration.
// One workgroup of 256 threads per (product, XCD).  Per chunk of SCHED_RC rounds: all threads fetch the costs and rank
// the entries of every round by cost; wave 0 deals the rounds one after the other (lane j < n_wg/8 stands for
// workgroup j*8 + x; what depends on the round before is only the order of the workgroups by work, 32 keys ranked by
// the 64 lanes against 16 keys each out of LDS); all threads write the descriptors to their queue slots.
#define SCHED_RC 128  // rounds per chunk
#define SCHED_WGS 16  // 2 products x 8 XCDs
#define SCHED_SCRATCH (5 * SCHED_RC * 32 + 256)  // bytes of LDS schedule_queues works in

__device__ __forceinline__ int work_item_cost(int rows)
{
    if (rows <= 0) return 0;
    const int nb = (rows + 31) >> 5;  // 32-row MFMA blocks of the item (the two waves of a SIMD share them)
    return 2 + (14 * nb) / 8;         // sixteenths of a full tile; the loads and the fixed part do not shrink
}

// where the entries of a table come from: the table in memory (the backward pass's products) ...
struct table_source {
    const omega_tile_desc *desc;
    int kcost;  // 0: an item costs by its rows; 1: by its k steps (weight-gradient items, all 256 rows high)
    __device__ __forceinline__ int cost(int L) const
    {
        return kcost ? min(255, 2 + desc[L].xrow0 / 8) : work_item_cost(desc[L].rows);
    }
    __device__ __forceinline__ omega_tile_desc get(int L) const { return desc[L]; }
};
// ... or the groups' row counts (the forward pass: the queue builders run beside the table writers, not behind them)
struct analytic_source {
    table_params tp;
    table_shape ts;
    const int *mt_s, *off_s;
    int E, G, T, bm;
    __device__ __forceinline__ omega_tile_desc get(int L) const { return item_desc(L, tp, ts, mt_s, off_s, E, G, T, bm); }
    __device__ __forceinline__ int cost(int L) const { return work_item_cost(get(L).rows); }
};

// (Dealing the rounds of a table in 2 or 4 independent chains, one workgroup each, shortens the one step that depends
// on the round before - the order of the workgroups by work - and was measured: the queue builders finish 5-9 us
// earlier, and the up product of 4096 tokens x 8 experts loses 2 %, 30 us, to the coarser levelling.)
template <class Source>
__device__ __forceinline__ void schedule_queues(const Source &src, omega_tile_desc *__restrict__ wq, int total, int n_wg, int x,
                                                unsigned char *scratch)
{
    unsigned char *cost_s = scratch;                                            // [round][place]
    unsigned short *sorted_s = (unsigned short *)(scratch + SCHED_RC * 32);     // [round][p] = cost << 8 | place of the p-th cheapest entry
    unsigned short *place_s = (unsigned short *)(scratch + 3 * SCHED_RC * 32);  // [round][workgroup j] = 0x8000 | (queue slot - len0) << 5 | source place
    int *len0_s = (int *)(scratch + 5 * SCHED_RC * 32);
    int *keys_s = len0_s + 32;
    const int tid = threadIdx.x, lane = tid & 63, nthr = blockDim.x;
    const int wpx = n_wg >> 3;
    const int rounds = (total + n_wg - 1) / n_wg;
    // entry of (round r, place i of this XCD), or -1
    auto entry = [&](int r, int i) {
        const int base = r * n_wg, left = min(n_wg, total - base);
        const int per = (left + 7) >> 3;
        const int L = base + x * per + i;
        return (i < per && L < base + left) ? L : -1;
    };
    // wave 0, lanes j and j + 32 alike: total cost and length of the queue of workgroup j*8 + x
    int work = 0, len = 0;
    for (int r0 = 0; r0 < rounds; r0 += SCHED_RC) {
        const int nr = min(SCHED_RC, rounds - r0);
        for (int idx = tid; idx < nr * 32; idx += nthr) {
            const int L = entry(r0 + (idx >> 5), idx & 31);
            cost_s[idx] = (unsigned char)(L >= 0 ? src.cost(L) : 0);
        }
        if (tid < 32) len0_s[tid] = len;
        __syncthreads();
        // every round's entries in the order of rising cost (ties to the lower place; places that stand for no workgroup
        // stay where they are): keys are unique, so an entry's rank is a count of smaller keys
        for (int idx = tid; idx < nr * 32; idx += nthr) {
            const int i = idx & 31;
            const uint4 *cs = (const uint4 *)(cost_s + (idx & ~31));
            const uint4 lo = cs[0], hi = cs[1];
            const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            const int c = cost_s[idx], key = (c << 5) | i;
            int rk = 0;
#pragma unroll
            for (int o = 0; o < 32; ++o) {
                const int ko = (int)(((w[o >> 2] >> ((o & 3) * 8)) & 255) << 5) | o;
                rk += (o < wpx && ko < key) ? 1 : 0;
            }
            sorted_s[(idx & ~31) + (i < wpx ? rk : i)] = (unsigned short)((c << 8) | i);
        }
        __syncthreads();
        if (tid < 64) {
            const int i = lane & 31, h = lane >> 5;
            int c_next = cost_s[i];
            for (int r = 0; r < nr; ++r) {
                const int c = c_next;
                c_next = r + 1 < nr ? cost_s[(r + 1) * 32 + i] : 0;
                int ce, srcp;
                // a round whose entries all cost the same (the common case: tiles of one expert after the even split)
                // needs no dealing - it adds the same work to every queue: each workgroup takes the entry of its place
                const int c0 = __builtin_amdgcn_readfirstlane(c);
                if (__ballot(i < wpx && c != c0) == 0) {
                    ce = c;
                    srcp = i;
                } else {
                    // place of the workgroup by falling work (ties to the lower workgroup): lanes i and i + 32 count the
                    // larger keys among 16 keys each; the workgroup at place p takes the p-th cheapest entry
                    const int key = i < wpx ? (work << 6) | (63 - i) : -1;
                    if (lane < 32) keys_s[lane] = key;
                    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");  // one wave: its LDS accesses complete in order
                    const int4 *kp = (const int4 *)(keys_s + 16 * h);
                    const int4 k0 = kp[0], k1 = kp[1], k2 = kp[2], k3 = kp[3];
                    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
                    const int cnt = (k0.x > key) + (k0.y > key) + (k0.z > key) + (k0.w > key) + (k1.x > key) + (k1.y > key) +
                                    (k1.z > key) + (k1.w > key) + (k2.x > key) + (k2.y > key) + (k2.z > key) + (k2.w > key) +
                                    (k3.x > key) + (k3.y > key) + (k3.z > key) + (k3.w > key);
                    const int rank_w = i < wpx ? cnt + __shfl_xor(cnt, 32, 64) : i;
                    const int mine = sorted_s[r * 32 + rank_w];
                    ce = mine >> 8;
                    srcp = mine & 31;
                }
                unsigned short pl = 0;
                if (i < wpx && ce > 0) {
                    pl = (unsigned short)(0x8000 | ((len - len0_s[i]) << 5) | srcp);
                    work += ce;
                    ++len;
                }
                if (lane < 32) place_s[r * 32 + lane] = pl;
            }
        }
        __syncthreads();
        for (int idx = tid; idx < nr * 32; idx += nthr) {
            const unsigned short pl = place_s[idx];
            if (pl) {
                const omega_tile_desc d = src.get(entry(r0 + (idx >> 5), pl & 31));
                wq[(size_t)(len0_s[idx & 31] + ((pl >> 5) & 0x3ff)) * n_wg + (idx & 31) * 8 + x] = d;
            }
        }
        __syncthreads();
    }
    if (tid < wpx) {  // a queue ends with an entry without rows
        omega_tile_desc z = {};
        wq[(size_t)len * n_wg + tid * 8 + x] = z;
    }
}

// up to three tables per launch: table p is scheduled by workgroups 8p .. 8p+7
struct sched_args {
    const omega_tile_desc *desc[3];
    omega_tile_desc *wq[3];
    int total_slot[3];  // index in tile_meta of the table's number of entries
    int kcost[3];       // see table_source
    const int32_t *tile_meta;
    int n_wg;
};

// The rows of one token tile into the packed image of the gathered rows (and of the shared experts' copy), by the
// workgroup that has just ranked the tile's pairs (gather semantics as img_token_drop,
// J/engine/nn/layer/dit/kernel/TokenDropKernel.cu:147-160).  In the packed image rows 2i and 2i+1 share every 128-byte
// line (64 bytes of a k step each).  The tile's pairs, sorted by destination row (pairs of one expert are
// consecutive rows), are therefore copied in units of such a row pair where the tile holds both rows: 8 lanes write one
// whole line (4 lanes per row), an instruction covers 8 k steps of the two rows; a row whose neighbour belongs to
// another tile goes by itself, 16 k steps per instruction.  (A wave per token writing 64-byte pieces wrote 1.4 times
// the bytes of the rows.)  The source rows are read in the same pattern, 512 or 1024 contiguous bytes of a row per
// instruction; a token's row is read K times, all but the first out of the L2.
template <bool NT>
__device__ __forceinline__ void copy_tile_rows(const unsigned char *__restrict__ x, int d, int t0, int ntok, int npairs,
                                               const int *sort_prow, const unsigned char *sort_tok,
                                               unsigned char *__restrict__ xg, unsigned char *__restrict__ xs)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
    const int KT = d >> 5;
    const size_t row_bytes = (size_t)d * 2;
    const int n_units = npairs + (xs != nullptr ? (ntok + 1) >> 1 : 0);
    for (int u = wave; u < n_units; u += n_waves) {
        // unit: destination row pa (token ta), and row pa + 1 (token tb) with it if it belongs to the tile as well
        int pa, ta, tb = -1;
        unsigned char *base = xg;
        if (u < npairs) {
            pa = sort_prow[u];
            if (u > 0 && (pa & 1) && sort_prow[u - 1] == pa - 1) continue;  // the second row of the unit before
            ta = sort_tok[u];
            if (!(pa & 1) && u + 1 < npairs && sort_prow[u + 1] == pa + 1) tb = sort_tok[u + 1];
        } else {
            ta = 2 * (u - npairs);
            pa = t0 + ta;  // row t of the shared experts' copy is token t; t0 is even
            if (ta + 1 < ntok) tb = ta + 1;
            base = xs;
        }
        const bool two = tb >= 0;
        // lane -> (row of the unit, k step within the instruction, chunk)
        const int sel = two ? (lane >> 2) & 1 : 0, kk = two ? lane >> 3 : lane >> 2, kpi = two ? 8 : 16, c = lane & 3;
        const int prow = pa + sel;
        const unsigned char *src = x + (size_t)(t0 + (sel ? tb : ta)) * row_bytes + c * 16;
        for (int kb0 = 0; kb0 < KT; kb0 += kpi * 4) {
            uint4 v[4];  // 4 KiB in flight per wave, 16 waves (the kernel keeps to 64 registers: two workgroups per compute unit)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int kb = kb0 + q * kpi + kk;
                v[q] = kb < KT ? *(const uint4 *)(src + (size_t)kb * 64) : uint4{0u, 0u, 0u, 0u};
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int kb = kb0 + q * kpi + kk;
                if (kb < KT) {
                    unsigned char *o = base + pk_chunk_off(prow, kb, c, KT);
                    if (NT) {
                        typedef unsigned v4u __attribute__((ext_vector_type(4)));
                        const v4u t4 = {v[q].x, v[q].y, v[q].z, v[q].w};
                        __builtin_nontemporal_store(t4, (v4u *)o);
                    } else {
                        *(uint4 *)o = v[q];
                    }
                }
            }
        }
    }
}

// MAXE: experts are limited to 256 per layer by the router kernels.
#define MAXE 256
#define RANK_CHUNKS (TOK_TILE_MAX * 64 / 64)  // 64-pair chunks of the largest token tile (K <= 64)
// One workgroup per token tile, behind n_sched workgroups that build the product kernels' queues (see the head of the file).
// 256 threads, or 1024 when the workgroups copy rows (x / xg given): the index work is done by the first 256; the
// kernel keeps to 64 registers so that two such workgroups share a compute unit and the queue builders run beside the
// tiles' workgroups, not behind them.
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(8, 8))) void dispatch_rank_kernel(const int32_t *__restrict__ ids,
                                                            const int32_t *__restrict__ tile_counts,
                                                            int32_t *__restrict__ counts, int n_tiles, int T, int tok_tile,
                                                            int K, int E, int Es, int bm, int32_t *__restrict__ offsets,
                                                            int32_t *__restrict__ dst, int32_t *__restrict__ dstp,
                                                            int32_t *__restrict__ src_row, int32_t *__restrict__ tokp,
                                                            omega_tile *__restrict__ tiles,
                                                            int32_t *__restrict__ tile_meta,
                                                            omega_tile_desc *__restrict__ desc_up, int nt_up, int ncols_up,
                                                            omega_tile_desc *__restrict__ desc_down, int nt_down,
                                                            int ncols_down, int ks_max_down, int kt_down, int tail_ks_down,
                                                            omega_tile_desc *__restrict__ wq_up,
                                                            omega_tile_desc *__restrict__ wq_down, int n_wg,
                                                            const unsigned char *__restrict__ x, int d,
                                                            unsigned char *__restrict__ xg, unsigned char *__restrict__ xs,
                                                            int nt_stores, int n_sched)
{
    __shared__ int off_s[MAXE + 1];        // logical first row of each expert
    __shared__ int mt_s[MAXE + 64 + 1];    // first row tile of each group (routed, then shared)
    __shared__ int id_s[TOK_TILE_MAX * 64];    // K <= 64
    __shared__ int base_s[MAXE];           // pairs of each expert in the token tiles before this one
    __shared__ int tot_s[MAXE];            // pairs of each expert in the whole batch
    __shared__ int part_s[2][256];
    // pairs of each expert in each 64-pair chunk of this tile; the queue builders, which rank nothing, work in it
    __shared__ __attribute__((aligned(16))) int ccount[RANK_CHUNKS][MAXE];
    static_assert(sizeof(int) * RANK_CHUNKS * MAXE >= SCHED_SCRATCH, "the queue builders' scratch fits the chunk counts");
    // the tile's pairs in the order of their destination rows (row copies by this workgroup): row and token within the tile
    __shared__ __attribute__((aligned(16))) int sort_prow[TOK_TILE_MAX * 64];
    __shared__ unsigned char sort_tok[TOK_TILE_MAX * 64];
    // (256 threads, or 1024 when the workgroup copies rows as well: the index work is done by the first 256)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nthr = blockDim.x;
    // the first n_sched workgroups build the product kernels' queues (bf16 layers): they need the experts' totals and
    // the scans of them like everybody else, and nothing that another workgroup of this launch writes
    const bool sched = (int)blockIdx.x < n_sched;
    const int tile = sched ? n_tiles : (int)blockIdx.x - n_sched;
    const int t0 = tile * tok_tile;
    const int npairs = sched ? 0 : min(tok_tile, T - t0) * K;
    const int nchunks = (npairs + 63) >> 6;

    // (row copies: the tile's rows are asked for now, one load per 128-byte line, so that they travel while the index
    //  work below keeps the memory idle; the copies then find them in the L2 or the last-level cache)
    int prefetched = 0;
    if (xg != nullptr && !sched) {
        const size_t tile_bytes = (size_t)min(tok_tile, T - t0) * d * 2;
        const unsigned char *xt = x + (size_t)t0 * d * 2;
        for (size_t o = (size_t)tid * 128; o < tile_bytes; o += (size_t)nthr * 128) prefetched ^= *(const int *)(xt + o);
    }
    for (int i = tid; i < npairs; i += nthr) id_s[i] = ids[(size_t)t0 * K + i];
    for (int i = tid; i < nchunks * E; i += nthr) ccount[i / E][i % E] = 0;
    {
        // thread (segment s of the token tiles, expert e): pairs of e in its tiles, and in those of them before this tile.
        // Every workgroup sums the whole histogram itself, so nobody waits for a scan launch or for another workgroup
        // (a second level of sums written by the router's last-arriving workgroups was tried: the device-scope fences
        // it needs between workgroups on different XCDs cost the router 30-45 us at 8192-16384 tokens).
        // Rows whose length is a multiple of four experts are read 16 bytes at a time (a quarter of the loads; the
        // partial sums then take four times the room and borrow the row-copy lists, which are filled much later).
        const bool vec = (E & 3) == 0;
        const int EU = vec ? E >> 2 : E;  // units of a row: groups of four experts, or experts
        int ES = 1;
        while (ES < EU) ES <<= 1;
        const int segs = min(256 / ES, 16), sg = tid / ES, eu = tid % ES;  // (at most 16 partial sums per expert to add up)
        const int per = (n_tiles + segs - 1) / segs;
        const int b = min(sg * per, n_tiles), en = min(b + per, n_tiles);
        int4 before = {0, 0, 0, 0}, all = {0, 0, 0, 0};
        if (eu < EU && sg < segs) {
            int t = b;
            if (vec) {
                const int4 *rows = (const int4 *)tile_counts;
                for (; t + 8 <= en; t += 8) {  // eight independent loads in flight
                    int4 c[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) c[u] = rows[(size_t)(t + u) * EU + eu];
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        all.x += c[u].x; all.y += c[u].y; all.z += c[u].z; all.w += c[u].w;
                        if (t + u < tile) { before.x += c[u].x; before.y += c[u].y; before.z += c[u].z; before.w += c[u].w; }
                    }
                }
                for (; t < en; ++t) {
                    const int4 c = rows[(size_t)t * EU + eu];
                    all.x += c.x; all.y += c.y; all.z += c.z; all.w += c.w;
                    if (t < tile) { before.x += c.x; before.y += c.y; before.z += c.z; before.w += c.w; }
                }
            } else {
                for (; t + 16 <= en; t += 16) {  // sixteen independent loads in flight
                    int c[16];
#pragma unroll
                    for (int u = 0; u < 16; ++u) c[u] = tile_counts[(size_t)(t + u) * E + eu];
#pragma unroll
                    for (int u = 0; u < 16; ++u) {
                        all.x += c[u];
                        before.x += t + u < tile ? c[u] : 0;
                    }
                }
                for (; t < en; ++t) {
                    const int c = tile_counts[(size_t)t * E + eu];
                    all.x += c;
                    before.x += t < tile ? c : 0;
                }
            }
        }
        int *pb = vec ? sort_prow : &part_s[0][0], *pa = vec ? sort_prow + 1024 : &part_s[1][0];  // [segment][expert]
        if (sg < segs && eu < EU) {
            if (vec) {
                *(int4 *)(pb + sg * E + 4 * eu) = before;
                *(int4 *)(pa + sg * E + 4 * eu) = all;
            } else {
                pb[sg * E + eu] = before.x;
                pa[sg * E + eu] = all.x;
            }
        }
        __syncthreads();
        if (tid < E) {
            int bsum = 0, asum = 0;
            for (int q = 0; q < segs; ++q) {
                bsum += pb[q * E + tid];
                asum += pa[q * E + tid];
            }
            base_s[tid] = bsum;
            tot_s[tid] = asum;
            if (tile == 0) counts[tid] = asum;
        }
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

    const int G = E + Es;
    if (sched) {
        __syncthreads();  // the scans above
        const int job = blockIdx.x, pass = job >> 3;
        const table_params tp = pass == 0 ? table_params{nt_up, ncols_up, 1, 0, 1}
                                          : table_params{nt_down, ncols_down, ks_max_down, kt_down, tail_ks_down};
        const table_shape ts(tp, mt_s[G]);
        const analytic_source src = {tp, ts, mt_s, off_s, E, G, T, bm};
        schedule_queues(src, pass == 0 ? wq_up : wq_down, ts.entries(), n_wg, job & 7, (unsigned char *)&ccount[0][0]);
        return;
    }

    // Stable rank of every pair among the pairs of its expert.  Within a 64-pair chunk (one wave): the lanes with one
    // expert find each other by ballot, a lane's rank is the number of them below it; across chunks: per-chunk counts
    // in LDS.  Each wave takes every fourth chunk.
    int my_re[RANK_CHUNKS / 4];  // rank within the chunk | expert << 8, or -1
#pragma unroll
    for (int cq = 0; cq < RANK_CHUNKS / 4; ++cq) {
        const int ch = wave + 4 * cq;
        my_re[cq] = -1;
        if (ch >= nchunks || wave >= 4) continue;  // uniform over the wave
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
            my_re[cq] = __popcll(below) | (e << 8);
            if (below == 0) ccount[ch][e] = __popcll(mine);  // the lowest lane of each expert of the chunk
        }
    }
    __syncthreads();
    // (row copies by this workgroup: where the pairs of each expert start in the tile's pair list sorted by destination row)
    int *run_off = &part_s[0][0];
    if (xg != nullptr && tid < 64) {
        int c[4], run = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid * 4 + i;
            c[i] = 0;
            if (e < E)
                for (int ch = 0; ch < nchunks; ++ch) c[i] += ccount[ch][e];
            run += c[i];
        }
        int incl = run;
#pragma unroll
        for (int m = 1; m < 64; m <<= 1) {
            const int o = __shfl_up(incl, m, 64);
            if (tid >= m) incl += o;
        }
        int ex = incl - run;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (tid * 4 + i < E) run_off[tid * 4 + i] = ex;
            ex += c[i];
        }
    }
    if (xg != nullptr) __syncthreads();
#pragma unroll
    for (int cq = 0; cq < RANK_CHUNKS / 4; ++cq) {
        const int ch = wave + 4 * cq, e = my_re[cq] >> 8;
        if (ch >= nchunks || e < 0 || wave >= 4) continue;
        const int i = ch * 64 + lane;
        int lrank = my_re[cq] & 255;  // rank among the tile's pairs of the expert
        for (int c2 = 0; c2 < ch; ++c2) lrank += ccount[c2][e];
        const int rank = base_s[e] + lrank;
        const int r = off_s[e] + rank;
        dst[(size_t)t0 * K + i] = r;
        dstp[(size_t)t0 * K + i] = mt_s[e] * bm + rank;
        src_row[r] = t0 + i / K;
        if (tokp != nullptr) tokp[mt_s[e] * bm + rank] = t0 + i / K;
        if (xg != nullptr) {
            sort_prow[run_off[e] + lrank] = mt_s[e] * bm + rank;
            sort_tok[run_off[e] + lrank] = (unsigned char)(i / K);
        }
    }

    if (tile == 0) {
        for (int e = tid; e <= E; e += nthr) offsets[e] = off_s[e];
        if (tid == 0) tile_meta[0] = mt_s[G];
        for (int g = tid; g <= G; g += nthr) tile_meta[1 + g] = mt_s[g];
    }
    // row-tile list: group g is written by workgroup g (mod grid), like the work-item tables below
    for (int g = tile; g < G; g += gridDim.x) {
        const int rows = g < E ? off_s[g + 1] - off_s[g] : T;
        const int nm = mt_s[g + 1] - mt_s[g];
        for (int mt = tid; mt < nm; mt += nthr) {
            omega_tile tl;
            tl.g = g;
            tl.row0 = (mt_s[g] + mt) * bm;
            tl.rows = min(bm, rows - mt * bm);
            tl.xrow0 = g < E ? -1 : mt * bm;
            tiles[mt_s[g] + mt] = tl;
        }
    }

    // ---- work-item tables of the two grouped products (bf16 layers) ----
    // (item_desc describes their order.)  Every workgroup writes a strided share of the entries; the product kernels
    // read the per-workgroup queues that the queue builders of this launch form from the same figures, the tables
    // serve what comes later (adding up the partial results of k slices).
    if (desc_up != nullptr || desc_down != nullptr) {
        const table_params tpu = {nt_up, ncols_up, 1, 0, 1}, tpd = {nt_down, ncols_down, ks_max_down, kt_down, tail_ks_down};
        const table_shape tsu(tpu, mt_s[G]), tsd(tpd, mt_s[G]);
        if (tile == 0 && tid == 0) {
            tile_meta[G + 2] = tsu.entries();
            tile_meta[G + 3] = tsd.entries();
            tile_meta[G + 7] = tsd.KS;
            // the k-sliced entries of the down table (their partial results are added up behind the product)
            tile_meta[G + 8] = tsd.KS > 1 ? 0 : tsd.Nt - tsd.r;
            tile_meta[G + 9] = tsd.KS > 1 ? tsd.Nt * tsd.KS : tsd.TKS > 1 ? tsd.r * tsd.TKS : 0;
        }
        if (desc_up != nullptr)
            for (int ent = tile * nthr + tid; ent < tsu.entries(); ent += n_tiles * nthr)
                desc_up[ent] = item_desc(ent, tpu, tsu, mt_s, off_s, E, G, T, bm);
        if (desc_down != nullptr)
            for (int ent = tile * nthr + tid; ent < tsd.entries(); ent += n_tiles * nthr)
                desc_down[ent] = item_desc(ent, tpd, tsd, mt_s, off_s, E, G, T, bm);
    }

    // ---- row copies (bf16 layers whose up product reads a gathered copy) ----
    if (xg != nullptr) {
        asm volatile("; the prefetched words are dropped here" ::"v"(prefetched));
        __syncthreads();  // sort_prow / sort_tok
        if (nt_stores) copy_tile_rows<true>(x, d, t0, min(tok_tile, T - t0), npairs, sort_prow, sort_tok, xg, xs);
        else copy_tile_rows<false>(x, d, t0, min(tok_tile, T - t0), npairs, sort_prow, sort_tok, xg, xs);
    }
}

// One wave per token; 16-byte chunks; up to 8 chunks in flight per lane.  PACKED: destination rows are in the
// packed tile image (chunk index = 4*kstep + c); when xs != nullptr, the token is also copied to row t of xs.
// NT: the rows are written with non-temporal stores, from half the last-level cache (256 MiB) of gathered rows on.
// 16384 tokens x 8 slots x 2048 (512 MiB): launch 0.204 -> 0.158 ms and the products that follow gain 2 %;
// 8192 x 6 x 2048 (192 MiB): launch 0.090 -> 0.073 ms, forward pass 1.332 -> 1.321 ms; 4096 x 2 x 4096 (64 MiB): launch
// -2.5 us, up product +3 us, the forward pass the same - left to the cache.
template <bool PACKED, bool NT>
__global__ __launch_bounds__(256) void dispatch_gather_kernel(const uint4 *__restrict__ x, const int32_t *__restrict__ dstp,
                                                              int T, int K, int chunks_per_row,
                                                              unsigned char *__restrict__ xg, unsigned char *__restrict__ xs)
{
    const int lane = threadIdx.x & 63;
    const int t = (int)blockIdx.x * 4 + (threadIdx.x >> 6);
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

// x != nullptr (bf16 layers): the workgroups also copy the rows of their token tiles into xg (and xs)
hipError_t launch_dispatch_index(const omega_moe *m, int T, int bm, hipStream_t s, const void *x)
{
    const omega_moe_config &c = m->cfg;
    const bool rows = x != nullptr && c.dtype == OMEGA_DTYPE_BF16;
    // from half the last-level cache of gathered rows on, the rows are written around it
    const int nt_stores = (size_t)T * c.K * c.d * 2 > OMEGA_LLC_BYTES / 2 ? 1 : 0;
    const int tok_tile = router_tok_tile(c.E);
    const int n_tiles = ceil_div(T, tok_tile);
    const int n_sched = m->desc_up != nullptr ? SCHED_WGS : 0;  // bf16 layers
    hipLaunchKernelGGL(dispatch_rank_kernel, dim3(n_tiles + n_sched), dim3(rows ? 1024 : 256), 0, s, m->ids, m->tile_counts, m->counts,
                       n_tiles, T, tok_tile, c.K, c.E, c.Es, bm, m->offsets, m->dst, m->dstp, m->src_row, m->tokp, m->tiles,
                       m->tile_meta, m->desc_up, c.H / 128, 128, m->desc_down, c.d / m->down_cols, m->down_cols,
                       m->down_ks_max, c.H / 32, m->down_tail_ks, m->wq_up, m->wq_down, m->n_wg, (const unsigned char *)x, c.d,
                       (unsigned char *)(rows ? m->xg : nullptr), (unsigned char *)(rows ? m->xs : nullptr), nt_stores, n_sched);
    return hipGetLastError();
}

hipError_t launch_dispatch_gather(const omega_moe *m, const void *x, int T, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const size_t row_bytes = (size_t)c.d * m->esize;
    if (c.dtype == OMEGA_DTYPE_BF16) {  // d % 256 == 0 is guaranteed at creation: rows are whole 64-byte k steps
        if ((size_t)T * c.K * row_bytes > OMEGA_LLC_BYTES / 2)
            hipLaunchKernelGGL((dispatch_gather_kernel<true, true>), dim3(ceil_div(T, 4)), dim3(256), 0, s, (const uint4 *)x,
                               m->dstp, T, c.K, (int)(row_bytes / 16), (unsigned char *)m->xg, (unsigned char *)m->xs);
        else
            hipLaunchKernelGGL((dispatch_gather_kernel<true, false>), dim3(ceil_div(T, 4)), dim3(256), 0, s, (const uint4 *)x,
                               m->dstp, T, c.K, (int)(row_bytes / 16), (unsigned char *)m->xg, (unsigned char *)m->xs);
    } else if (row_bytes % 16 == 0 && ((uintptr_t)x % 16) == 0) {
        hipLaunchKernelGGL((dispatch_gather_kernel<false, false>), dim3(ceil_div(T, 4)), dim3(256), 0, s, (const uint4 *)x,
                           m->dstp, T, c.K, (int)(row_bytes / 16), (unsigned char *)m->xg, (unsigned char *)nullptr);
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

__global__ __launch_bounds__(256) void bw_sched_kernel(sched_args sa)
{
    __shared__ __attribute__((aligned(16))) unsigned char scratch[SCHED_SCRATCH];
    const int pass = blockIdx.x >> 3, x = blockIdx.x & 7;
    const table_source src = {pass == 0 ? sa.desc[0] : pass == 1 ? sa.desc[1] : sa.desc[2],
                              pass == 0 ? sa.kcost[0] : pass == 1 ? sa.kcost[1] : sa.kcost[2]};
    const int total = sa.tile_meta[pass == 0 ? sa.total_slot[0] : pass == 1 ? sa.total_slot[1] : sa.total_slot[2]];
    schedule_queues(src, pass == 0 ? sa.wq[0] : pass == 1 ? sa.wq[1] : sa.wq[2], total, sa.n_wg, x, scratch);
}

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
