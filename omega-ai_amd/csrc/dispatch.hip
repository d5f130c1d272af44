// Dispatch: per-expert counts, prefix scan, stable permutation, row-tile list, coalesced row gather.
//
// Pair p = t*K+j goes to logical row dst[p] = offsets[id_p] + #{q<p : id_q == id_p} of the expert-contiguous
// order (a stable counting sort of the pair list by expert id); src_row[dst[p]] = t.  In the buffers the
// experts' segments start on row-tile boundaries (physical row dstp[p] = first_tile[id_p]*bm + rank).
// The router left one histogram row per 32-token tile in tile_counts[tile][e].  Three launches:
//   scan    one workgroup per 8 experts: exclusive prefix over the tiles of each expert (tile_base) and
//           the per-expert totals -> counts[e]
//   rank    one workgroup per token tile: offsets = exclusive scan of counts, first_tile = exclusive scan of
//           ceil(counts/bm); rank of each pair among the earlier pairs of its tile with the same expert;
//           dst/dstp/src_row; workgroup 0 also publishes offsets and the row-tile list that schedules the
//           grouped products
//   gather  one wave per token: the row of x is read once with 16-byte accesses and written to its K
//           destination rows (gather semantics as img_token_drop,
//           J/engine/nn/layer/dit/kernel/TokenDropKernel.cu:147-160); fp32 layers keep rows contiguous,
//           bf16 layers write the packed tile image the product kernels load (pack.h)
// No global atomics anywhere, so counts, offsets and the permutation are deterministic.
#include "common.h"
#include "pack.h"

#define TOK_TILE ROUTER_TOK_TILE
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

// MAXE: experts are limited to 256 per layer by the router kernels.
#define MAXE 256
__global__ __launch_bounds__(256) void dispatch_rank_kernel(const int32_t *__restrict__ ids,
                                                            const int32_t *__restrict__ tile_base,
                                                            const int32_t *__restrict__ counts, int T, int K, int E,
                                                            int Es, int bm, int32_t *__restrict__ offsets,
                                                            int32_t *__restrict__ dst, int32_t *__restrict__ dstp,
                                                            int32_t *__restrict__ src_row,
                                                            omega_tile *__restrict__ tiles,
                                                            int32_t *__restrict__ tile_meta,
                                                            omega_tile_desc *__restrict__ desc_up, int nt_up, int ncols_up,
                                                            omega_tile_desc *__restrict__ desc_down, int nt_down,
                                                            int ncols_down)
{
    __shared__ int off_s[MAXE + 1];        // logical first row of each expert
    __shared__ int mt_s[MAXE + 64 + 1];    // first row tile of each group (routed, then shared)
    __shared__ int id_s[TOK_TILE * 64];    // K <= 64
    const int tid = threadIdx.x, tile = blockIdx.x;
    const int t0 = tile * TOK_TILE;
    const int npairs = min(TOK_TILE, T - t0) * K;

    // exclusive scans of the E counts and of their tile counts: one wave, 4 experts per lane
    if (tid < 64) {
        int c[4], run = 0, runt = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid * 4 + i;
            c[i] = e < E ? counts[e] : 0;
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
    for (int i = tid; i < npairs; i += 256) id_s[i] = ids[(size_t)t0 * K + i];
    __syncthreads();

    for (int i = tid; i < npairs; i += 256) {
        const int e = id_s[i];
        int rank = 0;
        for (int q = 0; q < i; ++q) rank += (id_s[q] == e) ? 1 : 0;
        rank += tile_base[(size_t)tile * E + e];
        const int r = off_s[e] + rank;
        dst[(size_t)t0 * K + i] = r;
        dstp[(size_t)t0 * K + i] = mt_s[e] * bm + rank;
        src_row[r] = t0 + i / K;
    }

    if (tile == 0) {
        for (int e = tid; e <= E; e += 256) offsets[e] = off_s[e];
        const int G = E + Es;
        for (int g = 0; g < G; ++g) {
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
        if (tid == 0) tile_meta[0] = mt_s[G];
        for (int g = tid; g <= G; g += 256) tile_meta[1 + g] = mt_s[g];
    }

    // ---- work-item tables of the two grouped products (bf16 layers) ----
    // Tile number first_tile[g]*NT + n*Mg + m = (expert g, column tile n, row tile m): row tiles fastest, so that
    // tiles that run at the same time share weight tiles.  The compute units take 256 tiles at a time; when the
    // last r = Nt mod 256 tiles would occupy at most half of them, each of those tiles is cut into S = 2 or 4
    // slices of bm/S rows (adjacent entries, so that the slices of a tile run side by side on one XCD and share
    // the weight tile in its L2).  Group g is written by workgroup g (mod grid).
    if (desc_up != nullptr || desc_down != nullptr) {
        const int G = E + Es;
        if (tile == 0 && tid < 2) {
            const int Nt = mt_s[G] * (tid == 0 ? nt_up : nt_down), r = Nt % 256;
            const int S = (r == 0 || r > 128) ? 1 : (r > 64 ? 2 : 4);
            tile_meta[G + 2 + tid] = Nt - r + r * S;
        }
        for (int g = tile; g < G; g += gridDim.x) {
            const int rows = g < E ? off_s[g + 1] - off_s[g] : T;
            const int Mg = mt_s[g + 1] - mt_s[g];
            for (int pass = 0; pass < 2; ++pass) {
                omega_tile_desc *desc = pass == 0 ? desc_up : desc_down;
                const int NT = pass == 0 ? nt_up : nt_down, ncols = pass == 0 ? ncols_up : ncols_down;
                if (desc == nullptr) continue;
                const int Nt = mt_s[G] * NT, r = Nt % 256;
                const int S = (r == 0 || r > 128) ? 1 : (r > 64 ? 2 : 4);
                for (int l = tid; l < Mg * NT; l += 256) {
                    const int mt = l % Mg, n = l / Mg;
                    const int at = mt_s[g] * NT + l;
                    const int trows = min(bm, rows - mt * bm);
                    omega_tile_desc dsc;
                    dsc.g = g;
                    dsc.n0 = n * ncols;
                    dsc.pad[0] = dsc.pad[1] = dsc.pad[2] = 0;
                    if (at < Nt - r) {
                        dsc.row0 = (mt_s[g] + mt) * bm;
                        dsc.rows = trows;
                        dsc.xrow0 = g < E ? -1 : mt * bm;
                        desc[at] = dsc;
                    } else {
                        const int slice = bm / S;
                        for (int sl = 0; sl < S; ++sl) {
                            dsc.row0 = (mt_s[g] + mt) * bm + sl * slice;
                            dsc.rows = max(0, min(slice, trows - sl * slice));  // 0: nothing to do
                            dsc.xrow0 = g < E ? -1 : mt * bm + sl * slice;
                            desc[Nt - r + (at - (Nt - r)) * S + sl] = dsc;
                        }
                    }
                }
            }
        }
    }
}

// One wave per token; 16-byte chunks; up to 8 chunks in flight per lane.  PACKED: destination rows are in the
// packed tile image (chunk index = 4*kstep + c) and, when xs != nullptr, the token is also copied to row t of xs.
template <bool PACKED>
__global__ __launch_bounds__(256) void dispatch_gather_kernel(const uint4 *__restrict__ x, const int32_t *__restrict__ dstp,
                                                              int T, int K, int chunks_per_row,
                                                              unsigned char *__restrict__ xg, unsigned char *__restrict__ xs)
{
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= T) return;
    const uint4 *src = x + (size_t)t * chunks_per_row;
    const int KT = chunks_per_row >> 2;
    for (int c0 = 0; c0 < chunks_per_row; c0 += 64 * 8) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int c = c0 + u * 64 + lane;
            if (c < chunks_per_row) v[u] = src[c];
        }
        const int nd = K + ((PACKED && xs != nullptr) ? 1 : 0);
        for (int j = 0; j < nd; ++j) {
            const int prow = j < K ? dstp[(size_t)t * K + j] : t;
            unsigned char *base = j < K ? xg : xs;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int c = c0 + u * 64 + lane;
                if (c < chunks_per_row) {
                    if (PACKED) *(uint4 *)(base + pk_chunk_off(prow, c >> 2, c & 3, KT)) = v[u];
                    else *(uint4 *)(base + ((size_t)prow * chunks_per_row + c) * 16) = v[u];
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

hipError_t launch_dispatch_index(const omega_moe *m, int T, int bm, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const int n_tiles = ceil_div(T, TOK_TILE);
    hipLaunchKernelGGL(dispatch_scan_kernel, dim3(ceil_div(c.E, SCAN_EC)), dim3(256), 0, s, m->tile_counts,
                       m->tile_base, n_tiles, c.E, m->counts);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(dispatch_rank_kernel, dim3(n_tiles), dim3(256), 0, s, m->ids, m->tile_base, m->counts, T, c.K,
                       c.E, c.Es, bm, m->offsets, m->dst, m->dstp, m->src_row, m->tiles, m->tile_meta, m->desc_up, c.H / 128, 128,
                       m->desc_down, c.d / 256, 256);
    return hipGetLastError();
}

hipError_t launch_dispatch_gather(const omega_moe *m, const void *x, int T, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const size_t row_bytes = (size_t)c.d * m->esize;
    if (c.dtype == OMEGA_DTYPE_BF16) {  // d % 256 == 0 is guaranteed at creation: rows are whole 64-byte k steps
        hipLaunchKernelGGL(dispatch_gather_kernel<true>, dim3(ceil_div(T, 4)), dim3(256), 0, s, (const uint4 *)x, m->dstp,
                           T, c.K, (int)(row_bytes / 16), (unsigned char *)m->xg, (unsigned char *)m->xs);
    } else if (row_bytes % 16 == 0 && ((uintptr_t)x % 16) == 0) {
        hipLaunchKernelGGL(dispatch_gather_kernel<false>, dim3(ceil_div(T, 4)), dim3(256), 0, s, (const uint4 *)x,
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
