// Dispatch: per-expert counts, prefix scan, stable permutation, row-tile list, coalesced row gather.
//
// Pair p = t*K+j goes to row dst[p] = offsets[id_p] + #{q<p : id_q == id_p} of the expert-contiguous
// buffer (a stable counting sort of the pair list by expert id); src_row[dst[p]] = t.
// The router left one histogram row per 32-token tile in tile_counts[tile][e].  Three launches:
//   scan    one workgroup per 8 experts: exclusive prefix over the tiles of each expert (tile_base) and
//           the per-expert totals -> counts[e]
//   rank    one workgroup per token tile: offsets = exclusive scan of counts; rank of each pair among the
//           earlier pairs of its tile with the same expert; dst/src_row; workgroup 0 also publishes
//           offsets and the row-tile list that schedules the grouped products
//   gather  one wave per token: the row of x is read once and written to its K destination rows with
//           16-byte accesses (gather semantics as img_token_drop,
//           J/engine/nn/layer/dit/kernel/TokenDropKernel.cu:147-160)
// No global atomics anywhere, so counts, offsets and the permutation are deterministic.
#include "common.h"

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
                                                            int32_t *__restrict__ dst, int32_t *__restrict__ src_row,
                                                            omega_tile *__restrict__ tiles,
                                                            int32_t *__restrict__ tile_meta)
{
    __shared__ int off_s[MAXE + 1];
    __shared__ int id_s[TOK_TILE * 64];   // K <= 64
    __shared__ int mt_off[MAXE + 64 + 1];
    const int tid = threadIdx.x, tile = blockIdx.x;
    const int t0 = tile * TOK_TILE;
    const int npairs = min(TOK_TILE, T - t0) * K;

    // exclusive scan of the E counts: one wave, 4 experts per lane
    if (tid < 64) {
        int c[4], run = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid * 4 + i;
            c[i] = e < E ? counts[e] : 0;
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
            const int e = tid * 4 + i;
            if (e < E) off_s[e] = ex;
            ex += c[i];
        }
        if (tid == 63) off_s[E] = incl;  // counts beyond E are zero, so lane 63 holds the grand total
    }
    for (int i = tid; i < npairs; i += 256) id_s[i] = ids[(size_t)t0 * K + i];
    __syncthreads();

    for (int i = tid; i < npairs; i += 256) {
        const int e = id_s[i];
        int rank = 0;
        for (int q = 0; q < i; ++q) rank += (id_s[q] == e) ? 1 : 0;
        const int r = off_s[e] + tile_base[(size_t)tile * E + e] + rank;
        dst[(size_t)t0 * K + i] = r;
        src_row[r] = t0 + i / K;
    }

    if (tile == 0) {
        for (int e = tid; e <= E; e += 256) offsets[e] = off_s[e];
        const int G = E + Es;
        if (tid == 0) {
            int run = 0;
            for (int g = 0; g < G; ++g) {
                mt_off[g] = run;
                const int rows = g < E ? off_s[g + 1] - off_s[g] : T;
                run += (rows + bm - 1) / bm;
            }
            mt_off[G] = run;
            tile_meta[0] = run;
        }
        __syncthreads();
        const int P = T * K;
        for (int g = 0; g < G; ++g) {
            const int rows = g < E ? off_s[g + 1] - off_s[g] : T;
            const int row0 = g < E ? off_s[g] : P + (g - E) * T;
            const int nm = (rows + bm - 1) / bm;
            for (int mt = tid; mt < nm; mt += 256) {
                omega_tile tl;
                tl.g = g;
                tl.row0 = row0 + mt * bm;
                tl.rows = min(bm, rows - mt * bm);
                tl.xrow0 = g < E ? -1 : mt * bm;
                tiles[mt_off[g] + mt] = tl;
            }
        }
        for (int g = tid; g <= G; g += 256) tile_meta[1 + g] = mt_off[g];
    }
}

// One wave per token; 16-byte chunks; up to 8 chunks in flight per lane.
__global__ __launch_bounds__(256) void dispatch_gather_kernel(const uint4 *__restrict__ x, const int32_t *__restrict__ dst,
                                                              int T, int K, int chunks_per_row,
                                                              uint4 *__restrict__ xg)
{
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= T) return;
    const uint4 *src = x + (size_t)t * chunks_per_row;
    for (int c0 = 0; c0 < chunks_per_row; c0 += 64 * 8) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int c = c0 + u * 64 + lane;
            if (c < chunks_per_row) v[u] = src[c];
        }
        for (int j = 0; j < K; ++j) {
            uint4 *out = xg + (size_t)dst[(size_t)t * K + j] * chunks_per_row;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int c = c0 + u * 64 + lane;
                if (c < chunks_per_row) out[c] = v[u];
            }
        }
    }
}

// Fallback for rows that are not a multiple of 16 bytes: element-wise copy.
__global__ __launch_bounds__(256) void dispatch_gather_bytes_kernel(const unsigned char *__restrict__ x,
                                                                    const int32_t *__restrict__ dst, int T, int K,
                                                                    size_t row_bytes, unsigned char *__restrict__ xg)
{
    const int t = blockIdx.x;
    for (int j = 0; j < K; ++j) {
        unsigned char *out = xg + (size_t)dst[(size_t)t * K + j] * row_bytes;
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
                       c.E, c.Es, bm, m->offsets, m->dst, m->src_row, m->tiles, m->tile_meta);
    return hipGetLastError();
}

hipError_t launch_dispatch_gather(const omega_moe *m, const void *x, int T, hipStream_t s)
{
    const omega_moe_config &c = m->cfg;
    const size_t row_bytes = (size_t)c.d * m->esize;
    if (row_bytes % 16 == 0 && ((uintptr_t)x % 16) == 0) {
        hipLaunchKernelGGL(dispatch_gather_kernel, dim3(ceil_div(T, 4)), dim3(256), 0, s, (const uint4 *)x, m->dst, T,
                           c.K, (int)(row_bytes / 16), (uint4 *)m->xg);
    } else {
        hipLaunchKernelGGL(dispatch_gather_bytes_kernel, dim3(T), dim3(256), 0, s, (const unsigned char *)x, m->dst, T,
                           c.K, row_bytes, (unsigned char *)m->xg);
    }
    return hipGetLastError();
}
