// Packed "tile image" layout of the bf16 operands of the grouped products (weights, xg, a).
//
// A matrix with R rows (R a multiple of 128) and Kd columns (a multiple of 32) is stored as 1 KiB blocks of
// 16 rows x 32 columns, ordered [row group of 128][k step of 32][block of 16 rows]; inside a block, row r and
// 16-byte chunk c (8 columns) sit at (r % 16) * 64 + ((c ^ swz(r)) * 16).  A block is exactly what one
// wave-wide direct global->LDS load of the product kernels moves, already in the bank-conflict-free LDS
// order, so those loads read 1 KiB of contiguous memory instead of sixteen 64-byte row pieces.
#pragma once
#include <stdint.h>

// chunk swizzle: conflict-free operand reads for 8 consecutive rows on 32 LDS banks and 16 rows on 64 banks
__host__ __device__ static inline int pk_swz(int row) { return ((row >> 1) ^ (row >> 3)) & 3; }

// byte offset of the 16-byte chunk (row, k step kb, chunk c) in a packed matrix with KT k steps
__host__ __device__ static inline size_t pk_chunk_off(int row, int kb, int c, int KT)
{
    return ((((size_t)(row >> 7) * KT + kb) * 8 + ((row & 127) >> 4)) << 10) + ((row & 15) << 6) + ((c ^ pk_swz(row)) << 4);
}
