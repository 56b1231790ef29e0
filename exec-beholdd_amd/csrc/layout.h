// What the device code and the plain host twins (plain_twins.cpp) share: sizes, the order of a cache page's
// elements, and bfloat16 as its 16 bits.  Compiles with and without HIP.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define BH_BOTH __host__ __device__
#else
#define BH_BOTH
#endif

#define BH_WAVE 64
#define BH_PAGE 64  // tokens in one page of the key/value cache

enum BhDtype { BH_F32 = 0, BH_BF16 = 1 };

// ---- order of the elements of one head within one cache page --------------------------------
// A page holds, for each kv head, BH_PAGE x head_dim keys and as many values.
// BH_KV_ROWS:   keys [token][dim], values transposed [dim][token].
// BH_KV_PIECES: regrouped in pieces of 8 elements (16 bytes) the way the matrix-core attention
//               kernel takes them, so that each of its loads (64 lanes x 16 bytes) covers 1 KB of
//               contiguous memory.  Lane l = 16 g + j of a load holds
//               keys:   piece ((t * head_dim/32 + s) * 64 + l): token 32 (t/2) + 4 (t%2) + 8 (j/4) + j%4,
//                       dims 32 s + 8 g .. + 7                       (t < 4, s < head_dim/32)
//               values: piece ((dt * 2 + u) * 64 + l): dim 16 dt + j, tokens 32 u + 8 g .. + 7
//                                                                       (dt < head_dim/16, u < 2)
//               Needs head_dim to be a multiple of 32.
enum BhKvOrder { BH_KV_ROWS = 0, BH_KV_PIECES = 1 };

BH_BOTH inline int bh_key_index(int order, int token, int dim, int hd) {
  if (order == BH_KV_ROWS) return token * hd + dim;
  const int t = 2 * (token / 32) + (token / 4) % 2, j = 4 * ((token / 8) % 4) + token % 4;
  const int s = dim / 32, g = (dim % 32) / 8;
  return (((t * (hd / 32) + s) * 64) + 16 * g + j) * 8 + dim % 8;
}

BH_BOTH inline int bh_value_index(int order, int token, int dim, int hd) {
  if (order == BH_KV_ROWS) return dim * BH_PAGE + token;
  const int dt = dim / 16, j = dim % 16, u = token / 32, g = (token % 32) / 8;
  return (((dt * 2 + u) * 64) + 16 * g + j) * 8 + token % 8;
}

// ---- activation rows in blocks ---------------------------------------------------------------
// A bfloat16 matrix [rows][width] that a product of many rows reads as its activations may be kept in
// blocks of 16 rows x 32 columns, each 1 KB in the order in which one matrix-core operand lies in a
// wave's lanes: lane 16 q + r holds row r of the block, columns 8 q .. 8 q + 7.  The blocks of 16 rows
// follow each other along the width, then down the rows.  A wave then takes an operand with one load of
// contiguous memory instead of 64 bytes from each of 16 rows.  Needs width to be a multiple of 32; the
// buffer holds whole blocks (rows rounded up; the products of many rows read whole tiles of
// BH_BLOCKED_ROWS_PAD rows).  Steps of at most 8 rows use blocks of 8 rows instead (the same order with 8 in
// the place of 16: 512 bytes, of which the product of few rows reads each 16-byte piece into two lanes).
#define BH_BLOCKED_ROWS_PAD 256
BH_BOTH inline long bh_blocked_index_of(int block_rows, int row, int column, int width) {
  return ((long)(row / block_rows) * (width / 32) + column / 32) * (32 * block_rows) +
         (((column % 32) / 8) * block_rows + row % block_rows) * 8 + column % 8;
}
BH_BOTH inline long bh_blocked_index(int row, int column, int width) { return bh_blocked_index_of(16, row, column, width); }
// Where element (row, column) of a matrix lies whose rows are in blocks of `block_rows` (8 or 16), or one after
// the other (0).
BH_BOTH inline long bh_rows_index(int block_rows, int row, int column, int width) {
  return block_rows ? bh_blocked_index_of(block_rows, row, column, width) : (long)row * width + column;
}

// bfloat16 kept as its 16 bits; widening is a shift, narrowing rounds to nearest even.
struct bf16_t {
  uint16_t bits;
};

BH_BOTH inline float bf16_bits_to_f32(uint16_t bits) {
  union {
    uint32_t u;
    float f;
  } v;
  v.u = ((uint32_t)bits) << 16;
  return v.f;
}

BH_BOTH inline uint16_t f32_to_bf16_bits(float f) {
  union {
    uint32_t u;
    float f;
  } v;
  v.f = f;
  if ((v.u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((v.u >> 16) | 0x0040u);  // quiet NaN
  uint32_t rounding = 0x7fffu + ((v.u >> 16) & 1u);
  return (uint16_t)((v.u + rounding) >> 16);
}

