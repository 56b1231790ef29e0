// Shared definitions of the gfx950 kernel library: element types, conversions, wave and
// block reductions, error reporting.  Wavefronts are 64 lanes wide throughout.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

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

__host__ __device__ inline int bh_key_index(int order, int token, int dim, int hd) {
  if (order == BH_KV_ROWS) return token * hd + dim;
  const int t = 2 * (token / 32) + (token / 4) % 2, j = 4 * ((token / 8) % 4) + token % 4;
  const int s = dim / 32, g = (dim % 32) / 8;
  return (((t * (hd / 32) + s) * 64) + 16 * g + j) * 8 + dim % 8;
}

__host__ __device__ inline int bh_value_index(int order, int token, int dim, int hd) {
  if (order == BH_KV_ROWS) return dim * BH_PAGE + token;
  const int dt = dim / 16, j = dim % 16, u = token / 32, g = (token % 32) / 8;
  return (((dt * 2 + u) * 64) + 16 * g + j) * 8 + token % 8;
}

// bfloat16 kept as its 16 bits; widening is a shift, narrowing rounds to nearest even.
struct bf16_t {
  uint16_t bits;
};

__host__ __device__ inline float bf16_bits_to_f32(uint16_t bits) {
  union {
    uint32_t u;
    float f;
  } v;
  v.u = ((uint32_t)bits) << 16;
  return v.f;
}

__host__ __device__ inline uint16_t f32_to_bf16_bits(float f) {
  union {
    uint32_t u;
    float f;
  } v;
  v.f = f;
  if ((v.u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((v.u >> 16) | 0x0040u);  // quiet NaN
  uint32_t rounding = 0x7fffu + ((v.u >> 16) & 1u);
  return (uint16_t)((v.u + rounding) >> 16);
}

__device__ inline float to_f32(float x) { return x; }
__device__ inline float to_f32(bf16_t x) { return bf16_bits_to_f32(x.bits); }

template <typename T>
__device__ inline T from_f32(float x);
template <>
__device__ inline float from_f32<float>(float x) {
  return x;
}
template <>
__device__ inline bf16_t from_f32<bf16_t>(float x) {
  bf16_t r;
  r.bits = f32_to_bf16_bits(x);
  return r;
}

// ---- reductions -------------------------------------------------------------------------

__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int off = BH_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, BH_WAVE);
  return v;
}

__device__ inline float wave_max(float v) {
#pragma unroll
  for (int off = BH_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, BH_WAVE));
  return v;
}

// Block-wide sum; `scratch` holds at least blockDim.x / 64 floats.  Every thread gets the result.
__device__ inline float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (BH_WAVE - 1), wave = threadIdx.x / BH_WAVE;
  const int n_waves = (blockDim.x + BH_WAVE - 1) / BH_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int i = 0; i < n_waves; ++i) total += scratch[i];
  return total;
}

__device__ inline float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (BH_WAVE - 1), wave = threadIdx.x / BH_WAVE;
  const int n_waves = (blockDim.x + BH_WAVE - 1) / BH_WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int i = 1; i < n_waves; ++i) total = fmaxf(total, scratch[i]);
  return total;
}

// ---- errors ------------------------------------------------------------------------------

// Every entry point returns 0 on success; otherwise bh_last_error() gives the reason.
int bh_fail(const char* format, ...);
int bh_check_launch(const char* what);

#define BH_REQUIRE(cond, ...)                  \
  do {                                         \
    if (!(cond)) return bh_fail(__VA_ARGS__);  \
  } while (0)

// The cache of one layer as the kernels see it: pages of BH_PAGE tokens found through a
// per-sequence page table.  Keys lie [page][kv_head][token in page][head_dim]; values lie
// transposed, [page][kv_head][head_dim][token in page], so that a matrix-core operand of
// "head_dim rows x consecutive tokens" is a contiguous load.
