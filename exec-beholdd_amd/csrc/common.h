// Shared definitions of the gfx950 kernel library: element types, conversions, wave and
// block reductions, error reporting.  Wavefronts are 64 lanes wide throughout.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "layout.h"

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
// The compute units of the GPU that is current when it is first asked (256 on an MI355X): what launch plans count
// workgroups against.  Where no GPU is visible (a byte plan made on another machine) it says 256.
int bh_compute_units();

#define BH_REQUIRE(cond, ...)                  \
  do {                                         \
    if (!(cond)) return bh_fail(__VA_ARGS__);  \
  } while (0)

// The cache of one layer as the kernels see it: pages of BH_PAGE tokens found through a
// per-sequence page table.  Keys lie [page][kv_head][token in page][head_dim]; values lie
// transposed, [page][kv_head][head_dim][token in page], so that a matrix-core operand of
// "head_dim rows x consecutive tokens" is a contiguous load.
