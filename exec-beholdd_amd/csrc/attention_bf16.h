// What the two bfloat16 attention files share: vector types, small helpers, and the launcher of the
// prefill kernel (attention_prefill_bf16.hip) that bh_attention_bf16 (attention_bf16.hip) hands wide steps to.
#pragma once
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__device__ inline bf16x8_t as_bf16x8(u32x4_t v) { return __builtin_bit_cast(bf16x8_t, v); }
__device__ inline u32x4_t load16(const uint16_t* p) { return *reinterpret_cast<const u32x4_t*>(p); }
template <bool STREAM>
__device__ inline u32x4_t load16_cache(const uint16_t* p) {   // STREAM: nobody else reads these bytes soon
  if (STREAM) return __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  return *reinterpret_cast<const u32x4_t*>(p);
}

__device__ inline int wave_max_int(int v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = max(v, __shfl_xor(v, off, 64));
  return v;
}
__device__ inline int wave_min_int(int v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = min(v, __shfl_xor(v, off, 64));
  return v;
}

typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

// two float32 values rounded to nearest-even bfloat16 and packed (one v_cvt_pk_bf16_f32)
__device__ inline uint32_t pack_bf16(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// keep the first `n_valid` (0..8) bfloat16 elements of a 16-byte vector, zero the rest
__device__ inline u32x4_t keep_first(u32x4_t v, int n_valid) {
#pragma unroll
  for (int word = 0; word < 4; ++word) {
    const uint32_t mask = (2 * word + 1 < n_valid) ? 0xffffffffu : (2 * word < n_valid ? 0x0000ffffu : 0u);
    v[word] &= mask;
  }
  return v;
}

// Many columns per sequence (prefill): see attention_prefill_bf16.hip.  The caller has checked the sizes.
// out_blocked: the output [rows][H * hd] goes out in blocks of 16 rows x 32 columns (bh_blocked_index).
void bh_attention_prefill_launch(const void* q, void* out, const void* k_pages, const void* v_pages,
                                 const int32_t* page_table, int table_stride, const int32_t* positions,
                                 const int32_t* seq_start, int n_seqs, int tiles, int H, int KVH, int hd,
                                 float scale_log2, int window, int out_blocked, hipStream_t stream);
