// bfloat16 attention over the paged cache on the gfx950 matrix cores: the kernel for few columns per
// sequence (decode, short steps) and the entry point, which hands steps with many columns per sequence
// to the prefill kernel (attention_prefill_bf16.hip).
//
// A *column* is one (row, query head) pair.  A workgroup takes 16 columns that share a sequence
// and a kv head (consecutive rows x the heads of one group) and a range of that sequence's cache
// pages; its four waves take the pages of the range in turn.  For each page of 64 keys a wave
// computes, with v_mfma_f32_16x16x32_bf16,
//     S^T[key, column] = K[key, :] . Q[column, :]        (keys as rows: K is loaded straight from
//                                                          the cache in operand layout)
//     running maximum / sum per column in float32 (online softmax, exponent base 2)
//     O^T[d, column] += V^T[d, key] . P^T[key, column]   (the cache keeps V transposed inside a
//                                                          page, so this operand is a straight load too)
// The rows of an S^T tile are assigned to keys so that every lane ends up with the keys its P^T
// operand needs: tile t, row i <-> key 32*(t/2) + 4*(t%2) + 8*(i/4) + i%4.  Lane (column j, group g)
// then holds keys 8g..8g+7 (tiles 0, 1) and 32+8g..32+8g+7 (tiles 2, 3): the k-slices of the two
// P.V products of a page, whose V^T operands are 16 contiguous bytes per lane and 64 contiguous
// bytes per row and instruction.  The same holds for K along head_dim.
// The waves' results are merged through LDS.  When the keys of a sequence are split over several
// workgroups (decode: few columns, long caches) each writes an unnormalised partial result and
// its (maximum, sum) to scratch memory and a second kernel combines them.  (Letting the last
// workgroup combine, behind a device-wide fence and an arrival counter, was measured: the fences
// write back the L2 of every workgroup's XCD and cost several times what the second launch costs.)
//
// head_dim must be a multiple of 32, at most 256.  Masking is by position: column j sees keys
// lo_j .. pos_j.  Rows of a page beyond the last written key are never multiplied in: their
// probabilities are zero and their V values are zeroed before use.
#include "attention_bf16.h"

// A decode step can hand the kernel the fused projection rows themselves (struct FusedQkv) instead of
// finished queries and a cache that already holds the new keys: every workgroup then norms and rotates
// its own queries, and one wave of the sequence's last split norms and rotates the new key, treats it and
// the new value as one more page of a single visible key, and writes both into the cache for the steps
// to come.  The keys that come from the cache end one position earlier.  This takes the place of the
// launch of the norm/rotation/cache-write kernel.
struct FusedQkv {
  const uint16_t* qkv;      // [rows][(H + 2 KVH) * head_dim], one row per sequence; null: queries and cache are ready
  const void* q_weight;     // per-head RMSNorm weights [head_dim], or null for no norm
  const void* k_weight;
  int weight_f32;           // their element type: float32, else bfloat16
  float eps;
  const float* cos_table;   // [positions][head_dim / 2]: rotation over the whole head, or null for none
  const float* sin_table;
  int write_kv;             // 0: the cache entry belongs to another layer, which has written the new key already
  uint16_t* k_pages;        // the cache again, to write into
  uint16_t* v_pages;
};

// What a lane needs to norm and rotate its share of a head (elements 32 s + 8 g + e; the other three g share
// the head): asked for early (`ask`), used late (`apply`), so that the loads of the first cache page can be
// under way in between.
template <int NS>
struct HeadPrep {
  static constexpr int HD = 32 * NS, HS = NS / 2;
  u32x4_t weight_raw[NS][2];   // bfloat16 weights fill the first of each pair, float32 both
  float cos_v[HS > 0 ? HS : 1][8], sin_v[HS > 0 ? HS : 1][8];

  __device__ inline void ask(const void* weight, int weight_f32, const float* cos_table, const float* sin_table,
                             int pos, int g) {
    if (weight != nullptr) {
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        const int i = 32 * s + 8 * g;
        if (weight_f32) {
          weight_raw[s][0] = *reinterpret_cast<const u32x4_t*>(reinterpret_cast<const float*>(weight) + i);
          weight_raw[s][1] = *reinterpret_cast<const u32x4_t*>(reinterpret_cast<const float*>(weight) + i + 4);
        } else {
          weight_raw[s][0] = load16(reinterpret_cast<const uint16_t*>(weight) + i);
        }
      }
    }
    if (cos_table != nullptr) {
#pragma unroll
      for (int s = 0; s < HS; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int i = 32 * s + 8 * g + e;
          cos_v[s][e] = cos_table[(size_t)pos * (HD / 2) + i];
          sin_v[s][e] = sin_table[(size_t)pos * (HD / 2) + i];
        }
    }
  }

  // RMSNorm over the head, then split-half rotation: the partner of element i < HD / 2 is i + HD / 2, in the
  // same lane, HS slices on.
  __device__ inline void apply(float (&x)[NS][8], bool with_weight, int weight_f32, float eps, bool with_rotation) const {
    if (with_weight) {
      float ss = 0.f;
#pragma unroll
      for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += x[s][e] * x[s][e];
      ss += __shfl_xor(ss, 16, 64);
      ss += __shfl_xor(ss, 32, 64);
      const float inv = 1.0f / sqrtf(ss / (float)HD + eps);
#pragma unroll
      for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float w = weight_f32 ? __uint_as_float(weight_raw[s][e / 4][e % 4])
                                     : bf16_bits_to_f32((uint16_t)(weight_raw[s][0][e / 2] >> (16 * (e % 2))));
          x[s][e] = x[s][e] * inv * w;
        }
    }
    if (with_rotation) {
#pragma unroll
      for (int s = 0; s < HS; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float lo = x[s][e], hi = x[s + HS][e];
          x[s][e] = lo * cos_v[s][e] - hi * sin_v[s][e];
          x[s + HS][e] = lo * sin_v[s][e] + hi * cos_v[s][e];
        }
    }
  }
};

template <int NS>
__device__ inline void widen_head(float (&x)[NS][8], const u32x4_t (&raw)[NS]) {
#pragma unroll
  for (int s = 0; s < NS; ++s)
#pragma unroll
    for (int e = 0; e < 8; ++e) x[s][e] = bf16_bits_to_f32((uint16_t)(raw[s][e / 2] >> (16 * (e % 2))));
}

template <int NS>
__device__ inline void pack_head(u32x4_t (&out)[NS], const float (&x)[NS][8]) {
#pragma unroll
  for (int s = 0; s < NS; ++s)
#pragma unroll
    for (int word = 0; word < 4; ++word) out[s][word] = pack_bf16(x[s][2 * word], x[s][2 * word + 1]);
}

// NS = head_dim / 32.
// STREAM = one workgroup per (sequence, kv head, split): each cache byte is read once, past the caches.
// FUSED = the step is a decode step and `fused.qkv` is given.
// LEAN (with FUSED) = the queries are normed and rotated before the first page is asked for, and the new key's
// numbers are asked for after the last page: nothing of that overlaps with the pages any more, but what it needs
// in registers is gone while the pages stream, so that two workgroups fit a compute unit.  For launches of more
// workgroups than compute units, where the second workgroup is worth more than the overlap.
template <int NS, bool STREAM, bool FUSED, bool LEAN = false>
__global__ __launch_bounds__(256, (LEAN ? 2 : 1)) void attention_mfma_kernel(
    const uint16_t* __restrict__ q, uint16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, const uint16_t* __restrict__ k_pages, const uint16_t* __restrict__ v_pages,
    const int32_t* __restrict__ page_table, int table_stride, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ seq_start, int H, int KVH, float scale_log2, int window, int n_splits,
    int pages_per_split, int tile_groups, FusedQkv fused, int out_block_rows) {
  constexpr int HD = 32 * NS;
  __shared__ float sm_m[4][16];
  __shared__ float sm_l[4][16];
  __shared__ float sm_o[4][16][HD + 1];

  const int tile = blockIdx.x % tile_groups, unit = blockIdx.x / tile_groups;
  const int kvh = unit % KVH, z = unit / KVH;
  const int seq = z / n_splits, split = z % n_splits;
  const int G = H / KVH;
  // FUSED is a decode step: sequence s has the one row s, and nobody waits for `seq_start` to say so
  const int row0 = FUSED ? seq : seq_start[seq];
  const int n_cols = FUSED ? G : (seq_start[seq + 1] - row0) * G;
  if (tile * 16 >= n_cols) return;
  // The number of this wave's first page, if no window cuts the front off, is asked for beside the row's position
  // instead of after it: one trip to memory less before the first key is on its way.
  const int32_t* table = page_table + (size_t)seq * table_stride;
  const int first_guess = split * pages_per_split + (int)(threadIdx.x / 64);
  const int page_guess = first_guess < table_stride ? table[first_guess] : 0;

  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int j = lane % 16, g = lane / 16;
  const int wanted = tile * 16 + j;
  const int c = wanted < n_cols ? wanted : n_cols - 1;
  const int row = row0 + c / G, head = kvh * G + c % G;
  const int pos_row = positions[row];                   // the row's own position
  const bool new_key_apart = FUSED && fused.write_kv;   // the key at pos_row is not in the cache yet
  const int pos = new_key_apart ? pos_row - 1 : pos_row;   // the last key the row takes from the cache (-1: none)
  const int lo = (window > 0 && pos_row - window + 1 > 0) ? pos_row - window + 1 : 0;
  bf16x8_t q_vec[NS];
  // FUSED: the raw rows and what norms and rotates them are asked for here and used once the first page's
  // loads are under way (q) and after the pages (the new key and value).
  u32x4_t q_raw[NS], k_raw[NS];
  uint16_t new_value[2 * NS];   // dim 16 dt + j of the new value
  HeadPrep<NS> q_prep, k_prep;
  bool q_ready = !FUSED;
  const bool takes_new_key = FUSED && fused.write_kv && split == n_splits - 1 && wave == 0;
  auto ask_new_key = [&]() {   // one row per sequence: every lane's row is this row
    const uint16_t* qkv_row = fused.qkv + (size_t)row * (H + 2 * KVH) * HD;
#pragma unroll
    for (int s = 0; s < NS; ++s) k_raw[s] = load16(qkv_row + (size_t)(H + kvh) * HD + 32 * s + 8 * g);
#pragma unroll
    for (int dt = 0; dt < 2 * NS; ++dt) new_value[dt] = qkv_row[(size_t)(H + KVH + kvh) * HD + 16 * dt + j];
    // the rotation's numbers are q's, or (LEAN: q's are gone by then) asked for again
    k_prep.ask(fused.k_weight, fused.weight_f32, LEAN ? fused.cos_table : nullptr, LEAN ? fused.sin_table : nullptr, pos_row, g);
  };
  if (FUSED) {
    const uint16_t* qkv_row = fused.qkv + (size_t)row * (H + 2 * KVH) * HD;
#pragma unroll
    for (int s = 0; s < NS; ++s) q_raw[s] = load16(qkv_row + (size_t)head * HD + 32 * s + 8 * g);
    q_prep.ask(fused.q_weight, fused.weight_f32, fused.cos_table, fused.sin_table, pos_row, g);
    if (takes_new_key && !LEAN) ask_new_key();
  } else {
    const uint16_t* qp = q + ((size_t)row * H + head) * HD + 8 * g;
#pragma unroll
    for (int s = 0; s < NS; ++s) q_vec[s] = as_bf16x8(load16(qp + 32 * s));
  }
  auto finish_q = [&]() {
    float x[NS][8];
    widen_head<NS>(x, q_raw);
    q_prep.apply(x, fused.q_weight != nullptr, fused.weight_f32, fused.eps, fused.cos_table != nullptr);
    u32x4_t packed[NS];
    pack_head<NS>(packed, x);
#pragma unroll
    for (int s = 0; s < NS; ++s) q_vec[s] = as_bf16x8(packed[s]);
    q_ready = true;
  };
  if (FUSED && LEAN) finish_q();
  const int pos_max = wave_max_int(pos), pos_min = wave_min_int(pos);
  const int lo_min = wave_min_int(lo), lo_max = wave_max_int(lo);

  const int begin = lo_min / BH_PAGE + split * pages_per_split;
  const int last = pos_max >= 0 ? pos_max / BH_PAGE : -1;
  const int end = (begin + pages_per_split < last + 1) ? begin + pages_per_split : last + 1;

  f32x4_t o[2 * NS];
  float run_max = -INFINITY, run_sum = 0.f;  // run_sum: this lane's share of the column's sum
#pragma unroll
  for (int dt = 0; dt < 2 * NS; ++dt) o[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // One page of keys and values in operand order against the 16 columns: lane (j, g) holds keys
  // 64 p + 8 g + 32 (t / 2) + 4 (t % 2) + r.  A column sees keys see_lo .. see_hi; the bounds over the
  // wave say whether anything has to be masked at all.
  auto attend = [&](const u32x4_t (&k_vec)[4][NS], u32x4_t (&v_vec)[2 * NS][2], int p, int see_hi, int see_lo,
                    int hi_max, int hi_min, int lo_most) {
    const int key0 = p * BH_PAGE + 8 * g;
    const bool mask_needed = (p * BH_PAGE + BH_PAGE - 1 > hi_min) || (p * BH_PAGE < lo_most);
    f32x4_t st[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < NS; ++s)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(k_vec[t][s]), q_vec[s], acc, 0, 0, 0);
      st[t] = acc;
    }
    // Online softmax with few instructions: the maximum is taken over the raw scores, the scale
    // enters through one fused multiply-add per score, and the exponentials are bare v_exp_f32
    // (arguments <= 0; results below the normal range may flush to zero).
    if (mask_needed) {
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int key = key0 + 32 * (t / 2) + 4 * (t % 2) + r;
          if (key > see_hi || key < see_lo) st[t][r] = -INFINITY;
        }
    }
    float local_max = fmaxf(fmaxf(st[0][0], st[0][1]), fmaxf(st[0][2], st[0][3]));
#pragma unroll
    for (int t = 1; t < 4; ++t)
      local_max = fmaxf(local_max, fmaxf(fmaxf(st[t][0], st[t][1]), fmaxf(st[t][2], st[t][3])));
    local_max = fmaxf(local_max, __shfl_xor(local_max, 16, 64));
    local_max = fmaxf(local_max, __shfl_xor(local_max, 32, 64));
    const float new_max = fmaxf(run_max, local_max);              // raw (unscaled) scores
    const float shift = (new_max == -INFINITY) ? 0.f : -new_max * scale_log2;
    // exactly 1 while the maximum stands still, 0 when nothing was seen before
    const float alpha = (run_max == new_max) ? 1.0f : __builtin_amdgcn_exp2f((run_max - new_max) * scale_log2);
    float page_sum = 0.f;
    u32x4_t p_vec[2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int t = 2 * u + half;
        const float e0 = __builtin_amdgcn_exp2f(fmaf(st[t][0], scale_log2, shift));
        const float e1 = __builtin_amdgcn_exp2f(fmaf(st[t][1], scale_log2, shift));
        const float e2 = __builtin_amdgcn_exp2f(fmaf(st[t][2], scale_log2, shift));
        const float e3 = __builtin_amdgcn_exp2f(fmaf(st[t][3], scale_log2, shift));
        page_sum += (e0 + e1) + (e2 + e3);
        p_vec[u][2 * half] = pack_bf16(e0, e1);
        p_vec[u][2 * half + 1] = pack_bf16(e2, e3);
      }
    run_sum = run_sum * alpha + page_sum;
    run_max = new_max;
    if (p * BH_PAGE + BH_PAGE - 1 > hi_max) {  // the page's tail was never written: zero it
      const int valid = hi_max + 1 - key0;
#pragma unroll
      for (int dt = 0; dt < 2 * NS; ++dt) {
        v_vec[dt][0] = keep_first(v_vec[dt][0], valid);
        v_vec[dt][1] = keep_first(v_vec[dt][1], valid - 32);
      }
    }
    if (__any(alpha != 1.0f)) {   // after the first pages the maximum seldom moves
#pragma unroll
      for (int dt = 0; dt < 2 * NS; ++dt) o[dt] = o[dt] * alpha;
    }
#pragma unroll
    for (int dt = 0; dt < 2 * NS; ++dt) {
      f32x4_t acc = o[dt];
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(v_vec[dt][0]), as_bf16x8(p_vec[0]), acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(v_vec[dt][1]), as_bf16x8(p_vec[1]), acc, 0, 0, 0);
      o[dt] = acc;
    }
  };

  // a page's number is asked for one page early
  int page_ahead = (begin + wave < end) ? (begin + wave == first_guess ? page_guess : table[begin + wave]) : 0;
  for (int p = begin + wave; p < end; p += 4) {
    const int page = page_ahead;
    if (p + 4 < end) page_ahead = table[p + 4];
    const uint16_t* kb = k_pages + ((size_t)page * KVH + kvh) * BH_PAGE * HD;
    const uint16_t* vb = v_pages + ((size_t)page * KVH + kvh) * HD * BH_PAGE;
    u32x4_t k_vec[4][NS], v_vec[2 * NS][2];
    // the cache lies in pieces (BH_KV_PIECES): every load instruction covers 1 KB of contiguous memory
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int s = 0; s < NS; ++s) k_vec[t][s] = load16_cache<STREAM>(kb + ((t * NS + s) * 64 + lane) * 8);
#pragma unroll
    for (int dt = 0; dt < 2 * NS; ++dt) {
      v_vec[dt][0] = load16_cache<STREAM>(vb + ((dt * 2) * 64 + lane) * 8);
      v_vec[dt][1] = load16_cache<STREAM>(vb + ((dt * 2 + 1) * 64 + lane) * 8);
    }
    if (FUSED && !q_ready) finish_q();   // under the page's loads
    attend(k_vec, v_vec, p, pos, lo, pos_max, pos_min, lo_max);
  }

  if (takes_new_key) {
    // The new key and value of this (sequence, kv head): normed and rotated here, attended to as a page in
    // which only their own slot is visible, and written into the cache.
    if (!q_ready) finish_q();
    if (LEAN) ask_new_key();
    float x[NS][8];
    widen_head<NS>(x, k_raw);
    if (!LEAN) {
#pragma unroll
      for (int s = 0; s < HeadPrep<NS>::HS; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          k_prep.cos_v[s][e] = q_prep.cos_v[s][e];
          k_prep.sin_v[s][e] = q_prep.sin_v[s][e];
        }
    }
    k_prep.apply(x, fused.k_weight != nullptr, fused.weight_f32, fused.eps, fused.cos_table != nullptr);
    u32x4_t new_key[NS];
    pack_head<NS>(new_key, x);
    const int token = pos_row % BH_PAGE;
    const int token_t = 2 * (token / 32) + (token / 4) % 2, token_j = 4 * ((token / 8) % 4) + token % 4;
    const int token_u = token / 32, token_g = (token % 32) / 8, token_w = token % 8;
    const u32x4_t zero = {0u, 0u, 0u, 0u};
    u32x4_t k_vec[4][NS], v_vec[2 * NS][2];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int s = 0; s < NS; ++s) k_vec[t][s] = (t == token_t && j == token_j) ? new_key[s] : zero;
#pragma unroll
    for (int dt = 0; dt < 2 * NS; ++dt) {
      u32x4_t piece = zero;
      piece[token_w / 2] = (uint32_t)new_value[dt] << (16 * (token_w % 2));
      v_vec[dt][0] = (token_u == 0 && g == token_g) ? piece : zero;
      v_vec[dt][1] = (token_u == 1 && g == token_g) ? piece : zero;
    }
    attend(k_vec, v_vec, pos_row / BH_PAGE, pos_row, pos_row, pos_row, pos_row, pos_row);
    const int page = table[pos_row / BH_PAGE];
    uint16_t* kb = fused.k_pages + ((size_t)page * KVH + kvh) * BH_PAGE * HD;
    uint16_t* vb = fused.v_pages + ((size_t)page * KVH + kvh) * HD * BH_PAGE;
    if (j == 0) {
#pragma unroll
      for (int s = 0; s < NS; ++s)
        *reinterpret_cast<u32x4_t*>(kb + ((token_t * NS + s) * 64 + 16 * g + token_j) * 8) = new_key[s];
    }
    if (g == 0) {
#pragma unroll
      for (int dt = 0; dt < 2 * NS; ++dt) vb[bh_value_index(BH_KV_PIECES, token, 16 * dt + j, HD)] = new_value[dt];
    }
  }

  // merge the four waves: lane (j, g) holds O^T[16dt + 4g + r, j]
  {
    float lane_sum = run_sum;
    lane_sum += __shfl_xor(lane_sum, 16, 64);
    lane_sum += __shfl_xor(lane_sum, 32, 64);
    if (g == 0) {
      sm_m[wave][j] = run_max * scale_log2;   // in units of the base-2 exponent, as the merges use it
      sm_l[wave][j] = lane_sum;
    }
#pragma unroll
    for (int dt = 0; dt < 2 * NS; ++dt)
#pragma unroll
      for (int r = 0; r < 4; ++r) sm_o[wave][j][16 * dt + 4 * g + r] = o[dt][r];
    __syncthreads();
    for (int e = threadIdx.x; e < 16 * HD; e += 256) {
      const int col = e / HD, d = e % HD;
      const int cc = tile * 16 + col;
      if (cc >= n_cols) continue;
      float top = fmaxf(fmaxf(sm_m[0][col], sm_m[1][col]), fmaxf(sm_m[2][col], sm_m[3][col]));
      const float safe_top = (top == -INFINITY) ? 0.f : top;
      float sum = 0.f, value = 0.f;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float f = exp2f(sm_m[v][col] - safe_top);
        sum += sm_l[v][col] * f;
        value += sm_o[v][col][d] * f;
      }
      const size_t column = (size_t)(row0 + cc / G) * H + kvh * G + cc % G;
      if (n_splits == 1) {   // out_block_rows: the output [rows][H * HD] lies in blocks of that many rows (bh_rows_index)
        out[bh_rows_index(out_block_rows, row0 + cc / G, (kvh * G + cc % G) * HD + d, H * HD)] = f32_to_bf16_bits(value / sum);
      } else {
        part_o[(column * n_splits + split) * HD + d] = value;
        if (d == 0) {
          part_ml[(column * n_splits + split) * 2] = top;
          part_ml[(column * n_splits + split) * 2 + 1] = sum;
        }
      }
    }
  }
}

// One block per column.  Nothing here may wait for one split's numbers before asking for the next
// one's: with 32 splits that is 32 trips to the L2 in a row.  So the lanes of a wave fetch the splits'
// (maximum, sum) pairs side by side, and the partial outputs are fetched WIDTH splits at a time (8, or 4 where there are
// no more); the sums run over the splits in their order either way.
template <int WIDTH>
__global__ void attention_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                         uint16_t* __restrict__ out, int n_splits, int HD, int H, int out_block_rows) {
  const size_t column = blockIdx.x;
  const float* ml = part_ml + column * n_splits * 2;
  const int lane = threadIdx.x % BH_WAVE;
  // the first splits' outputs are asked for beside the maxima and sums, not after them
  float first_part[WIDTH];
#pragma unroll
  for (int u = 0; u < WIDTH; ++u)
    first_part[u] = threadIdx.x < HD ? part_o[(column * n_splits + (u < n_splits ? u : n_splits - 1)) * HD + threadIdx.x] : 0.f;
  float top = -INFINITY;
  for (int s = lane; s < n_splits; s += BH_WAVE) top = fmaxf(top, ml[2 * s]);
#pragma unroll
  for (int off = BH_WAVE / 2; off > 0; off >>= 1) top = fmaxf(top, __shfl_xor(top, off, BH_WAVE));
  float sum = 0.f;   // in the order: each lane its splits upwards, then the lanes pairwise
  for (int s = lane; s < n_splits; s += BH_WAVE) sum += ml[2 * s + 1] * exp2f(ml[2 * s] - top);
#pragma unroll
  for (int off = BH_WAVE / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off, BH_WAVE);
  const float inv = 1.0f / sum;
  for (int d = threadIdx.x; d < HD; d += blockDim.x) {
    float value = 0.f;
    for (int s0 = 0; s0 < n_splits; s0 += WIDTH) {
      float weight[WIDTH], part[WIDTH];
#pragma unroll
      for (int u = 0; u < WIDTH; ++u) {
        const int s = s0 + u < n_splits ? s0 + u : n_splits - 1;
        weight[u] = s0 + u < n_splits ? ml[2 * s] : -INFINITY;
        part[u] = (s0 == 0 && d == threadIdx.x) ? first_part[u] : part_o[(column * n_splits + s) * HD + d];
      }
#pragma unroll
      for (int u = 0; u < WIDTH; ++u) value += part[u] * exp2f(weight[u] - top);
    }
    out[bh_rows_index(out_block_rows, (int)(column / H), (int)(column % H) * HD + d, H * HD)] = f32_to_bf16_bits(value * inv);
  }
}

// The order of a cache page's elements that the kernels of this library expect for a cache of the
// given element type and head size: the writer, the attention for any size and this file's agree on it.
extern "C" int bh_kv_order(int dtype, int hd) {
  return (dtype == BH_BF16 && hd % 32 == 0 && hd >= 32 && hd <= 256) ? BH_KV_PIECES : BH_KV_ROWS;
}

// How many ways the keys are split for a given launch; the caller sizes the scratch from it.
extern "C" int bh_attention_bf16_splits(int n_seqs, int max_rows_per_seq, int H, int KVH, int max_position) {
  if (n_seqs <= 0 || max_rows_per_seq <= 0 || H <= 0 || KVH <= 0 || H % KVH) return 1;
  const int G = H / KVH;
  const long tiles = (long)((max_rows_per_seq * G + 15) / 16) * KVH * n_seqs;
  const int pages = max_position / BH_PAGE + 1;
  // Every wave of a workgroup at least one page.  The workgroups run in rounds of one per compute unit (256 on an
  // MI355X), so what a launch costs is its rounds times a workgroup's pages (and about four pages' worth of start and
  // merge): the split count with the least of that, the smaller one among equals.  One workgroup per compute unit or
  // just beyond, as it was before, made 288 to 384 workgroups of 9 to 14 and of 17 to 24 sequences: two rounds of
  // nearly whole-sized workgroups (decode steps of the Qwen3-8B shape at context 8,192, 8 layers: 6 sequences 1.18 ->
  // 1.11 ms, 10 1.48 -> 1.40, 12 1.63 -> 1.48, 20 2.18 -> 2.02, 24 2.23 -> 2.19; 8, 16 and 32 sequences as before).
  const int units = bh_compute_units();
  if (pages < 8) return 1;
  long want = 1, least = -1;
  if (tiles > units) {
    // More workgroups than compute units: two of the lean kernel's share a compute unit.  Just above one per compute
    // unit (and just above two) the few compute units that carry one more hold the launch up, and three (two) splits
    // spread the pages evenly; from about 1.4 per compute unit on the whole workgroups are as fast or faster
    // (Qwen3-8B shape, context 8,192, 8 layers, ms per step with 1 / 2 / 3 / 4 / 6 splits: 33 sequences 3.04 / 2.80 / 2.72 /
    // 2.69 / 2.66, 40: 3.20 / 2.92 / 2.89 / 2.90 / 2.91, 48: 3.27 / 3.35 / 3.25 / 3.25 / 3.25, 56: 3.66 / 3.75 / 3.75 / 3.69 /
    // 3.73, 72: 4.55 / 4.43 / 4.43 / 4.52 / 4.54).
    const double each_unit = (double)tiles / units;
    want = each_unit < 1.4 ? 3 : (each_unit > 2.0 && each_unit < 2.4) ? 2 : 1;
    if (want > pages / 4) want = pages / 4;
  } else {
    for (long splits = 1; splits <= pages / 4 && splits <= 64; ++splits) {
      const long rounds = (tiles * splits + units - 1) / units, each = (pages + splits - 1) / splits;
      const long cost = rounds * (each + 4);
      if (least < 0 || cost < least) least = cost, want = splits;
    }
  }
  const int per = (int)((pages + want - 1) / want);
  return (pages + per - 1) / per;
}

#define PREFILL_FROM_TILES 1024   // column tiles x kv heads x sequences from which the prefill kernel runs a step
// Whether a step of these sizes goes to the kernel for many columns per sequence, which writes its output in rows
// or in blocks of 16 rows x 32 columns (bh_blocked_index); the other steps' kernels write blocks of 8 or 16 rows.
extern "C" int bh_attention_bf16_writes_blocked(int n_seqs, int max_rows_per_seq, int H, int KVH, int max_position) {
  if (n_seqs <= 0 || max_rows_per_seq <= 0 || H <= 0 || KVH <= 0 || H % KVH) return 0;
  const long tiles = (long)((max_rows_per_seq * (H / KVH) + 15) / 16) * KVH * n_seqs;
  return bh_attention_bf16_splits(n_seqs, max_rows_per_seq, H, KVH, max_position) == 1 && tiles >= PREFILL_FROM_TILES ? 1 : 0;
}

static int attention_bf16_run(const void* q, void* out, void* part_o, void* part_ml, const void* k_pages,
                              const void* v_pages, const int32_t* page_table, int table_stride,
                              const int32_t* positions, const int32_t* seq_start, int n_seqs, int n_rows,
                              int max_rows_per_seq, int H, int KVH, int hd, float scale, int window,
                              int max_position, int n_splits, const FusedQkv& fused, int out_blocked,
                              hipStream_t stream) {
  BH_REQUIRE(n_seqs > 0 && n_rows > 0 && max_rows_per_seq > 0, "attention_bf16: empty batch");
  BH_REQUIRE(H > 0 && KVH > 0 && H % KVH == 0, "attention_bf16: %d query heads do not group evenly into %d kv heads", H, KVH);
  BH_REQUIRE(hd % 32 == 0 && hd >= 32 && hd <= 256, "attention_bf16: head size %d is not a multiple of 32 up to 256", hd);
  BH_REQUIRE(window >= 0 && max_position >= 0, "attention_bf16: window and positions must not be negative");
  BH_REQUIRE(n_splits >= 1 && (n_splits == 1 || (part_o && part_ml)), "attention_bf16: split keys need scratch memory");
  const int G = H / KVH;
  const int tiles = (max_rows_per_seq * G + 15) / 16;
  const int pages = max_position / BH_PAGE + 1;
  const int per = (pages + n_splits - 1) / n_splits;
  const float scale_log2 = scale * 1.4426950408889634f;
  BH_REQUIRE((long)tiles * KVH * n_seqs * n_splits < (1L << 31), "attention_bf16: too many workgroups");
  const bool is_fused = fused.qkv != nullptr;
  BH_REQUIRE(!is_fused || (tiles == 1 && max_rows_per_seq == 1 && n_rows == n_seqs),
             "attention_bf16: the fused projection rows are taken in decode steps of at most 16 heads per kv head only");
  if (!is_fused && n_splits == 1 && (long)tiles * KVH * n_seqs >= PREFILL_FROM_TILES) {   // many columns: the prefill kernel
    BH_REQUIRE(out_blocked == 0 || out_blocked == 16, "attention_bf16: a step of many columns writes rows or blocks of 16 rows, not of %d", out_blocked);
    bh_attention_prefill_launch(q, out, k_pages, v_pages, page_table, table_stride, positions, seq_start, n_seqs,
                                tiles, H, KVH, hd, scale_log2, window, out_blocked == 16, stream);
    return bh_check_launch("attention_prefill_bf16");
  }
  BH_REQUIRE(out_blocked == 0 || ((out_blocked == 8 || out_blocked == 16) && (H * hd) % 32 == 0),
             "attention_bf16: the output's rows lie in blocks of 8 or 16, or one after the other (0), not %d", out_blocked);
  const int tile_groups = tiles, z_count = n_seqs * n_splits;
  const bool lean = (long)tiles * KVH * z_count > bh_compute_units();   // more workgroups than compute units: two of them per unit
  dim3 grid(tile_groups * KVH * z_count), block(256);
#define BH_ATT_ONE(NS, STREAM, FUSED, ...)                                                                      \
  attention_mfma_kernel<NS, STREAM, FUSED, ##__VA_ARGS__><<<grid, block, 0, stream>>>(                          \
      (const uint16_t*)q, (uint16_t*)out, (float*)part_o, (float*)part_ml, (const uint16_t*)k_pages,            \
      (const uint16_t*)v_pages, page_table, table_stride, positions, seq_start, H, KVH, scale_log2, window,     \
      n_splits, per, tile_groups, fused, out_blocked)
#define BH_ATT(NS)                                      \
  do {                                                  \
    if (is_fused && lean && NS <= 4) BH_ATT_ONE(NS, true, true, (NS <= 4));   \
    else if (is_fused) BH_ATT_ONE(NS, true, true);      \
    else if (tile_groups == 1) BH_ATT_ONE(NS, true, false);  \
    else BH_ATT_ONE(NS, false, false);                  \
  } while (0)
  switch (hd / 32) {
    case 1: BH_ATT(1); break;
    case 2: BH_ATT(2); break;
    case 3: BH_ATT(3); break;
    case 4: BH_ATT(4); break;
    case 5: BH_ATT(5); break;
    case 6: BH_ATT(6); break;
    case 7: BH_ATT(7); break;
    default: BH_ATT(8); break;
  }
#undef BH_ATT
#undef BH_ATT_ONE
  if (int status = bh_check_launch("attention_mfma")) return status;
  if (n_splits > 1) {
    const dim3 columns(n_rows * H), threads(hd >= 128 ? 128 : 64);
    if (n_splits <= 4)
      attention_combine_kernel<4><<<columns, threads, 0, stream>>>((const float*)part_o, (const float*)part_ml, (uint16_t*)out,
                                                                   n_splits, hd, H, out_blocked);
    else
      attention_combine_kernel<8><<<columns, threads, 0, stream>>>((const float*)part_o, (const float*)part_ml, (uint16_t*)out,
                                                                   n_splits, hd, H, out_blocked);
    return bh_check_launch("attention_combine");
  }
  return 0;
}

extern "C" int bh_attention_bf16(const void* q, void* out, void* part_o, void* part_ml, const void* k_pages,
                                 const void* v_pages, const int32_t* page_table, int table_stride,
                                 const int32_t* positions, const int32_t* seq_start, int n_seqs, int n_rows,
                                 int max_rows_per_seq, int H, int KVH, int hd, float scale, int window,
                                 int max_position, int n_splits, int out_blocked, hipStream_t stream) {
  const FusedQkv none = {nullptr, nullptr, nullptr, 0, 0.f, nullptr, nullptr, 0, nullptr, nullptr};
  return attention_bf16_run(q, out, part_o, part_ml, k_pages, v_pages, page_table, table_stride, positions,
                            seq_start, n_seqs, n_rows, max_rows_per_seq, H, KVH, hd, scale, window, max_position,
                            n_splits, none, out_blocked, stream);
}

// A decode step (one row per sequence) straight from the fused projection rows [q heads | k heads | v heads]:
// per-head RMSNorm of q and k (weights may be null), rotation over the whole head at the row's position
// (tables may be null), the new key and value into the cache (unless write_kv is 0: the entry is another
// layer's), and attention over the cache and the new key.  See struct FusedQkv.  Row s is sequence s's: `seq_start`
// can only say so (0, 1, ..., n_seqs) and is not read.
extern "C" int bh_attention_decode_fused(const void* qkv, void* out, void* part_o, void* part_ml, void* k_pages,
                                         void* v_pages, const int32_t* page_table, int table_stride,
                                         const int32_t* positions, const int32_t* seq_start, int n_seqs, int H,
                                         int KVH, int hd, float scale, int window, int max_position, int n_splits,
                                         const void* q_weight, const void* k_weight, int w_dtype, float eps,
                                         const float* cos_table, const float* sin_table, int table_positions,
                                         int rot, int write_kv, int out_block_rows, hipStream_t stream) {
  BH_REQUIRE(qkv != nullptr, "attention_decode_fused: the projection rows are required");
  BH_REQUIRE((q_weight == nullptr) == (k_weight == nullptr), "attention_decode_fused: give both norm weights or neither");
  BH_REQUIRE(q_weight == nullptr || w_dtype == BH_F32 || w_dtype == BH_BF16, "attention_decode_fused: unknown weight dtype %d", w_dtype);
  BH_REQUIRE((cos_table == nullptr) == (sin_table == nullptr), "attention_decode_fused: cos and sin tables come together");
  BH_REQUIRE(cos_table == nullptr || (rot == hd && hd % 64 == 0),
             "attention_decode_fused: the rotation must span the whole head (%d of %d) and the head be a multiple of 64", rot, hd);
  BH_REQUIRE(cos_table == nullptr || max_position < table_positions,
             "attention_decode_fused: position %d is outside the rotation table of %d positions", max_position, table_positions);
  const FusedQkv fused = {(const uint16_t*)qkv, q_weight, k_weight, w_dtype == BH_F32, eps, cos_table, sin_table,
                          write_kv, (uint16_t*)k_pages, (uint16_t*)v_pages};
  return attention_bf16_run(nullptr, out, part_o, part_ml, k_pages, v_pages, page_table, table_stride, positions,
                            seq_start, n_seqs, n_seqs, 1, H, KVH, hd, scale, window, max_position, n_splits, fused,
                            out_block_rows, stream);
}
