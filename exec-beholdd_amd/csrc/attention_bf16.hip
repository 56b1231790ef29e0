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

// NS = head_dim / 32.
// STREAM = one workgroup per (sequence, kv head, split): each cache byte is read once, past the caches.
template <int NS, bool STREAM>
__global__ __launch_bounds__(256) void attention_mfma_kernel(
    const uint16_t* __restrict__ q, uint16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, const uint16_t* __restrict__ k_pages, const uint16_t* __restrict__ v_pages,
    const int32_t* __restrict__ page_table, int table_stride, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ seq_start, int H, int KVH, float scale_log2, int window, int n_splits,
    int pages_per_split, int tile_groups) {
  constexpr int HD = 32 * NS;
  constexpr int CT = 1;   // column tiles per workgroup
  __shared__ float sm_m[4][16];
  __shared__ float sm_l[4][16];
  __shared__ float sm_o[4][16][HD + 1];

  const int tile_group = blockIdx.x % tile_groups, unit = blockIdx.x / tile_groups;
  const int tile0 = tile_group * CT, kvh = unit % KVH, z = unit / KVH;
  const int seq = z / n_splits, split = z % n_splits;
  const int G = H / KVH;
  const int row0 = seq_start[seq];
  const int n_cols = (seq_start[seq + 1] - row0) * G;
  if (tile0 * 16 >= n_cols) return;

  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int j = lane % 16, g = lane / 16;
  int pos[CT], lo[CT];
  bf16x8_t q_vec[CT][NS];
  int pos_max = 0, pos_min = 0x7fffffff, lo_min = 0x7fffffff, lo_max = 0;
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int wanted = (tile0 + ct) * 16 + j;
    const int c = wanted < n_cols ? wanted : n_cols - 1;
    const int row = row0 + c / G, head = kvh * G + c % G;
    pos[ct] = positions[row];
    lo[ct] = (window > 0 && pos[ct] - window + 1 > 0) ? pos[ct] - window + 1 : 0;
    pos_max = max(pos_max, pos[ct]);
    pos_min = min(pos_min, pos[ct]);
    lo_min = min(lo_min, lo[ct]);
    lo_max = max(lo_max, lo[ct]);
    const uint16_t* qp = q + ((size_t)row * H + head) * HD + 8 * g;
#pragma unroll
    for (int s = 0; s < NS; ++s) q_vec[ct][s] = as_bf16x8(load16(qp + 32 * s));
  }
  pos_max = wave_max_int(pos_max);
  pos_min = wave_min_int(pos_min);
  lo_min = wave_min_int(lo_min);
  lo_max = wave_max_int(lo_max);

  const int begin = lo_min / BH_PAGE + split * pages_per_split;
  const int last = pos_max / BH_PAGE;
  const int end = (begin + pages_per_split < last + 1) ? begin + pages_per_split : last + 1;
  const int32_t* table = page_table + (size_t)seq * table_stride;

  f32x4_t o[CT][2 * NS];
  float run_max[CT], run_sum[CT];  // run_sum: this lane's share of the column's sum
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    run_max[ct] = -INFINITY;
    run_sum[ct] = 0.f;
#pragma unroll
    for (int dt = 0; dt < 2 * NS; ++dt) o[ct][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  int page_ahead = (begin + wave < end) ? table[begin + wave] : 0;   // a page's number is asked for one page early
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
    const int key0 = p * BH_PAGE + 8 * g;  // lane (j, g) holds keys key0 + 32 * (t / 2) + 4 * (t % 2) + r
    const bool mask_needed = (p * BH_PAGE + BH_PAGE - 1 > pos_min) || (p * BH_PAGE < lo_max);
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      if (CT > 1 && (tile0 + ct) * 16 >= n_cols) continue;  // a tile beyond the sequence's columns
      f32x4_t st[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < NS; ++s)
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(k_vec[t][s]), q_vec[ct][s], acc, 0, 0, 0);
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
            if (key > pos[ct] || key < lo[ct]) st[t][r] = -INFINITY;
          }
      }
      float local_max = fmaxf(fmaxf(st[0][0], st[0][1]), fmaxf(st[0][2], st[0][3]));
#pragma unroll
      for (int t = 1; t < 4; ++t)
        local_max = fmaxf(local_max, fmaxf(fmaxf(st[t][0], st[t][1]), fmaxf(st[t][2], st[t][3])));
      local_max = fmaxf(local_max, __shfl_xor(local_max, 16, 64));
      local_max = fmaxf(local_max, __shfl_xor(local_max, 32, 64));
      const float new_max = fmaxf(run_max[ct], local_max);              // raw (unscaled) scores
      const float shift = (new_max == -INFINITY) ? 0.f : -new_max * scale_log2;
      // exactly 1 while the maximum stands still, 0 when nothing was seen before
      const float alpha = (run_max[ct] == new_max) ? 1.0f : __builtin_amdgcn_exp2f((run_max[ct] - new_max) * scale_log2);
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
      run_sum[ct] = run_sum[ct] * alpha + page_sum;
      run_max[ct] = new_max;
      const bool rescale = __any(alpha != 1.0f);   // after the first pages the maximum seldom moves
      if (ct == 0 && p * BH_PAGE + BH_PAGE - 1 > pos_max) {  // the page's tail was never written: zero it
        const int valid = pos_max + 1 - key0;
#pragma unroll
        for (int dt = 0; dt < 2 * NS; ++dt) {
          v_vec[dt][0] = keep_first(v_vec[dt][0], valid);
          v_vec[dt][1] = keep_first(v_vec[dt][1], valid - 32);
        }
      }
      if (rescale) {
#pragma unroll
        for (int dt = 0; dt < 2 * NS; ++dt) o[ct][dt] = o[ct][dt] * alpha;
      }
#pragma unroll
      for (int dt = 0; dt < 2 * NS; ++dt) {
        f32x4_t acc = o[ct][dt];
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(v_vec[dt][0]), as_bf16x8(p_vec[0]), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(v_vec[dt][1]), as_bf16x8(p_vec[1]), acc, 0, 0, 0);
        o[ct][dt] = acc;
      }
    }
  }

  // merge the four waves, one column tile after the other: lane (j, g) holds O^T[16dt + 4g + r, j]
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int tile = tile0 + ct;
    if (tile * 16 >= n_cols) break;
    float lane_sum = run_sum[ct];
    lane_sum += __shfl_xor(lane_sum, 16, 64);
    lane_sum += __shfl_xor(lane_sum, 32, 64);
    if (ct > 0) __syncthreads();  // the previous tile's merge has read the buffers
    if (g == 0) {
      sm_m[wave][j] = run_max[ct] * scale_log2;   // in units of the base-2 exponent, as the merges use it
      sm_l[wave][j] = lane_sum;
    }
#pragma unroll
    for (int dt = 0; dt < 2 * NS; ++dt)
#pragma unroll
      for (int r = 0; r < 4; ++r) sm_o[wave][j][16 * dt + 4 * g + r] = o[ct][dt][r];
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
      if (n_splits == 1) {
        out[column * HD + d] = f32_to_bf16_bits(value / sum);
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
// (maximum, sum) pairs side by side, and the partial outputs are fetched eight splits at a time.
__global__ void attention_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                         uint16_t* __restrict__ out, int n_splits, int HD) {
  const size_t column = blockIdx.x;
  const float* ml = part_ml + column * n_splits * 2;
  const int lane = threadIdx.x % BH_WAVE;
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
    for (int s0 = 0; s0 < n_splits; s0 += 8) {
      float weight[8], part[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int s = s0 + u < n_splits ? s0 + u : n_splits - 1;
        weight[u] = s0 + u < n_splits ? ml[2 * s] : -INFINITY;
        part[u] = part_o[(column * n_splits + s) * HD + d];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) value += part[u] * exp2f(weight[u] - top);
    }
    out[column * HD + d] = f32_to_bf16_bits(value * inv);
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
  // about one workgroup per compute unit (256), every wave of a workgroup at least one page
  if (tiles >= 256 || pages < 8) return 1;
  long want = (256 + tiles - 1) / tiles;
  if (want > pages / 4) want = pages / 4;
  if (want < 1) want = 1;
  const int per = (int)((pages + want - 1) / want);
  return (pages + per - 1) / per;
}

extern "C" int bh_attention_bf16(const void* q, void* out, void* part_o, void* part_ml, const void* k_pages,
                                 const void* v_pages, const int32_t* page_table, int table_stride,
                                 const int32_t* positions, const int32_t* seq_start, int n_seqs, int n_rows,
                                 int max_rows_per_seq, int H, int KVH, int hd, float scale, int window,
                                 int max_position, int n_splits, hipStream_t stream) {
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
  if (n_splits == 1 && (long)tiles * KVH * n_seqs >= 1024) {   // many columns: the prefill kernel
    bh_attention_prefill_launch(q, out, k_pages, v_pages, page_table, table_stride, positions, seq_start, n_seqs,
                                tiles, H, KVH, hd, scale_log2, window, stream);
    return bh_check_launch("attention_prefill_bf16");
  }
  const int tile_groups = tiles, z_count = n_seqs * n_splits;
  dim3 grid(tile_groups * KVH * z_count), block(256);
#define BH_ATT_ONE(NS, STREAM)                                                                                  \
  attention_mfma_kernel<NS, STREAM><<<grid, block, 0, stream>>>(                                                \
      (const uint16_t*)q, (uint16_t*)out, (float*)part_o, (float*)part_ml, (const uint16_t*)k_pages,            \
      (const uint16_t*)v_pages, page_table, table_stride, positions, seq_start, H, KVH, scale_log2, window,     \
      n_splits, per, tile_groups)
#define BH_ATT(NS)                               \
  do {                                           \
    if (tile_groups == 1) BH_ATT_ONE(NS, true);  \
    else BH_ATT_ONE(NS, false);                  \
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
    attention_combine_kernel<<<dim3(n_rows * H), dim3(hd >= 128 ? 128 : 64), 0, stream>>>(
        (const float*)part_o, (const float*)part_ml, (uint16_t*)out, n_splits, hd);
    return bh_check_launch("attention_combine");
  }
  return 0;
}
