// bfloat16 attention for steps with many rows per sequence (prefill), on the gfx950 matrix cores.
//
// The decode kernel (attention_bf16.hip) gives every wave of a workgroup different cache pages and the
// same columns, and merges the waves at the end: right for few columns and long caches.  Here it is
// the other way round.  A workgroup takes 64 * CTW columns of one (sequence, kv head); each of its
// four waves owns CTW tiles of 16 columns for the whole kernel (its queries, running maximum and sum,
// output accumulators), and all four walk over the same cache pages.  A page's keys and values are
// brought into LDS once per workgroup (by loads that write LDS directly, the next page while the current
// one is multiplied) and every wave reads its matrix-core operands from there: the cache keeps a page in
// 16-byte pieces in exactly the order the lanes take them (BH_KV_PIECES), so the copy is linear and
// the LDS reads are conflict-free.  Nothing is merged at the end, a wave holds accumulators for its
// own columns only, and two workgroups fit a compute unit at head size 128.
//
// Products, softmax and masking are those of the decode kernel:
//     S^T[key, column] = K[key, :] . Q[column, :],   tile t, row i <-> key 32 (t/2) + 4 (t%2) + 8 (i/4) + i%4
//     online softmax per column in float32, exponent base 2
//     O^T[d, column] += V^T[d, key] . P^T[key, column]
// The walk over a page is bound by the vector instructions of the softmax, not by the products (counters: the
// vector units busy 57 % of the kernel's time, the matrix cores 38 %), so they are kept few: the maximum by
// v_maximum3_f32 (three numbers an instruction, no quieting of each score first as fmaxf needs), over the four
// lanes of a column by two row exchanges between registers instead of two shuffles through LDS, the sum of the
// probabilities by one more row of the value product, a page's operands asked of LDS in two goes ahead of
// the arithmetic that hides the wait, and the exponentials' reference moved (and the sums so far scaled) only
// when the maximum has grown by more than 2^8.  Measured, one sequence at 32 query and 8 kv heads of 128:
// 2,048 rows 72 -> 60 us, 4,096 rows 194 -> 166 us, 8,192 rows 604 -> 533 us.  With two column tiles a wave, one
// tile's softmax stands between the matrix instructions of the other (and the score products start from a constant
// instead of cleared registers): 56.5, 160 and 513 us.  Counters at 8,192 rows (SQ_VALU_MFMA_BUSY_CYCLES,
// SQ_ACTIVE_INST_VALU, SQ_VALU_MFMA_COEXEC_CYCLES): the matrix cores are busy half of the time and so is the vector
// issue port (three vector instructions per matrix instruction, the exponentials counting double), both at once
// a tenth of it.
// A wave skips pages none of whose keys any of its columns may see.  Values beyond the last position
// of the workgroup's columns are zeroed in LDS before the last page is used (their probabilities are
// zero, but what lies there may be anything).
#include "attention_bf16.h"
#include <type_traits>

// The larger of two numbers, a NaN if either is one (v_maximum3_f32, which takes its operands as they are; fmaxf
// has to make each of them a quiet number first, one more instruction per score).
__device__ inline float larger(float a, float b) { return __builtin_elementwise_maximum(a, b); }

// The largest of the values that the lanes j, 16 + j, 32 + j and 48 + j hold, in all four of them, by two
// exchanges of rows between registers (no trip through LDS as a shuffle takes): the first leaves rows 0 and 2 in
// one register and rows 1 and 3 in the other, each twice; the second the lower and the upper half.
__device__ inline float largest_of_column(float x) {
  const auto rows = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  const float pairs = larger(__uint_as_float(rows[0]), __uint_as_float(rows[1]));
  const auto halves = __builtin_amdgcn_permlane32_swap(__float_as_uint(pairs), __float_as_uint(pairs), false, false);
  return larger(__uint_as_float(halves[0]), __uint_as_float(halves[1]));
}

template <int NS, int CTW>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(NS <= 4 ? 2 : 1))) void attention_prefill_kernel(
    const uint16_t* __restrict__ q, uint16_t* __restrict__ out, const uint16_t* __restrict__ k_pages,
    const uint16_t* __restrict__ v_pages, const int32_t* __restrict__ page_table, int table_stride,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_start, int H, int KVH,
    float scale_log2, int window, int tile_groups, int n_seqs, int out_blocked) {
  constexpr int HD = 32 * NS;
  constexpr int PIECES = BH_PAGE * HD / 8;        // 16-byte pieces of one head's keys (or values) in a page
  constexpr int STAGE = 2 * PIECES / 256;         // pieces of a page (keys, then values) one thread copies
  constexpr int GROUP_TILES = 4 * CTW;            // column tiles of a workgroup
  constexpr float SLACK = 8.0f;
  __shared__ u32x4_t page_lds[2][2 * PIECES];

  // Workgroups go to the eight XCDs in turn, each with an L2 of its own: when the number of
  // (kv head, sequence) units allows it, all tile groups of a unit run on one XCD, one after the other,
  // so that the unit's keys and values stay in that L2; and the groups with the most keys (the last
  // rows of a causal prefill) start first.  (Handing them out so that the two workgroups of a compute unit carry
  // the same number of pages together, the heaviest with the lightest, changed nothing at 2,048 or 4,096 rows: there
  // the kernel takes as long as its heaviest workgroup alone, 1.8 us a page.)
  int tile_group, unit;
  const int units = KVH * n_seqs;
  if (units % 8 == 0) {
    const int xcd = blockIdx.x % 8, turn = blockIdx.x / 8;
    tile_group = tile_groups - 1 - turn % tile_groups;
    unit = (turn / tile_groups) * 8 + xcd;
  } else {
    tile_group = tile_groups - 1 - blockIdx.x % tile_groups;
    unit = blockIdx.x / tile_groups;
  }
  const int kvh = unit % KVH, seq = unit / KVH;
  const int G = H / KVH;
  const int row0 = seq_start[seq];
  const int n_cols = (seq_start[seq + 1] - row0) * G;
  const int group_col0 = tile_group * GROUP_TILES * 16;
  if (group_col0 >= n_cols) return;                // the whole workgroup: no barrier is left behind

  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);   // the same in all lanes: what depends on it alone stays out of the vector registers
  const int j = lane % 16, g = lane / 16;

  // rows of a sequence are consecutive and in position order: the workgroup's first and last row bound its keys
  const int group_last_col = min(n_cols, group_col0 + GROUP_TILES * 16) - 1;
  const int group_pos_max = positions[row0 + group_last_col / G];
  const int group_pos_first = positions[row0 + group_col0 / G];
  const int group_lo_min = (window > 0 && group_pos_first - window + 1 > 0) ? group_pos_first - window + 1 : 0;
  const int begin = group_lo_min / BH_PAGE, last = group_pos_max / BH_PAGE;
  const int32_t* table = page_table + (size_t)seq * table_stride;

  // this wave's columns
  const int wave_tile0 = tile_group * GROUP_TILES + wave * CTW;
  const bool wave_active = wave_tile0 * 16 < n_cols;
  int pos[CTW], lo[CTW];
  bf16x8_t q_vec[CTW][NS];
  int pos_max = 0, pos_min = 0x7fffffff, lo_min = 0x7fffffff, lo_max = 0;
#pragma unroll
  for (int ct = 0; ct < CTW; ++ct) {
    const int wanted = (wave_tile0 + ct) * 16 + j;
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

  // The sum of a column's probabilities is one more row of the value product: the probabilities, as they enter
  // that product (rounded to bfloat16), times a block of ones; every one of a lane's four sums is its column's.
  f32x4_t o[CTW][2 * NS], run_sum[CTW];
  float run_max[CTW];
  const u32x4_t ones = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
#pragma unroll
  for (int ct = 0; ct < CTW; ++ct) {
    run_max[ct] = -INFINITY;
    run_sum[ct] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int dt = 0; dt < 2 * NS; ++dt) o[ct][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  // global -> LDS directly (16-byte loads that write LDS at the wave's base + 16 * lane), piece by piece:
  // thread `tid` brings pieces tid, tid + 256, ... of the page's keys and then of its values, which is their
  // order in LDS too.  The loads are waited for (vmcnt) before the barrier that hands the page over.
  auto fetch = [&](int p, int buffer) {
    const int page = table[p];
    const uint16_t* kb = k_pages + ((size_t)page * KVH + kvh) * BH_PAGE * HD;
    const uint16_t* vb = v_pages + ((size_t)page * KVH + kvh) * HD * BH_PAGE;
    static_assert(PIECES % 256 == 0, "the first half of a thread's pieces are keys, the second half values");
#pragma unroll
    for (int i = 0; i < STAGE; ++i) {
      const uint16_t* src = (i < STAGE / 2 ? kb : vb) + (size_t)(tid + (i % (STAGE / 2)) * 256) * 8;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)&page_lds[buffer][i * 256 + wave * 64],
                                       16, 0, 0);
    }
  };
  // The last page's tail was never written: what lies there may be anything, and although its probabilities
  // are zero its values must be too.  Once the page is in LDS, every thread clears that part of its pieces.
  auto clear_tail = [&](int p, int buffer) {
    if (p * BH_PAGE + BH_PAGE - 1 <= group_pos_max) return;   // the same for the whole workgroup
#pragma unroll
    for (int i = 0; i < STAGE; ++i) {
      const int piece = tid + i * 256;
      if (piece < PIECES) continue;
      // value piece (dt * 2 + u) * 64 + l holds tokens 32 u + 8 (l / 16) .. + 7 of the page
      const int pv = piece - PIECES;
      const int first_token = p * BH_PAGE + 32 * ((pv / 64) % 2) + 8 * ((pv % 64) / 16);
      page_lds[buffer][piece] = keep_first(page_lds[buffer][piece], group_pos_max + 1 - first_token);
    }
    __syncthreads();
  };

  fetch(begin, 0);
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  // One column tile's scores of a page -> its probabilities (as bfloat16 operands of the value product) and the
  // factor for what was summed so far.  Vector instructions only, so that it can run between the matrix
  // instructions of another tile.
  auto softmax_of = [&](auto masked, int ct, f32x4_t (&st)[4], int key0, u32x4_t (&p_vec)[2]) -> float {
    if constexpr (decltype(masked)::value) {   // key k0 + d of the page is seen if lo <= k0 + d <= pos: two numbers per column, then constants
      const int d_last = pos[ct] - key0, d_first = lo[ct] - key0;
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int d = 32 * (t / 2) + 4 * (t % 2) + r;
          if (d > d_last || d < d_first) st[t][r] = -INFINITY;
        }
    }
    // Online softmax with few instructions: the maximum is taken over the raw scores, the scale
    // enters through one fused multiply-add per score, and the exponentials are bare v_exp_f32
    // (arguments <= 0; results below the normal range may flush to zero).
    float local_max = larger(larger(st[0][0], st[0][1]), st[0][2]);
    local_max = larger(larger(local_max, st[0][3]), st[1][0]);
#pragma unroll
    for (int t = 1; t < 4; ++t) {
      local_max = larger(larger(local_max, st[t][1]), st[t][2]);
      local_max = larger(larger(local_max, st[t][3]), t < 3 ? st[t + 1][0] : run_max[ct]);
    }
    const float new_max = largest_of_column(local_max);               // raw (unscaled) scores, the earlier pages' too
    // The exponentials' reference moves only when the maximum has grown by more than SLACK powers of two (or
    // from nothing): until then probabilities may reach 2^SLACK, which float32 sums and bfloat16 operands
    // hold as well as numbers up to one, and what was summed so far needs no factor.
    const bool stays = (new_max - run_max[ct]) * scale_log2 <= SLACK;   // false from -inf, and while nothing was seen
    const float reference = stays ? run_max[ct] : new_max;
    const float shift = (reference == -INFINITY) ? 0.f : -reference * scale_log2;
    // exactly 1 while the reference stands still, 0 when nothing was seen before
    const float alpha =
        (run_max[ct] == reference) ? 1.0f : __builtin_amdgcn_exp2f((run_max[ct] - reference) * scale_log2);
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int t = 2 * u + half;
        const float e0 = __builtin_amdgcn_exp2f(fmaf(st[t][0], scale_log2, shift));
        const float e1 = __builtin_amdgcn_exp2f(fmaf(st[t][1], scale_log2, shift));
        const float e2 = __builtin_amdgcn_exp2f(fmaf(st[t][2], scale_log2, shift));
        const float e3 = __builtin_amdgcn_exp2f(fmaf(st[t][3], scale_log2, shift));
        p_vec[u][2 * half] = pack_bf16(e0, e1);
        p_vec[u][2 * half + 1] = pack_bf16(e2, e3);
      }
    run_max[ct] = reference;
    return alpha;
  };
  auto scale_sums = [&](int ct, float alpha) {
    if (__any(alpha != 1.0f)) {   // after the first pages the reference seldom moves
      run_sum[ct] = run_sum[ct] * alpha;
#pragma unroll
      for (int dt = 0; dt < 2 * NS; ++dt) o[ct][dt] = o[ct][dt] * alpha;
    }
  };
  // The matrix instructions of one tile and the vector instructions of another are independent of each other: side
  // by side in one stretch of code they are issued in turn (a matrix instruction keeps the matrix core busy for 16
  // clocks and the issue port for 4; this asks the compiler for five vector instructions after each), so that a
  // wave's softmax runs under its own products and not only under another wave's.
#define BH_TAKE_TURNS(n)                                            \
  do {                                                              \
    _Pragma("unroll") for (int turn = 0; turn < (n); ++turn) {      \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);            \
      __builtin_amdgcn_sched_group_barrier(0x402, 5, 0);            \
    }                                                               \
  } while (0)
  auto scores_of = [&](int ct, const u32x4_t (&kop)[4 * NS], f32x4_t (&st)[4]) {   // 4 NS matrix instructions
    const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};   // (the first product of each chain adds to a constant: no registers to clear)
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        st[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kop[t * NS + s]), q_vec[ct][s], s == 0 ? zero : st[t], 0, 0, 0);
  };
  auto values_of = [&](int ct, const u32x4_t (&vop)[4 * NS], const u32x4_t (&p_vec)[2]) {   // 4 NS + 2 matrix instructions
    run_sum[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(ones), as_bf16x8(p_vec[0]), run_sum[ct], 0, 0, 0);
#pragma unroll
    for (int dt = 0; dt < 2 * NS; ++dt)
      o[ct][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vop[dt * 2]), as_bf16x8(p_vec[0]), o[ct][dt], 0, 0, 0);
    run_sum[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(ones), as_bf16x8(p_vec[1]), run_sum[ct], 0, 0, 0);
#pragma unroll
    for (int dt = 0; dt < 2 * NS; ++dt)
      o[ct][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vop[dt * 2 + 1]), as_bf16x8(p_vec[1]), o[ct][dt], 0, 0, 0);
  };
  auto attend_page = [&](auto masked, int p, int buffer) {
    const u32x4_t* kl = page_lds[buffer];
    const u32x4_t* vl = page_lds[buffer] + PIECES;
    const int key0 = p * BH_PAGE + 8 * g;  // lane (j, g) holds keys key0 + 32 * (t / 2) + 4 * (t % 2) + r
    // A page's operands are asked of LDS in two goes, each before the arithmetic that hides the wait: all the
    // keys' before the first score product, all the values' behind it.
    u32x4_t kop[4 * NS], vop[4 * NS];
#pragma unroll
    for (int i = 0; i < 4 * NS; ++i) kop[i] = kl[i * 64 + lane];
    __builtin_amdgcn_sched_barrier(0);
    f32x4_t st[CTW][4];
    u32x4_t p_vec[CTW][2];
    scores_of(0, kop, st[0]);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (CTW == 1) {
#pragma unroll
      for (int i = 0; i < 4 * NS; ++i) vop[i] = vl[i * 64 + lane];
      __builtin_amdgcn_sched_barrier(0);
      const float alpha = softmax_of(masked, 0, st[0], key0, p_vec[0]);
      scale_sums(0, alpha);
      values_of(0, vop, p_vec[0]);
    } else {
      static_assert(CTW <= 2, "a wave takes one or two column tiles");
      scores_of(1, kop, st[1]);                                              // the second tile's scores ...
      const float alpha0 = softmax_of(masked, 0, st[0], key0, p_vec[0]);     // ... with the first tile's softmax between them
#pragma unroll
      for (int i = 0; i < 4 * NS; ++i) vop[i] = vl[i * 64 + lane];          // (into the registers that the keys leave)
      BH_TAKE_TURNS(4 * NS);
      __builtin_amdgcn_sched_barrier(0);
      scale_sums(0, alpha0);
      __builtin_amdgcn_sched_barrier(0);
      values_of(0, vop, p_vec[0]);                                           // the first tile's values ...
      const float alpha1 = softmax_of(masked, 1, st[1], key0, p_vec[1]);     // ... with the second tile's softmax
      BH_TAKE_TURNS(4 * NS + 2);
      __builtin_amdgcn_sched_barrier(0);
      scale_sums(1, alpha1);
      __builtin_amdgcn_sched_barrier(0);
      values_of(1, vop, p_vec[1]);
    }
  };
  auto attend = [&](int p, int buffer) {
    // a page none of whose keys this wave's columns may see changes nothing
    const bool visible = wave_active && p * BH_PAGE <= pos_max && p * BH_PAGE + BH_PAGE - 1 >= lo_min;
    if (!visible) return;
    const bool mask_needed = (p * BH_PAGE + BH_PAGE - 1 > pos_min) || (p * BH_PAGE < lo_max);
    if (mask_needed) attend_page(std::true_type(), p, buffer);
    else attend_page(std::false_type(), p, buffer);
  };
  // all pages but the last in a loop whose body does not branch on the page count, so that the compiler may
  // interleave the next page's loads and staging writes with this page's arithmetic
  for (int p = begin; p < last; ++p) {
    const int buffer = (p - begin) & 1;
    fetch(p + 1, buffer ^ 1);   // everyone was done with that buffer at the last barrier
    attend(p, buffer);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();   // the next page is in place, and everyone is done with the one before it
  }
  clear_tail(last, (last - begin) & 1);
  attend(last, (last - begin) & 1);

  // lane (j, g) holds O^T[16 dt + 4 g + r, column j] and the column's sum
#pragma unroll
  for (int ct = 0; ct < CTW; ++ct) {
    const int cc = (wave_tile0 + ct) * 16 + j;
    if (cc >= n_cols) continue;
    const float inv = 1.0f / run_sum[ct][0];
    const int out_row = row0 + cc / G, out_column = (kvh * G + cc % G) * HD + 4 * g;
#pragma unroll
    for (int dt = 0; dt < 2 * NS; ++dt) {
      uint2 packed;
      packed.x = pack_bf16(o[ct][dt][0] * inv, o[ct][dt][1] * inv);
      packed.y = pack_bf16(o[ct][dt][2] * inv, o[ct][dt][3] * inv);
      const size_t at = out_blocked ? (size_t)bh_blocked_index(out_row, out_column + 16 * dt, H * HD)
                                    : (size_t)out_row * (H * HD) + out_column + 16 * dt;
      *reinterpret_cast<uint2*>(out + at) = packed;
    }
  }
}

#undef BH_TAKE_TURNS

void bh_attention_prefill_launch(const void* q, void* out, const void* k_pages, const void* v_pages,
                                 const int32_t* page_table, int table_stride, const int32_t* positions,
                                 const int32_t* seq_start, int n_seqs, int tiles, int H, int KVH, int hd,
                                 float scale_log2, int window, int out_blocked, hipStream_t stream) {
#define BH_PREFILL(NS, CTW)                                                                                  \
  do {                                                                                                       \
    const int tile_groups = (tiles + 4 * CTW - 1) / (4 * CTW);                                               \
    attention_prefill_kernel<NS, CTW><<<dim3(tile_groups * KVH * n_seqs), dim3(256), 0, stream>>>(           \
        (const uint16_t*)q, (uint16_t*)out, (const uint16_t*)k_pages, (const uint16_t*)v_pages, page_table,  \
        table_stride, positions, seq_start, H, KVH, scale_log2, window, tile_groups, n_seqs, out_blocked);   \
  } while (0)
  // Two column tiles per wave while the accumulators leave room for two workgroups per compute unit; one
  // where that gives fewer than two workgroups per compute unit (a page costs a workgroup nearly the same
  // time either way, so the steps are shorter with more and smaller workgroups: at 32 query and 8 kv heads
  // of 128, 512 rows 24.5 -> 18.1 us, 1,024 rows 38.6 -> 30.2 us; at 2,048 rows one tile is 3 % slower, at 4,096 rows
  // 20 %).
  const bool few = (long)((tiles + 7) / 8) * KVH * n_seqs < 512;
  switch (hd / 32) {
    case 1: if (few) BH_PREFILL(1, 1); else BH_PREFILL(1, 2); break;
    case 2: if (few) BH_PREFILL(2, 1); else BH_PREFILL(2, 2); break;
    case 3: if (few) BH_PREFILL(3, 1); else BH_PREFILL(3, 2); break;
    case 4: if (few) BH_PREFILL(4, 1); else BH_PREFILL(4, 2); break;
    case 5: BH_PREFILL(5, 1); break;
    case 6: BH_PREFILL(6, 1); break;
    case 7: BH_PREFILL(7, 1); break;
    default: BH_PREFILL(8, 1); break;
  }
#undef BH_PREFILL
}
