// Token selection from float32 logits.  One block per row does all of it (sample_kernel); long rows get help from
// blocks per chunk of the row where the work can be cut: the argmax in two steps, a draw from the whole distribution
// through the chunks' weight sums, a draw with a top-k through the chunks' own k largest (further down).
//   temperature <= 0: argmax, ties to the lowest id.
//   temperature  > 0: softmax(logits / temperature) with the maximum subtracted,
//                     optionally restricted to the top_k largest logits and then to the
//                     smallest set of most likely tokens whose mass reaches top_p (ties at a
//                     threshold are kept), then an inverse-CDF draw over the kept tokens in index order
//                     with the caller's uniform number in [0, 1).
// A row with a non-finite logit sets bad[row] = 1 and selects nothing (token -1).
//
// A token's weight exp((x - max) / temperature), a float32 in (0, 1], is taken as an integer: its value times 2^32,
// rounded (a weight below 2^-33 of the largest counts for nothing).  Sums of integers do not depend on the order
// they are added in, so a row's result depends neither on the other rows nor on how the threads share the row,
// and the sums can be made by atomic additions.  Both thresholds are found digit by digit (12, 12 and 8 bits of
// the order-preserving integer key of a logit): a pass over the row adds each token's count (top-k) or weight
// (top-p) to the bin of its digit, among the tokens whose higher digits are the ones found so far; the bins are
// walked from the top until the count reaches k, or the weight top_p of the total.  Three passes each, where a
// search bit by bit took 32 (a row of 151,936 logits, one row or eight: temperature alone 121 -> 48 us, with
// top-k of 50 711 -> 86, with top-p of 0.9 2,224 -> 110, with both 2,634 -> 128; 64 rows: 216 -> 52, 1,707 -> 94,
// 5,146 -> 117, 5,835 -> 142).  What is left there is arithmetic on the one compute unit that a row has: a pass costs
// 10 to 13 us, the draw's about 25 (holding twice the loads in flight changed nothing); hence the chunks.
#include "sampling.h"

#include <mutex>

#define SB 1024  // threads per block
#define SAMPLE_BINS 4096

typedef unsigned long long sample_u64;

// An integer that orders as the floats do; minus zero and zero, which compare equal, get one key (ties at a threshold
// are kept, and a tie must not depend on a sign bit).
__device__ inline uint32_t order_key(float x) {
  uint32_t u = __float_as_uint(x);
  if (u == 0x80000000u) u = 0u;
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// f(index, value) for every element of the row, each thread its share: four neighbours at a time where the row
// is aligned for it, every load of a trip asked for before the first is used.
template <typename F>
__device__ inline void over_the_row(const float* __restrict__ x, int vocab, F f) {
  const int tid = threadIdx.x;
  int head = (int)(((16 - (reinterpret_cast<uintptr_t>(x) & 15)) & 15) / 4);   // elements before the first 16-byte boundary
  if (head > vocab) head = vocab;
  const int quads = (vocab - head) / 4;
  const float4* x4 = reinterpret_cast<const float4*>(x + head);
  int q = tid;
  for (; q + 7 * SB < quads; q += 8 * SB) {   // 128 KB of a row on their way to a block
    float4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = x4[q + u * SB];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = head + 4 * (q + u * SB);
      f(i, v[u].x), f(i + 1, v[u].y), f(i + 2, v[u].z), f(i + 3, v[u].w);
    }
  }
  for (; q < quads; q += SB) {
    const float4 v = x4[q];
    const int i = head + 4 * q;
    f(i, v.x), f(i + 1, v.y), f(i + 2, v.z), f(i + 3, v.w);
  }
  if (tid < head) f(tid, x[tid]);
  const int tail = head + 4 * quads;
  if (tail + tid < vocab) f(tail + tid, x[tail + tid]);
}

// Sum over the block, the same in every thread (integers: any order gives the same).
__device__ inline sample_u64 block_total(sample_u64 v, sample_u64* scratch) {
#pragma unroll
  for (int off = BH_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, BH_WAVE);
  __syncthreads();
  if (threadIdx.x % BH_WAVE == 0) scratch[threadIdx.x / BH_WAVE] = v;
  __syncthreads();
  sample_u64 total = 0;
  for (int w = 0; w < SB / BH_WAVE; ++w) total += scratch[w];
  return total;
}

// The sum of the values of the threads before this one.
__device__ inline sample_u64 block_sum_before(sample_u64 v, sample_u64* scratch) {
  const int lane = threadIdx.x % BH_WAVE, wave = threadIdx.x / BH_WAVE;
  sample_u64 inclusive = v;
#pragma unroll
  for (int off = 1; off < BH_WAVE; off <<= 1) {
    const sample_u64 other = __shfl_up(inclusive, off, BH_WAVE);
    if (lane >= off) inclusive += other;
  }
  __syncthreads();
  if (lane == BH_WAVE - 1) scratch[wave] = inclusive;
  __syncthreads();
  sample_u64 before = 0;
  for (int w = 0; w < wave; ++w) before += scratch[w];
  return before + inclusive - v;
}

// The largest key t for which the weights of the tokens with key >= t add up to at least `need` (>= 1, at most the
// weights' total), among the tokens with key >= floor_key; weight(value) is a token's weight.  bins: SAMPLE_BINS
// words of LDS.  Every thread gets the key.
template <typename W>
__device__ inline uint32_t threshold_key(const float* __restrict__ x, int vocab, uint32_t floor_key, sample_u64 need,
                                         sample_u64* bins, sample_u64* scratch, uint32_t* found_bin, sample_u64* found_above,
                                         W weight) {
  uint32_t prefix = 0;   // the digits found so far, as the key's high bits
  int done_bits = 0;
  const int digit_bits[3] = {12, 12, 8};
#pragma unroll
  for (int pass = 0; pass < 3; ++pass) {
    const int bits = digit_bits[pass], shift = 32 - done_bits - bits;
    for (int b = threadIdx.x; b < SAMPLE_BINS; b += SB) bins[b] = 0;
    __syncthreads();
    over_the_row(x, vocab, [&](int, float v) {
      const uint32_t key = order_key(v);
      if (key < floor_key) return;
      if (done_bits > 0 && (key >> (32 - done_bits)) != prefix) return;
      const sample_u64 w = weight(v);
      if (w) atomicAdd(&bins[(key >> shift) & ((1u << bits) - 1u)], w);
    });
    __syncthreads();
    // from the top bin down: thread t has the bins SAMPLE_BINS - 1 - 4 t .. - 3, the highest first
    constexpr int PER = SAMPLE_BINS / SB;
    sample_u64 mine[PER], sum = 0;
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int bin = SAMPLE_BINS - 1 - (PER * (int)threadIdx.x + u);
      mine[u] = bin < (1 << bits) ? bins[bin] : 0;
      sum += mine[u];
    }
    sample_u64 above = block_sum_before(sum, scratch);   // the weight of the bins above this thread's
    if (above < need && above + sum >= need) {             // one thread: the bin where the sum reaches `need`
#pragma unroll
      for (int u = 0; u < PER; ++u) {
        if (above < need && above + mine[u] >= need) {
          *found_bin = (uint32_t)(SAMPLE_BINS - 1 - (PER * (int)threadIdx.x + u));
          *found_above = above;
        }
        above += mine[u];
      }
    }
    __syncthreads();
    prefix = (prefix << bits) | *found_bin;
    need -= *found_above;
    done_bits += bits;
    __syncthreads();
  }
  return prefix;
}

// What a block that selects for a row keeps in LDS.
struct SampleShared {
  sample_u64 bins[SAMPLE_BINS];
  sample_u64 scratch[SB / BH_WAVE];
  float wave_val[SB / BH_WAVE];
  int wave_idx[SB / BH_WAVE];
  int wave_bad[SB / BH_WAVE];
  uint32_t found_bin;
  sample_u64 found_above;
  int chosen;
};

// The draw from x[0..vocab) at a temperature above zero, the largest logit and its place known: the filters, then
// the inverse-CDF draw over the kept tokens in index order; thread 0 leaves the token.  `ids` (or null): the token
// that each element of x stands for, when x is a row's candidates and not the row itself.  `whole_total` (or 0):
// the weight of the whole row where top-p is to keep its share of that and not of what top-k leaves of x (
// x's elements from the key `complete_from` on are then all of the row's with such keys); false, and no token, if
// top-p's share reaches beyond them.
__device__ inline bool draw_from(const float* __restrict__ x, int vocab, const int32_t* __restrict__ ids, float max_logit,
                                 int arg_max, float temp, int k, float p_keep, float uniform_number, int32_t* token,
                                 SampleShared& sh, sample_u64 whole_total = 0, uint32_t complete_from = 0) {
  sample_u64* bins = sh.bins;
  sample_u64* scratch = sh.scratch;
  const int tid = threadIdx.x;
  // exp((v - max) / temperature) as 2^((v - max) * log2(e) / temperature): one multiplication and the hardware's
  // exponential; times 2^32 and rounded (the conversion stops at 2^32 - 1, which the largest token gets)
  const float per_logit = 1.4426950408889634f / temp;
  auto weight_of = [&](float v) -> sample_u64 {
    return (sample_u64)__float2uint_rn(__builtin_amdgcn_exp2f((v - max_logit) * per_logit) * 4294967296.f);
  };

  // top-k: the k-th largest logit's key; tokens with key >= floor_key are kept (ties at the k-th are)
  uint32_t floor_key = complete_from;
  if (k > 0 && k < vocab)
    floor_key = threshold_key(x, vocab, 0u, (sample_u64)k, bins, scratch, &sh.found_bin, &sh.found_above,
                              [](float) -> sample_u64 { return 1; });

  // top-p: the largest key whose tokens, with all above them, weigh top_p of what top-k has left
  if (p_keep > 0.f && p_keep < 1.f) {
    sample_u64 total = 0;
    if (whole_total != 0 && floor_key == 0u) {
      total = whole_total;   // x is the whole row, and its weight is known
    } else {
      over_the_row(x, vocab, [&](int, float v) {
        if (order_key(v) >= floor_key) total += weight_of(v);
      });
      total = block_total(total, scratch);
    }
    const sample_u64 of = whole_total != 0 ? whole_total : total;
    sample_u64 need = (sample_u64)__double2ull_rn((double)p_keep * (double)of);
    if (need < 1) need = 1;
    if (need > of) need = of;
    if (need > total) return false;   // (the same in every thread)
    const uint32_t key = threshold_key(x, vocab, floor_key, need, bins, scratch, &sh.found_bin, &sh.found_above, weight_of);
    if (key > floor_key) floor_key = key;
  }

  // The draw.  A wave owns a contiguous span of the vocabulary and walks it in trips of 256 tokens, lane l taking
  // tokens 64 u + l of a trip (u = 0..3): in index order a trip is its four quarters one after the other, a quarter its
  // lanes.  First every span's kept weight (a lane adds up its own tokens, one sum over the lanes at the end), which
  // says whose span holds the target; then all waves share that span's trips and leave each trip's weight in `bins`;
  // then one wave finds the trip, the quarter and the lane.  (A sum over the lanes for every trip of every span made
  // this pass 30 us of arithmetic on the one compute unit that a row has.)
  constexpr int WAVES = SB / BH_WAVE, TRIP = 4 * BH_WAVE;
  const int wave = tid / BH_WAVE, lane = tid % BH_WAVE;
  const int trips = ((vocab + WAVES - 1) / WAVES + TRIP - 1) / TRIP;   // per span; at most SAMPLE_BINS (the entry point checks)
  auto kept_weight = [&](int i) -> sample_u64 {
    if (i >= vocab) return 0;
    const float v = x[i];
    return order_key(v) >= floor_key ? weight_of(v) : 0;
  };
  auto wave_total = [&](sample_u64 v) {
#pragma unroll
    for (int off = BH_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, BH_WAVE);
    return v;
  };
  {
    const int begin = wave * trips * TRIP;
    sample_u64 mine = 0;
    constexpr int AHEAD = 8;   // trips whose loads are on their way together
    for (int trip0 = 0; trip0 < trips; trip0 += AHEAD) {
      float v[AHEAD][4];
#pragma unroll
      for (int a = 0; a < AHEAD; ++a)
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = begin + (trip0 + a) * TRIP + BH_WAVE * u + lane;
          v[a][u] = (trip0 + a < trips && i < vocab) ? x[i] : -INFINITY;   // what is not there weighs nothing
        }
#pragma unroll
      for (int a = 0; a < AHEAD; ++a)
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (v[a][u] != -INFINITY && order_key(v[a][u]) >= floor_key) mine += weight_of(v[a][u]);
    }
    mine = wave_total(mine);
    __syncthreads();
    if (lane == 0) scratch[wave] = mine;
    if (tid == 0) sh.chosen = arg_max;
    __syncthreads();
  }
  sample_u64 kept = 0;
  for (int w = 0; w < WAVES; ++w) kept += scratch[w];
  sample_u64 target = (sample_u64)__double2ull_rd((double)uniform_number * (double)kept);
  if (target >= kept) target = kept - 1;   // (uniform is below 1; the largest token alone weighs 2^32 - 1)
  int span = 0;
  sample_u64 before = 0;   // the kept weight of the spans before the target's
  for (; span < WAVES - 1 && before + scratch[span] <= target; ++span) before += scratch[span];
  const int span_begin = span * trips * TRIP;
  for (int trip = wave; trip < trips; trip += WAVES) {   // the waves share the span's trips
    sample_u64 w = 0;
#pragma unroll
    for (int u = 0; u < 4; ++u) w += kept_weight(span_begin + trip * TRIP + BH_WAVE * u + lane);
    w = wave_total(w);
    if (lane == 0) bins[trip] = w;
  }
  __syncthreads();
  if (wave == 0) {
    int trip = 0;
    for (; trip < trips - 1 && before + bins[trip] <= target; ++trip) before += bins[trip];
    const int base = span_begin + trip * TRIP;
    sample_u64 w[4], quarter[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      w[u] = kept_weight(base + BH_WAVE * u + lane);
      quarter[u] = wave_total(w[u]);
    }
    int u = 0;
    for (; u < 3 && before + quarter[u] <= target; ++u) before += quarter[u];
    const sample_u64 own = u == 0 ? w[0] : u == 1 ? w[1] : u == 2 ? w[2] : w[3];
    sample_u64 through = own;   // the quarter's weights up to and with this lane's
#pragma unroll
    for (int off = 1; off < BH_WAVE; off <<= 1) {
      const sample_u64 other = __shfl_up(through, off, BH_WAVE);
      if (lane >= off) through += other;
    }
    // the first lane whose token carries the sum beyond the target
    const unsigned long long beyond = __ballot(own > 0 && before + through > target);
    if (beyond != 0 && lane == __ffsll((long long)beyond) - 1) {
      const int place = base + BH_WAVE * u + lane;
      sh.chosen = ids ? ids[place] : place;
    }
  }
  __syncthreads();
  if (tid == 0) *token = sh.chosen;
  return true;
}

__global__ __launch_bounds__(SB) void sample_kernel(const float* __restrict__ logits,
                                                    const float* __restrict__ temperature,
                                                    const int32_t* __restrict__ top_k,
                                                    const float* __restrict__ top_p,
                                                    const float* __restrict__ uniform,
                                                    int32_t* __restrict__ tokens, int32_t* __restrict__ bad,
                                                    int vocab) {
  __shared__ SampleShared sh;
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)row * vocab;

  // the maximum with lowest-index ties, and the finiteness check
  float bv = -INFINITY;
  int bi = 0x7fffffff, not_finite = 0;
  over_the_row(x, vocab, [&](int i, float v) {
    if (!isfinite(v)) not_finite = 1;
    if (v > bv || (v == bv && i < bi) || bi == 0x7fffffff) bv = v, bi = i;
  });
#pragma unroll
  for (int off = BH_WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, BH_WAVE);
    const int oi = __shfl_xor(bi, off, BH_WAVE);
    not_finite |= __shfl_xor(not_finite, off, BH_WAVE);
    if (ov > bv || (ov == bv && oi < bi)) bv = ov, bi = oi;
  }
  if (tid % BH_WAVE == 0) sh.wave_val[tid / BH_WAVE] = bv, sh.wave_idx[tid / BH_WAVE] = bi, sh.wave_bad[tid / BH_WAVE] = not_finite;
  __syncthreads();
  for (int w = 0; w < SB / BH_WAVE; ++w) {
    not_finite |= sh.wave_bad[w];
    if (sh.wave_val[w] > bv || (sh.wave_val[w] == bv && sh.wave_idx[w] < bi)) bv = sh.wave_val[w], bi = sh.wave_idx[w];
  }
  const float temp = temperature ? temperature[row] : 0.f;
  if (not_finite || !(temp > 0.f)) {
    if (tid == 0) {
      tokens[row] = not_finite ? -1 : bi;
      bad[row] = not_finite ? 1 : 0;
    }
    return;
  }
  if (tid == 0) bad[row] = 0;
  draw_from(x, vocab, nullptr, bv, bi, temp, top_k ? top_k[row] : 0, top_p ? top_p[row] : 1.f, uniform[row], tokens + row, sh);
}

// ---- argmax of long rows in two steps ---------------------------------------------------------
// One block per row leaves all but a few compute units idle when there are few rows and a long
// vocabulary.  Step one: a block per (row, chunk of AC elements) writes the chunk's largest value and its
// lowest index, or index -1 if the chunk holds a non-finite value; step two: a wave per row takes the
// best of the chunks (lowest index among equals, as chunks are in index order).

#define AC 2048   // elements per chunk
#define AT 256    // threads per chunk

__global__ __launch_bounds__(AT) void argmax_chunk_kernel(const float* __restrict__ logits, float* __restrict__ part_val,
                                                          int32_t* __restrict__ part_idx, int vocab, int chunks) {
  __shared__ float val[AT];
  __shared__ int idx[AT];
  const int row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)row * vocab;
  const int end = min(vocab, (chunk + 1) * AC);
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  bool not_finite = false;
  for (int i = chunk * AC + tid; i < end; i += AT) {
    const float v = x[i];
    if (!isfinite(v)) not_finite = true;
    if (v > bv || bi == 0x7fffffff) {
      bv = v;
      bi = i;
    }
  }
  val[tid] = bv;
  idx[tid] = not_finite ? -1 : bi;
  __syncthreads();
  for (int stride = AT / 2; stride > 0; stride >>= 1) {
    if (tid < stride) {
      const float ov = val[tid + stride];
      const int oi = idx[tid + stride];
      // -1 (a non-finite value was seen) wins over everything
      if (idx[tid] != -1 && (oi == -1 || ov > val[tid] || (ov == val[tid] && oi < idx[tid]))) {
        val[tid] = ov;
        idx[tid] = oi;
      }
    }
    __syncthreads();
  }
  if (tid == 0) {
    part_val[(size_t)row * chunks + chunk] = val[0];
    part_idx[(size_t)row * chunks + chunk] = idx[0];
  }
}

__global__ __launch_bounds__(BH_WAVE) void argmax_rows_kernel(const float* __restrict__ part_val,
                                                              const int32_t* __restrict__ part_idx,
                                                              int32_t* __restrict__ tokens, int32_t* __restrict__ bad,
                                                              int chunks) {
  const int row = blockIdx.x, lane = threadIdx.x;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int c = lane; c < chunks; c += BH_WAVE) {
    const float v = part_val[(size_t)row * chunks + c];
    const int i = part_idx[(size_t)row * chunks + c];
    if (bi != -1 && (i == -1 || v > bv || (v == bv && i < bi))) {
      bv = v;
      bi = i;
    }
  }
#pragma unroll
  for (int off = BH_WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, BH_WAVE);
    const int oi = __shfl_xor(bi, off, BH_WAVE);
    if (bi != -1 && (oi == -1 || ov > bv || (ov == bv && oi < bi))) {
      bv = ov;
      bi = oi;
    }
  }
  if (lane == 0) {
    tokens[row] = bi == -1 ? -1 : bi;
    bad[row] = bi == -1 ? 1 : 0;
  }
}

// ---- a draw at a temperature alone, over chunks of the row ---------------------------------------
// Without top-k and top-p nothing has to be known of the whole row before its weights can be added up, so the row
// need not stay with one block: a block per (row, chunk of DC tokens) leaves the chunk's largest logit (with its
// lowest index, or -1 beside a logit that is not finite) and the chunk's weights relative to that logit, summed as
// integers; a block per row then scales the chunks' sums to the row's largest logit (one float32 factor each, a fixed
// computation), finds the chunk that holds the target, weighs that chunk's tokens against the row's largest logit
// and walks them in index order.  The target's place inside the chunk is taken in proportion, the chunk's scaled sum
// and the sum of its tokens' weights differing by their rounding.  (151,936 logits at a temperature: 48 us with a
// block per row, which is one compute unit; this way 1 to 64 rows take 12 to 16.)

#define DC 2048   // tokens per chunk
#define DT 256    // threads per block: eight tokens of a chunk each, token 256 u + thread in turn u

__device__ inline sample_u64 fixed_weight(float logit, float reference, float per_logit) {
  return (sample_u64)__float2uint_rn(__builtin_amdgcn_exp2f((logit - reference) * per_logit) * 4294967296.f);
}

// Sum over a block of DT threads, the same in every thread; `scratch` holds DT / 64 words.
__device__ inline sample_u64 draw_total(sample_u64 v, sample_u64* scratch) {
#pragma unroll
  for (int off = BH_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, BH_WAVE);
  __syncthreads();
  if (threadIdx.x % BH_WAVE == 0) scratch[threadIdx.x / BH_WAVE] = v;
  __syncthreads();
  sample_u64 total = 0;
  for (int w = 0; w < DT / BH_WAVE; ++w) total += scratch[w];
  return total;
}

__global__ __launch_bounds__(DT) void draw_chunk_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                        uint32_t* __restrict__ records, int vocab, int chunks) {
  __shared__ float wave_val[DT / BH_WAVE];
  __shared__ int wave_idx[DT / BH_WAVE];
  __shared__ sample_u64 scratch[DT / BH_WAVE];
  const int row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)row * vocab;
  float v[DC / DT];
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  bool not_finite = false;
#pragma unroll
  for (int u = 0; u < DC / DT; ++u) {
    const int i = chunk * DC + u * DT + tid;
    v[u] = i < vocab ? x[i] : -INFINITY;
    if (i < vocab && !isfinite(v[u])) not_finite = true;
    if (i < vocab && (v[u] > bv || bi == 0x7fffffff)) bv = v[u], bi = i;   // (a thread's indices rise with u)
  }
#pragma unroll
  for (int off = BH_WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, BH_WAVE);
    const int oi = __shfl_xor(bi, off, BH_WAVE);
    if (ov > bv || (ov == bv && oi < bi)) bv = ov, bi = oi;
  }
  const bool any_bad = __syncthreads_or(not_finite);
  if (tid % BH_WAVE == 0) wave_val[tid / BH_WAVE] = bv, wave_idx[tid / BH_WAVE] = bi;
  __syncthreads();
  for (int w = 0; w < DT / BH_WAVE; ++w)
    if (wave_val[w] > bv || (wave_val[w] == bv && wave_idx[w] < bi)) bv = wave_val[w], bi = wave_idx[w];
  const float temp = temperature[row];
  sample_u64 mass = 0;
  if (!any_bad && temp > 0.f) {
    const float per_logit = 1.4426950408889634f / temp;
#pragma unroll
    for (int u = 0; u < DC / DT; ++u)
      if (chunk * DC + u * DT + tid < vocab) mass += fixed_weight(v[u], bv, per_logit);
  }
  mass = draw_total(mass, scratch);
  if (tid == 0) {
    uint32_t* record = records + ((size_t)row * chunks + chunk) * 4;
    record[0] = __float_as_uint(bv);
    record[1] = (uint32_t)(any_bad ? -1 : bi);
    record[2] = (uint32_t)mass;
    record[3] = (uint32_t)(mass >> 32);
  }
}

#define DRAW_MOST_CHUNKS 1024
__global__ __launch_bounds__(DT) void draw_rows_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                       const float* __restrict__ uniform, const uint32_t* __restrict__ records,
                                                       int32_t* __restrict__ tokens, int32_t* __restrict__ bad, int vocab,
                                                       int chunks) {
  __shared__ sample_u64 scaled[DRAW_MOST_CHUNKS];
  __shared__ sample_u64 scratch[DT / BH_WAVE];
  __shared__ float wave_val[DT / BH_WAVE];
  __shared__ int wave_idx[DT / BH_WAVE];
  __shared__ int found_chunk;
  __shared__ sample_u64 found_before;
  __shared__ int chosen;
  const int row = blockIdx.x, tid = threadIdx.x;
  const uint32_t* mine = records + (size_t)row * chunks * 4;
  // the row's largest logit with its lowest index; chunks come in index order, so among equals the first chunk's
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  bool any_bad = false;
  for (int c = tid; c < chunks; c += DT) {
    const float value = __uint_as_float(mine[4 * c]);
    const int index = (int)mine[4 * c + 1];
    if (index < 0) any_bad = true;
    if (value > bv || bi == 0x7fffffff) bv = value, bi = index;   // (a thread's chunks rise)
  }
#pragma unroll
  for (int off = BH_WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, BH_WAVE);
    const int oi = __shfl_xor(bi, off, BH_WAVE);
    if (ov > bv || (ov == bv && oi < bi)) bv = ov, bi = oi;
  }
  any_bad = __syncthreads_or(any_bad);
  if (tid % BH_WAVE == 0) wave_val[tid / BH_WAVE] = bv, wave_idx[tid / BH_WAVE] = bi;
  __syncthreads();
  for (int w = 0; w < DT / BH_WAVE; ++w)
    if (wave_val[w] > bv || (wave_val[w] == bv && wave_idx[w] < bi)) bv = wave_val[w], bi = wave_idx[w];
  const float temp = temperature[row];
  if (any_bad || !(temp > 0.f)) {
    if (tid == 0) {
      tokens[row] = any_bad ? -1 : bi;
      bad[row] = any_bad ? 1 : 0;
    }
    return;
  }
  const float per_logit = 1.4426950408889634f / temp;
  sample_u64 sum = 0;
  for (int c = tid; c < chunks; c += DT) {
    const sample_u64 mass = (sample_u64)mine[4 * c + 2] | ((sample_u64)mine[4 * c + 3] << 32);
    const float factor = __builtin_amdgcn_exp2f((__uint_as_float(mine[4 * c]) - bv) * per_logit);   // 1 for the chunk of the largest logit
    const sample_u64 part = (sample_u64)__double2ull_rd((double)mass * (double)factor);
    scaled[c] = part;
    sum += part;
  }
  const sample_u64 kept = draw_total(sum, scratch);   // (its barriers also put `scaled` in place)
  sample_u64 target = (sample_u64)__double2ull_rd((double)uniform[row] * (double)kept);
  if (target >= kept) target = kept - 1;
  if (tid == 0) {
    int c = 0;
    sample_u64 before = 0;
    for (; c < chunks - 1 && before + scaled[c] <= target; ++c) before += scaled[c];
    found_chunk = c;
    found_before = before;
    chosen = bi;
  }
  __syncthreads();
  const int chunk = found_chunk;
  const float* x = logits + (size_t)row * vocab;
  sample_u64 w[DC / DT], of_chunk = 0;
#pragma unroll
  for (int u = 0; u < DC / DT; ++u) {
    const int i = chunk * DC + u * DT + tid;
    w[u] = i < vocab ? fixed_weight(x[i], bv, per_logit) : 0;
    of_chunk += w[u];
  }
  of_chunk = draw_total(of_chunk, scratch);
  if (of_chunk == 0) {   // every token of the chunk rounds to nothing against the row's largest: the chunk's own largest
    if (tid == 0) tokens[row] = (int)mine[4 * chunk + 1], bad[row] = 0;
    return;
  }
  // the target's place inside the chunk, in the units of its tokens' weights
  const sample_u64 inside = target - found_before, of_scaled = scaled[chunk];
  sample_u64 local = (sample_u64)__double2ull_rd((double)inside * ((double)of_chunk / (double)of_scaled));
  if (local >= of_chunk) local = of_chunk - 1;
  sample_u64 before = 0;
  int turn = 0;
  sample_u64 of_turn[DC / DT];
#pragma unroll
  for (int u = 0; u < DC / DT; ++u) of_turn[u] = draw_total(w[u], scratch);
  for (; turn < DC / DT - 1 && before + of_turn[turn] <= local; ++turn) before += of_turn[turn];
  sample_u64 own = 0;
#pragma unroll
  for (int u = 0; u < DC / DT; ++u)
    if (u == turn) own = w[u];
  // the weights of the turn's tokens before this thread's
  const int lane = tid % BH_WAVE, wave = tid / BH_WAVE;
  sample_u64 through = own;
#pragma unroll
  for (int off = 1; off < BH_WAVE; off <<= 1) {
    const sample_u64 other = __shfl_up(through, off, BH_WAVE);
    if (lane >= off) through += other;
  }
  __syncthreads();
  if (lane == BH_WAVE - 1) scratch[wave] = through;
  __syncthreads();
  for (int v = 0; v < wave; ++v) before += scratch[v];
  if (own > 0 && before + through - own <= local && local < before + through) chosen = chunk * DC + turn * DT + tid;
  __syncthreads();
  if (tid == 0) {
    tokens[row] = chosen;
    bad[row] = 0;
  }
}

// Words of scratch for a draw at a temperature alone over these rows (0: the rows are drawn by a block each).
extern "C" int bh_sample_draw_scratch(int n_rows, int vocab) {
  const int chunks = (vocab + DC - 1) / DC;
  if (n_rows <= 0 || n_rows > 65535 || vocab < 4 * DC || chunks > DRAW_MOST_CHUNKS) return 0;
  return 4 * n_rows * chunks;
}

// ---- a draw among the top k, from the candidates of the row's chunks ------------------------------
// Each of the k largest logits of a row is among the k largest of its chunk.  So a block per (row, chunk of DC tokens)
// leaves the chunk's largest logit and, in index order, every token of the chunk that is not below the chunk's k-th
// largest (ties kept; `used` places per chunk, filled up with minus infinity, which weighs nothing and lies below
// every threshold); the block of the row then does on these few thousand candidates exactly what it would do on the
// row: the k-th largest's key, top-p's threshold among what top-k leaves, the draw in index order.  The tokens kept
// are the same as over the whole row, and so are their integer weights, the target and the token drawn.  A row
// whose k is above CANDIDATES_UP_TO_K, or one of whose chunks has more ties at its threshold than fit, is
// drawn from the whole row as before, by the same block (only the search for the largest logit is saved).
// Up to 64 rows with a top-p and no top-k go the same way with the chunks' CANDIDATES_UP_TO_K largest: the chunks'
// blocks, which then know the row's largest logit from a launch before them (the argmax's first step), also leave
// their tokens' weight, so that the row's block knows the whole row's, and the key of their last candidate: from the
// largest of those keys on, the candidates are all of the row's tokens.  If top-p's share of the row's weight lies
// within these, threshold and draw among the candidates are those of the whole row; if not (a flat distribution),
// the row is drawn whole, its largest logit and its weight already known.  (One row of 151,936 random logits, top-p
// of 0.9: at a spread that keeps a thousand tokens or so 107 -> 42 us, at three times the spread 40, at a sixth of it,
// where most of the vocabulary is kept and the row is drawn whole, 106; the candidates are about the largest 6 % of the
// row.  64 rows: 125 -> 91, 120 -> 86 and, drawn whole, 135 -> 160.)
// 151,936 logits, top-k of 50: 86 -> 29 us for one row, 33 for eight, 94 -> 61 for 64; with top-p of 0.9 as well 128 -> 39, 42, 143 -> 70.

#define CANDIDATES_UP_TO_K 128
#define CANDIDATE_PLACES 144   // per chunk at most; used(k) = k + 8 rounded up to 16
#define CANDIDATES_FOR_TOP_P_UP_TO_ROWS 64

__host__ __device__ inline int candidate_places(int k) { return (k + 8 + 15) / 16 * 16; }

#define CANDIDATE_HEADER 8   // words a chunk leaves beside its candidates: largest logit, its place (-1: not finite), count (-1: none), last candidate's key, weight (2)

// The k whose candidates a row's chunks hand in: its top-k, or for a top-p alone the most there is room for.
__device__ inline int candidates_k(const int32_t* top_k, const float* top_p, int row) {
  if (top_k != nullptr) return top_k[row];
  const float p = top_p[row];
  return p > 0.f && p < 1.f ? CANDIDATES_UP_TO_K : 0;
}

__global__ __launch_bounds__(DT) void candidates_chunk_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                              const int32_t* __restrict__ top_k, const float* __restrict__ top_p,
                                                              const float* __restrict__ chunk_max,
                                                              uint32_t* __restrict__ headers, float* __restrict__ values,
                                                              int32_t* __restrict__ ids, int vocab, int chunks) {
  __shared__ float wave_val[DT / BH_WAVE];
  __shared__ int wave_idx[DT / BH_WAVE];
  __shared__ uint32_t counts[256];
  __shared__ uint32_t found_digit, found_above;
  __shared__ int wave_kept[DT / BH_WAVE];
  constexpr int PER = DC / DT;   // a thread's tokens: PER neighbours, so that the threads' order is the index order
  const int row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x, lane = tid % BH_WAVE, wave = tid / BH_WAVE;
  const float* x = logits + (size_t)row * vocab;
  const int first = chunk * DC + PER * tid;
  float v[PER];
  uint32_t key[PER];
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  bool not_finite = false;
#pragma unroll
  for (int u = 0; u < PER; ++u) v[u] = first + u < vocab ? x[first + u] : -INFINITY;
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const bool there = first + u < vocab;
    if (there && !isfinite(v[u])) not_finite = true;
    if (there && (v[u] > bv || bi == 0x7fffffff)) bv = v[u], bi = first + u;
    key[u] = there ? order_key(v[u]) : 0u;   // (no float has the key 0)
  }
#pragma unroll
  for (int off = BH_WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, BH_WAVE);
    const int oi = __shfl_xor(bi, off, BH_WAVE);
    if (ov > bv || (ov == bv && oi < bi)) bv = ov, bi = oi;
  }
  const bool any_bad = __syncthreads_or(not_finite);
  if (lane == 0) wave_val[wave] = bv, wave_idx[wave] = bi;
  __syncthreads();
  for (int w = 0; w < DT / BH_WAVE; ++w)
    if (wave_val[w] > bv || (wave_val[w] == bv && wave_idx[w] < bi)) bv = wave_val[w], bi = wave_idx[w];
  uint32_t* header = headers + ((size_t)row * chunks + chunk) * CANDIDATE_HEADER;
  const int k = candidates_k(top_k, top_p, row);
  if (chunk_max != nullptr) {   // the chunk's weight against the row's largest logit, which the launch before left chunk by chunk
    __shared__ sample_u64 sums[DT / BH_WAVE];
    float top = -INFINITY;
    for (int c = tid; c < chunks; c += DT) top = fmaxf(top, chunk_max[(size_t)row * chunks + c]);
#pragma unroll
    for (int off = BH_WAVE / 2; off > 0; off >>= 1) top = fmaxf(top, __shfl_xor(top, off, BH_WAVE));
    __syncthreads();
    if (lane == 0) wave_val[wave] = top;
    __syncthreads();
    for (int w = 0; w < DT / BH_WAVE; ++w) top = fmaxf(top, wave_val[w]);
    const float temp = temperature[row];
    sample_u64 weight = 0;
    if (!any_bad && temp > 0.f) {
      const float per_logit = 1.4426950408889634f / temp;
#pragma unroll
      for (int u = 0; u < PER; ++u)
        if (first + u < vocab) weight += fixed_weight(v[u], top, per_logit);
    }
    weight = draw_total(weight, sums);
    if (tid == 0) header[4] = (uint32_t)weight, header[5] = (uint32_t)(weight >> 32);
  }
  if (any_bad || k <= 0 || k > CANDIDATES_UP_TO_K || k >= vocab) {   // (the same for all of the row's chunks)
    if (tid == 0) {
      header[0] = __float_as_uint(bv);
      header[1] = (uint32_t)(any_bad ? -1 : bi);
      header[2] = (uint32_t)-1;   // no candidates
    }
    return;
  }
  // the key of the chunk's k-th largest logit, digit by digit from the top (all of a chunk that has no more than k)
  const int here = min(DC, vocab - chunk * DC);
  uint32_t floor_key = 0;
  if (here > k) {
    uint32_t need = (uint32_t)k;
#pragma unroll 1
    for (int shift = 24; shift >= 0; shift -= 8) {
      counts[tid] = 0;   // (DT == 256 bins)
      __syncthreads();
#pragma unroll
      for (int u = 0; u < PER; ++u)
        if (key[u] != 0u && (shift == 24 || (key[u] >> (shift + 8)) == (floor_key >> (shift + 8))))
          atomicAdd(&counts[(key[u] >> shift) & 255u], 1u);
      __syncthreads();
      if (wave == 0) {   // lane l has the bins 255 - 4 l .. 252 - 4 l, the highest first
        uint32_t mine[4], sum = 0;
#pragma unroll
        for (int u = 0; u < 4; ++u) mine[u] = counts[255 - (4 * lane + u)], sum += mine[u];
        uint32_t through = sum;
#pragma unroll
        for (int off = 1; off < BH_WAVE; off <<= 1) {
          const uint32_t other = __shfl_up(through, off, BH_WAVE);
          if (lane >= off) through += other;
        }
        uint32_t above = through - sum;
        if (above < need && above + sum >= need) {
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            if (above < need && above + mine[u] >= need) found_digit = 255u - (4 * lane + u), found_above = above;
            above += mine[u];
          }
        }
      }
      __syncthreads();
      floor_key |= found_digit << shift;
      need -= found_above;
      __syncthreads();
    }
  }
  // the kept tokens' places among the chunk's candidates, in index order
  int mine = 0;
#pragma unroll
  for (int u = 0; u < PER; ++u) mine += key[u] != 0u && key[u] >= floor_key;
  int through = mine;
#pragma unroll
  for (int off = 1; off < BH_WAVE; off <<= 1) {
    const int other = __shfl_up(through, off, BH_WAVE);
    if (lane >= off) through += other;
  }
  if (lane == BH_WAVE - 1) wave_kept[wave] = through;
  __syncthreads();
  int before = through - mine, kept = 0;
  for (int w = 0; w < DT / BH_WAVE; ++w) {
    if (w < wave) before += wave_kept[w];
    kept += wave_kept[w];
  }
  const int places = candidate_places(k);
  if (tid == 0) {
    header[0] = __float_as_uint(bv);
    header[1] = (uint32_t)bi;
    header[2] = (uint32_t)(kept <= places ? kept : -1);   // more ties than places: the row is drawn whole
    header[3] = floor_key;
  }
  if (kept > places) return;
  const size_t base = (size_t)row * chunks * CANDIDATE_PLACES + (size_t)chunk * places;
#pragma unroll
  for (int u = 0; u < PER; ++u)
    if (key[u] != 0u && key[u] >= floor_key) {
      values[base + before] = v[u];
      ids[base + before] = first + u;
      ++before;
    }
  for (int j = kept + tid; j < places; j += DT) values[base + j] = -INFINITY, ids[base + j] = 0;
}

__global__ __launch_bounds__(SB) void sample_candidates_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                               const int32_t* __restrict__ top_k, const float* __restrict__ top_p,
                                                               const float* __restrict__ uniform, const uint32_t* __restrict__ headers,
                                                               const float* __restrict__ values, const int32_t* __restrict__ ids,
                                                               int32_t* __restrict__ tokens, int32_t* __restrict__ bad, int vocab,
                                                               int chunks) {
  constexpr int HW = CANDIDATE_HEADER;
  __shared__ SampleShared sh;
  const int row = blockIdx.x, tid = threadIdx.x;
  const uint32_t* mine = headers + (size_t)row * chunks * HW;
  // the row's largest logit with its lowest index (chunks are in index order), from the chunks' own
  float bv = -INFINITY;
  int bi = 0x7fffffff, not_finite = 0, whole = 0;
  const bool share_of_the_row = top_k == nullptr;   // a top-p alone: the chunks have left their weights and last keys
  sample_u64 weight = 0;
  uint32_t complete_from = 0;
  for (int c = tid; c < chunks; c += SB) {
    const float value = __uint_as_float(mine[HW * c]);
    const int index = (int)mine[HW * c + 1];
    if (index < 0) not_finite = 1;
    if ((int)mine[HW * c + 2] < 0) whole = 1;
    if (value > bv || bi == 0x7fffffff) bv = value, bi = index;
    if (share_of_the_row) {
      weight += (sample_u64)mine[HW * c + 4] | ((sample_u64)mine[HW * c + 5] << 32);
      if ((int)mine[HW * c + 2] >= 0) complete_from = max(complete_from, mine[HW * c + 3]);
    }
  }
#pragma unroll
  for (int off = BH_WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, BH_WAVE);
    const int oi = __shfl_xor(bi, off, BH_WAVE);
    not_finite |= __shfl_xor(not_finite, off, BH_WAVE);
    whole |= __shfl_xor(whole, off, BH_WAVE);
    if (ov > bv || (ov == bv && oi < bi)) bv = ov, bi = oi;
  }
  if (tid % BH_WAVE == 0) sh.wave_val[tid / BH_WAVE] = bv, sh.wave_idx[tid / BH_WAVE] = bi, sh.wave_bad[tid / BH_WAVE] = not_finite | (whole << 1);
  __syncthreads();
  for (int w = 0; w < SB / BH_WAVE; ++w) {
    not_finite |= sh.wave_bad[w] & 1;
    whole |= sh.wave_bad[w] >> 1;
    if (sh.wave_val[w] > bv || (sh.wave_val[w] == bv && sh.wave_idx[w] < bi)) bv = sh.wave_val[w], bi = sh.wave_idx[w];
  }
  const float temp = temperature[row];
  if (not_finite || !(temp > 0.f)) {
    if (tid == 0) {
      tokens[row] = not_finite ? -1 : bi;
      bad[row] = not_finite ? 1 : 0;
    }
    return;
  }
  if (tid == 0) bad[row] = 0;
  const int k = top_k ? top_k[row] : 0;
  const float p_keep = top_p ? top_p[row] : 1.f;
  if (share_of_the_row) {
    weight = block_total(weight, sh.scratch);
#pragma unroll
    for (int off = BH_WAVE / 2; off > 0; off >>= 1) complete_from = max(complete_from, (uint32_t)__shfl_xor((int)complete_from, off, BH_WAVE));
    __syncthreads();
    if (tid % BH_WAVE == 0) sh.wave_idx[tid / BH_WAVE] = (int)complete_from;
    __syncthreads();
    for (int w = 0; w < SB / BH_WAVE; ++w) complete_from = max(complete_from, (uint32_t)sh.wave_idx[w]);
  }
  const int places = candidate_places(candidates_k(top_k, top_p, row));
  // with a top-k, top-p keeps its share of what top-k leaves; alone, its share of the whole row
  if (!whole && draw_from(values + (size_t)row * chunks * CANDIDATE_PLACES, chunks * places,
                          ids + (size_t)row * chunks * CANDIDATE_PLACES, bv, bi, temp, k, p_keep, uniform[row],
                          tokens + row, sh, weight, complete_from))
    return;
  __syncthreads();
  draw_from(logits + (size_t)row * vocab, vocab, nullptr, bv, bi, temp, k, p_keep, uniform[row], tokens + row, sh, weight);
}

// Words of scratch for draws with a top-k or a top-p over these rows (0: the rows are drawn by a block each from the whole row).
extern "C" int bh_sample_top_k_scratch(int n_rows, int vocab) {
  static_assert(AC == DC, "the argmax's chunks are the candidates' chunks");
  const long chunks = (vocab + DC - 1) / DC;
  const long words = (long)n_rows * chunks * (CANDIDATE_HEADER + 2 * CANDIDATE_PLACES + 2);
  if (n_rows <= 0 || n_rows > 65535 || vocab < 4 * DC || chunks > SB || words >= (1L << 31)) return 0;
  return (int)words;
}

// Float-sized words of scratch that bh_sample wants for these rows when every row is greedy (0: none).
extern "C" int bh_sample_scratch(int n_rows, int vocab) {
  if (n_rows <= 0 || vocab < 4 * AC || n_rows >= 128) return 0;   // enough rows fill the compute units by themselves
  return 2 * n_rows * ((vocab + AC - 1) / AC);
}

extern "C" int bh_sample(const float* logits, const float* temperature, const int32_t* top_k,
                         const float* top_p, const float* uniform, int32_t* tokens, int32_t* bad, void* scratch,
                         int n_rows, int vocab, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && vocab > 0, "sample: rows %d and vocabulary %d must be positive", n_rows, vocab);
  BH_REQUIRE(temperature == nullptr || uniform != nullptr, "sample: temperature sampling needs uniform numbers");
  if (temperature == nullptr && scratch != nullptr && bh_sample_scratch(n_rows, vocab) > 0) {
    const int chunks = (vocab + AC - 1) / AC;
    BH_REQUIRE(n_rows <= 65535, "sample: too many rows");
    float* part_val = (float*)scratch;
    int32_t* part_idx = (int32_t*)scratch + (size_t)n_rows * chunks;
    argmax_chunk_kernel<<<dim3(chunks, n_rows), dim3(AT), 0, stream>>>(logits, part_val, part_idx, vocab, chunks);
    if (int status = bh_check_launch("argmax_chunk")) return status;
    argmax_rows_kernel<<<dim3(n_rows), dim3(BH_WAVE), 0, stream>>>(part_val, part_idx, tokens, bad, chunks);
    return bh_check_launch("argmax_rows");
  }
  BH_REQUIRE(temperature == nullptr || vocab <= SAMPLE_BINS * 256 * (SB / BH_WAVE),
             "sample: a draw takes vocabularies of up to %d tokens, not %d", SAMPLE_BINS * 256 * (SB / BH_WAVE), vocab);
  if (temperature != nullptr && top_k == nullptr && top_p == nullptr && scratch != nullptr && bh_sample_draw_scratch(n_rows, vocab) > 0) {
    const int chunks = (vocab + DC - 1) / DC;
    draw_chunk_kernel<<<dim3(chunks, n_rows), dim3(DT), 0, stream>>>(logits, temperature, (uint32_t*)scratch, vocab, chunks);
    if (int status = bh_check_launch("draw_chunk")) return status;
    draw_rows_kernel<<<dim3(n_rows), dim3(DT), 0, stream>>>(logits, temperature, uniform, (const uint32_t*)scratch, tokens, bad,
                                                            vocab, chunks);
    return bh_check_launch("draw_rows");
  }
  if (temperature != nullptr && (top_k != nullptr || (top_p != nullptr && n_rows <= CANDIDATES_FOR_TOP_P_UP_TO_ROWS)) && scratch != nullptr &&
      bh_sample_top_k_scratch(n_rows, vocab) > 0) {
    const int chunks = (vocab + DC - 1) / DC;
    uint32_t* headers = (uint32_t*)scratch;
    float* values = (float*)scratch + (size_t)n_rows * chunks * CANDIDATE_HEADER;
    int32_t* ids = (int32_t*)values + (size_t)n_rows * chunks * CANDIDATE_PLACES;
    float* chunk_max = nullptr;
    if (top_k == nullptr) {   // a top-p alone: the chunks' weights need the row's largest logit first
      chunk_max = (float*)(ids + (size_t)n_rows * chunks * CANDIDATE_PLACES);
      argmax_chunk_kernel<<<dim3(chunks, n_rows), dim3(AT), 0, stream>>>(logits, chunk_max, (int32_t*)chunk_max + (size_t)n_rows * chunks,
                                                                         vocab, chunks);
      if (int status = bh_check_launch("argmax_chunk")) return status;
    }
    candidates_chunk_kernel<<<dim3(chunks, n_rows), dim3(DT), 0, stream>>>(logits, temperature, top_k, top_p, chunk_max, headers, values,
                                                                           ids, vocab, chunks);
    if (int status = bh_check_launch("candidates_chunk")) return status;
    sample_candidates_kernel<<<dim3(n_rows), dim3(SB), 0, stream>>>(logits, temperature, top_k, top_p, uniform, headers, values,
                                                                    ids, tokens, bad, vocab, chunks);
    return bh_check_launch("sample_candidates");
  }
  sample_kernel<<<dim3(n_rows), dim3(SB), 0, stream>>>(logits, temperature, top_k, top_p, uniform, tokens, bad,
                                                       vocab);
  return bh_check_launch("sample");
}

// ---- greedy selection without an allocation ----------------------------------------------------
// The per-chunk maxima of the two-step argmax in a fixed array of the library's own.  In host code the
// array's name is only a handle: its address on the current GPU comes from hipGetSymbolAddress, once per
// device, and that address is what the kernels get.

static __device__ __align__(256) float greedy_scratch[BH_GREEDY_STATIC_WORDS];

#define BH_MAX_DEVICES 64
static float* greedy_scratch_at[BH_MAX_DEVICES];   // the array's address on each device, null until asked
static std::mutex greedy_scratch_lock;

static int greedy_scratch_here(float** out) {
  int device = -1;
  hipError_t status = hipGetDevice(&device);
  if (status != hipSuccess) return bh_fail("sample: no current device: %s", hipGetErrorString(status));
  BH_REQUIRE(device >= 0 && device < BH_MAX_DEVICES, "sample: device %d is beyond the %d this library keeps scratch for",
             device, BH_MAX_DEVICES);
  std::lock_guard<std::mutex> guard(greedy_scratch_lock);
  if (greedy_scratch_at[device] == nullptr) {
    void* address = nullptr;
    status = hipGetSymbolAddress(&address, HIP_SYMBOL(greedy_scratch));
    if (status != hipSuccess || address == nullptr)
      return bh_fail("sample: the address of the static scratch on device %d is not known: %s", device,
                     hipGetErrorString(status));
    greedy_scratch_at[device] = (float*)address;
  }
  *out = greedy_scratch_at[device];
  return 0;
}

extern "C" int bh_sample_greedy_static(const float* logits, int32_t* tokens, int32_t* bad, int n_rows, int vocab,
                                       hipStream_t stream) {
  BH_REQUIRE(logits != nullptr && tokens != nullptr && bad != nullptr, "sample: logits, tokens and flags are required");
  BH_REQUIRE(n_rows > 0 && vocab > 0, "sample: rows %d and vocabulary %d must be positive", n_rows, vocab);
  BH_REQUIRE(n_rows <= 65535, "sample: too many rows");
  const long chunks = ((long)vocab + AC - 1) / AC;
  BH_REQUIRE(2 * (long)n_rows * chunks <= BH_GREEDY_STATIC_WORDS,
             "sample: %d rows of %d logits need %ld words of scratch, the static array holds %d "
             "(2 x rows x ceil(vocabulary / %d) words)", n_rows, vocab, 2 * (long)n_rows * chunks,
             BH_GREEDY_STATIC_WORDS, AC);
  float* scratch = nullptr;
  if (int status = greedy_scratch_here(&scratch)) return status;
  float* part_val = scratch;
  int32_t* part_idx = (int32_t*)scratch + (size_t)n_rows * chunks;
  argmax_chunk_kernel<<<dim3((int)chunks, n_rows), dim3(AT), 0, stream>>>(logits, part_val, part_idx, vocab, (int)chunks);
  if (int status = bh_check_launch("argmax_chunk")) return status;
  argmax_rows_kernel<<<dim3(n_rows), dim3(BH_WAVE), 0, stream>>>(part_val, part_idx, tokens, bad, (int)chunks);
  return bh_check_launch("argmax_rows");
}
