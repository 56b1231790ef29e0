// Token selection from float32 logits, one block per row.
//   temperature <= 0: argmax, ties to the lowest id.
//   temperature  > 0: softmax(logits / temperature) in float32 with the maximum subtracted,
//                     optionally restricted to the top_k largest logits and then to the
//                     smallest set of most likely tokens whose mass reaches top_p (ties at a
//                     threshold are kept), then an inverse-CDF draw with the caller's uniform
//                     number in [0, 1).  Sums run in a fixed order, so a row's result does not
//                     depend on the other rows.
// A row with a non-finite logit sets bad[row] = 1 and selects nothing (token -1).
#include "sampling.h"

#include <mutex>

#define SB 1024  // threads per block

__device__ inline uint32_t order_key(float x) {
  uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__global__ __launch_bounds__(SB) void sample_kernel(const float* __restrict__ logits,
                                                    const float* __restrict__ temperature,
                                                    const int32_t* __restrict__ top_k,
                                                    const float* __restrict__ top_p,
                                                    const float* __restrict__ uniform,
                                                    int32_t* __restrict__ tokens, int32_t* __restrict__ bad,
                                                    int vocab) {
  __shared__ float scratch[SB / BH_WAVE];
  __shared__ float best_val[SB];
  __shared__ int best_idx[SB];
  __shared__ float prefix[SB + 1];
  __shared__ int chosen;

  const int row = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)row * vocab;

  // pass 1: maximum with lowest-index ties, and the finiteness check
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  float not_finite = 0.f;
  for (int i = tid; i < vocab; i += SB) {
    const float v = x[i];
    if (!isfinite(v)) not_finite = 1.f;
    if (v > bv || bi == 0x7fffffff) {
      bv = v;
      bi = i;
    }
  }
  not_finite = block_sum(not_finite, scratch);
  if (not_finite > 0.f) {
    if (tid == 0) {
      tokens[row] = -1;
      bad[row] = 1;
    }
    return;
  }
  best_val[tid] = bv;
  best_idx[tid] = bi;
  __syncthreads();
  for (int stride = SB / 2; stride > 0; stride >>= 1) {
    if (tid < stride) {
      const float ov = best_val[tid + stride];
      const int oi = best_idx[tid + stride];
      if (ov > best_val[tid] || (ov == best_val[tid] && oi < best_idx[tid])) {
        best_val[tid] = ov;
        best_idx[tid] = oi;
      }
    }
    __syncthreads();
  }
  const float max_logit = best_val[0];
  const int arg_max = best_idx[0];
  const float temp = temperature ? temperature[row] : 0.f;
  if (!(temp > 0.f)) {
    if (tid == 0) {
      tokens[row] = arg_max;
      bad[row] = 0;
    }
    return;
  }
  const float inv_temp = 1.0f / temp;

  // top-k: the k-th largest logit, found bit by bit on the order-preserving integer key
  uint32_t floor_key = 0;  // tokens with key >= floor_key are kept
  const int k = top_k ? top_k[row] : 0;
  if (k > 0 && k < vocab) {
    uint32_t found = 0;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t candidate = found | (1u << bit);
      float count = 0.f;
      for (int i = tid; i < vocab; i += SB) count += (order_key(x[i]) >= candidate) ? 1.f : 0.f;
      count = block_sum(count, scratch);
      if (count >= (float)k) found = candidate;
    }
    floor_key = found;
  }

  // each thread owns a contiguous range of the vocabulary
  const int per = (vocab + SB - 1) / SB;
  const int lo = tid * per < vocab ? tid * per : vocab;
  const int hi = lo + per < vocab ? lo + per : vocab;

  // top-p: the largest key threshold whose kept mass still reaches top_p of the total
  const float p_keep = top_p ? top_p[row] : 1.f;
  if (p_keep > 0.f && p_keep < 1.f) {
    float total = 0.f;
    for (int i = lo; i < hi; ++i)
      if (order_key(x[i]) >= floor_key) total += expf((x[i] - max_logit) * inv_temp);
    total = block_sum(total, scratch);
    const float need = p_keep * total;
    uint32_t found = 0;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t candidate = found | (1u << bit);
      float mass = 0.f;
      if (candidate >= floor_key) {
        for (int i = lo; i < hi; ++i)
          if (order_key(x[i]) >= candidate) mass += expf((x[i] - max_logit) * inv_temp);
      } else {
        mass = 0.f;  // below the top-k floor nothing changes; handled by taking the floor below
      }
      mass = block_sum(mass, scratch);
      if (candidate < floor_key || mass >= need) found = candidate;
    }
    if (found > floor_key) floor_key = found;
  }

  // inverse CDF over the kept tokens in index order
  float mine = 0.f;
  for (int i = lo; i < hi; ++i)
    if (order_key(x[i]) >= floor_key) mine += expf((x[i] - max_logit) * inv_temp);
  best_val[tid] = mine;
  if (tid == 0) chosen = arg_max;
  __syncthreads();
  if (tid == 0) {
    float running = 0.f;
    for (int t = 0; t < SB; ++t) {
      prefix[t] = running;
      running += best_val[t];
    }
    prefix[SB] = running;
  }
  __syncthreads();
  const float target = uniform[row] * prefix[SB];
  const bool last_owner = (tid == SB - 1);
  if (mine > 0.f && target >= prefix[tid] && (target < prefix[tid + 1] || last_owner)) {
    float running = prefix[tid];
    int pick = -1, last_kept = -1;
    for (int i = lo; i < hi; ++i) {
      if (order_key(x[i]) < floor_key) continue;
      last_kept = i;
      running += expf((x[i] - max_logit) * inv_temp);
      if (running > target) {
        pick = i;
        break;
      }
    }
    chosen = pick >= 0 ? pick : last_kept;
  }
  __syncthreads();
  if (tid == 0) {
    tokens[row] = chosen;
    bad[row] = 0;
  }
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
