// Kernels that take every size and both element types: embedding gather, RMSNorm, a tiled
// FMA matrix product, per-head q/k norm + rotation + cache write, attention over the paged
// cache, SwiGLU.  The float32 engine runs on these alone (true 32-bit arithmetic: plain FMA,
// no matrix-core mode); the bfloat16 engine uses them wherever no faster kernel fits a size.
// All reductions, norms, softmax and rotation are computed in float32.
#include "common.h"
#include <algorithm>

#include <stdarg.h>
#include <stdio.h>

// ---- errors ------------------------------------------------------------------------------

static thread_local char g_error[512] = "";

int bh_fail(const char* format, ...) {
  va_list args;
  va_start(args, format);
  vsnprintf(g_error, sizeof(g_error), format, args);
  va_end(args);
  return 1;
}

int bh_check_launch(const char* what) {
  hipError_t status = hipGetLastError();
  if (status != hipSuccess) return bh_fail("%s: launch failed: %s", what, hipGetErrorString(status));
  return 0;
}

int bh_compute_units() {
  static const int units = [] {
    int device = 0;
    hipDeviceProp_t properties;
    if (hipGetDevice(&device) != hipSuccess || hipGetDeviceProperties(&properties, device) != hipSuccess ||
        properties.multiProcessorCount <= 0) {
      (void)hipGetLastError();   // no GPU here: the error is not a launch's
      return 256;
    }
    return properties.multiProcessorCount;
  }();
  return units;
}

extern "C" const char* bh_last_error() { return g_error; }
extern "C" int bh_page_size() { return BH_PAGE; }

// ---- embedding ---------------------------------------------------------------------------
// hidden[row, :] = table[token[row], :], widened to float32.  A row's token is tokens[row], or, where
// token_src is given and token_src[row] >= 0, fed[token_src[row]]: a token that an earlier kernel chose
// and the host has not seen yet.  Such a token may be anything (the selection kernel writes -1 for a row
// it refuses), so ids outside the table read row 0; the host finds out from the selection itself.

template <typename T>
__global__ void embed_kernel(const int32_t* __restrict__ tokens, const int32_t* __restrict__ token_src,
                             const int32_t* __restrict__ fed, const T* __restrict__ table,
                             float* __restrict__ out, int width, int table_rows) {
  const int row = blockIdx.x;
  int token = tokens[row];
  if (token_src != nullptr && token_src[row] >= 0) token = fed[token_src[row]];
  if (token < 0 || token >= table_rows) token = 0;
  const T* src = table + (size_t)token * width;
  float* dst = out + (size_t)row * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = to_f32(src[i]);
}

extern "C" int bh_embed(const int32_t* tokens, const int32_t* token_src, const int32_t* fed, const void* table,
                        int table_dtype, float* out, int n_rows, int width, int table_rows, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && width > 0 && table_rows > 0, "embed: rows %d, width %d and table rows %d must be positive",
             n_rows, width, table_rows);
  BH_REQUIRE((token_src == nullptr) == (fed == nullptr), "embed: fed tokens and their row indices come together");
  dim3 grid(n_rows), block(256);
  if (table_dtype == BH_F32)
    embed_kernel<float><<<grid, block, 0, stream>>>(tokens, token_src, fed, (const float*)table, out, width, table_rows);
  else if (table_dtype == BH_BF16)
    embed_kernel<bf16_t><<<grid, block, 0, stream>>>(tokens, token_src, fed, (const bf16_t*)table, out, width,
                                                     table_rows);
  else
    return bh_fail("embed: unknown table dtype %d", table_dtype);
  return bh_check_launch("embed");
}

// ---- RMSNorm -----------------------------------------------------------------------------
// out[r, i] = (x[src, i] * inv) * w[i], inv = 1/sqrt(mean(x^2) + eps), src = rows ? rows[r] : r.

// PER > 0: the row fits PER elements per thread; x and w are loaded into registers before the
// reduction so that both memory round trips overlap (a decode step runs this on a handful of rows,
// where latency is all there is).  PER == 0: any width, in loops.
template <typename TW, typename TO, int PER>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows,
                               const TW* __restrict__ w, TO* __restrict__ out, int width, float eps, int block_rows) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  const float* xr = x + (size_t)src * width;
  // block_rows: the output's rows lie in blocks of that many (bh_rows_index), or one after the other (0)
  auto at = [&](int i) { return out + bh_rows_index(block_rows, r, i, width); };
  if (PER > 0) {
    float xv[PER > 0 ? PER : 1], wv[PER > 0 ? PER : 1];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int i = threadIdx.x + j * blockDim.x;
      xv[j] = i < width ? xr[i] : 0.f;
      wv[j] = (w && i < width) ? to_f32(w[i]) : 1.f;
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) ss += xv[j] * xv[j];
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)width + eps);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int i = threadIdx.x + j * blockDim.x;
      if (i < width) *at(i) = from_f32<TO>(xv[j] * inv * wv[j]);
    }
    return;
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = xr[i];
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float y = xr[i] * inv;
    if (w) y *= to_f32(w[i]);
    *at(i) = from_f32<TO>(y);
  }
}

// The same for widths that are multiples of 4 and many rows: a thread takes NV groups of four neighbouring
// elements (16-byte loads of the row, 8- or 16-byte loads of the weight, 8- or 16-byte stores), which moves the
// same bytes in a quarter of the memory instructions.  The order of the sum differs from the kernel above
// (a thread adds its four elements first), like that kernel's differs between widths.
typedef float norm_f32x4_t __attribute__((ext_vector_type(4)));
typedef uint16_t norm_u16x4_t __attribute__((ext_vector_type(4)));
template <typename TW, typename TO, int NV>
__global__ void rmsnorm_wide_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows,
                                    const TW* __restrict__ w, TO* __restrict__ out, int width, float eps,
                                    int block_rows) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  const norm_f32x4_t* xr = reinterpret_cast<const norm_f32x4_t*>(x + (size_t)src * width);
  const int fours = width / 4;
  const norm_f32x4_t zero = {0.f, 0.f, 0.f, 0.f}, one = {1.f, 1.f, 1.f, 1.f};
  norm_f32x4_t xv[NV], wv[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + j * blockDim.x;
    xv[j] = i < fours ? xr[i] : zero;
    wv[j] = one;
    if (w && i < fours) {
      if constexpr (sizeof(TW) == 4) {
        wv[j] = reinterpret_cast<const norm_f32x4_t*>(w)[i];
      } else {
        const norm_u16x4_t bits = reinterpret_cast<const norm_u16x4_t*>(w)[i];
#pragma unroll
        for (int e = 0; e < 4; ++e) wv[j][e] = bf16_bits_to_f32(bits[e]);
      }
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) ss += xv[j][0] * xv[j][0] + xv[j][1] * xv[j][1] + xv[j][2] * xv[j][2] + xv[j][3] * xv[j][3];
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + j * blockDim.x;
    if (i >= fours) continue;
    if constexpr (sizeof(TO) == 4) {
      *reinterpret_cast<norm_f32x4_t*>(out + bh_rows_index(block_rows, r, 4 * i, width)) = xv[j] * inv * wv[j];
    } else {
      norm_u16x4_t bits;
#pragma unroll
      for (int e = 0; e < 4; ++e) bits[e] = f32_to_bf16_bits(xv[j][e] * inv * wv[j][e]);
      *reinterpret_cast<norm_u16x4_t*>(out + bh_rows_index(block_rows, r, 4 * i, width)) = bits;
    }
  }
}

#define NORM_WIDE_FROM_ROWS 64   // fewer rows are latency, not bytes: the kernel above with its scalar loads was measured for them
template <typename TW, typename TO>
static void launch_rmsnorm(const float* x, const int32_t* rows, const void* w, void* out, int n_rows, int width,
                           float eps, int block_rows, hipStream_t stream) {
  if (n_rows >= NORM_WIDE_FROM_ROWS && width % 4 == 0 && width <= 4 * 4 * 1024 &&
      ((uintptr_t)x | (uintptr_t)w | (uintptr_t)out) % 16 == 0) {
    const int fours = width / 4;
    const int wide_threads = std::min(1024, ((fours + 3) / 4 + 63) / 64 * 64);   // four groups per thread where that fits
    const int each = (fours + wide_threads - 1) / wide_threads;
    dim3 grid(n_rows), block(wide_threads);
#define BH_NORM_WIDE(NV) \
  rmsnorm_wide_kernel<TW, TO, NV><<<grid, block, 0, stream>>>(x, rows, (const TW*)w, (TO*)out, width, eps, block_rows)
    if (each == 1) BH_NORM_WIDE(1);
    else if (each == 2) BH_NORM_WIDE(2);
    else BH_NORM_WIDE(4);
#undef BH_NORM_WIDE
    return;
  }
  const int threads = width >= 4096 ? 1024 : (width >= 1024 ? 512 : 256);
  const int per = (width + threads - 1) / threads;
  dim3 grid(n_rows), block(threads);
#define BH_NORM(PER) \
  rmsnorm_kernel<TW, TO, PER><<<grid, block, 0, stream>>>(x, rows, (const TW*)w, (TO*)out, width, eps, block_rows)
  if (per <= 4) BH_NORM(4);
  else if (per <= 8) BH_NORM(8);
  else BH_NORM(0);
#undef BH_NORM
}

// out_block_rows: the output's rows lie in blocks of 8 or 16 rows x 32 columns (bh_rows_index; bfloat16, width a
// multiple of 32), or one after the other (0).
extern "C" int bh_rmsnorm(const float* x, const int32_t* rows, const void* w, int w_dtype, void* out,
                          int out_dtype, int n_rows, int width, float eps, int out_block_rows, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && width > 0, "rmsnorm: rows %d and width %d must be positive", n_rows, width);
  BH_REQUIRE(eps >= 0.f, "rmsnorm: eps must not be negative");
  BH_REQUIRE(out_block_rows == 0 || ((out_block_rows == 8 || out_block_rows == 16) && out_dtype == BH_BF16 && width % 32 == 0),
             "rmsnorm: rows in blocks of %d need bfloat16 and a width that is a multiple of 32 (got %d)", out_block_rows, width);
  const int b = out_block_rows;
  if (w_dtype == BH_F32 && out_dtype == BH_F32) launch_rmsnorm<float, float>(x, rows, w, out, n_rows, width, eps, b, stream);
  else if (w_dtype == BH_F32 && out_dtype == BH_BF16) launch_rmsnorm<float, bf16_t>(x, rows, w, out, n_rows, width, eps, b, stream);
  else if (w_dtype == BH_BF16 && out_dtype == BH_F32) launch_rmsnorm<bf16_t, float>(x, rows, w, out, n_rows, width, eps, b, stream);
  else if (w_dtype == BH_BF16 && out_dtype == BH_BF16) launch_rmsnorm<bf16_t, bf16_t>(x, rows, w, out, n_rows, width, eps, b, stream);
  else return bh_fail("rmsnorm: unknown dtypes %d/%d", w_dtype, out_dtype);
  return bh_check_launch("rmsnorm");
}

// ---- matrix product, plain FMA -------------------------------------------------------------
// C[M, N] (+)= A[M, K] * W[N, K]^T with float32 accumulation; 64x64 tile, 16-wide k slices.

#define GT 64
#define GK 16

template <typename TA, typename TW, typename TC, bool ACCUMULATE>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TA* __restrict__ a, const TW* __restrict__ w,
                                                           TC* __restrict__ c, int M, int N, int K) {
  __shared__ float as[GK][GT + 1];
  __shared__ float ws[GK][GT + 1];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
  const int tx = tid % 16, ty = tid / 16;  // thread computes rows ty*4.., columns tx*4..
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += GK) {
    // 64 rows x 16 k = 1024 elements per operand, 4 per thread
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = tid + i * 256;
      const int r = e / GK, kk = e % GK;
      const int gm = m0 + r, gn = n0 + r, gk = k0 + kk;
      as[kk][r] = (gm < M && gk < K) ? to_f32(a[(size_t)gm * K + gk]) : 0.f;
      ws[kk][r] = (gn < N && gk < K) ? to_f32(w[(size_t)gn * K + gk]) : 0.f;
    }
    __syncthreads();
    // blocked summation: each 16-wide slice is summed on its own and then added, so the
    // rounding error grows with K/16 + 16 terms instead of K
    float part[4][4] = {};
#pragma unroll
    for (int kk = 0; kk < GK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = as[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) part[i][j] = fmaf(av[i], wv[j], part[i][j]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] += part[i][j];
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + ty * 4 + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn >= N) continue;
      const size_t at = (size_t)gm * N + gn;
      float v = acc[i][j];
      if (ACCUMULATE) v += to_f32(c[at]);
      c[at] = from_f32<TC>(v);
    }
  }
}

template <typename TA, typename TW>
static int gemm_generic_out(const void* a, const void* w, void* c, int c_dtype, int accumulate, int M, int N,
                            int K, hipStream_t stream) {
  dim3 grid((N + GT - 1) / GT, (M + GT - 1) / GT), block(256);
#define BH_GEMM(TC, ACC) \
  gemm_generic_kernel<TA, TW, TC, ACC><<<grid, block, 0, stream>>>((const TA*)a, (const TW*)w, (TC*)c, M, N, K)
  if (c_dtype == BH_F32 && accumulate) BH_GEMM(float, true);
  else if (c_dtype == BH_F32) BH_GEMM(float, false);
  else if (c_dtype == BH_BF16 && accumulate) BH_GEMM(bf16_t, true);
  else if (c_dtype == BH_BF16) BH_GEMM(bf16_t, false);
  else return bh_fail("gemm: unknown output dtype %d", c_dtype);
#undef BH_GEMM
  return bh_check_launch("gemm_generic");
}

extern "C" int bh_gemm_generic(const void* a, int a_dtype, const void* w, int w_dtype, void* c, int c_dtype,
                               int accumulate, int M, int N, int K, hipStream_t stream) {
  BH_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: sizes M=%d N=%d K=%d must be positive", M, N, K);
  BH_REQUIRE((N + GT - 1) / GT <= 2147483647 && (M + GT - 1) / GT <= 65535,
             "gemm: M=%d needs more than 65535 row tiles", M);
  if (a_dtype == BH_F32 && w_dtype == BH_F32)
    return gemm_generic_out<float, float>(a, w, c, c_dtype, accumulate, M, N, K, stream);
  if (a_dtype == BH_BF16 && w_dtype == BH_BF16)
    return gemm_generic_out<bf16_t, bf16_t>(a, w, c, c_dtype, accumulate, M, N, K, stream);
  if (a_dtype == BH_BF16 && w_dtype == BH_F32)
    return gemm_generic_out<bf16_t, float>(a, w, c, c_dtype, accumulate, M, N, K, stream);
  if (a_dtype == BH_F32 && w_dtype == BH_BF16)
    return gemm_generic_out<float, bf16_t>(a, w, c, c_dtype, accumulate, M, N, K, stream);
  return bh_fail("gemm: unknown operand dtypes %d/%d", a_dtype, w_dtype);
}

// ---- q/k norm + rotation + cache write -------------------------------------------------------
// One wave per (row, head) of the fused projection row [q heads | k heads | v heads].
// q head: optional RMSNorm over the head, rotation at the row's position, written to q_out.
// k head: the same, written into the cache page of (sequence, position).
// v head: copied into the cache.  Where an element lies within its page follows `kv_order`.  Rotation pairs are (i, i + rot/2) for i < rot/2; elements
// from rot to head_dim pass through.  With write_kv == 0 only the q heads are processed.

template <typename T, typename TW>
__global__ __launch_bounds__(64) void qk_norm_rope_cache_kernel(
    const T* __restrict__ qkv, T* __restrict__ q_out, const TW* __restrict__ q_weight,
    const TW* __restrict__ k_weight, float eps, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, int rot, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ row_seq, T* __restrict__ k_pages, T* __restrict__ v_pages,
    const int32_t* __restrict__ page_table, int table_stride, int H, int KVH, int hd, int kv_order) {
  const int row = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int fused = (H + 2 * KVH) * hd;
  const T* src = qkv + (size_t)row * fused + (size_t)head * hd;
  const int pos = positions[row];

  T* dst;
  const TW* weight;
  int order = BH_KV_ROWS, token = 0;   // a q head is one row of its own
  if (head < H) {
    dst = q_out + ((size_t)row * H + head) * hd;
    weight = q_weight;
  } else {
    const int seq = row_seq[row];
    const int page = page_table[(size_t)seq * table_stride + pos / BH_PAGE];
    const int kv_head = (head - H) % KVH;
    const bool is_value = head >= H + KVH;
    weight = k_weight;
    order = kv_order;
    token = pos % BH_PAGE;
    if (is_value) {
      T* block = v_pages + ((size_t)page * KVH + kv_head) * BH_PAGE * hd;
      for (int i = lane; i < hd; i += BH_WAVE) block[bh_value_index(order, token, i, hd)] = src[i];
      return;
    }
    dst = k_pages + ((size_t)page * KVH + kv_head) * BH_PAGE * hd;
  }
  float inv = 1.f;
  if (weight) {
    float ss = 0.f;
    for (int i = lane; i < hd; i += BH_WAVE) {
      float v = to_f32(src[i]);
      ss += v * v;
    }
    ss = wave_sum(ss);
    inv = 1.0f / sqrtf(ss / (float)hd + eps);
  }
  const int half = rot / 2;
  for (int i = lane; i < half; i += BH_WAVE) {
    float a = to_f32(src[i]), b = to_f32(src[i + half]);
    if (weight) {
      a = a * inv * to_f32(weight[i]);
      b = b * inv * to_f32(weight[i + half]);
    }
    float c = 1.f, s = 0.f;
    if (cos_table) {
      c = cos_table[(size_t)pos * half + i];
      s = sin_table[(size_t)pos * half + i];
    }
    dst[bh_key_index(order, token, i, hd)] = from_f32<T>(a * c - b * s);
    dst[bh_key_index(order, token, i + half, hd)] = from_f32<T>(a * s + b * c);
  }
  for (int i = rot + lane; i < hd; i += BH_WAVE) {
    float a = to_f32(src[i]);
    if (weight) a = a * inv * to_f32(weight[i]);
    dst[bh_key_index(order, token, i, hd)] = from_f32<T>(a);
  }
}

// eight consecutive elements at an 8-element boundary, in one or two loads
__device__ inline void load_eight(const float* p, float (&v)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ inline void load_eight(const bf16_t* p, float (&v)[8]) {
  const uint4 q = *reinterpret_cast<const uint4*>(p);
  const uint32_t words[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = bf16_bits_to_f32((uint16_t)(words[e / 2] >> (16 * (e % 2))));
}

// The same for many bfloat16 rows: a lane takes 8 consecutive elements of a head (16 bytes), LPH = head_dim / 8
// lanes a head, 64 / LPH heads of RPW rows a wave, four waves a block.  The rotation spans the whole head or is absent, so
// that an element's partner sits LPH / 2 lanes away.  Per q or k head: one 16-byte load, one 16-byte store.
// The values have waves of their own, behind the `main_waves` that take the q and k heads (`n_heads` of them):
// a value's neighbours in memory are the same dim of other tokens, eight tokens to a 16-byte piece in either
// cache order, so a wave takes eight rows and (up to) 64 / LPH kv heads, and where the eight tokens of a piece
// are consecutive rows of this step (the same sequence, positions 8 x .. 8 x + 7) the lanes of its first row load all eight
// rows, turn the 8 x 8 elements and store whole pieces; rows whose piece is not whole in this step (a step's
// first and last tokens) store their eight elements one by one.  (8,192 rows of 32 query and 8 kv heads of
// 128: the stores of the values one by one were 35 of the kernel's 57 us.)
// The value that the lane LPH / 2 further on (or back) in the same head holds, and a sum over a head's LPH lanes, in
// all of them.  A head of 16 lanes is a row of the wave's data-parallel moves: rotations within the row, no trip through LDS.
template <int LPH>
__device__ inline float head_partner(float v) {
  if constexpr (LPH == 16) return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x128, 0xf, 0xf, false));   // row_ror:8
  else return __shfl_xor(v, LPH / 2, BH_WAVE);
}
template <int LPH>
__device__ inline float head_sum(float v) {
  if constexpr (LPH == 16) {
    v += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x128, 0xf, 0xf, false));   // row_ror:8, 4, 2, 1
    v += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x124, 0xf, 0xf, false));
    v += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x122, 0xf, 0xf, false));
    v += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x121, 0xf, 0xf, false));
  } else {
#pragma unroll
    for (int off = LPH / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, BH_WAVE);
  }
  return v;
}

// PARTS: `qkv` holds no bfloat16 rows but the float32 sums of a product whose K was cut into parts,
// [parts][n_rows][(H + 2 KVH) * HD], as the kernel left them whose wave groups take turns: an element is the sum
// of its parts in their order, rounded to bfloat16 (what that product's finishing kernel would have written, which
// this takes the place of, and the bfloat16 rows' trip to memory and back with it).
template <bool PARTS, int RN>
__device__ inline void eight_of_each_row(const uint16_t* qkv, const size_t (&at)[RN], size_t part_stride, int parts,
                                         uint4 (&raw)[RN]) {   // at[r]: element offset in a [rows][width] matrix
  if constexpr (!PARTS) {
#pragma unroll
    for (int r = 0; r < RN; ++r) raw[r] = *reinterpret_cast<const uint4*>(qkv + at[r]);
  } else {
    const float* sums = reinterpret_cast<const float*>(qkv);
    float4 lo[RN], hi[RN];
#pragma unroll
    for (int r = 0; r < RN; ++r) lo[r] = hi[r] = make_float4(0.f, 0.f, 0.f, 0.f);
    constexpr int GROUP = RN >= 8 ? 2 : 4;   // parts whose loads, of all the rows, are on their way together
    for (int p0 = 0; p0 < parts; p0 += GROUP) {
      float4 a[GROUP][RN], b[GROUP][RN];
#pragma unroll
      for (int u = 0; u < GROUP; ++u)
#pragma unroll
        for (int r = 0; r < RN; ++r) {
          const float* from = sums + (size_t)min(p0 + u, parts - 1) * part_stride + at[r];
          const bool there = p0 + u < parts;
          a[u][r] = there ? *reinterpret_cast<const float4*>(from) : make_float4(0.f, 0.f, 0.f, 0.f);
          b[u][r] = there ? *reinterpret_cast<const float4*>(from + 4) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
      for (int u = 0; u < GROUP; ++u)   // in the parts' order; a part that is not there adds zero
#pragma unroll
        for (int r = 0; r < RN; ++r) {
          lo[r].x += a[u][r].x, lo[r].y += a[u][r].y, lo[r].z += a[u][r].z, lo[r].w += a[u][r].w;
          hi[r].x += b[u][r].x, hi[r].y += b[u][r].y, hi[r].z += b[u][r].z, hi[r].w += b[u][r].w;
        }
    }
#pragma unroll
    for (int r = 0; r < RN; ++r) {
      raw[r].x = (uint32_t)f32_to_bf16_bits(lo[r].x) | ((uint32_t)f32_to_bf16_bits(lo[r].y) << 16);
      raw[r].y = (uint32_t)f32_to_bf16_bits(lo[r].z) | ((uint32_t)f32_to_bf16_bits(lo[r].w) << 16);
      raw[r].z = (uint32_t)f32_to_bf16_bits(hi[r].x) | ((uint32_t)f32_to_bf16_bits(hi[r].y) << 16);
      raw[r].w = (uint32_t)f32_to_bf16_bits(hi[r].z) | ((uint32_t)f32_to_bf16_bits(hi[r].w) << 16);
    }
  }
}

template <typename TW, int LPH, int RPW, bool PARTS>   // RPW: rows that a wave of the q and k heads takes
__global__ __launch_bounds__(256) void qk_norm_rope_cache_rows_kernel(
    const uint16_t* __restrict__ qkv, int parts, uint16_t* __restrict__ q_out, const TW* __restrict__ q_weight,
    const TW* __restrict__ k_weight, float eps, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, const int32_t* __restrict__ positions, const int32_t* __restrict__ row_seq,
    uint16_t* __restrict__ k_pages, uint16_t* __restrict__ v_pages, const int32_t* __restrict__ page_table,
    int table_stride, int H, int KVH, int kv_order, int n_rows, int n_heads, int main_waves, int value_waves) {
  constexpr int HD = 8 * LPH, HPW = BH_WAVE / LPH;
  const int waves_per_row = (n_heads + HPW - 1) / HPW;
  const int wave = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + threadIdx.x / BH_WAVE), lane = threadIdx.x % BH_WAVE;
  if (wave >= main_waves) {   // the values of eight rows and HPW kv heads
    if (wave - main_waves >= value_waves) return;   // the last block's waves beyond the work (none at all without write_kv)
    const int chunks = (KVH + HPW - 1) / HPW, group = (wave - main_waves) / chunks;
    // lanes without a kv head of their own follow the last one and store nothing: every lane stays to the end,
    // because the rows' positions below are read out of the first 24 lanes' registers
    const int wanted_head = ((wave - main_waves) % chunks) * HPW + lane / LPH, c = lane % LPH;
    const bool mine = wanted_head < KVH;
    const int kv_head = mine ? wanted_head : KVH - 1;
    const size_t fused = (size_t)(H + 2 * KVH) * HD, part_stride = (size_t)n_rows * fused;
    const size_t src = (size_t)(H + KVH + kv_head) * HD + 8 * c;   // + row * fused
    // Positions and sequences of the rows 8 group - 8 .. 8 group + 15, one in each of the first 24 lanes, in one load
    // each: everything that the eight rows' decisions below look at (asked for row by row inside the loop, eight
    // waits for memory in a row were most of this kernel's time at a few hundred rows).
    const int base = 8 * group - 8;
    const int near = min(max(base + lane, 0), n_rows - 1);
    const int near_pos = positions[near], near_seq = row_seq[near];
    auto pos_of = [&](int row) { return __builtin_amdgcn_readlane(near_pos, __builtin_amdgcn_readfirstlane(row - base)); };
    auto seq_of = [&](int row) { return __builtin_amdgcn_readlane(near_seq, __builtin_amdgcn_readfirstlane(row - base)); };
    for (int row = 8 * group; row < 8 * group + 8 && row < n_rows; ++row) {
      const int pos = pos_of(row), seq = seq_of(row);
      const int first = row - pos % 8;   // where the row of the piece's first token would lie
      bool whole = first >= 0 && first + 7 < n_rows;   // the piece's eight tokens are the rows first .. first + 7, in order
      if (whole) {
#pragma unroll
        for (int t = 0; t < 8; ++t) whole = whole && seq_of(first + t) == seq && pos_of(first + t) == pos - pos % 8 + t;
      }
      if (whole && pos % 8 != 0) continue;   // the first row of the piece stores it
      const int page = page_table[(size_t)seq * table_stride + pos / BH_PAGE];
      uint16_t* block = v_pages + ((size_t)page * KVH + kv_head) * BH_PAGE * HD;
      if (!whole) {
        const size_t one_at[1] = {src + (size_t)row * fused};
        uint4 one[1];
        eight_of_each_row<PARTS, 1>(qkv, one_at, part_stride, parts, one);
        const uint32_t words[4] = {one[0].x, one[0].y, one[0].z, one[0].w};
        if (mine) {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            block[bh_value_index(kv_order, pos % BH_PAGE, 8 * c + e, HD)] = (uint16_t)(words[e / 2] >> (16 * (e % 2)));
        }
        continue;
      }
      uint4 raw[8];   // token t's dims 8 c .. 8 c + 7
      size_t raw_at[8];
#pragma unroll
      for (int t = 0; t < 8; ++t) raw_at[t] = src + (size_t)(row + t) * fused;
      eight_of_each_row<PARTS, 8>(qkv, raw_at, part_stride, parts, raw);
#pragma unroll
      for (int e = 0; e < 8; ++e) {   // dim 8 c + e of the eight tokens: the halves e % 2 of the words e / 2
        const uint32_t pick = e % 2 ? 0x07060302u : 0x05040100u;
        uint32_t word[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) word[t] = e / 2 == 0 ? raw[t].x : e / 2 == 1 ? raw[t].y : e / 2 == 2 ? raw[t].z : raw[t].w;
        uint4 piece;
        piece.x = __builtin_amdgcn_perm(word[1], word[0], pick);
        piece.y = __builtin_amdgcn_perm(word[3], word[2], pick);
        piece.z = __builtin_amdgcn_perm(word[5], word[4], pick);
        piece.w = __builtin_amdgcn_perm(word[7], word[6], pick);
        if (mine) *reinterpret_cast<uint4*>(block + bh_value_index(kv_order, pos % BH_PAGE, 8 * c + e, HD)) = piece;
      }
    }
    return;
  }
  const int first_row = (wave / waves_per_row) * RPW;
  if (first_row >= n_rows) return;   // whole waves leave; nothing below synchronises the block
  const int wanted = (wave % waves_per_row) * HPW + lane / LPH, c = lane % LPH;
  const bool active = wanted < n_heads;
  const int head = active ? wanted : n_heads - 1;   // lanes without a head of their own follow the last one and store nothing
  const bool is_q = head < H;
  // All of a wave's loads are asked for before anything is computed: RPW rows' 16 bytes, their positions and, behind
  // those, their angles.  (With one row per wave the three waits in a row, for so little data each, were the kernel's time.)
  int pos[RPW];
  uint4 raw[RPW];
  size_t raw_at[RPW];
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    const int row = min(first_row + r, n_rows - 1);
    pos[r] = positions[row];
    raw_at[r] = ((size_t)row * (H + 2 * KVH) + head) * HD + 8 * c;
  }
  eight_of_each_row<PARTS, RPW>(qkv, raw_at, (size_t)n_rows * (H + 2 * KVH) * HD, parts, raw);
  const TW* weight = is_q ? q_weight : k_weight;
  float wv[8];
  if (weight != nullptr) load_eight(weight + 8 * c, wv);
  constexpr int HALF = HD / 2;
  float cs[RPW][8], sn[RPW][8];
  if (cos_table != nullptr) {
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
      load_eight(cos_table + (size_t)pos[r] * HALF + 8 * (c % (LPH / 2)), cs[r]);
      load_eight(sin_table + (size_t)pos[r] * HALF + 8 * (c % (LPH / 2)), sn[r]);
    }
  }
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    const int row = first_row + r;
    const uint32_t words[4] = {raw[r].x, raw[r].y, raw[r].z, raw[r].w};
    float x[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = bf16_bits_to_f32((uint16_t)(words[e / 2] >> (16 * (e % 2))));
    if (weight != nullptr) {
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
      ss = head_sum<LPH>(ss);
      const float inv = 1.0f / sqrtf(ss / (float)HD + eps);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = x[e] * inv * wv[e];
    }
    if (cos_table != nullptr) {
      const bool lower = c < LPH / 2;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float other = head_partner<LPH>(x[e]);
        x[e] = lower ? x[e] * cs[r][e] - other * sn[r][e] : other * sn[r][e] + x[e] * cs[r][e];
      }
    }   // (all the lanes of a head take the same way through this: the exchanges stay within the head)
    if (!active || row >= n_rows) continue;
    uint4 packed;
    packed.x = (uint32_t)f32_to_bf16_bits(x[0]) | ((uint32_t)f32_to_bf16_bits(x[1]) << 16);
    packed.y = (uint32_t)f32_to_bf16_bits(x[2]) | ((uint32_t)f32_to_bf16_bits(x[3]) << 16);
    packed.z = (uint32_t)f32_to_bf16_bits(x[4]) | ((uint32_t)f32_to_bf16_bits(x[5]) << 16);
    packed.w = (uint32_t)f32_to_bf16_bits(x[6]) | ((uint32_t)f32_to_bf16_bits(x[7]) << 16);
    if (is_q) {
      *reinterpret_cast<uint4*>(q_out + ((size_t)row * H + head) * HD + 8 * c) = packed;
      continue;
    }
    const int page = page_table[(size_t)row_seq[row] * table_stride + pos[r] / BH_PAGE];
    const int token = pos[r] % BH_PAGE, kv_head = head - H;
    uint16_t* block = k_pages + ((size_t)page * KVH + kv_head) * BH_PAGE * HD;
    *reinterpret_cast<uint4*>(block + bh_key_index(kv_order, token, 8 * c, HD)) = packed;   // 8 dims lie together in both orders
  }
}

// The form for many bfloat16 rows (or, parts > 0, for a product's float32 sums in `parts` parts of K): whether it
// takes these sizes, and its launch.
static bool qk_rows_form_takes(int n_rows, int hd, int rot) {
  return n_rows >= 64 && (hd == 64 || hd == 128 || hd == 256) && (rot == 0 || rot == hd);
}
static int qk_rows_form(const void* qkv, int parts, void* q_out, const void* q_weight, const void* k_weight, int w_dtype,
                        float eps, const float* cos_table, const float* sin_table, int rot, const int32_t* positions,
                        const int32_t* row_seq, void* k_pages, void* v_pages, const int32_t* page_table, int table_stride,
                        int n_rows, int H, int KVH, int hd, int write_kv, int kv_order, hipStream_t stream) {
  // waves for the q and k heads of every row, then (write_kv) waves for the values of eight rows each
  const int lanes_per_head = hd / 8, heads_per_wave = 64 / lanes_per_head, main_heads = write_kv ? H + KVH : H;
  constexpr int RPW = 4;
  const long main_waves = (long)((n_rows + RPW - 1) / RPW) * ((main_heads + heads_per_wave - 1) / heads_per_wave);
  const long value_waves = write_kv ? (long)((n_rows + 7) / 8) * ((KVH + heads_per_wave - 1) / heads_per_wave) : 0;
  BH_REQUIRE(main_waves + value_waves < (1L << 31), "qk_norm_rope: too many rows");
  BH_REQUIRE(w_dtype == BH_F32 || w_dtype == BH_BF16, "qk_norm_rope: unknown weight dtype %d", w_dtype);
  dim3 wide_grid((unsigned)((main_waves + value_waves + 3) / 4)), wide_block(4 * BH_WAVE);
#define BH_QK_ROWS(TW, LPH, PARTS)                                                                                  \
  qk_norm_rope_cache_rows_kernel<TW, LPH, RPW, PARTS><<<wide_grid, wide_block, 0, stream>>>(                        \
      (const uint16_t*)qkv, parts, (uint16_t*)q_out, (const TW*)q_weight, (const TW*)k_weight, eps,                 \
      rot ? cos_table : nullptr, rot ? sin_table : nullptr,                                                          \
      positions, row_seq, (uint16_t*)k_pages, (uint16_t*)v_pages, page_table, table_stride, H, KVH, kv_order,      \
      n_rows, main_heads, (int)main_waves, (int)value_waves)
#define BH_QK_ROWS_W(LPH)                                      \
  do {                                                         \
    if (parts > 0 && w_dtype == BH_F32) BH_QK_ROWS(float, LPH, true);   \
    else if (parts > 0) BH_QK_ROWS(bf16_t, LPH, true);         \
    else if (w_dtype == BH_F32) BH_QK_ROWS(float, LPH, false); \
    else BH_QK_ROWS(bf16_t, LPH, false);                       \
  } while (0)
  if (hd == 64) BH_QK_ROWS_W(8);
  else if (hd == 128) BH_QK_ROWS_W(16);
  else BH_QK_ROWS_W(32);
#undef BH_QK_ROWS_W
#undef BH_QK_ROWS
  return bh_check_launch("qk_norm_rope_cache_rows");
}

// Rows may come in any order (every (sequence, position) once).  The form for many rows stores the values of eight
// consecutive positions as one piece where the step holds all eight as consecutive rows of one sequence, which it
// checks row by row (a step lays a sequence's rows out that way); any other row stores its own elements.
extern "C" int bh_qk_norm_rope_cache(const void* qkv, int dtype, void* q_out, const void* q_weight,
                                     const void* k_weight, int w_dtype, float eps, const float* cos_table,
                                     const float* sin_table, int table_positions, int rot,
                                     const int32_t* positions, const int32_t* row_seq, void* k_pages,
                                     void* v_pages, const int32_t* page_table, int table_stride, int n_rows,
                                     int H, int KVH, int hd, int write_kv, int kv_order, int max_position,
                                     hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && H > 0 && KVH > 0 && hd > 0, "qk_norm_rope: sizes must be positive");
  BH_REQUIRE(rot >= 0 && rot <= hd && rot % 2 == 0, "qk_norm_rope: rotary width %d must be even and at most %d", rot, hd);
  BH_REQUIRE((q_weight == nullptr) == (k_weight == nullptr), "qk_norm_rope: give both norm weights or neither");
  BH_REQUIRE(cos_table == nullptr || max_position < table_positions,
             "qk_norm_rope: position %d is outside the rotation table of %d positions", max_position, table_positions);
  BH_REQUIRE(H + 2 * KVH <= 65535, "qk_norm_rope: too many heads");
  BH_REQUIRE(kv_order == BH_KV_ROWS || (kv_order == BH_KV_PIECES && hd % 32 == 0),
             "qk_norm_rope: cache order %d does not exist for head size %d", kv_order, hd);
  if (cos_table == nullptr) rot = 0;
  const int n_heads = write_kv ? H + 2 * KVH : H;
  if (dtype == BH_BF16 && qk_rows_form_takes(n_rows, hd, rot))
    return qk_rows_form(qkv, 0, q_out, q_weight, k_weight, w_dtype, eps, cos_table, sin_table, rot, positions, row_seq,
                        k_pages, v_pages, page_table, table_stride, n_rows, H, KVH, hd, write_kv, kv_order, stream);
  dim3 grid(n_rows, n_heads), block(BH_WAVE);
#define BH_QK(T, TW)                                                                                         \
  qk_norm_rope_cache_kernel<T, TW><<<grid, block, 0, stream>>>(                                              \
      (const T*)qkv, (T*)q_out, (const TW*)q_weight, (const TW*)k_weight, eps, cos_table, sin_table, rot,    \
      positions, row_seq, (T*)k_pages, (T*)v_pages, page_table, table_stride, H, KVH, hd, kv_order)
  if (dtype == BH_F32 && w_dtype == BH_F32) BH_QK(float, float);
  else if (dtype == BH_F32 && w_dtype == BH_BF16) BH_QK(float, bf16_t);
  else if (dtype == BH_BF16 && w_dtype == BH_F32) BH_QK(bf16_t, float);
  else if (dtype == BH_BF16 && w_dtype == BH_BF16) BH_QK(bf16_t, bf16_t);
  else return bh_fail("qk_norm_rope: unknown dtypes %d/%d", dtype, w_dtype);
#undef BH_QK
  return bh_check_launch("qk_norm_rope_cache");
}

// The same from the float32 sums that a product of many rows left in `parts` parts of K
// ([parts][n_rows][(H + 2 KVH) * hd]; bh_gemm_bf16_bare_parts says which products do): every element is the sum of
// its parts in their order, rounded to bfloat16, as that product's finishing kernel would have written it; q_out,
// the cache and the weights as above, bfloat16 outputs.  bh_qk_norm_rope_cache_takes_sums: whether these sizes go.
extern "C" int bh_qk_norm_rope_cache_takes_sums(int n_rows, int hd, int rot) {
  return qk_rows_form_takes(n_rows, hd, rot) ? 1 : 0;
}
extern "C" int bh_qk_norm_rope_cache_sums(const float* sums, int parts, void* q_out, const void* q_weight,
                                          const void* k_weight, int w_dtype, float eps, const float* cos_table,
                                          const float* sin_table, int table_positions, int rot,
                                          const int32_t* positions, const int32_t* row_seq, void* k_pages,
                                          void* v_pages, const int32_t* page_table, int table_stride, int n_rows,
                                          int H, int KVH, int hd, int write_kv, int kv_order, int max_position,
                                          hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && H > 0 && KVH > 0 && hd > 0 && parts > 0, "qk_norm_rope: sizes must be positive");
  BH_REQUIRE((q_weight == nullptr) == (k_weight == nullptr), "qk_norm_rope: give both norm weights or neither");
  BH_REQUIRE(cos_table == nullptr || max_position < table_positions,
             "qk_norm_rope: position %d is outside the rotation table of %d positions", max_position, table_positions);
  BH_REQUIRE(H + 2 * KVH <= 65535, "qk_norm_rope: too many heads");
  BH_REQUIRE(kv_order == BH_KV_ROWS || (kv_order == BH_KV_PIECES && hd % 32 == 0),
             "qk_norm_rope: cache order %d does not exist for head size %d", kv_order, hd);
  if (cos_table == nullptr) rot = 0;
  BH_REQUIRE(qk_rows_form_takes(n_rows, hd, rot),
             "qk_norm_rope: sums in parts are taken for at least 64 rows, heads of 64, 128 or 256 and a rotation over "
             "the whole head or none (rows %d, head %d, rotation %d)", n_rows, hd, rot);
  BH_REQUIRE(((uintptr_t)sums % 16) == 0 && ((long)(H + 2 * KVH) * hd) % 4 == 0, "qk_norm_rope: the sums must be 16-byte aligned");
  return qk_rows_form(sums, parts, q_out, q_weight, k_weight, w_dtype, eps, cos_table, sin_table, rot, positions, row_seq,
                      k_pages, v_pages, page_table, table_stride, n_rows, H, KVH, hd, write_kv, kv_order, stream);
}

// ---- attention over the paged cache, any size -------------------------------------------------
// One block per (row, query head).  The row at position p of sequence s sees keys
// max(0, p - window + 1) .. p of that sequence (window 0: all of them).  Keys are taken 256
// at a time: scores (one thread per key), running maximum and sum in float32 (online softmax),
// then the value sum with threads spread over (key subset, dimension).

#define AG_THREADS 256

template <typename T>
__global__ __launch_bounds__(AG_THREADS) void attention_generic_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int32_t* __restrict__ page_table, int table_stride, const int32_t* __restrict__ row_seq,
    const int32_t* __restrict__ positions, int H, int KVH, int hd, float scale, int window, int kv_order) {
  extern __shared__ float smem[];
  float* qs = smem;                    // [hd]
  float* probs = qs + hd;              // [AG_THREADS]
  float* partial = probs + AG_THREADS; // [AG_THREADS]
  __shared__ float scratch[AG_THREADS / BH_WAVE];

  const int row = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
  const int kv_head = head / (H / KVH);
  const int pos = positions[row];
  const int32_t* table = page_table + (size_t)row_seq[row] * table_stride;
  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;

  const T* qr = q + ((size_t)row * H + head) * hd;
  for (int i = tid; i < hd; i += AG_THREADS) qs[i] = to_f32(qr[i]);
  __syncthreads();

  // value phase: groups of hd threads; group g takes keys g, g + n_groups, ... of a chunk
  const int n_groups = AG_THREADS / hd > 0 ? AG_THREADS / hd : 1;
  const int group = tid / hd, dim = tid % hd;
  const bool value_thread = tid < n_groups * hd;  // hd <= AG_THREADS is checked on the host

  float run_max = -INFINITY, run_sum = 0.f, acc = 0.f;
  for (int c0 = first; c0 <= pos; c0 += AG_THREADS) {
    const int j = c0 + tid;
    float s = -INFINITY;
    if (j <= pos) {
      const int page = table[j / BH_PAGE];
      const T* block = k_pages + ((size_t)page * KVH + kv_head) * BH_PAGE * hd;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], to_f32(block[bh_key_index(kv_order, j % BH_PAGE, d, hd)]), dot);
      s = dot * scale;
    }
    const float chunk_max = block_max(s, scratch);
    const float new_max = fmaxf(run_max, chunk_max);
    const float p = (j <= pos) ? expf(s - new_max) : 0.f;
    probs[tid] = p;
    const float chunk_sum = block_sum(p, scratch);  // its barriers also publish probs[]
    const float alpha = (run_max == -INFINITY) ? 0.f : expf(run_max - new_max);
    run_sum = run_sum * alpha + chunk_sum;
    run_max = new_max;
    if (value_thread) {
      acc *= alpha;
      const int n_keys = (pos - c0 + 1 < AG_THREADS) ? pos - c0 + 1 : AG_THREADS;
      for (int jj = group; jj < n_keys; jj += n_groups) {
        const int key = c0 + jj;
        const int page = table[key / BH_PAGE];
        const T* block = v_pages + ((size_t)page * KVH + kv_head) * BH_PAGE * hd;
        acc = fmaf(probs[jj], to_f32(block[bh_value_index(kv_order, key % BH_PAGE, dim, hd)]), acc);
      }
    }
    __syncthreads();  // probs[] is rewritten by the next chunk
  }
  partial[tid] = value_thread ? acc : 0.f;
  __syncthreads();
  if (tid < hd) {
    float total = 0.f;
    for (int g = 0; g < n_groups; ++g) total += partial[g * hd + tid];
    out[((size_t)row * H + head) * hd + tid] = from_f32<T>(total / run_sum);
  }
}

extern "C" int bh_attention_generic(const void* q, void* out, int dtype, const void* k_pages,
                                    const void* v_pages, const int32_t* page_table, int table_stride,
                                    const int32_t* row_seq, const int32_t* positions, int n_rows, int H,
                                    int KVH, int hd, float scale, int window, int kv_order,
                                    hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && H > 0 && KVH > 0 && hd > 0, "attention: sizes must be positive");
  BH_REQUIRE(H % KVH == 0, "attention: %d query heads do not group evenly into %d kv heads", H, KVH);
  BH_REQUIRE(hd <= AG_THREADS, "attention: head size %d is above the limit of %d", hd, AG_THREADS);
  BH_REQUIRE(H <= 65535, "attention: too many heads");
  BH_REQUIRE(window >= 0, "attention: window must not be negative");
  BH_REQUIRE(kv_order == BH_KV_ROWS || (kv_order == BH_KV_PIECES && hd % 32 == 0),
             "attention: cache order %d does not exist for head size %d", kv_order, hd);
  dim3 grid(n_rows, H), block(AG_THREADS);
  const size_t smem = (size_t)(hd + 2 * AG_THREADS) * sizeof(float);
  if (dtype == BH_F32)
    attention_generic_kernel<float><<<grid, block, smem, stream>>>(
        (const float*)q, (float*)out, (const float*)k_pages, (const float*)v_pages, page_table, table_stride,
        row_seq, positions, H, KVH, hd, scale, window, kv_order);
  else if (dtype == BH_BF16)
    attention_generic_kernel<bf16_t><<<grid, block, smem, stream>>>(
        (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)k_pages, (const bf16_t*)v_pages, page_table,
        table_stride, row_seq, positions, H, KVH, hd, scale, window, kv_order);
  else
    return bh_fail("attention: unknown dtype %d", dtype);
  return bh_check_launch("attention_generic");
}

// ---- SwiGLU ---------------------------------------------------------------------------------
// out[r, i] = silu(gu[r, i]) * gu[r, F + i], silu(x) = x / (1 + exp(-x)).

template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int F, size_t total) {
  const size_t at = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (at >= total) return;
  const size_t r = at / F;
  const int i = (int)(at % F);
  const float g = to_f32(gu[r * 2 * F + i]);
  const float u = to_f32(gu[r * 2 * F + F + i]);
  out[at] = from_f32<T>(g / (1.0f + expf(-g)) * u);
}

extern "C" int bh_swiglu(const void* gu, void* out, int dtype, int n_rows, int F, hipStream_t stream) {
  BH_REQUIRE(n_rows > 0 && F > 0, "swiglu: sizes must be positive");
  const size_t total = (size_t)n_rows * F;
  const size_t blocks = (total + 255) / 256;
  BH_REQUIRE(blocks <= 2147483647u, "swiglu: too many elements");
  dim3 grid((unsigned)blocks), block(256);
  if (dtype == BH_F32)
    swiglu_kernel<float><<<grid, block, 0, stream>>>((const float*)gu, (float*)out, F, total);
  else if (dtype == BH_BF16)
    swiglu_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, F, total);
  else
    return bh_fail("swiglu: unknown dtype %d", dtype);
  return bh_check_launch("swiglu");
}

// ---- activation rows in blocks ---------------------------------------------------------------------
// A bfloat16 matrix [rows][width] into the blocks of 16 rows x 32 columns that products of many rows read
// fastest (bh_blocked_index in layout.h), and back.  One thread moves one piece of 16 bytes (8 columns of a
// row).  Producers that know their reader write the blocks themselves; this is for the ones that do not.
// Rows of the last block that the matrix does not have are filled with zeros.
typedef uint32_t blocked_u32x4_t __attribute__((ext_vector_type(4)));
template <bool TO_BLOCKS>
__global__ __launch_bounds__(256) void rows_blocked_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                           int n_rows, int width, long pieces, int block_rows) {
  const long piece = (long)blockIdx.x * 256 + threadIdx.x;   // in the order of the blocked matrix
  if (piece >= pieces) return;
  const int r = piece % block_rows, q = (piece / block_rows) % 4;
  const long block = piece / (4 * block_rows);
  const int column = (int)(block % (width / 32)) * 32 + 8 * q, row = (int)(block / (width / 32)) * block_rows + r;
  const blocked_u32x4_t zero = {0u, 0u, 0u, 0u};
  if (TO_BLOCKS) {
    reinterpret_cast<blocked_u32x4_t*>(dst)[piece] =
        row < n_rows ? *reinterpret_cast<const blocked_u32x4_t*>(src + (size_t)row * width + column) : zero;
  } else if (row < n_rows) {
    *reinterpret_cast<blocked_u32x4_t*>(dst + (size_t)row * width + column) = reinterpret_cast<const blocked_u32x4_t*>(src)[piece];
  }
}

extern "C" int bh_rows_blocked(const void* src, void* dst, int n_rows, int width, int to_blocks, int block_rows,
                               hipStream_t stream) {
  BH_REQUIRE(src != nullptr && dst != nullptr && n_rows > 0 && width > 0, "rows_blocked: a matrix with rows and a width");
  BH_REQUIRE(width % 32 == 0, "rows_blocked: the width %d must be a multiple of 32", width);
  BH_REQUIRE(block_rows == 8 || block_rows == 16, "rows_blocked: blocks of 8 or 16 rows, not %d", block_rows);
  BH_REQUIRE(((uintptr_t)src | (uintptr_t)dst) % 16 == 0, "rows_blocked: buffers must be 16-byte aligned");
  const long pieces = (long)((n_rows + block_rows - 1) / block_rows) * (width / 32) * 4 * block_rows;
  BH_REQUIRE((pieces + 255) / 256 < (1L << 31), "rows_blocked: too many blocks");
  dim3 grid((unsigned)((pieces + 255) / 256)), block(256);
  if (to_blocks) rows_blocked_kernel<true><<<grid, block, 0, stream>>>((const uint16_t*)src, (uint16_t*)dst, n_rows, width, pieces, block_rows);
  else rows_blocked_kernel<false><<<grid, block, 0, stream>>>((const uint16_t*)src, (uint16_t*)dst, n_rows, width, pieces, block_rows);
  return bh_check_launch("rows_blocked");
}

// ---- a yardstick for the memory system ----------------------------------------------------------
// Not a product kernel: reads `bytes` of device memory once, the way the streaming kernels of this library
// read weights and cache pages (16 bytes a lane, sixteen loads of 1 KB in flight per wave, four waves a
// workgroup, every workgroup a contiguous share), with or without the hint that nobody reads the bytes again
// soon.  Its rate is what a kernel that does nothing but read can reach on this GPU; bench.py --hbm-ceiling
// prints it beside the library routines' rates.
typedef uint32_t bh_u32x4_t __attribute__((ext_vector_type(4)));

template <bool STREAM>
__global__ __launch_bounds__(256) void stream_read_kernel(const uint8_t* __restrict__ data, long per_workgroup,
                                                          uint32_t* __restrict__ sink) {
  const int wave = threadIdx.x / BH_WAVE, lane = threadIdx.x % BH_WAVE;
  const uint8_t* mine = data + (size_t)blockIdx.x * per_workgroup + lane * 16;
  bh_u32x4_t seen = {0u, 0u, 0u, 0u};
  for (long at = (long)wave * 16384; at + 16384 <= per_workgroup; at += 4 * 16384) {
    bh_u32x4_t piece[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const bh_u32x4_t* p = reinterpret_cast<const bh_u32x4_t*>(mine + at + u * 1024);
      piece[u] = STREAM ? __builtin_nontemporal_load(p) : *p;
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) seen ^= piece[u];
  }
  if ((seen[0] ^ seen[1] ^ seen[2] ^ seen[3]) == 0x9e3779b9u) sink[0] = 1;   // keeps the loads alive
}

// Reads the first workgroups * (bytes / workgroups rounded down to 64 KB) bytes; returns that count through `read`.
extern "C" int bh_stream_read(const void* data, long bytes, int workgroups, int nontemporal, void* sink, long* read,
                              hipStream_t stream) {
  BH_REQUIRE(data != nullptr && sink != nullptr && read != nullptr, "stream_read: data, sink and count are required");
  BH_REQUIRE(workgroups > 0 && bytes >= (long)workgroups * 65536, "stream_read: at least 64 KB per workgroup");
  const long per_workgroup = bytes / workgroups / 65536 * 65536;
  *read = per_workgroup * workgroups;
  if (nontemporal) stream_read_kernel<true><<<dim3(workgroups), dim3(256), 0, stream>>>((const uint8_t*)data, per_workgroup, (uint32_t*)sink);
  else stream_read_kernel<false><<<dim3(workgroups), dim3(256), 0, stream>>>((const uint8_t*)data, per_workgroup, (uint32_t*)sink);
  return bh_check_launch("stream_read");
}
