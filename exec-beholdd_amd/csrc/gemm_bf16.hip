// bfloat16 matrix products on the gfx950 matrix cores: C[M, N] (+)= A[M, K] * W[N, K]^T,
// float32 accumulation, C in float32 or bfloat16.
//
// Two kernels.
//   skinny (M <= 64, the decode shapes): the product is bound by reading W once from HBM.  A
//     workgroup owns 16 rows of W; its waves split K between them in 64-wide chunks, each lane
//     reading 32 contiguous bytes of a row so that four lanes cover a 128-byte line, and feed
//     v_mfma_f32_16x16x32_bf16 with W as the row operand and the activations as the column
//     operand; the waves' partial tiles are summed through LDS in a fixed order.
//   tiled (M > 64, the prefill shapes): 128x128 output tile per workgroup of four waves, 64-wide
//     k slices staged through padded LDS with the next slice's global loads in flight during
//     the multiplies; v_mfma_f32_32x32x16_bf16, each wave a 64x64 quarter.
// K must be a multiple of 8 (16-byte loads); other sizes are free.
//
// Operand layouts relied on (wave of 64 lanes, l = lane):
//   16x16x32: A row l%16, k 8*(l/16)..+7;  B column l%16, the same k;  D column l%16, rows 4*(l/16)..+3
//   32x32x16: A row l%32, k 8*(l/32)..+7;  B column l%32, the same k;  D column l%32,
//             rows 8*(i/4) + 4*(l/32) + i%4 for i = 0..15
// Which 8 of the k values a lane group multiplies is free as long as both operands agree.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__device__ inline bf16x8_t as_bf16x8(u32x4_t v) { return __builtin_bit_cast(bf16x8_t, v); }

__device__ inline u32x4_t load16(const uint16_t* p) { return *reinterpret_cast<const u32x4_t*>(p); }
__device__ inline u32x4_t load16_stream(const uint16_t* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
}

template <typename TC>
__device__ inline void store_out(TC* c, size_t at, float v, bool accumulate);
template <>
__device__ inline void store_out<float>(float* c, size_t at, float v, bool accumulate) {
  c[at] = accumulate ? c[at] + v : v;
}
template <>
__device__ inline void store_out<bf16_t>(bf16_t* c, size_t at, float v, bool accumulate) {
  if (accumulate) v += to_f32(c[at]);
  c[at] = from_f32<bf16_t>(v);
}

// ---- skinny --------------------------------------------------------------------------------

template <int MB, int WAVES, typename TC>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const uint16_t* __restrict__ a,
                                                                 const uint16_t* __restrict__ w,
                                                                 TC* __restrict__ c, int M, int N, int K,
                                                                 int accumulate) {
  __shared__ float partial[WAVES][MB][256];
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int i = lane % 16, g = lane / 16;
  const int n0 = blockIdx.x * 16;
  const int w_row = (n0 + i < N) ? n0 + i : N - 1;
  const uint16_t* wp = w + (size_t)w_row * K + g * 16;
  const uint16_t* xp[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    const int row = (b * 16 + i < M) ? b * 16 + i : M - 1;
    xp[b] = a + (size_t)row * K + g * 16;
  }
  f32x4_t acc[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) acc[b] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const int full = K / 64;
  int chunk = wave;
  // U chunks per trip, all their loads issued before the first multiply, to keep bytes in flight
  constexpr int U = MB <= 2 ? 4 : 2;
  for (; chunk + (U - 1) * WAVES < full; chunk += U * WAVES) {
    u32x4_t wv[U][2], xv[U][MB][2];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (chunk + u * WAVES) * 64;
      wv[u][0] = load16_stream(wp + k);
      wv[u][1] = load16_stream(wp + k + 8);
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        xv[u][b][0] = load16(xp[b] + k);
        xv[u][b][1] = load16(xp[b] + k + 8);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wv[u][0]), as_bf16x8(xv[u][b][0]), acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wv[u][1]), as_bf16x8(xv[u][b][1]), acc[b], 0, 0, 0);
      }
  }
  for (; chunk < full; chunk += WAVES) {
    const int k = chunk * 64;
    const u32x4_t w0 = load16_stream(wp + k), w1 = load16_stream(wp + k + 8);
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      const u32x4_t x0 = load16(xp[b] + k), x1 = load16(xp[b] + k + 8);
      acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(w0), as_bf16x8(x0), acc[b], 0, 0, 0);
      acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(w1), as_bf16x8(x1), acc[b], 0, 0, 0);
    }
  }
  if (chunk == full && full * 64 < K) {  // the last, partial chunk: 8-element pieces beyond K are zero
    const int k = full * 64, at = k + g * 16;
    const u32x4_t zero = {0u, 0u, 0u, 0u};
    const u32x4_t w0 = at < K ? load16_stream(wp + k) : zero, w1 = at + 8 < K ? load16_stream(wp + k + 8) : zero;
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      const u32x4_t x0 = at < K ? load16(xp[b] + k) : zero, x1 = at + 8 < K ? load16(xp[b] + k + 8) : zero;
      acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(w0), as_bf16x8(x0), acc[b], 0, 0, 0);
      acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(w1), as_bf16x8(x1), acc[b], 0, 0, 0);
    }
  }
  // D: lane holds column (activation row) i and rows (W rows) 4g..4g+3; lay it out as [m][n]
#pragma unroll
  for (int b = 0; b < MB; ++b)
#pragma unroll
    for (int r = 0; r < 4; ++r) partial[wave][b][i * 16 + 4 * g + r] = acc[b][r];
  __syncthreads();
  for (int e = threadIdx.x; e < MB * 256; e += WAVES * 64) {
    const int b = e / 256, m = b * 16 + (e % 256) / 16, n = n0 + e % 16;
    if (m >= M || n >= N) continue;
    float sum = 0.f;
#pragma unroll
    for (int v = 0; v < WAVES; ++v) sum += partial[v][b][e % 256];
    store_out<TC>(c, (size_t)m * N + n, sum, accumulate != 0);
  }
}

template <int MB, typename TC>
static void launch_skinny(const void* a, const void* w, void* c, int M, int N, int K, int accumulate,
                          hipStream_t stream) {
  constexpr int WAVES = 8;
  dim3 grid((N + 15) / 16), block(WAVES * 64);
  gemm_skinny_kernel<MB, WAVES, TC><<<grid, block, 0, stream>>>((const uint16_t*)a, (const uint16_t*)w, (TC*)c, M,
                                                                N, K, accumulate);
}

// ---- tiled -----------------------------------------------------------------------------------

#define TB 128          // output tile edge
#define TK 64           // k slice
#define TPITCH (TK + 8) // LDS row pitch in elements: 144 bytes, so 16-byte reads of 16 rows hit 64 distinct banks

template <typename TC>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const uint16_t* __restrict__ a,
                                                         const uint16_t* __restrict__ w, TC* __restrict__ c,
                                                         int M, int N, int K, int accumulate) {
  __shared__ __attribute__((aligned(16))) uint16_t as[2][TB * TPITCH];
  __shared__ __attribute__((aligned(16))) uint16_t ws[2][TB * TPITCH];
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int m0 = blockIdx.y * TB, n0 = blockIdx.x * TB;
  const int wm = (wave / 2) * 64, wn = (wave % 2) * 64;  // this wave's quarter of the tile

  // global -> LDS staging: a slice is 128 rows x 8 pieces of 16 bytes; a thread moves 4 pieces per operand
  int st_row[4], st_piece[4];
  const uint16_t* a_src[4];
  const uint16_t* w_src[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int e = tid + s * 256;
    st_row[s] = e / 8;
    st_piece[s] = e % 8;
    const int am = (m0 + st_row[s] < M) ? m0 + st_row[s] : M - 1;
    const int wr = (n0 + st_row[s] < N) ? n0 + st_row[s] : N - 1;
    a_src[s] = a + (size_t)am * K + st_piece[s] * 8;
    w_src[s] = w + (size_t)wr * K + st_piece[s] * 8;
  }
  u32x4_t a_reg[4], w_reg[4];
  const u32x4_t zero = {0u, 0u, 0u, 0u};
  auto fetch = [&](int k0) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const bool inside = k0 + st_piece[s] * 8 < K;
      a_reg[s] = inside ? load16(a_src[s] + k0) : zero;
      w_reg[s] = inside ? load16(w_src[s] + k0) : zero;
    }
  };
  auto stash = [&](int buffer) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int at = st_row[s] * TPITCH + st_piece[s] * 8;
      *reinterpret_cast<u32x4_t*>(&as[buffer][at]) = a_reg[s];
      *reinterpret_cast<u32x4_t*>(&ws[buffer][at]) = w_reg[s];
    }
  };

  f32x16_t acc[2][2];
#pragma unroll
  for (int x = 0; x < 2; ++x)
#pragma unroll
    for (int y = 0; y < 2; ++y)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[x][y][e] = 0.f;

  const int slices = (K + TK - 1) / TK;
  fetch(0);
  stash(0);
  __syncthreads();
  const int frag_row = lane % 32, frag_k = (lane / 32) * 8;
  for (int s = 0; s < slices; ++s) {
    const int buffer = s & 1;
    if (s + 1 < slices) fetch((s + 1) * TK);
#pragma unroll
    for (int kk = 0; kk < TK; kk += 16) {
      bf16x8_t af[2], wf[2];
#pragma unroll
      for (int x = 0; x < 2; ++x)
        af[x] = as_bf16x8(*reinterpret_cast<const u32x4_t*>(&as[buffer][(wm + x * 32 + frag_row) * TPITCH + kk + frag_k]));
#pragma unroll
      for (int y = 0; y < 2; ++y)
        wf[y] = as_bf16x8(*reinterpret_cast<const u32x4_t*>(&ws[buffer][(wn + y * 32 + frag_row) * TPITCH + kk + frag_k]));
#pragma unroll
      for (int x = 0; x < 2; ++x)
#pragma unroll
        for (int y = 0; y < 2; ++y)
          acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[x], wf[y], acc[x][y], 0, 0, 0);
    }
    if (s + 1 < slices) stash(buffer ^ 1);
    __syncthreads();
  }
  // D of one 32x32 block: column (n) lane%32, rows (m) 8*(e/4) + 4*(lane/32) + e%4
#pragma unroll
  for (int x = 0; x < 2; ++x)
#pragma unroll
    for (int y = 0; y < 2; ++y) {
      const int n = n0 + wn + y * 32 + lane % 32;
      if (n >= N) continue;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = m0 + wm + x * 32 + 8 * (e / 4) + 4 * (lane / 32) + e % 4;
        if (m < M) store_out<TC>(c, (size_t)m * N + n, acc[x][y][e], accumulate != 0);
      }
    }
}

// ---- entry -------------------------------------------------------------------------------------

extern "C" int bh_gemm_bf16(const void* a, const void* w, void* c, int c_dtype, int accumulate, int M, int N, int K,
                            hipStream_t stream) {
  BH_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_bf16: sizes M=%d N=%d K=%d must be positive", M, N, K);
  BH_REQUIRE(K % 8 == 0, "gemm_bf16: K=%d must be a multiple of 8", K);
  BH_REQUIRE(c_dtype == BH_F32 || c_dtype == BH_BF16, "gemm_bf16: unknown output dtype %d", c_dtype);
  BH_REQUIRE(((uintptr_t)a | (uintptr_t)w) % 16 == 0, "gemm_bf16: operands must be 16-byte aligned");
  if (M <= 64) {
    const int blocks = (M + 15) / 16;
#define BH_SKINNY(MB)                                                                               \
  if (c_dtype == BH_F32) launch_skinny<MB, float>(a, w, c, M, N, K, accumulate, stream);             \
  else launch_skinny<MB, bf16_t>(a, w, c, M, N, K, accumulate, stream)
    if (blocks == 1) { BH_SKINNY(1); }
    else if (blocks == 2) { BH_SKINNY(2); }
    else if (blocks == 3) { BH_SKINNY(3); }
    else { BH_SKINNY(4); }
#undef BH_SKINNY
    return bh_check_launch("gemm_skinny");
  }
  const int row_tiles = (M + TB - 1) / TB;
  BH_REQUIRE(row_tiles <= 65535, "gemm_bf16: M=%d needs more than 65535 row tiles", M);
  dim3 grid((N + TB - 1) / TB, row_tiles), block(256);
  if (c_dtype == BH_F32)
    gemm_tiled_kernel<float><<<grid, block, 0, stream>>>((const uint16_t*)a, (const uint16_t*)w, (float*)c, M, N, K,
                                                         accumulate);
  else
    gemm_tiled_kernel<bf16_t><<<grid, block, 0, stream>>>((const uint16_t*)a, (const uint16_t*)w, (bf16_t*)c, M, N,
                                                          K, accumulate);
  return bh_check_launch("gemm_tiled");
}
