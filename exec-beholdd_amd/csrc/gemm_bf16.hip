// bfloat16 matrix products on the gfx950 matrix cores: C[M, N] (+)= A[M, K] * W[N, K]^T,
// float32 accumulation, C in float32 or bfloat16; optionally C[M, F] = silu(A Wg^T) * (A Wu^T)
// for W = [Wg; Wu] stacked (the SwiGLU feed-forward's first half in one pass).
//
// Weight layouts.  `rows`: W as checkpoints store it, [N, K] row-major.  `tiles`: the same
// numbers regrouped at load time into blocks of 16 rows x 64 k, block (nb, kb) at
// (nb * K/64 + kb) * 1024 elements, and inside a block [half u][lane l][8] with
// row = l % 16, k = 16 * (l / 16) + 8 * u + e.  A wave then reads a block as two fully
// contiguous 1 KB loads that are already in matrix-core operand order; streaming a weight once
// from HBM (decode) runs about a third faster from this layout than from strided rows.
// Tiles need K % 64 == 0; rows beyond N in the last block are zero.
//
// Two ways, by the number of rows M.
//   skinny (M <= 16; up to 64 where the tiled way below does not take the shape): bound by reading W once.
//     A workgroup owns 16 rows of W (a gate block and its up block for SwiGLU); its 8 waves split K in
//     64-wide chunks and feed v_mfma_f32_16x16x32_bf16 with W as the row operand and the activations as the
//     column operand; the waves' partial tiles are summed through LDS in a fixed order.
//   tiled (M > 16): output tiles of 32 x 128, 64 x 128, 128 x 128 (four waves) or 256 x 256 (eight), 64-wide
//     k slices staged through padded LDS (one or two buffers) with the next slice's global loads in flight
//     during the multiplies; v_mfma_f32_32x32x16_bf16.  For SwiGLU a wave's columns are the gate and the up
//     columns of the same outputs.  `gemm_tiled_whole_kernel` is the variant for whole tiles of the tiles
//     layout: it can carry a norm (struct RidingNorm), and where the tiles are too few to fill the chip
//     (17 to about 512 rows at these widths) it cuts K into parts over workgroups and a finishing kernel adds
//     them (needs scratch memory).  `gemm_tiled_kernel` takes every shape and both layouts.
// K must be a multiple of 8 (16-byte loads); other sizes are free.
//
// Operand layouts relied on (wave of 64 lanes, l = lane):
//   16x16x32: A row l%16, k 8*(l/16)..+7;  B column l%16, the same k;  D column l%16, rows 4*(l/16)..+3
//   32x32x16: A row l%32, k 8*(l/32)..+7;  B column l%32, the same k;  D column l%32,
//             rows 8*(i/4) + 4*(l/32) + i%4 for i = 0..15
// Which 8 of the k values a lane group multiplies is free as long as both operands agree.
#include "common.h"
#include "gemm_bf16_slices.h"
#include "gemm_bf16_turns.h"
#include <algorithm>
#include <type_traits>

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

__device__ inline float silu_mul(float gate, float up) { return gate / (1.0f + expf(-gate)) * up; }

// every lane's value of the lane eight further on in its group of 16 (lanes 8 to 15: nothing that matters)
__device__ inline u32x4_t from_lane_plus_8(u32x4_t v) {
  u32x4_t out;
#pragma unroll
  for (int word = 0; word < 4; ++word)
    out[word] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v[word], 0x108 /* row_shl:8 */, 0xf, 0xf, true);
  return out;
}

#define MFMA16(a, b, c) __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a), as_bf16x8(b), c, 0, 0, 0)

// ---- skinny --------------------------------------------------------------------------------
// RT = 1: plain product.  RT = 2: SwiGLU; the second row block lies `pair_blocks` blocks after the first.

// An RMSNorm between two products can ride on them (struct RidingNorm):
//   behind: the product that completes the float32 residual h also writes bfloat16(h[m][n] * g[n]) (the
//           norm's output but for the row factor) and, per workgroup, the sum of h[m][n]^2 over its
//           columns (16 of them in the skinny kernel, 64 in the finishing kernel, a tile's width in whole tiles);
//   ahead:  the product that consumes the norm's output takes those unscaled rows as its activations and
//           multiplies its result by 1 / sqrt(sum of the partial sums / K + eps) of the row.
// The row factor commutes with the product, so the result is the norm's up to the rounding of the
// activations; the partial sums are added in a fixed order.  The skinny kernel and whole tiles (with or
// without the finishing kernel) do this; the tiled kernel for every shape does not.
struct RidingNorm {
  const float* ahead_ss;   // [M][ahead_blocks] partial sums of squares for the rows of `a`, or null
  int ahead_blocks;
  float ahead_eps;
  const void* behind_weight;  // [N] norm weight for the rows this product completes, or null
  int behind_weight_f32;      // its element type: float32, else bfloat16
  uint16_t* behind_rows;      // [M][N] bfloat16 out
  float* behind_ss;           // [M][bh_gemm_bf16_norm_blocks()] out
};

// Rows in blocks (bh_rows_index in layout.h; 0: rows one after the other) for the skinny kernel's bfloat16
// matrices: its activations, its output (SwiGLU's, which the next product reads) and the rows it prepares for a
// norm behind it.  A lane's two loads of a 64-wide chunk of activations then are the pieces 2 g and 2 g + 1 of the
// chunk's two 32-wide steps: 16 lanes read 256 contiguous bytes (128 with blocks of 8 rows, where the lanes of
// rows 8 to 15 read what the first eight read) instead of 64 bytes from each of 16 rows, which weighs as much as
// the weights' loads do: the eight waves of every workgroup read all of the activations.
// Measured (Qwen3-8B sizes, us per product, qkv / o / gate+up / down): 8 rows 12.7 / 9.2 / 34.1 / 21.0 -> 11.4 /
// 8.6 / 33.7 / 19.9; 16 rows 15.3 / 10.4 / 35.9 / 24.2 -> 12.4 / 8.9 / 33.1 / 20.4; 32 rows (tiles with K in
// parts before) 16.2 / 12.6 / 49.4 / 26.4 -> 14.9 / 10.0 / 40.5 / 23.1; 48 rows 18.2 / 14.3 / 50.1 / 28.7 -> 18.6 /
// 11.8 / 46.0 / 28.4; at 64 rows the tiles are as fast.  (Each product alone; inside a decode step 48 rows did not
// gain, see SKINNY_UP_TO_ROWS, and a single row, which alone is read as fast as it lies (10.9 / 8.4 / 33.7 / 19.6
// against 11.2 / 8.6 / 33.8 / 19.9), did: the step of one sequence 3.61 -> 3.55 ms, of two 3.79 -> 3.71.)
struct RowBlocks {
  int a, c, behind;
};

// XB: the rows per block of the activations (RowBlocks::a), known when the kernel is compiled: as a number that
// only the launch knows it cost the kernel for rows 2 % of a decode step.
template <int MB, int WAVES, bool TILES, int RT, typename TC, int XB = 0>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const uint16_t* __restrict__ a,
                                                                 const uint16_t* __restrict__ w,
                                                                 TC* __restrict__ c, int M, int N, int K,
                                                                 int accumulate, int pair_blocks,
                                                                 RidingNorm norm, RowBlocks blocks) {
  __shared__ float partial[WAVES][RT][MB][256];
  __shared__ float row_factor[MB * 16];
  // The norm ahead: 32 threads per row, each with every 32nd partial sum.  The first 256 of a row are asked
  // for here and added up after the product's main loop, so that nobody waits for them.
  constexpr int ROWS_PER_PASS = WAVES * 2, PASSES = (MB * 16 + ROWS_PER_PASS - 1) / ROWS_PER_PASS;
  const int part = threadIdx.x % 32;
  float early[PASSES][8];
  if (norm.ahead_ss) {
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
      const int r = pass * ROWS_PER_PASS + threadIdx.x / 32;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int block = part + 32 * u;
        early[pass][u] = (r < M && block < norm.ahead_blocks) ? norm.ahead_ss[(size_t)r * norm.ahead_blocks + block] : 0.f;
      }
    }
  }
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int i = lane % 16, g = lane / 16;
  const int n0 = blockIdx.x * 16;
  const int full = K / 64;
  // What a float32 output holds before this product adds to it, and the weight of the norm behind: each thread knows
  // the elements it will write, and asks for them here, so that nobody waits for them behind the main loop (the
  // residual was written by another kernel, on other XCDs: it comes from beyond this XCD's L2).
  constexpr int OUT_PASSES = (MB * 256 + WAVES * 64 - 1) / (WAVES * 64);
  constexpr bool OUT_EARLY = RT == 1 && sizeof(TC) == 4;
  float before[OUT_PASSES], behind_gain[OUT_PASSES];
  if (OUT_EARLY) {
#pragma unroll
    for (int pass = 0; pass < OUT_PASSES; ++pass) {
      const int e = threadIdx.x + pass * WAVES * 64;
      const int m = e / 256 * 16 + (e % 256) / 16, n = n0 + e % 16;
      const bool valid = e < MB * 256 && m < M && n < N;
      before[pass] = (valid && accumulate) ? reinterpret_cast<const float*>(c)[(size_t)m * N + n] : 0.f;
      behind_gain[pass] = 0.f;
      if (valid && norm.behind_weight)
        behind_gain[pass] = norm.behind_weight_f32 ? reinterpret_cast<const float*>(norm.behind_weight)[n]
                                                   : bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(norm.behind_weight)[n]);
    }
  }
  // per row block: base pointer, distance between consecutive 64-wide chunks, distance to the second half
  const uint16_t* wp[RT];
  const size_t chunk_stride = TILES ? 1024 : 64;
  const int half_offset = TILES ? 512 : 8;
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const int block = blockIdx.x + t * pair_blocks;
    if (TILES) {
      wp[t] = w + (size_t)block * full * 1024 + lane * 8;
    } else {
      const int rows = RT == 2 ? 2 * N : N;  // SwiGLU: N counts outputs, W has twice as many rows
      const int row = (block * 16 + i < rows) ? block * 16 + i : rows - 1;
      wp[t] = w + (size_t)row * K + g * 16;
    }
  }
  const uint16_t* xp[MB];
  // from a chunk's first piece of this lane to its second, and to the next chunk
  constexpr int x_half = XB ? XB * 8 : 8, x_chunk = XB ? 64 * XB : 64;
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    if (XB) {   // piece p = 2 g + u of a chunk is lane group p % 4 of its step p / 4
      constexpr int step = 32 * (XB ? XB : 1);
      // (blocks of 8 rows: lanes 8 to 15 of a group take the second piece of rows 0 to 7, which lies right behind
      // the first pieces, so that one load brings both and a lane move hands the second to the lane of its row)
      xp[b] = a + (size_t)(b * 16 / (XB ? XB : 1)) * (K / 32) * step + (g / 2) * step + ((2 * g) % 4 * XB + (XB == 8 ? i : i % (XB ? XB : 1))) * 8;
    } else {
      const int row = (b * 16 + i < M) ? b * 16 + i : M - 1;
      xp[b] = a + (size_t)row * K + g * 16;
    }
  }
  f32x4_t acc[RT][MB];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[t][b] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  int chunk = wave;
  // U chunks per trip, all their loads issued before the first multiply, to keep bytes in flight
  constexpr int U = (MB * RT <= 2) ? 4 : (MB * RT <= 4 ? (MB == 4 ? 4 : 2) : 2);
  for (; chunk + (U - 1) * WAVES < full; chunk += U * WAVES) {
    u32x4_t wv[U][RT][2], xv[U][MB][2];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int at = chunk + u * WAVES;
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        const uint16_t* p = wp[t] + (size_t)at * chunk_stride;
        wv[u][t][0] = TILES ? load16_stream(p) : load16(p);
        wv[u][t][1] = TILES ? load16_stream(p + half_offset) : load16(p + half_offset);
      }
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        xv[u][b][0] = load16(xp[b] + at * x_chunk);
        if (XB != 8) xv[u][b][1] = load16(xp[b] + at * x_chunk + x_half);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int b = 0; b < MB; ++b) {
          if (XB == 8 && t == 0) xv[u][b][1] = from_lane_plus_8(xv[u][b][0]);
          acc[t][b] = MFMA16(wv[u][t][0], xv[u][b][0], acc[t][b]);
          acc[t][b] = MFMA16(wv[u][t][1], xv[u][b][1], acc[t][b]);
        }
  }
  for (; chunk < full; chunk += WAVES) {
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const uint16_t* p = wp[t] + (size_t)chunk * chunk_stride;
      const u32x4_t w0 = load16(p), w1 = load16(p + half_offset);
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        const u32x4_t x0 = load16(xp[b] + chunk * x_chunk);
        const u32x4_t x1 = XB == 8 ? from_lane_plus_8(x0) : load16(xp[b] + chunk * x_chunk + x_half);
        acc[t][b] = MFMA16(w0, x0, acc[t][b]);
        acc[t][b] = MFMA16(w1, x1, acc[t][b]);
      }
    }
  }
  if (!TILES && chunk == full && full * 64 < K) {  // rows layout: the last, partial chunk; pieces beyond K are zero
    const int k = full * 64, at = k + g * 16;
    const u32x4_t zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const u32x4_t w0 = at < K ? load16(wp[t] + k) : zero, w1 = at + 8 < K ? load16(wp[t] + k + 8) : zero;
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        const u32x4_t x0 = at < K ? load16(xp[b] + k) : zero, x1 = at + 8 < K ? load16(xp[b] + k + 8) : zero;
        acc[t][b] = MFMA16(w0, x0, acc[t][b]);
        acc[t][b] = MFMA16(w1, x1, acc[t][b]);
      }
    }
  }
  if (norm.ahead_ss) {
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
      const int r = pass * ROWS_PER_PASS + threadIdx.x / 32;
      float ss = 0.f;
#pragma unroll
      for (int u = 0; u < 8; ++u) ss += early[pass][u];
      if (r < M)
        for (int block = part + 256; block < norm.ahead_blocks; block += 32) ss += norm.ahead_ss[(size_t)r * norm.ahead_blocks + block];
#pragma unroll
      for (int off = 16; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
      if (part == 0 && r < MB * 16) row_factor[r] = (r < M) ? 1.0f / sqrtf(ss / (float)K + norm.ahead_eps) : 0.f;
    }
  }
  // D: lane holds column (activation row) i and rows (W rows) 4g..4g+3; lay it out as [m][n]
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int b = 0; b < MB; ++b)
#pragma unroll
      for (int r = 0; r < 4; ++r) partial[wave][t][b][i * 16 + 4 * g + r] = acc[t][b][r];
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < OUT_PASSES; ++pass) {
    const int e = threadIdx.x + pass * WAVES * 64;
    if (e >= MB * 256) break;   // whole waves enter or stay out
    const int b = e / 256, m = b * 16 + (e % 256) / 16, n = n0 + e % 16;
    const bool valid = m < M && n < N;
    float sum[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      sum[t] = 0.f;
#pragma unroll
      for (int v = 0; v < WAVES; ++v) sum[t] += partial[v][t][b][e % 256];
      if (norm.ahead_ss) sum[t] *= row_factor[m];
    }
    float value = 0.f;   // what the residual holds afterwards (norm.behind_weight: float32 output, RT == 1)
    if (valid) {
      if (RT == 2) {
        store_out<TC>(c, (size_t)bh_rows_index(blocks.c, m, n, N), silu_mul(sum[0], sum[RT - 1]), false);
      } else if (OUT_EARLY) {
        value = accumulate ? before[pass] + sum[0] : sum[0];
        reinterpret_cast<float*>(c)[(size_t)m * N + n] = value;
      } else {
        store_out<TC>(c, (size_t)m * N + n, sum[0], accumulate != 0);
      }
    }
    if (RT == 1 && norm.behind_weight) {   // (float32 output)
      float sq = value * value;   // 0 where there is no element
      sq += __shfl_xor(sq, 8, 64);   // the 16 columns of a row sit in 16 neighbouring lanes
      sq += __shfl_xor(sq, 4, 64);
      sq += __shfl_xor(sq, 2, 64);
      sq += __shfl_xor(sq, 1, 64);
      if (valid) {
        norm.behind_rows[bh_rows_index(blocks.behind, m, n, N)] = f32_to_bf16_bits(value * behind_gain[pass]);
        if (e % 16 == 0) norm.behind_ss[(size_t)m * gridDim.x + blockIdx.x] = sq;
      }
    }
  }
}

// The skinny product of packed weights with workgroups that own 20 or 24 weight rows instead of 16 (parts of two
// neighbouring blocks of the packed layout), for products whose blocks of 16 rows are
// more than the compute units but fewer than twice as many: a quarter of the compute units would carry two blocks,
// the others one, and the product takes as long as one with twice the compute units' blocks (Qwen3-14B's down
// projection, 5120 x 17408 at 8 rows: 40.3 us, where 4096 x 17408 takes 25.4 and 8192 x 17408 47.2; with spans of
// 20 rows 35.3 us, at 32 rows 59.6 -> 48.6; Qwen3-32B's, 5120 x 25600: 57.8 -> 49.9 and 86.8 -> 68.1; decode steps of 8,
// 16 and 32 sequences at the 14B sizes 3 to 5 % faster, at the 32B sizes 6 to 8 %).  A lane asks
// only for the rows its workgroup owns (the rows of a block lie side by side, 16 bytes each, so these are runs of 64
// bytes and more), multiplies every block it touches and keeps what it owns.  Workgroups that run on one XCD own
// neighbouring rows, so that a line of the weights that two of them share is fetched into that L2 once.  RT = 1 only.
#define SPAN_TILES 2
template <int MB, int WAVES, typename TC, int XB>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_span_kernel(const uint16_t* __restrict__ a,
                                                                      const uint16_t* __restrict__ w,
                                                                      TC* __restrict__ c, int M, int N, int K,
                                                                      int accumulate, int span, RidingNorm norm,
                                                                      RowBlocks blocks) {
  __shared__ float partial[WAVES][SPAN_TILES][MB][256];
  __shared__ float row_factor[MB * 16];
  constexpr int ROWS_PER_PASS = WAVES * 2, PASSES = (MB * 16 + ROWS_PER_PASS - 1) / ROWS_PER_PASS;
  const int part = threadIdx.x % 32;
  float early[PASSES][8];
  if (norm.ahead_ss) {
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
      const int r = pass * ROWS_PER_PASS + threadIdx.x / 32;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int block = part + 32 * u;
        early[pass][u] = (r < M && block < norm.ahead_blocks) ? norm.ahead_ss[(size_t)r * norm.ahead_blocks + block] : 0.f;
      }
    }
  }
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int i = lane % 16, g = lane / 16;
  const int full = K / 64;
  // workgroups go to the XCDs in turn: the ones of an XCD own a run of neighbouring spans
  const int owner = gridDim.x % 8 == 0 ? (int)(blockIdx.x % 8) * (int)(gridDim.x / 8) + (int)(blockIdx.x / 8) : (int)blockIdx.x;
  const int first_row = owner * span, first_tile = first_row / 16;
  int lo[SPAN_TILES], hi[SPAN_TILES];   // the rows of each block that this workgroup owns: lo <= row < hi (none: hi <= lo)
  const uint16_t* wp[SPAN_TILES];
#pragma unroll
  for (int t = 0; t < SPAN_TILES; ++t) {
    const int tile_row = (first_tile + t) * 16;
    lo[t] = max(first_row, tile_row) - tile_row;
    hi[t] = min(min(first_row + span, N), tile_row + 16) - tile_row;
    const int tile = min(first_tile + t, N / 16 - 1);   // (a block beyond the matrix is never loaded; its address stays inside)
    wp[t] = w + (size_t)tile * full * 1024 + lane * 8;
  }
  // what a float32 output holds before this product adds to it, and the weight of the norm behind, asked for here as
  // in the kernel above
  constexpr int OUT_PASSES = (MB * 256 + WAVES * 64 - 1) / (WAVES * 64);
  constexpr bool OUT_EARLY = sizeof(TC) == 4;
  float before[OUT_PASSES][SPAN_TILES], behind_gain[OUT_PASSES][SPAN_TILES];
  if (OUT_EARLY) {
#pragma unroll
    for (int pass = 0; pass < OUT_PASSES; ++pass)
#pragma unroll
      for (int t = 0; t < SPAN_TILES; ++t) {
        const int e = threadIdx.x + pass * WAVES * 64;
        const int m = e / 256 * 16 + (e % 256) / 16, column = e % 16, n = (first_tile + t) * 16 + column;
        const bool valid = e < MB * 256 && m < M && column >= lo[t] && column < hi[t];
        before[pass][t] = (valid && accumulate) ? reinterpret_cast<const float*>(c)[(size_t)m * N + n] : 0.f;
        behind_gain[pass][t] = 0.f;
        if (valid && norm.behind_weight)
          behind_gain[pass][t] = norm.behind_weight_f32 ? reinterpret_cast<const float*>(norm.behind_weight)[n]
                                                        : bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(norm.behind_weight)[n]);
      }
  }
  const uint16_t* xp[MB];
  constexpr int x_half = XB ? XB * 8 : 8, x_chunk = XB ? 64 * XB : 64;
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    if (XB) {
      constexpr int step = 32 * (XB ? XB : 1);
      xp[b] = a + (size_t)(b * 16 / (XB ? XB : 1)) * (K / 32) * step + (g / 2) * step + ((2 * g) % 4 * XB + (XB == 8 ? i : i % (XB ? XB : 1))) * 8;
    } else {
      const int row = (b * 16 + i < M) ? b * 16 + i : M - 1;
      xp[b] = a + (size_t)row * K + g * 16;
    }
  }
  f32x4_t acc[SPAN_TILES][MB];
#pragma unroll
  for (int t = 0; t < SPAN_TILES; ++t)
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[t][b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const u32x4_t zero = {0u, 0u, 0u, 0u};
  bool mine[SPAN_TILES];
#pragma unroll
  for (int t = 0; t < SPAN_TILES; ++t) mine[t] = i >= lo[t] && i < hi[t];

  constexpr int U = MB == 1 ? 4 : 2;   // chunks per trip, all their loads issued before the first multiply
  int chunk = wave;
  for (; chunk + (U - 1) * WAVES < full; chunk += U * WAVES) {
    u32x4_t wv[U][SPAN_TILES][2], xv[U][MB][2];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int at = chunk + u * WAVES;
#pragma unroll
      for (int t = 0; t < SPAN_TILES; ++t) {
        const uint16_t* p = wp[t] + (size_t)at * 1024;
        wv[u][t][0] = mine[t] ? load16_stream(p) : zero;
        wv[u][t][1] = mine[t] ? load16_stream(p + 512) : zero;
      }
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        xv[u][b][0] = load16(xp[b] + at * x_chunk);
        if (XB != 8) xv[u][b][1] = load16(xp[b] + at * x_chunk + x_half);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        if (XB == 8) xv[u][b][1] = from_lane_plus_8(xv[u][b][0]);
#pragma unroll
        for (int t = 0; t < SPAN_TILES; ++t) {
          if (hi[t] <= lo[t]) continue;   // the same for the whole workgroup
          acc[t][b] = MFMA16(wv[u][t][0], xv[u][b][0], acc[t][b]);
          acc[t][b] = MFMA16(wv[u][t][1], xv[u][b][1], acc[t][b]);
        }
      }
  }
  for (; chunk < full; chunk += WAVES) {
    u32x4_t x0[MB], x1[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      x0[b] = load16(xp[b] + chunk * x_chunk);
      x1[b] = XB == 8 ? from_lane_plus_8(x0[b]) : load16(xp[b] + chunk * x_chunk + x_half);
    }
#pragma unroll
    for (int t = 0; t < SPAN_TILES; ++t) {
      if (hi[t] <= lo[t]) continue;
      const uint16_t* p = wp[t] + (size_t)chunk * 1024;
      const u32x4_t w0 = mine[t] ? load16(p) : zero, w1 = mine[t] ? load16(p + 512) : zero;
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        acc[t][b] = MFMA16(w0, x0[b], acc[t][b]);
        acc[t][b] = MFMA16(w1, x1[b], acc[t][b]);
      }
    }
  }
  if (norm.ahead_ss) {
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
      const int r = pass * ROWS_PER_PASS + threadIdx.x / 32;
      float ss = 0.f;
#pragma unroll
      for (int u = 0; u < 8; ++u) ss += early[pass][u];
      if (r < M)
        for (int block = part + 256; block < norm.ahead_blocks; block += 32) ss += norm.ahead_ss[(size_t)r * norm.ahead_blocks + block];
#pragma unroll
      for (int off = 16; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
      if (part == 0 && r < MB * 16) row_factor[r] = (r < M) ? 1.0f / sqrtf(ss / (float)K + norm.ahead_eps) : 0.f;
    }
  }
  // D: lane holds column (activation row) i and rows (W rows) 4g..4g+3 of each block; lay it out as [m][n]
#pragma unroll
  for (int t = 0; t < SPAN_TILES; ++t)
#pragma unroll
    for (int b = 0; b < MB; ++b)
#pragma unroll
      for (int r = 0; r < 4; ++r) partial[wave][t][b][i * 16 + 4 * g + r] = acc[t][b][r];
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < OUT_PASSES; ++pass) {
    const int e = threadIdx.x + pass * WAVES * 64;
    if (e >= MB * 256) break;   // whole waves enter or stay out
    const int b = e / 256, m = b * 16 + (e % 256) / 16, column = e % 16;
    float sq = 0.f;   // of what this workgroup adds to row m of the residual (norm.behind_weight)
#pragma unroll
    for (int t = 0; t < SPAN_TILES; ++t) {
      const int n = (first_tile + t) * 16 + column;
      const bool valid = m < M && column >= lo[t] && column < hi[t];
      float sum = 0.f;
#pragma unroll
      for (int v = 0; v < WAVES; ++v) sum += partial[v][t][b][e % 256];
      if (norm.ahead_ss) sum *= row_factor[m];
      if (!valid) continue;
      if (OUT_EARLY) {
        const float value = accumulate ? before[pass][t] + sum : sum;
        reinterpret_cast<float*>(c)[(size_t)m * N + n] = value;
        if (norm.behind_weight) {
          sq += value * value;
          norm.behind_rows[bh_rows_index(blocks.behind, m, n, N)] = f32_to_bf16_bits(value * behind_gain[pass][t]);
        }
      } else {
        store_out<TC>(c, (size_t)m * N + n, sum, accumulate != 0);
      }
    }
    if (norm.behind_weight) {
      sq += __shfl_xor(sq, 8, 64);   // the 16 columns of a row sit in 16 neighbouring lanes
      sq += __shfl_xor(sq, 4, 64);
      sq += __shfl_xor(sq, 2, 64);
      sq += __shfl_xor(sq, 1, 64);
      if (column == 0 && m < M) norm.behind_ss[(size_t)m * gridDim.x + blockIdx.x] = sq;
    }
  }
}

// ---- K in parts: the finishing kernel ---------------------------------------------------------
// Whole tiles that are too few to fill the chip cut K into parts over workgroups (gemm_tiled_whole_kernel
// with `parts_out`); the bare sums go to scratch memory as [K part][row][weight row].  This kernel adds the
// parts in order and does what the other kernels do with their sums: the row factor of a norm ahead,
// SwiGLU, accumulation into the residual, a norm behind.
// One block per 16 rows x 64 outputs: thread (r, col) = (tid / 16, tid % 16) has the four outputs
// 64 * blockIdx.x + 4 col .. + 3 of row 16 * blockIdx.y + r (N is a multiple of 16 here).  All of a thread's
// loads are asked for before the first is used.  A norm behind gets one partial sum per row and block.
#define MAX_PARTS 16
#define MAX_TURNS_PARTS 8   // what gemm_turns_parts cuts K into at most
#define FINISH_COLUMNS 64
typedef uint16_t u16x4_t __attribute__((ext_vector_type(4)));
// blocks.c: a SwiGLU's bfloat16 output goes out in blocks of that many rows (bh_rows_index; 0: rows); blocks.behind: so do
// the rows prepared for a norm behind (a thread's four columns lie in one 16-byte piece of a block).
template <bool SWIGLU, typename TC>
__global__ __launch_bounds__(256) void gemm_parts_finish_kernel(const float* __restrict__ sums, TC* __restrict__ c,
                                                                int M, int N, int K, int parts, int accumulate,
                                                                RidingNorm norm, RowBlocks blocks) {
  const int w_rows = SWIGLU ? 2 * N : N;
  const int col = threadIdx.x % 16, n = blockIdx.x * FINISH_COLUMNS + 4 * col, m = blockIdx.y * 16 + threadIdx.x / 16;
  const bool valid = m < M && n < N;
  const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
  f32x4_t first_part[MAX_PARTS], second_part[SWIGLU ? MAX_PARTS : 1];
#pragma unroll
  for (int part = 0; part < MAX_PARTS; ++part) {
    const bool there = valid && part < parts;
    const float* row = sums + ((size_t)(there ? part : 0) * M + (valid ? m : 0)) * w_rows;
    first_part[part] = there ? *reinterpret_cast<const f32x4_t*>(row + n) : zero;
    if (SWIGLU) second_part[part] = there ? *reinterpret_cast<const f32x4_t*>(row + N + n) : zero;
  }
  float factor = 1.f;
  if (norm.ahead_ss) {   // 16 lanes share a row: each adds every 16th partial sum, then the 16 are added pairwise
    float ss = 0.f;
    for (int block0 = col; block0 < norm.ahead_blocks; block0 += 16 * 8) {
      float piece[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int block = block0 + 16 * u;
        piece[u] = (m < M && block < norm.ahead_blocks) ? norm.ahead_ss[(size_t)m * norm.ahead_blocks + block] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) ss += piece[u];
    }
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
    factor = 1.0f / sqrtf(ss / (float)K + norm.ahead_eps);
  }
  f32x4_t first = zero, second = zero;   // the outputs' sums over the parts, in their order; for SwiGLU the gates' and the up rows'
#pragma unroll
  for (int part = 0; part < MAX_PARTS; ++part) {
    first += first_part[part];
    if (SWIGLU) second += second_part[part];
  }
  first *= factor;
  second *= factor;
  const size_t at = (size_t)(valid ? m : 0) * N + (valid ? n : 0);
  f32x4_t value = zero;   // what the outputs hold afterwards; 0 where there is no element
  if (valid) {
    if (SWIGLU) {
#pragma unroll
      for (int i = 0; i < 4; ++i) value[i] = silu_mul(first[i], second[i]);
    } else {
      value = first;
      if (accumulate) {
        if constexpr (sizeof(TC) == 4) {
          value += *reinterpret_cast<const f32x4_t*>(reinterpret_cast<const float*>(c) + at);
        } else {
          const u16x4_t old = *reinterpret_cast<const u16x4_t*>(reinterpret_cast<const uint16_t*>(c) + at);
#pragma unroll
          for (int i = 0; i < 4; ++i) value[i] += bf16_bits_to_f32(old[i]);
        }
      }
    }
    if constexpr (sizeof(TC) == 4) {
      *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(c) + at) = value;
    } else {
      u16x4_t packed;
#pragma unroll
      for (int i = 0; i < 4; ++i) packed[i] = f32_to_bf16_bits(value[i]);
      *reinterpret_cast<u16x4_t*>(reinterpret_cast<uint16_t*>(c) + (SWIGLU ? (size_t)bh_rows_index(blocks.c, m, n, N) : at)) = packed;
    }
  }
  if (!SWIGLU && norm.behind_weight) {   // float32 output
    float sq = value[0] * value[0] + value[1] * value[1] + value[2] * value[2] + value[3] * value[3];
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) sq += __shfl_xor(sq, off, 64);   // the 64 columns of a row are 16 neighbouring lanes
    if (valid) {
      u16x4_t rows;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float g = norm.behind_weight_f32 ? reinterpret_cast<const float*>(norm.behind_weight)[n + i]
                                               : bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(norm.behind_weight)[n + i]);
        rows[i] = f32_to_bf16_bits(value[i] * g);
      }
      *reinterpret_cast<u16x4_t*>(norm.behind_rows + (size_t)bh_rows_index(blocks.behind, m, n, N)) = rows;
    }
    if (col == 0 && m < M) norm.behind_ss[(size_t)m * gridDim.x + blockIdx.x] = sq;
  }
}

// ---- tiled -----------------------------------------------------------------------------------

// The same for a product that completes the float32 residual right before an RMSNorm reads it, with many rows
// (the parts come from the kernel whose wave groups take turns): a block owns eight whole rows, so it can finish
// the norm itself and the norm needs no launch and no second pass over the residual.  Lane l of wave w has row
// l % 8 of the block's rows and the pieces of eight columns 8 w + l / 8, + 128, ...: a wave reads 256 contiguous
// bytes of each of its rows and writes 128 contiguous bytes of the norm's output per row, or, with
// normed_blocked (the output in blocks of 16 rows x 32 columns, bh_blocked_index, for a product that reads it
// that way), the 128 bytes that eight rows' pieces of the same columns fill there.  The parts are added in their
// order, then the residual's old values, as the kernel above does; a row's sum of squares is added up in an
// order that depends on the width only.
#define FINISH_NORM_PIECES 8   // pieces of eight columns per thread: rows of up to 8,192
typedef uint32_t finish_u32x4_t __attribute__((ext_vector_type(4)));
template <int PARTS, int ROWS>   // PARTS: at least `parts`, what the loop over them is unrolled to; ROWS per block, 128 threads each
__global__ __launch_bounds__(128 * ROWS) void gemm_parts_finish_norm_kernel(const float* __restrict__ sums, float* __restrict__ c,
                                                                      int M, int N, int parts, const void* __restrict__ weight,
                                                                      int weight_f32, float eps, uint16_t* __restrict__ normed,
                                                                      int normed_blocked) {
  constexpr int WAVES = 2 * ROWS, WAVE_PIECES = 64 / ROWS;   // a step over the row is 128 pieces wide
  __shared__ float partial[WAVES][ROWS];
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int r = lane % ROWS, row = blockIdx.x * ROWS + r, pieces = N / 8;
  const bool row_there = row < M;
  const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
  constexpr bool KEEP = PARTS <= 4;   // with more parts the registers do not hold the new values too: they are read again
  f32x4_t value[KEEP ? FINISH_NORM_PIECES : 1][2];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < FINISH_NORM_PIECES; ++j) {
    const int piece = WAVE_PIECES * wave + lane / ROWS + 128 * j;
    const bool there = row_there && piece < pieces;
    if (KEEP) value[j][0] = value[j][1] = zero;
    if (!there) continue;
    f32x4_t* residual = reinterpret_cast<f32x4_t*>(c + (size_t)row * N + 8 * piece);
    constexpr int GROUP = PARTS < 4 ? PARTS : 4;   // parts whose loads are on their way together
    const f32x4_t old[2] = {residual[0], residual[1]};
    f32x4_t sum[2] = {zero, zero};
#pragma unroll
    for (int p0 = 0; p0 < PARTS; p0 += GROUP) {
      f32x4_t part[GROUP][2];
#pragma unroll
      for (int u = 0; u < GROUP; ++u) {
        const int p = p0 + u;
        const f32x4_t* from = reinterpret_cast<const f32x4_t*>(sums + ((size_t)(p < parts ? p : 0) * M + row) * N + 8 * piece);
        part[u][0] = p < parts ? from[0] : zero;
        part[u][1] = p < parts ? from[1] : zero;
      }
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int u = 0; u < GROUP; ++u) sum[half] = p0 + u == 0 ? part[u][half] : sum[half] + part[u][half];
    }
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const f32x4_t v = sum[half] + old[half];
      if (KEEP) value[j][half] = v;
      residual[half] = v;
      ss += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
    }
  }
#pragma unroll
  for (int step = ROWS; step < 64; step *= 2) ss += __shfl_xor(ss, step, 64);
  if (lane < ROWS) partial[wave][lane] = ss;
  __syncthreads();
  float total = 0.f;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) total += partial[w][r];
  const float inv = 1.0f / sqrtf(total / (float)N + eps);
#pragma unroll
  for (int j = 0; j < FINISH_NORM_PIECES; ++j) {
    const int piece = WAVE_PIECES * wave + lane / ROWS + 128 * j;
    if (!row_there || piece >= pieces) continue;
    f32x4_t g[2];
    if (weight_f32) {
      g[0] = reinterpret_cast<const f32x4_t*>(weight)[2 * piece];
      g[1] = reinterpret_cast<const f32x4_t*>(weight)[2 * piece + 1];
    } else {
      const finish_u32x4_t raw = reinterpret_cast<const finish_u32x4_t*>(weight)[piece];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        g[e / 2][2 * (e % 2)] = bf16_bits_to_f32((uint16_t)(raw[e] & 0xffffu));
        g[e / 2][2 * (e % 2) + 1] = bf16_bits_to_f32((uint16_t)(raw[e] >> 16));
      }
    }
    f32x4_t v[2];
    if (KEEP) {
      v[0] = value[j][0], v[1] = value[j][1];
    } else {
      const f32x4_t* residual = reinterpret_cast<const f32x4_t*>(c + (size_t)row * N + 8 * piece);
      v[0] = residual[0], v[1] = residual[1];
    }
    finish_u32x4_t bits;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int half = e / 2, i = 2 * (e % 2);
      bits[e] = (uint32_t)f32_to_bf16_bits(v[half][i] * inv * g[half][i]) |
                ((uint32_t)f32_to_bf16_bits(v[half][i + 1] * inv * g[half][i + 1]) << 16);
    }
    const size_t at = normed_blocked ? (size_t)bh_blocked_index(row, 8 * piece, N) : (size_t)row * N + 8 * piece;
    *reinterpret_cast<finish_u32x4_t*>(normed + at) = bits;
  }
}

#define TK 64           // k slice
#define TPITCH (TK + 8) // LDS row pitch in elements: 144 bytes, so 16-byte reads of 16 rows hit 64 distinct banks

// A workgroup of WM x WN waves computes a (32 WX WM) x (32 WY WN) tile; a wave WX x WY blocks of 32 x 32.
// SWIGLU: a wave's 32 WY rows of W are the gate rows of its 16 WY outputs and then the up rows of the
// same outputs; N counts outputs and the up rows start `N` rows (N/16 blocks) further on.
template <bool TILES, bool SWIGLU, int WX, int WY, int WM, int WN, int BUFFERS, typename TC>
__global__ __launch_bounds__(64 * WM * WN) void gemm_tiled_kernel(const uint16_t* __restrict__ a,
                                                                   const uint16_t* __restrict__ w,
                                                                   TC* __restrict__ c, int M, int N, int K,
                                                                   int accumulate) {
  constexpr int THREADS = 64 * WM * WN;
  constexpr int TBM = 32 * WX * WM, TBN = 32 * WY * WN;
  constexpr int A_PIECES = TBM * 8 / THREADS;   // 16-byte pieces of a slice that one thread stages
  constexpr int W_PIECES = TBN * 8 / THREADS;
  static_assert(TBM * 8 % THREADS == 0 && TBN * 8 % THREADS == 0, "the tile is staged in whole rounds of the workgroup");
  static_assert(!SWIGLU || WY % 2 == 0, "gate and up blocks come in pairs");
  __shared__ __attribute__((aligned(16))) uint16_t as[BUFFERS][TBM * TPITCH];
  __shared__ __attribute__((aligned(16))) uint16_t ws[BUFFERS][TBN * TPITCH];
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int m0 = blockIdx.y * TBM;
  const int n0 = blockIdx.x * (SWIGLU ? TBN / 2 : TBN);      // first output column of the tile
  const int wm = (wave / WN) * 32 * WX, wn = (wave % WN) * 32 * WY;  // this wave's part of the tile (in LDS rows)
  const int w_rows = SWIGLU ? 2 * N : N;
  const int w_blocks = (w_rows + 15) / 16;

  // LDS row r of the W tile -> row of W
  auto w_row_of = [&](int r) {
    if (!SWIGLU) return n0 + r;
    constexpr int OUTS = 16 * WY;                          // outputs of one wave column
    const int part = r / (2 * OUTS), inner = r % (2 * OUTS);
    return (inner < OUTS ? 0 : N) + n0 + part * OUTS + inner % OUTS;
  };

  // global -> LDS staging: a slice is rows x 8 pieces of 16 bytes
  int a_at[A_PIECES], w_at[W_PIECES], a_piece[A_PIECES], w_piece[W_PIECES];
  const uint16_t* a_src[A_PIECES];
  const uint16_t* w_src[W_PIECES];
#pragma unroll
  for (int s = 0; s < A_PIECES; ++s) {
    const int e = tid + s * THREADS;
    const int row = e / 8, piece = e % 8;
    const int am = (m0 + row < M) ? m0 + row : M - 1;
    a_src[s] = a + (size_t)am * K + piece * 8;
    a_at[s] = row * TPITCH + piece * 8;
    a_piece[s] = piece;
  }
#pragma unroll
  for (int s = 0; s < W_PIECES; ++s) {
    const int e = tid + s * THREADS;
    const int row = e / 8, piece = e % 8;
    w_piece[s] = piece;
    if (TILES) {
      // blocks of 16 rows; inside a block piece p = u * 64 + l holds row l % 16, k 16 * (l / 16) + 8 * u
      const int block = e / 128, p = e % 128, u = p / 64, l = p % 64;
      int global_block = w_row_of(block * 16) / 16;
      if (global_block >= w_blocks) global_block = w_blocks - 1;
      w_src[s] = w + (size_t)global_block * (K / 64) * 1024 + p * 8;
      w_at[s] = (block * 16 + l % 16) * TPITCH + 16 * (l / 16) + 8 * u;
    } else {
      int wr = w_row_of(row);
      if (wr >= w_rows) wr = w_rows - 1;
      w_src[s] = w + (size_t)wr * K + piece * 8;
      w_at[s] = row * TPITCH + piece * 8;
    }
  }
  const size_t w_step = TILES ? 1024 : TK;
  u32x4_t a_reg[A_PIECES], w_reg[W_PIECES];
  const u32x4_t zero = {0u, 0u, 0u, 0u};
  const bool whole_slices = K % TK == 0;   // then no piece of a slice lies beyond K and no load is predicated
  auto fetch = [&](int slice) {
    const int k0 = slice * TK;
    if (whole_slices) {
#pragma unroll
      for (int s = 0; s < A_PIECES; ++s) a_reg[s] = load16(a_src[s] + k0);
#pragma unroll
      for (int s = 0; s < W_PIECES; ++s) w_reg[s] = load16(w_src[s] + (size_t)slice * w_step);
    } else {
#pragma unroll
      for (int s = 0; s < A_PIECES; ++s) a_reg[s] = (k0 + a_piece[s] * 8 < K) ? load16(a_src[s] + k0) : zero;
#pragma unroll
      for (int s = 0; s < W_PIECES; ++s)
        w_reg[s] = (TILES || k0 + w_piece[s] * 8 < K) ? load16(w_src[s] + (size_t)slice * w_step) : zero;
    }
  };
  auto stash = [&](int buffer) {
#pragma unroll
    for (int s = 0; s < A_PIECES; ++s) *reinterpret_cast<u32x4_t*>(&as[buffer][a_at[s]]) = a_reg[s];
#pragma unroll
    for (int s = 0; s < W_PIECES; ++s) *reinterpret_cast<u32x4_t*>(&ws[buffer][w_at[s]]) = w_reg[s];
  };

  f32x16_t acc[WX][WY];
#pragma unroll
  for (int x = 0; x < WX; ++x)
#pragma unroll
    for (int y = 0; y < WY; ++y)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[x][y][e] = 0.f;

  const int slices = (K + TK - 1) / TK;
  fetch(0);
  stash(0);
  __syncthreads();
  const int frag_row = lane % 32, frag_k = (lane / 32) * 8;
  for (int s = 0; s < slices; ++s) {
    const int buffer = BUFFERS == 2 ? (s & 1) : 0;
    if (s + 1 < slices) fetch(s + 1);
#pragma unroll
    for (int kk = 0; kk < TK; kk += 16) {
      bf16x8_t af[WX], wf[WY];
#pragma unroll
      for (int x = 0; x < WX; ++x)
        af[x] = as_bf16x8(*reinterpret_cast<const u32x4_t*>(&as[buffer][(wm + x * 32 + frag_row) * TPITCH + kk + frag_k]));
#pragma unroll
      for (int y = 0; y < WY; ++y)
        wf[y] = as_bf16x8(*reinterpret_cast<const u32x4_t*>(&ws[buffer][(wn + y * 32 + frag_row) * TPITCH + kk + frag_k]));
#pragma unroll
      for (int x = 0; x < WX; ++x)
#pragma unroll
        for (int y = 0; y < WY; ++y)
          acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[x], wf[y], acc[x][y], 0, 0, 0);
    }
    if (BUFFERS == 1) __syncthreads();   // one buffer: everyone has read the slice before it is overwritten
    if (s + 1 < slices) stash(BUFFERS == 2 ? buffer ^ 1 : 0);   // (writing it half-way through the multiplies measured slower)
    __syncthreads();
  }
  // D of one 32x32 block: column (n) lane%32, rows (m) 8*(e/4) + 4*(lane/32) + e%4
#pragma unroll
  for (int x = 0; x < WX; ++x) {
    if (SWIGLU) {
#pragma unroll
      for (int y = 0; y < WY / 2; ++y) {
        const int n = n0 + (wave % WN) * 16 * WY + y * 32 + lane % 32;
        if (n >= N) continue;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int m = m0 + wm + x * 32 + 8 * (e / 4) + 4 * (lane / 32) + e % 4;
          if (m < M) store_out<TC>(c, (size_t)m * N + n, silu_mul(acc[x][y][e], acc[x][y + WY / 2][e]), false);
        }
      }
    } else {
#pragma unroll
      for (int y = 0; y < WY; ++y) {
        const int n = n0 + wn + y * 32 + lane % 32;
        if (n >= N) continue;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int m = m0 + wm + x * 32 + 8 * (e / 4) + 4 * (lane / 32) + e % 4;
          if (m < M) store_out<TC>(c, (size_t)m * N + n, acc[x][y][e], accumulate != 0);
        }
      }
    }
  }
}

// ---- tiled, whole tiles of the packed layout ---------------------------------------------------
// The same product for the common case: W in the tiles layout, K a multiple of 64, N a multiple of 16, and
// M and N at least a tile.  Then no load needs a bounds check: a tile that would stick out is moved back
// inside (its last row or column on the matrix's last) and stores only what the tile it stands for owns.
// Every thread's loads of a slice differ from one another by amounts that are the same for all threads,
// so a thread keeps one offset for A and one for W instead of a pointer per load; with the registers this
// frees, the compiler reads the next operand fragments from LDS while the current ones are multiplied.

template <bool SWIGLU, int WX, int WY, int WM, int WN, int BUFFERS, typename TC>
__global__ __launch_bounds__(64 * WM * WN) void gemm_tiled_whole_kernel(const uint16_t* __restrict__ a,
                                                                         const uint16_t* __restrict__ w,
                                                                         TC* __restrict__ c, int M, int N, int K,
                                                                         int accumulate, RidingNorm norm,
                                                                         float* __restrict__ parts_out,
                                                                         int slices_per_part) {
  constexpr int THREADS = 64 * WM * WN;
  constexpr int TBM = 32 * WX * WM, TBN = 32 * WY * WN;
  static_assert(TBM <= THREADS, "one thread per row of the tile adds up the norm's partial sums");
  constexpr int A_PIECES = TBM * 8 / THREADS, W_PIECES = TBN * 8 / THREADS;
  constexpr int A_ROWS = THREADS / 8;      // rows of A that one round of the workgroup's loads covers
  constexpr int W_BLOCKS = THREADS / 128;  // 16-row blocks of W per round
  constexpr int OUTS = SWIGLU ? TBN / 2 : TBN;   // output columns of a tile
  static_assert(TBM * 8 % THREADS == 0 && TBN * 8 % THREADS == 0, "the tile is staged in whole rounds of the workgroup");
  static_assert(!SWIGLU || W_BLOCKS == WY, "a round of W loads is the gate half or the up half of one wave column");
  __shared__ __attribute__((aligned(16))) uint16_t as[BUFFERS][TBM * TPITCH];
  __shared__ __attribute__((aligned(16))) uint16_t ws[BUFFERS][TBN * TPITCH];
  __shared__ __attribute__((aligned(16))) float row_factor[TBM];   // norm ahead: what each row's result is multiplied by
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int m_own = blockIdx.y * TBM, n_own = blockIdx.x * OUTS;   // what this tile stands for
  // Tiles of 32 or 64 rows (WX == 1) also take fewer rows than a tile: loads repeat the last row, and
  // nothing beyond it is stored.
  constexpr bool SHORT = WX == 1;
  const int m0 = SHORT && M < TBM ? 0 : min(m_own, M - TBM), n0 = min(n_own, N - OUTS);   // where it computes
  const int wm = (wave / WN) * 32 * WX, wn = (wave % WN) * 32 * WY;

  // A: piece e = tid + s * THREADS is row e / 8, 16 bytes e % 8 of the slice
  const uint16_t* a_tile = a + (size_t)m0 * K;
  const int a_off = (tid / 8) * K + (tid % 8) * 8;                 // + s * A_ROWS * K, the same for all threads
  const int a_lds = (tid / 8) * TPITCH + (tid % 8) * 8;            // + s * A_ROWS * TPITCH
  int a_short[SHORT ? A_PIECES : 1];                               // short tiles: an offset per round, rows clamped
  if (SHORT) {
#pragma unroll
    for (int s = 0; s < A_PIECES; ++s) a_short[s] = min(tid / 8 + s * A_ROWS, M - 1 - m0) * K + (tid % 8) * 8;
  }
  // W: piece e is block e / 128 of the tile's rows in LDS, piece p = e % 128 = u * 64 + l of that block's slice:
  // row l % 16, k 16 * (l / 16) + 8 u.  LDS block b of round s holds W rows starting at
  //   plain:  n0 + 16 (b + s * W_BLOCKS)
  //   SwiGLU: wave column s / 2; s even: gate rows n0 + (s / 2) * 16 WY + 16 b; s odd: the up rows, N further on
  const int w_block = tid / 128, w_p = tid % 128, w_l = w_p % 64, w_u = w_p / 64;
  const size_t block_stride = (size_t)(K / 64) * 1024;             // elements from one 16-row block to the next
  const uint16_t* w_tile = w + (size_t)(n0 / 16) * block_stride;
  const int w_off = w_block * (int)block_stride + w_p * 8;         // + what round s adds, the same for all threads
  const int w_lds = (w_block * 16 + w_l % 16) * TPITCH + 16 * (w_l / 16) + 8 * w_u;   // + s * W_BLOCKS * 16 * TPITCH
  size_t w_round[W_PIECES];
#pragma unroll
  for (int s = 0; s < W_PIECES; ++s)
    w_round[s] = SWIGLU ? ((size_t)(s / 2) * WY + (s % 2 ? (size_t)(N / 16) : 0)) * block_stride
                        : (size_t)s * W_BLOCKS * block_stride;

  u32x4_t a_reg[A_PIECES], w_reg[W_PIECES];
  auto fetch = [&](int slice) {
#pragma unroll
    for (int s = 0; s < A_PIECES; ++s)
      a_reg[s] = load16(a_tile + (SHORT ? (size_t)a_short[s] : (size_t)s * A_ROWS * K + a_off) + slice * TK);
#pragma unroll
    for (int s = 0; s < W_PIECES; ++s) w_reg[s] = load16(w_tile + w_round[s] + (size_t)slice * 1024 + w_off);
  };
  auto stash = [&](int buffer) {
#pragma unroll
    for (int s = 0; s < A_PIECES; ++s)
      *reinterpret_cast<u32x4_t*>(&as[buffer][a_lds + s * A_ROWS * TPITCH]) = a_reg[s];
#pragma unroll
    for (int s = 0; s < W_PIECES; ++s)
      *reinterpret_cast<u32x4_t*>(&ws[buffer][w_lds + s * W_BLOCKS * 16 * TPITCH]) = w_reg[s];
  };

  f32x16_t acc[WX][WY];
#pragma unroll
  for (int x = 0; x < WX; ++x)
#pragma unroll
    for (int y = 0; y < WY; ++y)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[x][y][e] = 0.f;

  // K in parts (parts_out): workgroup z multiplies its part of the slices and leaves the bare sums to
  // gemm_parts_finish_kernel.
  const int first_slice = parts_out ? blockIdx.z * slices_per_part : 0;
  const int end_slice = parts_out ? min(K / TK, first_slice + slices_per_part) : K / TK;
  fetch(first_slice);
  if (norm.ahead_ss && !parts_out && tid < TBM) {   // while the first slice is on its way
    const float* partial = norm.ahead_ss + (size_t)min(m0 + tid, M - 1) * norm.ahead_blocks;
    float total = 0.f;
    if (norm.ahead_blocks % 4 == 0) {   // 32 sums per round of loads, added in their order
      const f32x4_t* four = reinterpret_cast<const f32x4_t*>(partial);
      const int fours = norm.ahead_blocks / 4;
      for (int b = 0; b < fours; b += 8) {
        f32x4_t v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = b + i < fours ? four[b + i] : f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 8; ++i) total += v[i][0], total += v[i][1], total += v[i][2], total += v[i][3];
      }
    } else {
      for (int b = 0; b < norm.ahead_blocks; ++b) total += partial[b];
    }
    row_factor[tid] = rsqrtf(total / (float)K + norm.ahead_eps);
  }
  stash(0);
  __syncthreads();
  const int frag = (lane % 32) * TPITCH + (lane / 32) * 8;
  auto multiply = [&](int buffer) {
#pragma unroll
    for (int kk = 0; kk < TK; kk += 16) {
      bf16x8_t af[WX], wf[WY];
#pragma unroll
      for (int x = 0; x < WX; ++x)
        af[x] = as_bf16x8(*reinterpret_cast<const u32x4_t*>(&as[buffer][(wm + x * 32) * TPITCH + kk + frag]));
#pragma unroll
      for (int y = 0; y < WY; ++y)
        wf[y] = as_bf16x8(*reinterpret_cast<const u32x4_t*>(&ws[buffer][(wn + y * 32) * TPITCH + kk + frag]));
#pragma unroll
      for (int x = 0; x < WX; ++x)
#pragma unroll
        for (int y = 0; y < WY; ++y)
          acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[x], wf[y], acc[x][y], 0, 0, 0);
    }
  };
  // All slices but the last in a loop without a branch in its body: loads, multiplies and staging writes
  // are one stretch of code that the compiler may interleave.
  for (int s = first_slice; s + 1 < end_slice; ++s) {
    const int buffer = BUFFERS == 2 ? ((s - first_slice) & 1) : 0;
    fetch(s + 1);
    __builtin_amdgcn_sched_barrier(0);   // the loads go out first: a slice of multiplies is their time to land
    multiply(buffer);
    if (BUFFERS == 1) __syncthreads();   // one buffer: everyone has read the slice before it is overwritten
    stash(BUFFERS == 2 ? buffer ^ 1 : 0);
    __syncthreads();
  }
  multiply(BUFFERS == 2 ? ((end_slice - 1 - first_slice) & 1) : 0);
  // D of one 32x32 block: column (n) lane%32, rows (m) 8*(e/4) + 4*(lane/32) + e%4
  if (parts_out) {   // [part][row][weight row]; a SwiGLU's up rows lie N after its gate rows
    const int w_rows = SWIGLU ? 2 * N : N;
    float* out = parts_out + (size_t)blockIdx.z * M * w_rows;
#pragma unroll
    for (int x = 0; x < WX; ++x)
#pragma unroll
      for (int y = 0; y < WY; ++y) {
        const int n = SWIGLU ? n0 + (wave % WN) * 16 * WY + (y % (WY / 2)) * 32 + lane % 32 : n0 + wn + y * 32 + lane % 32;
        if (n < n_own) continue;
        const int w_row = SWIGLU && y >= WY / 2 ? N + n : n;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int m = m0 + wm + x * 32 + 8 * (e / 4) + 4 * (lane / 32) + e % 4;
          if (m >= m_own && m < M) out[(size_t)m * w_rows + w_row] = acc[x][y][e];
        }
      }
    return;
  }
  if (norm.ahead_ss) {
#pragma unroll
    for (int x = 0; x < WX; ++x)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const f32x4_t f = *reinterpret_cast<const f32x4_t*>(&row_factor[wm + x * 32 + 8 * q + 4 * (lane / 32)]);
#pragma unroll
        for (int y = 0; y < WY; ++y)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[x][y][4 * q + i] *= f[i];
      }
  }
  if constexpr (!SWIGLU && sizeof(TC) == 4) {
    if (norm.behind_weight) {
      // The residual's new values, the norm's unscaled output, and the sum of squares of each row over the
      // columns this tile owns: within a wave by lane exchanges, across the WN waves of a row through LDS,
      // always in the same order.
      __syncthreads();   // the operand buffers are free now
      float* partial = reinterpret_cast<float*>(&as[0][0]);   // [WN][TBM]
      static_assert(WN * TBM * 4 <= (int)sizeof(as), "the partial sums fit in the A buffers");
      float g[WY];
#pragma unroll
      for (int y = 0; y < WY; ++y) {
        const int n = n0 + wn + y * 32 + lane % 32;
        g[y] = norm.behind_weight_f32 ? reinterpret_cast<const float*>(norm.behind_weight)[n]
                                      : bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(norm.behind_weight)[n]);
      }
#pragma unroll
      for (int x = 0; x < WX; ++x) {
        float sq[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) sq[e] = 0.f;
#pragma unroll
        for (int y = 0; y < WY; ++y) {
          const int n = n0 + wn + y * 32 + lane % 32;
          if (n < n_own) continue;
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int m = m0 + wm + x * 32 + 8 * (e / 4) + 4 * (lane / 32) + e % 4;
            if (m < m_own || m >= M) continue;
            const size_t at = (size_t)m * N + n;
            const float value = accumulate ? c[at] + acc[x][y][e] : acc[x][y][e];
            c[at] = value;
            norm.behind_rows[at] = f32_to_bf16_bits(value * g[y]);
            sq[e] += value * value;
          }
        }
#pragma unroll
        for (int e = 0; e < 16; ++e) {
#pragma unroll
          for (int step = 16; step >= 1; step >>= 1) sq[e] += __shfl_xor(sq[e], step);
          if (lane % 32 == 0) partial[(wave % WN) * TBM + wm + x * 32 + 8 * (e / 4) + 4 * (lane / 32) + e % 4] = sq[e];
        }
      }
      __syncthreads();
      if (tid < TBM && m0 + tid >= m_own && m0 + tid < M) {
        float total = 0.f;
#pragma unroll
        for (int part = 0; part < WN; ++part) total += partial[part * TBM + tid];
        norm.behind_ss[(size_t)(m0 + tid) * gridDim.x + blockIdx.x] = total;
      }
      return;
    }
  }
#pragma unroll
  for (int x = 0; x < WX; ++x) {
    if (SWIGLU) {
#pragma unroll
      for (int y = 0; y < WY / 2; ++y) {
        const int n = n0 + (wave % WN) * 16 * WY + y * 32 + lane % 32;
        if (n < n_own) continue;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int m = m0 + wm + x * 32 + 8 * (e / 4) + 4 * (lane / 32) + e % 4;
          if (m >= m_own && m < M) store_out<TC>(c, (size_t)m * N + n, silu_mul(acc[x][y][e], acc[x][y + WY / 2][e]), false);
        }
      }
    } else {
#pragma unroll
      for (int y = 0; y < WY; ++y) {
        const int n = n0 + wn + y * 32 + lane % 32;
        if (n < n_own) continue;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int m = m0 + wm + x * 32 + 8 * (e / 4) + 4 * (lane / 32) + e % 4;
          if (m >= m_own && m < M) store_out<TC>(c, (size_t)m * N + n, acc[x][y][e], accumulate != 0);
        }
      }
    }
  }
}

// ---- entry -------------------------------------------------------------------------------------

// The weight rows per workgroup (20 or 24) with which the skinny product of packed weights runs as
// gemm_skinny_span_kernel, or 0: where its blocks of 16 rows are more than the compute units and fewer than twice as
// many, and some such span divides the rows into no more workgroups than there are compute units.
static int skinny_span_rows(int M, int N, int K) {
  if (M > 32 || N % 16 != 0 || K % 64 != 0) return 0;
  const int tiles = N / 16, units = bh_compute_units();
  if (tiles <= units || tiles >= 2 * units) return 0;
  for (int rows = 20; rows <= 24; rows += 4)   // (28 rows can lie in three blocks: 7168 x 5120 at 8 rows 14.6 -> 17.1 us)
    if (N % rows == 0 && N / rows <= units) return rows;
  return 0;
}

template <bool TILES, int RT, typename TC>
static void launch_skinny(const void* a, const void* w, void* c, int M, int N, int K, int accumulate,
                          int pair_blocks, const RidingNorm& norm, const RowBlocks& blocks, hipStream_t stream) {
  constexpr int WAVES = 8;
  if constexpr (TILES && RT == 1) {
    if (const int span = skinny_span_rows(M, N, K)) {
      dim3 span_grid(N / span), span_block(WAVES * 64);
#define BH_SPAN(MB, XB)                                                                                  \
  gemm_skinny_span_kernel<MB, WAVES, TC, XB><<<span_grid, span_block, 0, stream>>>(                      \
      (const uint16_t*)a, (const uint16_t*)w, (TC*)c, M, N, K, accumulate, span, norm, blocks)
      if (blocks.a == 8) BH_SPAN(1, 8);
      else if (blocks.a == 16 && M <= 16) BH_SPAN(1, 16);
      else if (blocks.a == 16) BH_SPAN(2, 16);
      else if (M <= 16) BH_SPAN(1, 0);
      else BH_SPAN(2, 0);
#undef BH_SPAN
      return;
    }
  }
  dim3 grid((N + 15) / 16), block(WAVES * 64);
#define BH_SKINNY(MB, XB)                                                                                 \
  gemm_skinny_kernel<MB, WAVES, TILES, RT, TC, XB><<<grid, block, 0, stream>>>(                           \
      (const uint16_t*)a, (const uint16_t*)w, (TC*)c, M, N, K, accumulate, pair_blocks, norm, blocks)
  if constexpr (TILES) {   // activations in blocks come with packed weights only, up to SKINNY_UP_TO_ROWS rows
    if (blocks.a == 8) {
      BH_SKINNY(1, 8);
      return;
    }
    if (blocks.a == 16) {
      switch ((M + 15) / 16) {
        case 1: BH_SKINNY(1, 16); break;
        default: BH_SKINNY(2, 16); break;
      }
      return;
    }
  }
  switch ((M + 15) / 16) {
    case 1: BH_SKINNY(1, 0); break;
    case 2: BH_SKINNY(2, 0); break;
    case 3: BH_SKINNY(3, 0); break;
    default: BH_SKINNY(4, 0); break;
  }
#undef BH_SKINNY
}

// Measured at the Qwen3-8B shapes (2,048 rows).  The multiplies of a 128 x 128 tile need as many LDS
// cycles (operand reads and the staging writes) as MFMA cycles, so LDS bounds them; a 256 x 256 tile
// of eight waves, each 64 x 128, reads a quarter less per multiply and wins once it still gives every
// compute unit three tiles.  Below that the smaller tile keeps more compute units busy.  Two LDS buffers
// (one barrier per slice, two workgroups per compute unit) are the better choice unless a single one
// (four workgroups per compute unit) lets the whole grid run at once: between two and four tiles for
// each of the 256 compute units.
// Fewer than 128 rows (decode steps of many sequences, short prompts) are still bound by reading W: tiles
// of 64 rows, or of 32 for up to 32 rows, which the kernel also takes when there are fewer rows than a tile.
enum TiledConfig { TILED_256 = 0, TILED_128_ONE_BUFFER = 1, TILED_128 = 2, TILED_64_ROWS = 3, TILED_32_ROWS = 4 };
static TiledConfig tiled_config(int M, int N, bool swiglu, int* rows, int* columns) {
  if (M <= 32) {
    *rows = 32;
    *columns = 128;
    return TILED_32_ROWS;
  }
  if (M < 128) {
    *rows = 64;
    *columns = swiglu ? 64 : 128;
    return TILED_64_ROWS;
  }
  const long tiles_128 = (long)((N + (swiglu ? 63 : 127)) / (swiglu ? 64 : 128)) * ((M + 127) / 128);
  const long tiles_256 = (long)((N + (swiglu ? 127 : 255)) / (swiglu ? 128 : 256)) * ((M + 255) / 256);
  const int units = bh_compute_units();   // measured with 256: two tiles each, and between two and four
  const bool big = tiles_256 >= 2 * units;
  *rows = big ? 256 : 128;
  *columns = (big ? 256 : 128) / (swiglu ? 2 : 1);
  return big ? TILED_256 : tiles_128 > 2 * units && tiles_128 <= 4 * units ? TILED_128_ONE_BUFFER : TILED_128;
}
// Up to how many rows the skinny kernel takes a product of packed weights (it reads its activations in blocks,
// see struct RowBlocks); without packed weights, or where the tiles do not fit, up to 64.
// Decode steps of the Qwen3-8B sizes at context 8,192, against tiles with K in parts from 17 rows on: 16
// sequences 6.88 -> 6.64 ms, 32 sequences 10.38 -> 9.93 ms, 48 sequences 14.24 -> 14.43 ms (so not those).
#define SKINNY_UP_TO_ROWS 32
static bool skinny_first(int M, int N, int K, int layout, int activation) {
  // (but for the products of 17 to 32 rows and very many outputs that the kernel for 33 to 128 rows takes)
  return layout == 1 && K % TK == 0 && N % 16 == 0 && M <= SKINNY_UP_TO_ROWS && !gemm_slices_takes(M, N, K, layout, activation);
}
// Whether the product runs as whole tiles (gemm_tiled_whole_kernel): the way that cuts K into parts and
// the only tiled way a norm rides on.
static bool tiled_whole(int M, int N, int K, int layout, int rows, int columns) {
  return layout == 1 && K % TK == 0 && N % 16 == 0 && M > SKINNY_UP_TO_ROWS && (M >= rows || rows <= 64) && N >= columns &&
         (long)rows * K < (1L << 31);
}

// Whole tiles that are too few to fill the chip cut K into parts (gemm_parts_finish_kernel adds them): the
// number of parts and the 64-wide slices in each; one part means no cut.
// Measured at the Qwen3-8B shapes.  Up to 512 rows (much of the time still goes to reading W, and there is
// little scratch traffic): about 384 workgroups, whatever the number of tiles, was the best of 256 to 2,048
// in decode steps of 17 to 64 sequences and in prompts of 128 to 512 tokens (512 tokens, per layer: o 70 ->
// 40 us, down 250 -> 82 us).  Beyond that the cut pays up to half a tile per compute unit and no longer at
// one; one workgroup per compute unit is then enough (more parts only add scratch traffic) unless a part
// would still be longer than 64 slices.
#define TILED_FEW_ROWS 512
#define TILED_FEW_ROWS_WORKGROUPS 384   // on 256 compute units; scaled to the chip's (bh_compute_units)
#define TILED_FEW_TILES 128             // likewise
static void tiled_parts(int M, int N, int K, int layout, bool swiglu, int* parts, int* slices_per_part) {
  int rows, columns;
  tiled_config(M, N, swiglu, &rows, &columns);
  *parts = 1;
  *slices_per_part = K / TK;
  if (!tiled_whole(M, N, K, layout, rows, columns)) return;
  const long tiles = (long)((N + columns - 1) / columns) * ((M + rows - 1) / rows);
  const int slices = K / TK;
  int p;
  const int units = bh_compute_units();
  const int few_rows_workgroups = TILED_FEW_ROWS_WORKGROUPS * units / 256, few_tiles = TILED_FEW_TILES * units / 256;
  if (M <= TILED_FEW_ROWS) {
    p = (int)((few_rows_workgroups + tiles - 1) / tiles);
  } else {
    if (tiles > few_tiles) return;
    p = (int)(2 * few_tiles / tiles);
    if (slices / p > 64) p *= 2;
  }
  p = std::min(std::min(p, MAX_PARTS), slices / 4);    // at least four slices each
  if (p < 2) return;
  *slices_per_part = (slices + p - 1) / p;
  *parts = (slices + *slices_per_part - 1) / *slices_per_part;
}

template <bool TILES, bool SWIGLU, typename TC>
static void launch_tiled(const void* a, const void* w, void* c, int M, int N, int K, int accumulate,
                         const RidingNorm& norm, float* parts_out, hipStream_t stream) {
  int rows, columns;
  const TiledConfig config = tiled_config(M, N, SWIGLU, &rows, &columns);
  const bool whole = tiled_whole(M, N, K, TILES ? 1 : 0, rows, columns);
  int parts = 1, slices_per_part = 0;
  if (parts_out) tiled_parts(M, N, K, TILES ? 1 : 0, SWIGLU, &parts, &slices_per_part);
  if (parts == 1) parts_out = nullptr;
  dim3 grid((N + columns - 1) / columns, (M + rows - 1) / rows, parts);
#define BH_TILED(WX, WY, WM, WN, BUFFERS)                                                                 \
  do {                                                                                                     \
    dim3 block(64 * WM * WN);                                                                              \
    if (TILES && whole)                                                                                    \
      gemm_tiled_whole_kernel<SWIGLU, WX, WY, WM, WN, BUFFERS, TC><<<grid, block, 0, stream>>>(            \
          (const uint16_t*)a, (const uint16_t*)w, (TC*)c, M, N, K, accumulate, norm, parts_out,            \
          slices_per_part);                                                                                \
    else                                                                                                   \
      gemm_tiled_kernel<TILES, SWIGLU, WX, WY, WM, WN, BUFFERS, TC><<<grid, block, 0, stream>>>(           \
          (const uint16_t*)a, (const uint16_t*)w, (TC*)c, M, N, K, accumulate);                            \
  } while (0)
  switch (config) {
    case TILED_256: BH_TILED(2, 4, 4, 2, 2); break;
    case TILED_128_ONE_BUFFER: BH_TILED(2, 2, 2, 2, 1); break;
    case TILED_64_ROWS: BH_TILED(1, 2, 2, 2, 1); break;   // one LDS buffer: more workgroups per compute unit, more loads in flight
    case TILED_32_ROWS:
      if constexpr (SWIGLU) BH_TILED(1, 2, 1, 4, 1);
      else BH_TILED(1, 1, 1, 4, 1);
      break;
    default: BH_TILED(2, 2, 2, 2, 2); break;
  }
#undef BH_TILED
}

// How many partial sums per row a product of these sizes writes when a norm rides behind it (0: it cannot
// carry one), and whether it can take prepared norm rows as its activations.
// Beyond 256 rows a product carries no norm: at the Qwen3-8B shapes, whole model, the prompt of 128 tokens
// ran 2 % faster with riding norms, that of 512 the same, those of 1,024 to 4,096 tokens 1 to 2 % slower
// than with norms as launches of their own (the producers' longer epilogues cost more than the norms).
#define NORM_RIDES_UP_TO_ROWS 256
extern "C" int bh_gemm_bf16_norm_blocks(int M, int N, int K, int layout, int activation) {
  if (activation || M <= 0 || M > NORM_RIDES_UP_TO_ROWS || N <= 0 || K % 8 != 0) return 0;
  int rows, columns, parts, each;
  if (gemm_slices_takes(M, N, K, layout, 0)) return (N + FINISH_COLUMNS - 1) / FINISH_COLUMNS;   // always finished by that kernel
  tiled_config(M, N, false, &rows, &columns);
  if (!tiled_whole(M, N, K, layout, rows, columns)) {   // the skinny kernel's blocks, or its workgroups of wider spans
    if (layout == 1 && skinny_first(M, N, K, layout, 0))
      if (const int span = skinny_span_rows(M, N, K)) return N / span;
    return M <= 64 ? (N + 15) / 16 : 0;
  }
  tiled_parts(M, N, K, layout, false, &parts, &each);
  return parts > 1 ? (N + FINISH_COLUMNS - 1) / FINISH_COLUMNS : (N + columns - 1) / columns;   // the finishing kernel's blocks, or the tiles'
}
extern "C" int bh_gemm_bf16_takes_norm(int M, int N, int K, int layout, int activation) {
  if (M <= 0 || N <= 0 || K % 8 != 0 || (activation && N % 16 != 0)) return 0;
  if (M <= 64) return 1;
  int rows, columns;
  tiled_config(M, N, activation != 0, &rows, &columns);
  return tiled_whole(M, N, K, layout, rows, columns) ? 1 : 0;
}

// The rows per block (16 or 8) if a product of these sizes reads its activations faster from blocks of that
// many rows x 32 columns (bh_rows_index, layout.h) and takes them that way, else 0: the products of the kernel
// whose wave groups take turns (16), and those of up to 32 rows of the skinny kernel (8 up to 8 rows, else 16).
extern "C" int bh_gemm_bf16_reads_blocked(int M, int N, int K, int layout, int activation) {
  if (M <= 0 || N <= 0 || K <= 0 || K % 32 != 0) return 0;
  if (gemm_turns_blocks(M, N, K, layout, activation) || gemm_turns_parts(M, N, K, layout, activation) > 1) return 16;
  if (skinny_first(M, N, K, layout, activation)) return M <= 8 ? 8 : 16;
  if (gemm_slices_takes(M, N, K, layout, activation)) return 16;
  return 0;
}

// In what form a product of these sizes can write the bfloat16 rows it produces for the next product (a SwiGLU's
// output, the rows prepared for a norm behind it): 2 = rows or blocks of 8 or 16 rows (the skinny kernel),
// 1 = rows or, for SwiGLU, blocks of 16 (the kernel whose wave groups take turns), 0 = rows only.
extern "C" int bh_gemm_bf16_writes_blocked(int M, int N, int K, int layout, int activation) {
  if (M <= 0 || N <= 0 || K <= 0 || N % 32 != 0) return 0;
  if (gemm_turns_blocks(M, N, K, layout, activation)) return activation ? 1 : 0;
  if (gemm_slices_takes(M, N, K, layout, activation)) return 2;    // the finishing kernel writes any blocks
  int rows, columns;
  tiled_config(M, N, activation != 0, &rows, &columns);
  return M <= 64 && !tiled_whole(M, N, K, layout, rows, columns) ? 2 : 0;
}

// layout: 0 = rows, 1 = tiles.  activation: 0 = none; 1 = SwiGLU (W has 2 * N rows: gate rows then up rows).
// Bytes of scratch memory that bh_gemm_bf16 wants for this product (0: none).
// In how many parts of K the tiled kernels (whole tiles, or the kernel whose wave groups take turns) multiply a
// product when they are given scratch memory (1: in one go).
static int tiled_or_turns_parts(int M, int N, int K, int layout, int activation) {
  if (gemm_turns_blocks(M, N, K, layout, activation)) return 1;
  if (const int turns_parts = gemm_turns_parts(M, N, K, layout, activation); turns_parts > 1) return turns_parts;
  int parts, each;
  tiled_parts(M, N, K, layout, activation != 0, &parts, &each);
  return parts;
}
extern "C" long bh_gemm_bf16_scratch(int M, int N, int K, int layout, int activation) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  int parts = tiled_or_turns_parts(M, N, K, layout, activation);
  if (gemm_slices_takes(M, N, K, layout, activation))   // (a caller whose activations lie in rows gets the tiles: room for either)
    parts = std::max(parts, gemm_slices_parts(M, N, K, activation, nullptr));
  else if (parts == 1) return 0;
  return (long)parts * M * (activation ? 2 * N : N) * (long)sizeof(float);
}

// The `ahead_*` and `behind_*` arguments (null when unused) let an RMSNorm ride on the products before and
// after it (struct RidingNorm) where bh_gemm_bf16_takes_norm / bh_gemm_bf16_norm_blocks say so.  `scratch`: bh_gemm_bf16_scratch() bytes, or
// null (then K is not cut into parts where that would be faster).
// a_block_rows: the activations (for a norm ahead: its unscaled rows) lie in blocks of that many rows, as
// bh_gemm_bf16_reads_blocked says this product reads them, or in rows (0).  c_block_rows: a SwiGLU's output goes out
// that way (16 in the kernel for many rows; 0, 8 or 16 in the skinny one); behind_block_rows: so do the rows
// prepared for a norm behind (the skinny kernel's).
extern "C" int bh_gemm_bf16(const void* a, const void* w, void* c, int c_dtype, int accumulate, int M, int N, int K,
                            int layout, int activation, const float* ahead_ss, int ahead_blocks, float ahead_eps,
                            const void* behind_weight, int behind_weight_dtype, void* behind_rows,
                            float* behind_ss, void* scratch, int a_block_rows, int c_block_rows, int behind_block_rows,
                            hipStream_t stream) {
  BH_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_bf16: sizes M=%d N=%d K=%d must be positive", M, N, K);
  BH_REQUIRE(K % 8 == 0, "gemm_bf16: K=%d must be a multiple of 8", K);
  BH_REQUIRE(c_dtype == BH_F32 || c_dtype == BH_BF16, "gemm_bf16: unknown output dtype %d", c_dtype);
  BH_REQUIRE(((uintptr_t)a | (uintptr_t)w) % 16 == 0, "gemm_bf16: operands must be 16-byte aligned");
  BH_REQUIRE(layout == 0 || (layout == 1 && K % 64 == 0), "gemm_bf16: the tiles layout needs K=%d to be a multiple of 64", K);
  BH_REQUIRE(activation == 0 || activation == 1, "gemm_bf16: unknown activation %d", activation);
  BH_REQUIRE(activation == 0 || (N % 16 == 0 && !accumulate),
             "gemm_bf16: SwiGLU needs a multiple of 16 outputs (got %d) and no accumulation", N);
  BH_REQUIRE((M + 127) / 128 <= 65535, "gemm_bf16: M=%d needs more than 65535 row tiles", M);
  BH_REQUIRE(!ahead_ss || bh_gemm_bf16_takes_norm(M, N, K, layout, activation),
             "gemm_bf16: a product of M=%d N=%d K=%d cannot take prepared norm rows (bh_gemm_bf16_takes_norm)", M, N, K);
  BH_REQUIRE(!behind_weight || bh_gemm_bf16_norm_blocks(M, N, K, layout, activation) > 0,
             "gemm_bf16: a product of M=%d N=%d K=%d cannot carry a norm (bh_gemm_bf16_norm_blocks)", M, N, K);
  BH_REQUIRE(!ahead_ss || (ahead_blocks > 0 && ahead_eps > 0.f), "gemm_bf16: the norm ahead needs partial sums and an epsilon");
  BH_REQUIRE(!behind_weight || (behind_rows && behind_ss && c_dtype == BH_F32 && activation == 0),
             "gemm_bf16: the norm behind needs its outputs, a float32 product and no activation");
  BH_REQUIRE(!behind_weight || behind_weight_dtype == BH_F32 || behind_weight_dtype == BH_BF16,
             "gemm_bf16: unknown norm weight dtype %d", behind_weight_dtype);
  const RidingNorm norm = {ahead_ss, ahead_blocks, ahead_eps, behind_weight, behind_weight_dtype == BH_F32,
                           (uint16_t*)behind_rows, behind_ss};
  const bool f32 = c_dtype == BH_F32;
  const auto block_rows_ok = [](int rows) { return rows == 0 || rows == 8 || rows == 16; };
  BH_REQUIRE(block_rows_ok(a_block_rows) && block_rows_ok(c_block_rows) && block_rows_ok(behind_block_rows),
             "gemm_bf16: rows lie in blocks of 8 or 16, or one after the other (0)");
  BH_REQUIRE(a_block_rows == 0 || a_block_rows == bh_gemm_bf16_reads_blocked(M, N, K, layout, activation),
             "gemm_bf16: a product of M=%d N=%d K=%d does not read rows in blocks of %d (bh_gemm_bf16_reads_blocked)", M, N, K, a_block_rows);
  BH_REQUIRE(c_block_rows == 0 || (activation && N % 32 == 0), "gemm_bf16: only SwiGLU's output goes out in blocks, N=%d a multiple of 32", N);
  BH_REQUIRE(behind_block_rows == 0 || (behind_weight && N % 32 == 0), "gemm_bf16: rows in blocks for a norm behind need that norm, N=%d a multiple of 32", N);
  const bool skinny = [&] {
    int rows, columns;
    tiled_config(M, N, activation != 0, &rows, &columns);
    return M <= 64 && !tiled_whole(M, N, K, layout, rows, columns) && !(M <= SKINNY_UP_TO_ROWS && gemm_slices_takes(M, N, K, layout, activation));
  }();
  // 33 to 128 rows from blocks of 16: the kernel whose waves share the activations through LDS, then the finishing kernel
  const bool slices = scratch != nullptr && a_block_rows == 16 && !skinny && gemm_slices_takes(M, N, K, layout, activation);
  BH_REQUIRE(skinny || slices || (c_block_rows != 8 && behind_block_rows == 0 && (c_block_rows == 0 || gemm_turns_blocks(M, N, K, layout, activation))),
             "gemm_bf16: a product of M=%d N=%d K=%d does not write these blocks", M, N, K);
  dim3 finish_grid((N + FINISH_COLUMNS - 1) / FINISH_COLUMNS, (M + 15) / 16);
  const RowBlocks finish_blocks = {0, slices ? c_block_rows : 0, slices ? behind_block_rows : 0};
#define BH_FINISH(SWIGLU, TC)                                                                                \
  gemm_parts_finish_kernel<SWIGLU, TC><<<finish_grid, 256, 0, stream>>>((const float*)scratch, (TC*)c, M, N, K, \
                                                                         parts, accumulate, norm, finish_blocks)
  if (!f32 && a_block_rows == 16 && layout == 1 && gemm_slices_gated(M, N, K, activation))   // the SwiGLU of many outputs: no parts, no finishing kernel
    return gemm_slices_launch_gated(a, w, c, c_block_rows, M, N, K, ahead_ss, ahead_blocks, ahead_eps, stream);
  if (slices) {
    BH_REQUIRE(((uintptr_t)c | (uintptr_t)scratch | (uintptr_t)behind_rows) % 16 == 0,
               "gemm_bf16: output, scratch memory and norm rows must be 16-byte aligned");
    const int parts = gemm_slices_parts(M, N, K, activation, nullptr);
    // One part, float32 rows out, nothing to add, to scale or to prepare: the sums are the output, in its own order
    // (the head product of 33 to 128 rows: 151,936 x 4,096 at 64 rows 279 us with the finishing kernel's copy).
    if (parts == 1 && f32 && !activation && !accumulate && !ahead_ss && !behind_weight)
      return gemm_slices_launch(a, w, (float*)c, M, N, K, activation, stream);
    if (int status = gemm_slices_launch(a, w, (float*)scratch, M, N, K, activation, stream)) return status;
    if (activation) { if (f32) BH_FINISH(true, float); else BH_FINISH(true, bf16_t); }
    else { if (f32) BH_FINISH(false, float); else BH_FINISH(false, bf16_t); }
    return bh_check_launch("gemm_parts_finish");
  }
  const int a_blocked = a_block_rows == 16 && !skinny, c_blocked = c_block_rows == 16 && !skinny;
  if (!ahead_ss && !behind_weight && (f32 || !accumulate)) {   // many rows: the kernel whose wave groups take turns
    if (const int blocks = gemm_turns_blocks(M, N, K, layout, activation))
      return gemm_turns_launch(a, w, c, c_dtype, accumulate, M, N, K, activation, blocks, a_blocked, c_blocked, stream);
  }
#define BH_PICK(FN, TILES, EXTRA, ...)                                             \
  do {                                                                              \
    if (f32) FN<TILES, EXTRA, float>(__VA_ARGS__);                                  \
    else FN<TILES, EXTRA, bf16_t>(__VA_ARGS__);                                     \
  } while (0)
  const bool in_parts = scratch != nullptr && tiled_or_turns_parts(M, N, K, layout, activation) > 1;
  BH_REQUIRE(!a_blocked || (in_parts && gemm_turns_parts(M, N, K, layout, activation) > 1),
             "gemm_bf16: a product of M=%d N=%d K=%d that reads rows in blocks needs its scratch memory", M, N, K);
  BH_REQUIRE(in_parts || !behind_weight || tiled_or_turns_parts(M, N, K, layout, activation) == 1,
             "gemm_bf16: a product of M=%d N=%d K=%d carries a norm through its finishing kernel and needs scratch memory", M, N, K);
  if (in_parts) {   // K in parts, then the finishing kernel
    BH_REQUIRE(((uintptr_t)c | (uintptr_t)scratch | (uintptr_t)behind_rows) % 16 == 0,
               "gemm_bf16: output, scratch memory and norm rows must be 16-byte aligned");
    int parts, each;
    if (const int turns_parts = gemm_turns_parts(M, N, K, layout, activation); turns_parts > 1) {
      parts = turns_parts;
      if (int status = gemm_turns_launch_parts(a, w, (float*)scratch, M, N, K, parts, a_blocked, stream)) return status;
    } else {
      tiled_parts(M, N, K, layout, activation != 0, &parts, &each);
      const RidingNorm none = {};
      if (activation) launch_tiled<true, true, float>(a, w, nullptr, M, N, K, 0, none, (float*)scratch, stream);
      else launch_tiled<true, false, float>(a, w, nullptr, M, N, K, 0, none, (float*)scratch, stream);
      if (int status = bh_check_launch("gemm_tiled")) return status;
    }
    if (activation) { if (f32) BH_FINISH(true, float); else BH_FINISH(true, bf16_t); }
    else { if (f32) BH_FINISH(false, float); else BH_FINISH(false, bf16_t); }
#undef BH_FINISH
    return bh_check_launch("gemm_parts_finish");
  }
  if (skinny) {
    const int pair_blocks = N / 16;
    const RowBlocks blocks = {a_block_rows, c_block_rows, behind_block_rows};
    if (activation) {
      if (layout) BH_PICK(launch_skinny, true, 2, a, w, c, M, N, K, 0, pair_blocks, norm, blocks, stream);
      else BH_PICK(launch_skinny, false, 2, a, w, c, M, N, K, 0, pair_blocks, norm, blocks, stream);
    } else {
      if (layout) BH_PICK(launch_skinny, true, 1, a, w, c, M, N, K, accumulate, 0, norm, blocks, stream);
      else BH_PICK(launch_skinny, false, 1, a, w, c, M, N, K, accumulate, 0, norm, blocks, stream);
    }
    return bh_check_launch("gemm_skinny");
  }
  if (activation) {
    if (layout) BH_PICK(launch_tiled, true, true, a, w, c, M, N, K, 0, norm, nullptr, stream);
    else BH_PICK(launch_tiled, false, true, a, w, c, M, N, K, 0, norm, nullptr, stream);
  } else {
    if (layout) BH_PICK(launch_tiled, true, false, a, w, c, M, N, K, accumulate, norm, nullptr, stream);
    else BH_PICK(launch_tiled, false, false, a, w, c, M, N, K, accumulate, norm, nullptr, stream);
  }
#undef BH_PICK
  return bh_check_launch("gemm_tiled");
}

// residual[M, N] += A W^T and normed = RMSNorm(residual; weight, eps) as bfloat16, in one go: for the products of
// many rows whose K the turns kernel multiplies in parts (bh_gemm_bf16_finishes_norm says which), whose finishing
// kernel streams the residual anyway.  `scratch`: bh_gemm_bf16_scratch() bytes.
extern "C" int bh_gemm_bf16_finishes_norm(int M, int N, int K, int layout) {
  if (M <= 0 || N <= 0 || K <= 0 || N % 8 != 0 || N > 8 * 128 * FINISH_NORM_PIECES) return 0;
  const int parts = gemm_turns_parts(M, N, K, layout, 0);
  return parts > 1 && parts <= MAX_TURNS_PARTS ? 1 : 0;
}
extern "C" int bh_gemm_bf16_then_norm(const void* a, const void* w, float* residual, int M, int N, int K, int layout,
                                      const void* norm_weight, int norm_weight_dtype, float eps, void* normed,
                                      void* scratch, int a_blocked, int normed_blocked, hipStream_t stream) {
  BH_REQUIRE(bh_gemm_bf16_finishes_norm(M, N, K, layout),
             "gemm_bf16_then_norm: a product of M=%d N=%d K=%d does not finish a norm (bh_gemm_bf16_finishes_norm)", M, N, K);
  BH_REQUIRE(a && w && residual && norm_weight && normed && scratch, "gemm_bf16_then_norm: every operand is needed");
  BH_REQUIRE(norm_weight_dtype == BH_F32 || norm_weight_dtype == BH_BF16, "gemm_bf16_then_norm: unknown norm weight dtype %d", norm_weight_dtype);
  BH_REQUIRE(eps >= 0.f, "gemm_bf16_then_norm: eps must not be negative");
  BH_REQUIRE(((uintptr_t)a | (uintptr_t)w | (uintptr_t)residual | (uintptr_t)normed | (uintptr_t)scratch | (uintptr_t)norm_weight) % 16 == 0,
             "gemm_bf16_then_norm: operands must be 16-byte aligned");
  BH_REQUIRE(!normed_blocked || N % 32 == 0, "gemm_bf16_then_norm: rows in blocks need N=%d to be a multiple of 32", N);
  const int parts = gemm_turns_parts(M, N, K, layout, 0);
  if (int status = gemm_turns_launch_parts(a, w, (float*)scratch, M, N, K, parts, a_blocked, stream)) return status;
#define BH_FINISH_NORM_ROWS(PARTS, ROWS)                                                                              \
  gemm_parts_finish_norm_kernel<PARTS, ROWS><<<(M + ROWS - 1) / ROWS, 128 * ROWS, 0, stream>>>(                        \
      (const float*)scratch, residual, M, N, parts, norm_weight, norm_weight_dtype == BH_F32, eps, (uint16_t*)normed, \
      normed_blocked)
  // Rows per block: at 1,024 rows two ran 4 % faster than eight (more and smaller blocks), from 2,048 rows on all ran
  // alike; full 128-byte lines of the blocked output take eight.
  const int rows_per_block = M >= 4096 ? 8 : M >= 2048 ? 4 : 2;
#define BH_FINISH_NORM(PARTS)                          \
  do {                                                 \
    if (rows_per_block == 8) BH_FINISH_NORM_ROWS(PARTS, 8); \
    else if (rows_per_block == 4) BH_FINISH_NORM_ROWS(PARTS, 4); \
    else BH_FINISH_NORM_ROWS(PARTS, 2); \
  } while (0)
  if (parts <= 2) BH_FINISH_NORM(2);
  else if (parts <= 4) BH_FINISH_NORM(4);
  else BH_FINISH_NORM(MAX_TURNS_PARTS);
#undef BH_FINISH_NORM_ROWS
#undef BH_FINISH_NORM
  return bh_check_launch("gemm_parts_finish_norm");
}

// A W^T of many rows left as the float32 sums of K's parts, [parts][M][N], for a consumer that adds them up itself
// (the q/k norm, rotation and cache write: bh_qk_norm_rope_cache_sums): the product without its finishing kernel.
// bh_gemm_bf16_bare_parts: how many parts such a product of these sizes has, 0 where the product is not one whose
// K goes in parts through the kernel for many rows.  `sums`: parts * M * N floats.
extern "C" int bh_gemm_bf16_bare_parts(int M, int N, int K, int layout) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const int parts = gemm_turns_parts(M, N, K, layout, 0);
  return parts > 1 && parts <= MAX_TURNS_PARTS ? parts : 0;
}
extern "C" int bh_gemm_bf16_bare(const void* a, const void* w, float* sums, int M, int N, int K, int layout, int a_blocked,
                                 hipStream_t stream) {
  const int parts = bh_gemm_bf16_bare_parts(M, N, K, layout);
  BH_REQUIRE(parts > 0, "gemm_bf16_bare: a product of M=%d N=%d K=%d is not left in parts (bh_gemm_bf16_bare_parts)", M, N, K);
  BH_REQUIRE(a && w && sums, "gemm_bf16_bare: every operand is needed");
  BH_REQUIRE(((uintptr_t)a | (uintptr_t)w | (uintptr_t)sums) % 16 == 0, "gemm_bf16_bare: operands must be 16-byte aligned");
  return gemm_turns_launch_parts(a, w, sums, M, N, K, parts, a_blocked, stream);
}
