// bfloat16 products of 33 to 128 rows (decode steps of many sequences, short prompts): still bound by reading W
// once, but the activations are no longer small.  A wave that multiplies a 2 KB chunk of W (16 weight rows x 64 k)
// needs the 8 KB of 64 activation rows for the same k; with a workgroup per 16 weight rows (the kernel for up to
// 32 rows, gemm_bf16.hip) every wave fetches those itself, and the L2 then hands out five bytes for each byte of
// W, which is what bounds it.  Here the waves of a workgroup own neighbouring blocks of 16 weight rows and walk
// over k together, a stage of 128 or 256 k at a time: the stage's activations go into LDS once per workgroup, each
// wave asks for its own W of the next stage while this one is multiplied, and takes the activation operands from
// LDS, which has a path of its own.  Two forms:
//   K in parts over workgroups of four waves, so that the chip is full (about 512 workgroups); the bare sums go to
//   scratch memory as [part][row][weight row] and gemm_parts_finish_kernel (gemm_bf16.hip) adds them and applies
//   norm factors, SwiGLU and accumulation;
//   a SwiGLU of so many outputs that workgroups of six waves per 48 outputs fill the chip walks over all of K
//   and finishes itself (GATED below): no scratch memory, no second launch.
//
// Needs: W in the tiles layout (16 rows x 64 k blocks), the activations in blocks of 16 rows x 32 k in operand
// order (bh_blocked_index; their buffer holds whole blocks, so rows beyond M may be read and hold anything: a
// column of the product depends on its own activation row only, and those columns are not stored).
//
// Where the time goes (Qwen3-8B sizes, 64 rows, qkv; a copy of the first form with parts switched off): W loads alone
// 9.9 us (5.1 TB/s; one workgroup per 16 weight rows reads at 5.5), with the activations' loads, LDS writes and
// meetings 10.9, with the LDS reads and products too 11.2; storing the partial sums of 8 parts (12.6 MB) 14.5; with
// the finishing kernel 22.  The products themselves run as fast as those of 8 rows; cutting K costs as much again.
#include "gemm_bf16_slices.h"

#include <algorithm>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

namespace {

__device__ inline bf16x8_t as_bf16x8(u32x4_t v) { return __builtin_bit_cast(bf16x8_t, v); }
__device__ inline u32x4_t load16_stream(const uint16_t* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
}

// s_waitcnt immediate of gfx9 (vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8): until the wave's LDS accesses are
// done; nothing is asked of the other counters.
#define WAIT_LDS() __builtin_amdgcn_s_waitcnt(15 | (3 << 14) | (7 << 4) | (0 << 8))
// All waves of the workgroup have written their share of LDS and are done with what they read before.
#define MEET()                            \
  do {                                    \
    WAIT_LDS();                           \
    __builtin_amdgcn_sched_barrier(0);    \
    __builtin_amdgcn_s_barrier();         \
    __builtin_amdgcn_sched_barrier(0);    \
  } while (0)

constexpr int STAGE_K = 256;             // K is cut into parts at multiples of this

// MB: blocks of 16 activation rows (2 to 8).  A stage is SC chunks of 64 k: each wave holds its SC x 2 KB of W for it
// in registers and the workgroup the activations' MB x SC x 2 KB in LDS; while a stage is multiplied the next one's
// loads are on their way (registers and LDS hold two stages), one meeting of the waves per stage.
// DEEP: W is asked for two stages ahead (three sets of registers; the activations, which come from the L2, stay one
// stage ahead).  Qwen3-8B sizes, each product alone, us without / with: K in parts, 64 rows qkv 18.6 / 18.1, down 28.3 /
// 27.5, 96 rows qkv 21.2 / 20.5, down 33.4 / 32.1, o the same; the SwiGLU that finishes itself 48 rows 39.4 / 41.3, 64 rows
// 47.3 / 44.5, 96 rows 50.7 / 55.4, so that one takes it at 49 to 64 rows only; a decode step of 64 sequences at context
// 640 5.50 -> 5.40 ms.
// GATED: SwiGLU with all of K in one workgroup (one part): waves 0 to 3 own four blocks of gate rows, waves 4 to 7 the
// blocks of up rows of the same outputs (N / 16 blocks further on); at the end the up waves hand their sums over
// through LDS and the gate waves write bfloat16(silu(gate) * up), times the row factors of a norm ahead, into `gated`
// (in blocks of gated_block_rows rows, or rows): no scratch memory and no finishing kernel.
struct GatedOut {
  uint16_t* gated;        // [M][N] bfloat16
  int gated_block_rows;
  int N;                  // outputs; W has 2 N rows
  const float* ahead_ss;  // [M][ahead_blocks] partial sums of squares of the activations' rows, or null
  int ahead_blocks;
  float ahead_eps;
};

__device__ inline float silu_mul(float gate, float up) { return gate / (1.0f + expf(-gate)) * up; }

template <int MB, int SC, int WAVES, bool GATED, bool DEEP = false>
__global__ __launch_bounds__(64 * WAVES, GATED ? (WAVES + 3) / 4 : (MB > 4 || WAVES > 4) ? 2 : 4) void gemm_slices_kernel(const uint16_t* __restrict__ a,
                                                                    const uint16_t* __restrict__ w,
                                                                    float* __restrict__ sums, int M, int w_rows, int K,
                                                                    int stages_per_part, GatedOut out) {
  constexpr int STEPS = 2 * SC, PIECES = MB * STEPS, MINE = (PIECES + WAVES - 1) / WAVES;   // per stage: steps of 32 k; 1 KB pieces; a wave's
  __shared__ __attribute__((aligned(16))) u32x4_t xs[2][PIECES * 64];   // [stage in turn][block of 16 rows][step of 32 k][lane]
  const int lane = threadIdx.x % 64;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int blocks = w_rows / 16, chunks = K / 64, stages = chunks / SC;
  // GATED: blocks of gate rows 4 x .. 4 x + 3 and, `blocks / 2` further on, their up rows
  const int block_own = GATED ? blockIdx.x * (WAVES / 2) + wave % (WAVES / 2) + (wave / (WAVES / 2)) * (blocks / 2)
                              : blockIdx.x * WAVES + wave;
  const bool owned = GATED ? blockIdx.x * (WAVES / 2) + wave % (WAVES / 2) < blocks / 2 : block_own < blocks;
  const int block = owned ? block_own : blocks - 1;    // a wave beyond the last block repeats it and stores nothing
  const int first = blockIdx.y * stages_per_part, end = min(stages, first + stages_per_part);
  const uint16_t* wp = w + (size_t)block * chunks * 1024 + lane * 8;
  const int q = lane / 16, r = lane % 16;
  // Half u of a chunk holds, for lane group q, k 16 q + 8 u .. + 7 of the chunk's 64: in the activations' blocks
  // that is step (2 q + u) / 4 of the chunk's two, lane group (2 q + u) % 4.
  int x_at[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) x_at[u] = ((2 * q + u) / 4) * 64 + 16 * ((2 * q + u) % 4) + r;
  // This wave's share of a stage's activations: the pieces of 1 KB (a block of 16 rows x 32 k) wave, wave + 8, ...
  const int a_row_block = (K / 32) * 512;              // elements from one block of 16 rows to the next
  int x_from[MINE];
#pragma unroll
  for (int j = 0; j < MINE; ++j) {
    const int e = min(j * WAVES + wave, PIECES - 1);   // (a wave without a piece repeats the last one)
    x_from[j] = (e / STEPS) * a_row_block + (e % STEPS) * 512 + lane * 8;
  }

  f32x4_t acc[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) acc[b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  // The norm ahead: eight threads per row add up its partial sums, each every eighth, in a fixed order.
  __shared__ float row_factor[GATED ? 16 * MB : 1];
  if (GATED && out.ahead_ss) {
    const int part = threadIdx.x % 4;    // four threads per row, 16 WAVES rows at a time
#pragma unroll
    for (int row0 = 0; row0 < 16 * MB; row0 += 16 * WAVES) {
      const int row = row0 + threadIdx.x / 4;
      float ss = 0.f;
      if (row < M)
        for (int block0 = part; block0 < out.ahead_blocks; block0 += 4) ss += out.ahead_ss[(size_t)row * out.ahead_blocks + block0];
      ss += __shfl_xor(ss, 2, 64);
      ss += __shfl_xor(ss, 1, 64);
      if (part == 0 && row < 16 * MB) row_factor[row] = row < M ? 1.0f / sqrtf(ss / (float)K + out.ahead_eps) : 0.f;   // visible after the first meeting
    }
  }

  auto ask_x = [&](int t, u32x4_t (&xv)[MINE]) {
#pragma unroll
    for (int j = 0; j < MINE; ++j) xv[j] = *reinterpret_cast<const u32x4_t*>(a + (size_t)(x_from[j] + t * (STEPS * 512)));
  };
  auto ask_w = [&](int t, u32x4_t (&wv)[SC][2]) {
#pragma unroll
    for (int c = 0; c < SC; ++c)
#pragma unroll
      for (int u = 0; u < 2; ++u) wv[c][u] = load16_stream(wp + ((size_t)t * SC + c) * 1024 + u * 512);
  };
  auto ask = [&](int t, u32x4_t (&wv)[SC][2], u32x4_t (&xv)[MINE]) {
    ask_x(t, xv);
    ask_w(t, wv);
  };
  auto stash = [&](int turn, const u32x4_t (&xv)[MINE]) {
#pragma unroll
    for (int j = 0; j < MINE; ++j)
      if (PIECES % WAVES == 0 || j * WAVES + wave < PIECES) xs[turn][(j * WAVES + wave) * 64 + lane] = xv[j];
  };
  auto multiply = [&](int turn, const u32x4_t (&wv)[SC][2]) {
#pragma unroll
    for (int c = 0; c < SC; ++c)
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int b = 0; b < MB; ++b)
          acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wv[c][u]), as_bf16x8(xs[turn][(b * STEPS + 2 * c) * 64 + x_at[u]]),
                                                           acc[b], 0, 0, 0);
  };

  // Stage t lies in turn (t - first) % 2.  Before a wave writes a turn's LDS again, every wave has passed the
  // meeting that follows the other turn's writes, which it reaches only after it has multiplied this turn's.
  u32x4_t w0[SC][2], w1[SC][2], x0[MINE], x1[MINE];
  if (DEEP) {
    // W two stages ahead (three sets of registers), the activations one (they come from the L2): a stage's
    // activations are asked for before the W of the stage after it, so that waiting for them leaves that W on its way.
    u32x4_t w2[SC][2];
    ask_x(first, x0);
    ask_w(first, w0);
    if (first + 1 < end) ask_w(first + 1, w1);
#define BH_STAGE(at, turn, w_now, w_then, x_now, x_then)  \
    stash(turn, x_now);                                   \
    MEET();                                               \
    if (t + (at) + 1 < end) ask_x(t + (at) + 1, x_then);  \
    if (t + (at) + 2 < end) ask_w(t + (at) + 2, w_then);  \
    multiply(turn, w_now);                                \
    if (t + (at) + 1 >= end) break;
    for (int t = first; t < end; t += 6) {
      BH_STAGE(0, 0, w0, w2, x0, x1)
      BH_STAGE(1, 1, w1, w0, x1, x0)
      BH_STAGE(2, 0, w2, w1, x0, x1)
      BH_STAGE(3, 1, w0, w2, x1, x0)
      BH_STAGE(4, 0, w1, w0, x0, x1)
      BH_STAGE(5, 1, w2, w1, x1, x0)
    }
#undef BH_STAGE
  } else {
    ask(first, w0, x0);
    for (int t = first; t < end; t += 2) {
      stash(0, x0);
      MEET();
      if (t + 1 < end) ask(t + 1, w1, x1);
      multiply(0, w0);
      if (t + 1 >= end) break;
      stash(1, x1);
      MEET();
      if (t + 2 < end) ask(t + 2, w0, x0);
      multiply(1, w1);
    }
  }
  // acc[b][i]: activation row 16 b + r, weight row 16 block + 4 q + i
  if (GATED) {
    f32x4_t* handed = reinterpret_cast<f32x4_t*>(&xs[0][0]);   // [up wave][block of 16 rows][lane]: WAVES / 2 x MB KB of the 2 PIECES KB
    static_assert(WAVES / 2 * MB <= 2 * PIECES, "the up waves' sums fit where the activations stood");
    MEET();   // everyone has read the last stage
    if (wave >= WAVES / 2) {
#pragma unroll
      for (int b = 0; b < MB; ++b) handed[((wave - WAVES / 2) * MB + b) * 64 + lane] = acc[b];
    }
    MEET();
    if (wave >= WAVES / 2 || !owned) return;
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      const int m = 16 * b + r, n = 16 * block_own + 4 * q;
      if (m >= M) continue;
      const f32x4_t up = handed[(wave * MB + b) * 64 + lane];
      const float f = out.ahead_ss ? row_factor[m] : 1.f;
      uint32_t packed[2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        packed[i] = (uint32_t)f32_to_bf16_bits(silu_mul(acc[b][2 * i] * f, up[2 * i] * f)) |
                    ((uint32_t)f32_to_bf16_bits(silu_mul(acc[b][2 * i + 1] * f, up[2 * i + 1] * f)) << 16);
      uint32_t* at = reinterpret_cast<uint32_t*>(out.gated + bh_rows_index(out.gated_block_rows, m, n, out.N));
      at[0] = packed[0];
      at[1] = packed[1];
    }
    return;
  }
  if (!owned) return;
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    const int m = 16 * b + r;
    if (m < M)
      *reinterpret_cast<f32x4_t*>(sums + ((size_t)blockIdx.y * M + m) * w_rows + 16 * block_own + 4 * q) = acc[b];
  }
}

constexpr int MOST_PARTS = 16;           // what the finishing kernel adds up at most
// Up to how many rows (Qwen3-8B sizes, each product alone, us against the tiles with K in parts): 96 rows qkv 21.2 / 23.5,
// o 17.6 / 20.6, gate+up 55.4 / 66.2, down 33.3 / 42.5; 128 rows qkv 23.5 / 24.2, o 20.0 / 23.4, down 37.9 / 39.4, but
// gate+up 74.2 / 63.1 (eight blocks of rows in registers at stages of four chunks).
constexpr int MOST_ROWS = 128, MOST_ROWS_GATED = 96;

}  // namespace

// From 33 rows on; a product of very many outputs (the head over a long vocabulary, whose workgroups fill the chip many
// times over without a cut of K) from 17 rows on: 151,936 x 4,096, us with the kernel for up to 32 rows / here: 17 rows
// 275 / 221, 32 rows 286 / 234 (16 rows there 225).
constexpr int FEW_ROWS_FROM = 17, FEW_ROWS_OUTPUTS = 32768;
bool gemm_slices_takes(int M, int N, int K, int layout, int activation) {
  const bool rows_fit = M > 32 || (M >= FEW_ROWS_FROM && !activation && N >= FEW_ROWS_OUTPUTS);
  return layout == 1 && rows_fit && M <= (activation ? MOST_ROWS_GATED : MOST_ROWS) && K >= 512 && K % STAGE_K == 0 && N % 16 == 0 && N >= 128 &&
         (long)64 * K < (1L << 31);
}

// Measured at the Qwen3-8B sizes, 64 rows, each product alone with its finishing kernel (us: qkv / o / down), against
// 21.6 / 18.1 / 32.5 of the tiles with K in parts: eight waves a workgroup, stages of two chunks, about 384 workgroups
// 22.2 / 17.5 / 31.3; four waves (twice the activations' bytes from the L2, half the bytes of partial sums), stages of
// four chunks, 384 workgroups 18.1 / 15.9 / 29.7; four waves, two chunks, 512 workgroups 18.6 / 15.6 / 28.2, and in the
// whole model (decode step of 64 sequences, context 640) 5.50 against 5.56 and 5.67 ms for the other two, 5.98 before.
constexpr int WAVES = 4;
static int target_workgroups() { return 2 * bh_compute_units(); }      // 512 on the chip these were measured on
// The SwiGLU that finishes itself has one workgroup per compute unit at most, so a wave may use twice the registers:
// stages of four chunks, 8 to 16 KB of W on their way per wave (gate+up at 64 rows with eight waves per 64 outputs
// 46.4 us; with stages of two chunks 56.1; four waves per 32 outputs 49.7; K in two parts and the finishing kernel
// 52.1; the tiles 47.4).
// How many blocks of gate rows a workgroup takes (twice as many waves): a workgroup walks over all of K, so the
// kernel lasts as long as the compute unit that carries the most bytes, and workgroups that share a compute unit share
// its bandwidth: the fewest bytes per compute unit, ceil(workgroups / compute units) x blocks, decides, the smaller
// workgroup at a tie.  Qwen3-8B (768 blocks of gate rows, 256 compute units): three blocks, 256 workgroups of six
// waves; gate+up alone against four blocks (192 workgroups of eight waves): 40 rows 39.7 / 44.5 us, 64 rows 47.1 / 46.7,
// 96 rows 50.6 / 54.9.  Qwen3-14B (1,088 blocks): five, gate+up at 64 rows 71.6 us (5.0 TB/s); three, with 363 workgroups,
// 99.7.  Qwen3-32B (1,600 blocks): seven, 117.5 us (4.5 TB/s; 18 registers of a wave spilled); three 145.7.
constexpr int GATED_CHUNKS = 4, GATED_MOST_BLOCKS = 8;
// (Beyond 64 rows the registers of a wave hold six blocks of rows: more than eight waves a workgroup leave a wave too few
// and it spills, 96 rows at Qwen3-14B's sizes 101.8 us with ten waves.)
static int gated_blocks(int M, int N) {
  const int gate_blocks = N / 16, units = bh_compute_units();
  int best = 3, best_cost = 1 << 30;
  for (int b = 3; b <= (M > 64 ? 4 : GATED_MOST_BLOCKS); ++b) {
    const int workgroups = (gate_blocks + b - 1) / b, cost = ((workgroups + units - 1) / units) * b;
    if (cost < best_cost) best = b, best_cost = cost;
  }
  return best;
}

bool gemm_slices_gated(int M, int N, int K, int activation) {
  // With enough outputs that its workgroups fill the chip, a SwiGLU needs no parts.  (Also tried for 9 to 32 rows, which
  // the kernel with a workgroup per 16 weight rows takes: gate+up alone 38.4 against 40.1 us at 17 to 32 rows, 35.6 against
  // 34.7 at 16, but the whole decode step slower, 16 sequences 4.53 against 4.30 ms, 32 sequences 5.53 against 5.48.)
  return activation && gemm_slices_takes(M, N, K, 1, activation) && N % 32 == 0 &&
         (N / 16 + gated_blocks(M, N) - 1) / gated_blocks(M, N) >= bh_compute_units() * 5 / 8;
}

int gemm_slices_parts(int M, int N, int K, int activation, int* stages_per_part) {
  const int w_blocks = (activation ? 2 * N : N) / 16, groups = (w_blocks + WAVES - 1) / WAVES;
  const int stages = K / STAGE_K;
  if (gemm_slices_gated(M, N, K, activation)) {
    if (stages_per_part) *stages_per_part = stages;
    return 1;
  }
  int parts = std::max(1, std::min({stages / 2, MOST_PARTS, (target_workgroups() + groups / 2) / groups}));   // 512 k each at least
  const int each = (stages + parts - 1) / parts;
  parts = (stages + each - 1) / each;
  if (stages_per_part) *stages_per_part = each;       // in units of STAGE_K
  (void)M;
  return parts;
}

int gemm_slices_launch(const void* a, const void* w, float* sums, int M, int N, int K, int activation,
                       hipStream_t stream) {
  BH_REQUIRE(gemm_slices_takes(M, N, K, 1, activation), "gemm_slices: a product of M=%d N=%d K=%d is not one this kernel takes", M, N, K);
  BH_REQUIRE(((uintptr_t)a | (uintptr_t)w | (uintptr_t)sums) % 16 == 0, "gemm_slices: operands must be 16-byte aligned");
  const int w_rows = activation ? 2 * N : N;
  int each;
  const int parts = gemm_slices_parts(M, N, K, activation, &each);
  const GatedOut none = {};
  constexpr int SC = 2;
  // One part and many times the chip's workgroups (the head over a long vocabulary): eight waves a workgroup, so that half
  // as many bytes of activations cross from the L2, pay at 49 to 96 rows (151,936 x 4,096, us with four / eight waves: 32 rows
  // 230 / 244, 48 rows 249 / 252, 64 rows 262 / 254, 96 rows 282 / 252, 128 rows 306 / 303).
  if (parts == 1 && M > 48 && M <= 96 && w_rows / 16 >= 16 * bh_compute_units()) {
    const dim3 grid((w_rows / 16 + 7) / 8, parts), block(64 * 8);
#define BH_SLICES8(MB) gemm_slices_kernel<MB, SC, 8, false, true><<<grid, block, 0, stream>>>((const uint16_t*)a, (const uint16_t*)w, sums, M, w_rows, K, each * (STAGE_K / 64 / SC), none)
    if (M <= 64) BH_SLICES8(4);
    else BH_SLICES8(6);
#undef BH_SLICES8
    return bh_check_launch("gemm_slices");
  }
  const dim3 grid((w_rows / 16 + WAVES - 1) / WAVES, parts), block(64 * WAVES);
#define BH_SLICES(MB) gemm_slices_kernel<MB, SC, WAVES, false, true><<<grid, block, 0, stream>>>((const uint16_t*)a, (const uint16_t*)w, sums, M, w_rows, K, each * (STAGE_K / 64 / SC), none)
  if (M <= 32) BH_SLICES(2);
  else if (M <= 48) BH_SLICES(3);
  else if (M <= 64) BH_SLICES(4);
  else if (M <= 96) BH_SLICES(6);
  else BH_SLICES(8);
#undef BH_SLICES
  return bh_check_launch("gemm_slices");
}

int gemm_slices_launch_gated(const void* a, const void* w, void* gated, int gated_block_rows, int M, int N, int K,
                             const float* ahead_ss, int ahead_blocks, float ahead_eps, hipStream_t stream) {
  BH_REQUIRE(gemm_slices_gated(M, N, K, 1), "gemm_slices: a SwiGLU of M=%d N=%d K=%d is not one this kernel finishes itself", M, N, K);
  BH_REQUIRE(((uintptr_t)a | (uintptr_t)w | (uintptr_t)gated) % 16 == 0, "gemm_slices: operands must be 16-byte aligned");
  BH_REQUIRE(!ahead_ss || (ahead_blocks > 0 && ahead_eps > 0.f), "gemm_slices: the norm ahead needs partial sums and an epsilon");
  constexpr int SC = GATED_CHUNKS;
  const int blocks_each = gated_blocks(M, N), WAVES = 2 * blocks_each;
  const GatedOut out = {(uint16_t*)gated, gated_block_rows, N, ahead_ss, ahead_blocks, ahead_eps};
  const dim3 grid((N / 16 + WAVES / 2 - 1) / (WAVES / 2)), block(64 * WAVES);
  const int stages = K / (64 * SC);
#define BH_GATED(MB, NW) gemm_slices_kernel<MB, SC, NW, true, MB == 4><<<grid, block, 0, stream>>>((const uint16_t*)a, (const uint16_t*)w, nullptr, M, 2 * N, K, stages, out)
#define BH_GATED_ROWS(NW) do { if (M <= 48) BH_GATED(3, NW); else if (M <= 64) BH_GATED(4, NW); else BH_GATED(6, NW); } while (0)
  static_assert(MOST_ROWS_GATED <= 96 && GATED_MOST_BLOCKS == 8, "the forms below");
  switch (blocks_each) {
    case 3: BH_GATED_ROWS(6); break;
    case 4: BH_GATED_ROWS(8); break;
    case 5: BH_GATED_ROWS(10); break;
    case 6: BH_GATED_ROWS(12); break;
    case 7: BH_GATED_ROWS(14); break;
    default: BH_GATED_ROWS(16); break;
  }
#undef BH_GATED_ROWS
#undef BH_GATED
  return bh_check_launch("gemm_slices");
}
