// bfloat16 matrix products of many rows, C[M, N] (+)= A[M, K] * W[N, K]^T with W in the tiles layout
// (see gemm_bf16.hip), for the shapes where a 256-row tile fills the chip: prompts from 320 tokens on.
//
// A workgroup of eight waves owns 256 rows x 32 YB weight rows.  Its waves form two groups of four (one wave
// of each group per SIMD) that take turns: while one group multiplies (32, 24 or 16 MFMAs on operands it holds
// in registers), the other reads its next operands from LDS and asks for data that is three steps ahead; a
// barrier ends every turn.  So the matrix cores always have one wave per SIMD that does nothing but multiply,
// and no wave waits for memory in the middle of its multiplies.  A step is half a 64-wide k slice: the 32 k
// values that one 16x16x32 MFMA takes.
//
// Global memory goes to LDS directly (16-byte loads that write LDS at the wave's base + 16 * lane): 1 KB per
// load, which is one operand of 16 rows x 32 k in lane order, so that reading it back is one conflict-free
// 16-byte read per lane.  Four lanes bring 256 bytes of a block of W; of A they bring 64 consecutive bytes of a
// row when A lies in rows, so that a quarter of a wave touches 16 cache lines, each for a quarter of its bytes,
// and every line is asked for again by the next step.  A in blocks of 16 rows x 32 k in operand order
// (bh_blocked_index in layout.h; the kernels that produce activations write it that way for this reader) makes
// an operand 1 KB of contiguous memory like W's: gate/up at 2,048 rows 333 -> 293 us (1.41 PFLOP/s), qkv 100 -> 85,
// down with 128-wide tiles 247 -> 181, with 256-wide tiles at 4,096 rows 348 -> 284 (1.45).  The vendor library's
// product (torch.matmul, bfloat16) takes 287 us for the gate/up shape without the gate (1.44 PFLOP/s), 81 us for qkv,
// and reaches 1.51 to 1.55 at its best shapes (4,096 and 8,192 rows): that, not 2.5, is what these matrix cores
// give with operands from memory.
// LDS holds four steps (4 x (16 + 2 YB) KB); a step's region is loaded again as soon as both groups have read
// it, which is five to six turns before it is read next.
//
// Measured at the Qwen3-8B shapes, 2,048 rows, activations in rows, each product alone: gate/up with SwiGLU 404 -> 330 us
// (1.25 PFLOP/s), qkv 132 -> 104 us with tiles of 192 weight rows (256 of them, one per compute unit), o 102 ->
// 84 us with 128; in the whole model 381 -> 338, 115 -> 101 and 87 -> 94 us (which is why the o and down
// projections there go through K in parts of the widest tile instead, see turns_plan: 77 us for o, finishing
// kernel included).
// What bounds it (activations in rows): the loads alone (no multiplies) take 0.9 of the whole kernel's time, the
// multiplies alone 0.6, the multiplies with their operand reads from LDS 0.8 (1.46 to 1.58 PFLOP/s).  It is not the loads' latency (five or six steps in LDS instead of four changed nothing; touching the
// lines three slices ahead with 4-byte loads made it slower, 0.9 PFLOP/s for gate/up: loads retire in order, so
// the loads for LDS waited behind the touches), not LDS (a compute unit reads 256 bytes per clock from it and
// needs a third of that) and not memory beyond L2 (87 % of the L2 requests hit; 0.3 to 0.6 GB come from beyond
// it).  The 32 compute units of an XCD ask its L2 for 1 MB per step, which at the matrix cores' full speed
// would be all that its 16 channels of 64 bytes per clock can give; a compute unit alone gets at most about
// 43 bytes per clock out of L1 and L2 (loads only, to LDS or to registers alike), and a tile of 256 x 128 asks
// for 47 where 256 x 256 asks for 32, which is why the narrower tiles lose.
// Tried for the products with 4,096 weight rows, which have only 128 tiles of 256 x 256: a tile of 256 x 128
// in which the two groups divide the k steps between them (every wave 64 x 128, sums exchanged through LDS at
// the end) ran like the 128-wide tile (0.8 PFLOP/s); A brought in whole 128-byte lines and kept permuted in
// LDS was slower (its slice buffer is free only four turns before it is read again).
#include "gemm_bf16_turns.h"
#include <type_traits>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

namespace {

__device__ inline bf16x8_t as_bf16x8(u32x4_t v) { return __builtin_bit_cast(bf16x8_t, v); }
__device__ inline float silu_mul(float gate, float up) { return gate / (1.0f + expf(-gate)) * up; }

// s_waitcnt immediates of gfx9: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8.  Both wait for all
// LDS reads; the first also until at most `vm` of the wave's global loads are still on their way.
#define WAIT_VM_LGKM0(vm) __builtin_amdgcn_s_waitcnt(((vm) & 15) | (((vm) >> 4) << 14) | (7 << 4) | (0 << 8))
#define WAIT_LGKM0() __builtin_amdgcn_s_waitcnt(15 | (3 << 14) | (7 << 4) | (0 << 8))
// The end of a turn.  Nothing may be moved across it by the compiler.
#define TICK()                            \
  do {                                    \
    __builtin_amdgcn_sched_barrier(0);    \
    __builtin_amdgcn_s_barrier();         \
    __builtin_amdgcn_sched_barrier(0);    \
  } while (0)

// Which tile a workgroup takes.  Workgroups go to the eight XCDs in turn (workgroup i to XCD i % 8), and each
// XCD has an L2 of its own: neighbours in the order below are workgroups of one XCD, and the 32 of them that
// run at one time (one per compute unit, walking over k in step) should ask that L2 for as few different bytes
// as possible.  So the order goes through the tiles in blocks of 8 row tiles x 4 weight tiles (row tiles
// first): a slice of rows is then fetched once for four compute units and a slice of weights once for eight,
// 12 slices for 32 tiles, where a whole column of row tiles under one weight tile would fetch 33 (measured
// with the chip full: L2 delivers 26 TB/s to the compute units, what lies beyond it 7; at 149,070 rows x
// 51,200 weight rows the column order read 305 GB per product and ran at 1.14 PFLOP/s).  Up to eight row tiles
// (2,048 rows) both orders are the same; at 8,192 rows x 4,096 the gate and up product went from 1,245 to
// 1,165 us (1.42 PFLOP/s) and the down projection from 600 to 563 us (1.46).  Only speed depends on where
// the workgroups really run.
__device__ inline void tile_of_workgroup(int n_tiles, int m_tiles, int* tile_n, int* tile_m) {
  constexpr int BM = 8, BN = 4;
  const int total = n_tiles * m_tiles, xcd = blockIdx.x % 8, each = total / 8, more = total % 8;
  int v = xcd * each + min(xcd, more) + blockIdx.x / 8;
  const int whole_columns = n_tiles / BN;                   // groups of BN weight tiles
  int first_n = 0, columns = BN;
  if (v >= whole_columns * BN * m_tiles) {                  // the weight tiles that fill no group
    v -= whole_columns * BN * m_tiles;
    first_n = whole_columns * BN;
    columns = n_tiles - first_n;
  } else {
    first_n = (v / (BN * m_tiles)) * BN;
    v %= BN * m_tiles;
  }
  const int chunk = v / (BM * columns), within = v % (BM * columns);   // chunks of BM row tiles; the last may be shorter
  const int rows = min(BM, m_tiles - chunk * BM);
  *tile_m = chunk * BM + within % rows;
  *tile_n = first_n + within / rows;
}

// MODE 0: bfloat16 output.  1: float32 output, optionally added to what is there.  2: SwiGLU, bfloat16 output
// (N outputs; W has 2 N rows, gate rows then up rows; a wave's weight rows are the gate and the up rows of
// the same outputs).  YB: blocks of 16 weight rows per wave.
// A tile that would stick out of the matrix is moved back inside and stores only what it owns.
// a_blocked: A lies in blocks of 16 rows x 32 k in operand order (bh_blocked_index), so that a wave's load of an
// operand is 1 KB of contiguous memory; its buffer holds whole tiles of 256 rows, and a tile that sticks out
// below stays where it is and stores only the rows that exist.  c_blocked (MODE 2): the output likewise.
template <int MODE, int YB>
__global__ __launch_bounds__(512) void gemm_turns_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ w,
                                                      void* __restrict__ c, int M, int N, int K, int accumulate,
                                                      int a_blocked, int c_blocked) {
  constexpr int OUTS = MODE == 2 ? 16 * YB : 32 * YB;
  constexpr int CHUNKS = 16 + 2 * YB;
  constexpr int WL = YB / 2;   // W chunks per loading wave
  constexpr int R = 4;                 // steps that LDS holds (with five or six of them it ran no faster)
  __shared__ __attribute__((aligned(16))) u32x4_t lds[R * CHUNKS * 64];   // [region][16 A blocks, then 2 YB W blocks][lane]
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int g = wave / 4, i4 = wave % 4;
  int tile_n, tile_m;
  tile_of_workgroup((N + OUTS - 1) / OUTS, (M + 255) / 256, &tile_n, &tile_m);
  const int m_own = tile_m * 256, n_own = tile_n * OUTS;
  const int m0 = a_blocked ? m_own : min(m_own, M - 256), n0 = min(n_own, N - OUTS);
  // K in parts (blockIdx.y, MODE 1 only): part p multiplies its share of k and leaves the bare sums at
  // c + p * M * N for the finishing kernel of gemm_bf16.hip; one part is the whole product.
  const int k_part = K / gridDim.y, k_first = blockIdx.y * k_part;
  const int J = k_part / 32;   // steps: half slices; k_part % 128 == 0

  // The first group brings A (four blocks of 16 rows per wave), the second W (YB / 2 blocks per wave).
  // A step takes 32 consecutive k: lane (row r = lane % 16, group q = lane / 16) holds k 8 q .. 8 q + 7 of them,
  // so four lanes bring 64 consecutive bytes of a row.  In W's tiles layout those are the 16-byte pieces
  // 4 v + q of the row (v: first or second step of the slice), piece p at half p % 2, lane 16 (p / 2) + r.
  const uint16_t* a_src = a_blocked ? a + ((size_t)((m0 + 64 * i4) / 16) * (K / 32) + k_first / 32) * 512 + lane * 8
                                    : a + (size_t)(m0 + 64 * i4 + lane % 16) * K + k_first + 8 * (lane / 16);
  const size_t a_block = a_blocked ? (size_t)(K / 32) * 512 : (size_t)16 * K;   // from 16 rows to the next
  const int w_lane = ((lane / 16) % 2) * 512 + (16 * (lane / 32) + lane % 16) * 8;   // + 256 elements for the second step
  const uint16_t* w_src[WL];
#pragma unroll
  for (int b = 0; b < WL; ++b) {
    const int rb = i4 * WL + b, gg = rb / YB, y = rb % YB;
    const int nb = MODE == 2 ? (y < YB / 2 ? 0 : N / 16) + n0 / 16 + (YB / 2) * gg + y % (YB / 2) : n0 / 16 + rb;
    w_src[b] = w + ((size_t)nb * (K / 64) + k_first / 64) * 1024 + w_lane;
  }
  auto fetch_a = [&](int j, int region) {   // step j = half u of slice s
    const int s = j >> 1, u = j & 1;
#pragma unroll
    for (int b = 0; b < 4; ++b)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a_src + b * a_block + (a_blocked ? j * 512 : s * 64 + u * 32)),
                                       (__attribute__((address_space(3))) void*)&lds[(region * CHUNKS + 4 * i4 + b) * 64], 16, 0, 0);
  };
  auto fetch_w = [&](int j, int region) {
    const int s = j >> 1, u = j & 1;
#pragma unroll
    for (int b = 0; b < WL; ++b)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(w_src[b] + (size_t)s * 1024 + u * 256),
                                       (__attribute__((address_space(3))) void*)&lds[(region * CHUNKS + 16 + i4 * WL + b) * 64], 16, 0, 0);
  };

  f32x4_t acc[4][YB];
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int y = 0; y < YB; ++y) acc[x][y] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  u32x4_t af[4], wf[YB];

  auto read_operands = [&](int region) {
#pragma unroll
    for (int x = 0; x < 4; ++x) af[x] = lds[(region * CHUNKS + 4 * i4 + x) * 64 + lane];
#pragma unroll
    for (int y = 0; y < YB; ++y) wf[y] = lds[(region * CHUNKS + 16 + YB * g + y) * 64 + lane];
  };
  auto multiply = [&]() {
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int x = 0; x < 4; ++x)
#pragma unroll
      for (int y = 0; y < YB; ++y)
        acc[x][y] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wf[y]), as_bf16x8(af[x]), acc[x][y], 0, 0, 0);
    __builtin_amdgcn_s_setprio(0);
  };

  // Step j lies in region j % R.  A wave asks for step j + R - 1 while it reads step j (into the region that
  // step j - 1 has left); before the turn in which the first group reads step j + 1, all that was asked for
  // it must have landed: what may still be on its way are the loads of the steps after it.
  auto wait_for_next = [&](int j, auto per_step) {   // per_step: this wave's loads per step
    constexpr int each = decltype(per_step)::value;
    const int later = min(R - 2, J - 2 - j);   // steps after j + 1 that have been asked for
    if (later >= 2) WAIT_VM_LGKM0(2 * each);
    else if (later == 1) WAIT_VM_LGKM0(each);
    else WAIT_VM_LGKM0(0);
  };
  static_assert(R == 4, "wait_for_next knows of two steps on their way after the next");
  if (g == 0) {
    for (int j = 0; j < R - 1 && j < J; ++j) fetch_a(j, j);
    WAIT_VM_LGKM0(0);
    TICK();
    int region = 0;
    for (int j = 0; j < J; ++j) {
      if (j + R - 1 < J) fetch_a(j + R - 1, region == 0 ? R - 1 : region - 1);
      read_operands(region);
      WAIT_LGKM0();
      TICK();
      multiply();
      wait_for_next(j, std::integral_constant<int, 4>());
      TICK();
      region = region == R - 1 ? 0 : region + 1;
    }
    TICK();
  } else {
    for (int j = 0; j < R - 1 && j < J; ++j) fetch_w(j, j);
    WAIT_VM_LGKM0(0);
    TICK();
    TICK();   // the second group runs one tick behind
    int region = 0;
    for (int j = 0; j < J; ++j) {
      if (j + R - 1 < J) fetch_w(j + R - 1, region == 0 ? R - 1 : region - 1);
      read_operands(region);
      wait_for_next(j, std::integral_constant<int, WL>());
      TICK();
      multiply();
      TICK();
      region = region == R - 1 ? 0 : region + 1;
    }
  }
  // acc[x][y][i]: row 64 i4 + 16 x + lane % 16 of the tile, weight row 16 (YB g + y) + 4 (lane / 16) + i
  const int m = m0 + 64 * i4 + lane % 16;
  if (MODE == 2) {
    uint16_t* out = reinterpret_cast<uint16_t*>(c);
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int row = m + 16 * x;
      if (row < m_own || row >= M) continue;
#pragma unroll
      for (int y = 0; y < YB / 2; ++y) {
        const int n = n0 + 8 * YB * g + 16 * y + 4 * (lane / 16);
        if (n < n_own) continue;
        u32x2_t packed;
        packed[0] = f32_to_bf16_bits(silu_mul(acc[x][y][0], acc[x][y + YB / 2][0])) | ((uint32_t)f32_to_bf16_bits(silu_mul(acc[x][y][1], acc[x][y + YB / 2][1])) << 16);
        packed[1] = f32_to_bf16_bits(silu_mul(acc[x][y][2], acc[x][y + YB / 2][2])) | ((uint32_t)f32_to_bf16_bits(silu_mul(acc[x][y][3], acc[x][y + YB / 2][3])) << 16);
        *reinterpret_cast<u32x2_t*>(out + (c_blocked ? (size_t)bh_blocked_index(row, n, N) : (size_t)row * N + n)) = packed;
      }
    }
  } else {
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int row = m + 16 * x;
      if (row < m_own || row >= M) continue;
#pragma unroll
      for (int y = 0; y < YB; ++y) {
        const int n = n0 + 16 * YB * g + 16 * y + 4 * (lane / 16);
        if (n < n_own) continue;
        if (MODE == 1) {
          f32x4_t* at = reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(c) + ((size_t)blockIdx.y * M + row) * N + n);
          f32x4_t v = acc[x][y];
          if (accumulate) v += *at;
          *at = v;
        } else {
          u32x2_t packed;
          packed[0] = f32_to_bf16_bits(acc[x][y][0]) | ((uint32_t)f32_to_bf16_bits(acc[x][y][1]) << 16);
          packed[1] = f32_to_bf16_bits(acc[x][y][2]) | ((uint32_t)f32_to_bf16_bits(acc[x][y][3]) << 16);
          *reinterpret_cast<u32x2_t*>(reinterpret_cast<uint16_t*>(c) + (size_t)row * N + n) = packed;
        }
      }
    }
  }
}


#undef WAIT_VM_LGKM0
#undef WAIT_LGKM0
#undef TICK

template <int MODE>
void launch(const void* a, const void* w, void* c, int blocks, int M, int N, int K, int accumulate, int a_blocked,
            int c_blocked, hipStream_t stream, int parts = 1) {
  const int outs = (MODE == 2 ? 16 : 32) * blocks;
  dim3 grid(((N + outs - 1) / outs) * ((M + 255) / 256), parts);
#define BH_TURNS(YB) \
  gemm_turns_kernel<MODE, YB><<<grid, 512, 0, stream>>>((const uint16_t*)a, (const uint16_t*)w, c, M, N, K, accumulate, a_blocked, c_blocked)
  if (blocks == 8) BH_TURNS(8);
  else if (blocks == 6) BH_TURNS(6);
  else BH_TURNS(4);
#undef BH_TURNS
}

}  // namespace

bool gemm_turns_can(int M, int N, int K, int layout, int activation, int blocks) {
  if (blocks != 8 && blocks != 6 && blocks != 4) return false;
  const int outs = (activation ? 16 : 32) * blocks;
  return layout == 1 && M >= 256 && N >= outs && N % 16 == 0 && K >= 128 && K % 128 == 0 &&
         (long)((N + outs - 1) / outs) * ((M + 255) / 256) < (1L << 31);   // offsets into A, W and C are 64-bit
}

// Which way, if any.  A tile of YB blocks per wave costs a compute unit YB x cost(YB) units of time, where cost
// is what the narrower tiles lose (measured 1.43, 1.16 and 1.07 PFLOP/s for 8, 6 and 4 with the chip full and the
// activations in blocks; 1.25, 1.11 and 0.90 with activations in rows), and
// the chip works in rounds of 256 tiles; a tile of its own is taken if that estimate reaches 0.6 PFLOP/s, which
// the other tiled kernels stay below at these sizes (with 0.8 as the bar, prefill steps of 320 to 768 tokens were 2 to
// 18 % slower at the Qwen3-8B, 14B and 32B widths, and no length was faster).  Products with so few of the widest tiles that much of the
// chip would idle can instead cut K into parts over as many times the workgroups, each leaving its bare sums in
// scratch memory ([part][row][weight row], float32) for a finishing kernel of gemm_bf16.hip; that costs about
// 0.85 of the tile's rate (for the o projection of the Qwen3-8B shape at 2,048 rows the parts and the 128-wide
// tile run alike alone, but the whole prefill went 31.8 -> 30.5 ms with the parts).
namespace {
struct TurnsPlan {
  int blocks;   // tile width for the product in one launch, or 0
  int parts;    // parts of K, or 1
  int part_blocks = 8;   // the tile width of the parts
};
TurnsPlan turns_plan(int M, int N, int K, int layout, int activation) {
  TurnsPlan plan = {0, 1};
  if (M <= 256) return plan;   // up to there a norm may ride on the product, which this kernel does not carry
  double best_rate = 600.0;    // TFLOP/s: what a tile of its own has to reach
  double direct_rate = 0.0;
  const double work = (double)M * (activation ? 2.0 * N : (double)N);   // rows x weight rows
  const int units = bh_compute_units();   // a round is one tile per compute unit (the rates below were measured with 256)
  for (int blocks = 8; blocks >= 4; blocks -= 2) {
    if (!gemm_turns_can(M, N, K, layout, activation, blocks)) continue;
    const int outs = (activation ? 16 : 32) * blocks;
    const long tiles = (long)((N + outs - 1) / outs) * ((M + 255) / 256);
    const long rounds = (tiles + units - 1) / units;
    const double cost = blocks == 8 ? 1.0 : blocks == 6 ? 1.23 : 1.34;
    const double rate = 1430.0 * (units / 256.0) * work / ((double)rounds * units * 256 * (activation ? 2 : 1) * outs * cost);
    if (rate >= best_rate) best_rate = direct_rate = rate, plan.blocks = blocks;
  }
  if (!activation && M >= 320 && gemm_turns_can(M, N, K, layout, 0, 8)) {
    // As many parts (8, 4 or 2) as keep the workgroups within one round and every part at least 512 long; worth
    // it from about five eighths of the chip on.  Measured at the Qwen3-8B widths against the other kernels, us:
    // 512 rows: down in 8 parts 88 -> 72 (o in 4 parts, half the chip, 41 -> 45; in 8 parts of 512 the prefill step of
    // 512 tokens is 0.5 % faster than with the older tiles); 768 rows: o 71 -> 53,
    // down 195 -> 102 in 4; 1,024 rows: o 72 -> 57, down 196 -> 111 in 4; 1,536 rows: o 93 -> 77, down 219 -> 173 in 2;
    // 2,048 rows: down 240 -> 199 in 2.  From 320 rows on (a whole prefill step of the Qwen3-8B shape with the parts from 257
    // rows on instead of from 512 on: 272 tokens 9.15 -> 9.24 ms, 320 tokens 9.34 -> 9.25, 384 tokens 9.62 -> 9.48, 448 tokens
    // 10.88 -> 9.77).
    // With the widest tile first; where that needs eight parts (257 to 512 rows at these widths), four parts of the
    // 128-wide tile instead: half the bare sums to write and to read again (512 rows at the Qwen3-8B widths, product +
    // finishing kernel, o and down on average: 42.5 + 19.9 -> 40.9 + 14.1 us; where the widest tile needs four parts or
    // two, the narrower one lost: 640 rows 51.8 + 16.0 -> 64.0 + 13.1, 1,024 rows 60.8 + 21.7 -> 73.8 + 17.4; the
    // 192-wide tile lost everywhere).
    auto parts_of = [&](int pb) {
      const int outs = 32 * pb;
      const long tiles = (long)((N + outs - 1) / outs) * ((M + 255) / 256);
      int parts = 8;
      while (parts > 1 && (tiles * parts > units || K / parts < 512 || K % (128 * parts) != 0)) parts /= 2;
      return parts > 1 && tiles * parts >= units * 5 / 8 ? parts : 1;
    };
    int pb = 8, parts = parts_of(8);
    if (parts == 8 && gemm_turns_can(M, N, K, layout, 0, 4) && parts_of(4) == 4) pb = 4, parts = 4;
    // Where the widest tile finds no cut that fills five eighths of the chip within one round (the q/k/v projection of the
    // Qwen3-8B shape at 513 to 768 rows: 72 tiles, 144 workgroups in two parts, 288 in four) and no tile of its own is worth it
    // either, the 192-wide tile may (96 tiles, 192 workgroups in two parts), then the 128-wide one.
    if (parts == 1 && plan.blocks == 0)
      for (int narrower = 6; narrower >= 4 && parts == 1; narrower -= 2)
        if (gemm_turns_can(M, N, K, layout, 0, narrower) && parts_of(narrower) > 1) pb = narrower, parts = parts_of(narrower);
    if (parts > 1) {
      const double rate = 0.85 * 1430.0 * (units / 256.0) * work / ((double)units * 256 * 32 * pb / parts * (pb == 8 ? 1.0 : pb == 6 ? 1.23 : 1.34));
      if (rate > direct_rate) plan.blocks = 0, plan.parts = parts, plan.part_blocks = pb;
    }
  }
  return plan;
}
}  // namespace

int gemm_turns_blocks(int M, int N, int K, int layout, int activation) {
  return turns_plan(M, N, K, layout, activation).blocks;
}
int gemm_turns_parts(int M, int N, int K, int layout, int activation) {
  return turns_plan(M, N, K, layout, activation).parts;
}

int gemm_turns_launch_parts(const void* a, const void* w, float* sums, int M, int N, int K, int parts, int a_blocked,
                            hipStream_t stream) {
  const int pb = turns_plan(M, N, K, 1, 0).part_blocks;
  BH_REQUIRE(parts >= 1 && K % (128 * parts) == 0 && gemm_turns_can(M, N, K / parts, 1, 0, pb),
             "gemm_turns: M=%d N=%d K=%d cannot be multiplied in %d parts of K", M, N, K, parts);
  BH_REQUIRE(((uintptr_t)a | (uintptr_t)w | (uintptr_t)sums) % 16 == 0, "gemm_turns: operands must be 16-byte aligned");
  launch<1>(a, w, sums, pb, M, N, K, 0, a_blocked, 0, stream, parts);
  return bh_check_launch("gemm_turns");
}

int gemm_turns_launch(const void* a, const void* w, void* c, int c_dtype, int accumulate, int M, int N, int K,
                      int activation, int blocks, int a_blocked, int c_blocked, hipStream_t stream) {
  BH_REQUIRE(gemm_turns_can(M, N, K, 1, activation, blocks),
             "gemm_turns: a product of M=%d N=%d K=%d with %d blocks per wave is not one this kernel takes "
             "(M >= 256, K a multiple of 128, N a multiple of 16 and at least a tile)", M, N, K, blocks);
  BH_REQUIRE(c_dtype == BH_F32 || (c_dtype == BH_BF16 && !accumulate),
             "gemm_turns: output float32, or bfloat16 without accumulation");
  BH_REQUIRE(!activation || c_dtype == BH_BF16, "gemm_turns: SwiGLU writes bfloat16");
  BH_REQUIRE(((uintptr_t)a | (uintptr_t)w | (uintptr_t)c) % 16 == 0 && (c_dtype == BH_F32 || N % 4 == 0),
             "gemm_turns: operands and output must be 16-byte aligned");
  BH_REQUIRE(!c_blocked || (activation && N % 32 == 0), "gemm_turns: only SwiGLU writes its output in blocks, and N=%d must be a multiple of 32", N);
  if (activation) launch<2>(a, w, c, blocks, M, N, K, 0, a_blocked, c_blocked, stream);
  else if (c_dtype == BH_F32) launch<1>(a, w, c, blocks, M, N, K, accumulate, a_blocked, 0, stream);
  else launch<0>(a, w, c, blocks, M, N, K, 0, a_blocked, 0, stream);
  return bh_check_launch("gemm_turns");
}

// For tests and measurements: the kernel at a given tile width, whatever gemm_turns_blocks would choose.
extern "C" int bh_gemm_bf16_turns(const void* a, const void* w, void* c, int c_dtype, int accumulate, int M, int N,
                                  int K, int activation, int blocks, int a_blocked, int c_blocked, hipStream_t stream) {
  return gemm_turns_launch(a, w, c, c_dtype, accumulate, M, N, K, activation, blocks, a_blocked, c_blocked, stream);
}
extern "C" int bh_gemm_bf16_turns_blocks(int M, int N, int K, int layout, int activation) {
  return gemm_turns_blocks(M, N, K, layout, activation);
}
