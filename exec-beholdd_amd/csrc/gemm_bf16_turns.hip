// bfloat16 matrix products of many rows, C[M, N] (+)= A[M, K] * W[N, K]^T with W in the tiles layout
// (see gemm_bf16.hip), for the shapes where a 256-row tile fills the chip: prompts from about 512 tokens on.
//
// A workgroup of eight waves owns 256 rows x 32 YB weight rows.  Its waves form two groups of four (one wave
// of each group per SIMD) that take turns: while one group multiplies (32, 24 or 16 MFMAs on operands it holds
// in registers), the other reads its next operands from LDS and asks for data that is three steps ahead; a
// barrier ends every turn.  So the matrix cores always have one wave per SIMD that does nothing but multiply,
// and no wave waits for memory in the middle of its multiplies.  A step is half a 64-wide k slice: the 32 k
// values that one 16x16x32 MFMA takes, in the order in which the tiles layout holds them.
//
// Global memory goes to LDS directly (16-byte loads that write LDS at the wave's base + 16 * lane): 1 KB per
// load, which is one operand of 16 rows x 32 k in lane order, so that reading it back is one conflict-free
// 16-byte read per lane.  W's tiles layout already is that order (contiguous 1 KB loads); for A a lane loads
// its 16 bytes from its row.  LDS holds four steps (4 x (16 + 2 YB) KB); a step's region is loaded again as
// soon as both groups have read it, which is five to six turns before it is read next: time enough for
// loads that miss every cache.
//
// Measured at the Qwen3-8B shapes, 2,048 rows: gate/up with SwiGLU 404 -> 330 us (1.25 PFLOP/s), qkv
// 132 -> 104 us with tiles of 192 weight rows (256 of them, one per compute unit), o 102 -> 83 us with 128.
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

// MODE 0: bfloat16 output.  1: float32 output, optionally added to what is there.  2: SwiGLU, bfloat16 output
// (N outputs; W has 2 N rows, gate rows then up rows; a wave's weight rows are the gate and the up rows of
// the same outputs).  YB: blocks of 16 weight rows per wave.
// A tile that would stick out of the matrix is moved back inside and stores only what it owns.
template <int MODE, int YB>
__global__ __launch_bounds__(512) void gemm_turns_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ w,
                                                      void* __restrict__ c, int M, int N, int K, int accumulate) {
  constexpr int OUTS = MODE == 2 ? 16 * YB : 32 * YB;
  constexpr int CHUNKS = 16 + 2 * YB;
  constexpr int WL = YB / 2;   // W chunks per loading wave
  __shared__ __attribute__((aligned(16))) u32x4_t lds[4][CHUNKS][64];   // [region][16 A blocks, then 2 YB W blocks][lane]
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int g = wave / 4, i4 = wave % 4;
  const int n_tiles = (N + OUTS - 1) / OUTS;
  const int tile_n = blockIdx.x % n_tiles, tile_m = blockIdx.x / n_tiles;
  const int m_own = tile_m * 256, n_own = tile_n * OUTS;
  const int m0 = min(m_own, M - 256), n0 = min(n_own, N - OUTS);
  const int J = K / 32;   // half slices; K % 128 == 0

  // The first group brings A (four blocks of 16 rows per wave), the second W (YB / 2 blocks per wave).
  const uint16_t* a_src = a + (size_t)(m0 + 64 * i4 + lane % 16) * K + 16 * (lane / 16);
  const uint16_t* w_src[WL];
#pragma unroll
  for (int b = 0; b < WL; ++b) {
    const int rb = i4 * WL + b, gg = rb / YB, y = rb % YB;
    const int nb = MODE == 2 ? (y < YB / 2 ? 0 : N / 16) + n0 / 16 + (YB / 2) * gg + y % (YB / 2) : n0 / 16 + rb;
    w_src[b] = w + (size_t)nb * (K / 64) * 1024 + lane * 8;
  }
  auto fetch_a = [&](int j, int region) {
    const int s = j >> 1, u = j & 1;
#pragma unroll
    for (int b = 0; b < 4; ++b)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a_src + (size_t)b * 16 * K + s * 64 + u * 8),
                                       (__attribute__((address_space(3))) void*)&lds[region][4 * i4 + b][0], 16, 0, 0);
  };
  auto fetch_w = [&](int j, int region) {
    const int s = j >> 1, u = j & 1;
#pragma unroll
    for (int b = 0; b < WL; ++b)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(w_src[b] + (size_t)s * 1024 + u * 512),
                                       (__attribute__((address_space(3))) void*)&lds[region][16 + i4 * WL + b][0], 16, 0, 0);
  };

  f32x4_t acc[4][YB];
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int y = 0; y < YB; ++y) acc[x][y] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  u32x4_t af[4], wf[YB];

  auto read_operands = [&](int region) {
#pragma unroll
    for (int x = 0; x < 4; ++x) af[x] = lds[region][4 * i4 + x][lane];
#pragma unroll
    for (int y = 0; y < YB; ++y) wf[y] = lds[region][16 + YB * g + y][lane];
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

  if (g == 0) {
    fetch_a(0, 0); fetch_a(1, 1); fetch_a(2, 2);
    WAIT_VM_LGKM0(0);
    TICK();
    auto step = [&](auto fetch, auto pending, int j, int region) {
      if (fetch.value) fetch_a(j + 3, (region + 3) % 4);
      read_operands(region);
      WAIT_LGKM0();
      TICK();
      multiply();
      // half slice j + 1 must have landed before the next tick, in which this group reads it
      WAIT_VM_LGKM0(4 * pending.value);
      TICK();
    };
    using std::integral_constant;
    typedef integral_constant<bool, true> yes;
    typedef integral_constant<bool, false> no;
    int j = 0;
    for (; j + 4 < J; j += 4) {
      step(yes(), integral_constant<int, 2>(), j, 0); step(yes(), integral_constant<int, 2>(), j + 1, 1);
      step(yes(), integral_constant<int, 2>(), j + 2, 2); step(yes(), integral_constant<int, 2>(), j + 3, 3);
    }
    step(yes(), integral_constant<int, 2>(), j, 0); step(no(), integral_constant<int, 1>(), j + 1, 1);
    step(no(), integral_constant<int, 0>(), j + 2, 2); step(no(), integral_constant<int, 0>(), j + 3, 3);
    TICK();
  } else {
    fetch_w(0, 0); fetch_w(1, 1); fetch_w(2, 2);
    WAIT_VM_LGKM0(0);
    TICK();
    TICK();   // the second group runs one tick behind
    auto step = [&](auto fetch, auto pending, int j, int region) {
      if (fetch.value) fetch_w(j + 3, (region + 3) % 4);
      read_operands(region);
      WAIT_VM_LGKM0(WL * pending.value);
      TICK();
      multiply();
      TICK();
    };
    using std::integral_constant;
    typedef integral_constant<bool, true> yes;
    typedef integral_constant<bool, false> no;
    int j = 0;
    for (; j + 4 < J; j += 4) {
      step(yes(), integral_constant<int, 2>(), j, 0); step(yes(), integral_constant<int, 2>(), j + 1, 1);
      step(yes(), integral_constant<int, 2>(), j + 2, 2); step(yes(), integral_constant<int, 2>(), j + 3, 3);
    }
    step(yes(), integral_constant<int, 2>(), j, 0); step(no(), integral_constant<int, 1>(), j + 1, 1);
    step(no(), integral_constant<int, 0>(), j + 2, 2); step(no(), integral_constant<int, 0>(), j + 3, 3);
  }

  // acc[x][y][i]: row 64 i4 + 16 x + lane % 16 of the tile, weight row 16 (YB g + y) + 4 (lane / 16) + i
  const int m = m0 + 64 * i4 + lane % 16;
  if (MODE == 2) {
    uint16_t* out = reinterpret_cast<uint16_t*>(c);
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int row = m + 16 * x;
      if (row < m_own) continue;
#pragma unroll
      for (int y = 0; y < YB / 2; ++y) {
        const int n = n0 + 8 * YB * g + 16 * y + 4 * (lane / 16);
        if (n < n_own) continue;
        u32x2_t packed;
        packed[0] = f32_to_bf16_bits(silu_mul(acc[x][y][0], acc[x][y + YB / 2][0])) | ((uint32_t)f32_to_bf16_bits(silu_mul(acc[x][y][1], acc[x][y + YB / 2][1])) << 16);
        packed[1] = f32_to_bf16_bits(silu_mul(acc[x][y][2], acc[x][y + YB / 2][2])) | ((uint32_t)f32_to_bf16_bits(silu_mul(acc[x][y][3], acc[x][y + YB / 2][3])) << 16);
        *reinterpret_cast<u32x2_t*>(out + (size_t)row * N + n) = packed;
      }
    }
  } else {
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int row = m + 16 * x;
      if (row < m_own) continue;
#pragma unroll
      for (int y = 0; y < YB; ++y) {
        const int n = n0 + 16 * YB * g + 16 * y + 4 * (lane / 16);
        if (n < n_own) continue;
        if (MODE == 1) {
          f32x4_t* at = reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(c) + (size_t)row * N + n);
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
void launch(const void* a, const void* w, void* c, int blocks, int M, int N, int K, int accumulate, hipStream_t stream) {
  const int outs = (MODE == 2 ? 16 : 32) * blocks;
  dim3 grid(((N + outs - 1) / outs) * ((M + 255) / 256));
#define BH_TURNS(YB) \
  gemm_turns_kernel<MODE, YB><<<grid, 512, 0, stream>>>((const uint16_t*)a, (const uint16_t*)w, c, M, N, K, accumulate)
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
         (long)M * K < (1L << 31) && (long)((N + outs - 1) / outs) * ((M + 255) / 256) < (1L << 31);
}

// Which tile, if any.  A tile of YB blocks per wave costs a compute unit YB x cost(YB) units of time, where
// cost is what the narrower tiles lose (more LDS reads and loads per multiply: measured 1.25, 1.11 and 0.90
// PFLOP/s for 8, 6 and 4 with the chip full), and the chip works in rounds of 256 tiles.  The estimate is
// compared with what the other tiled kernels reach (about 0.85 PFLOP/s at their best, less for short K,
// where their start and end of a tile weigh more).
int gemm_turns_blocks(int M, int N, int K, int layout, int activation) {
  if (M <= 256) return 0;   // up to there a norm may ride on the product, which this kernel does not carry
  int best = 0;
  double best_rate = 0.0;
  const double work = (double)M * (activation ? 2.0 * N : (double)N);   // rows x weight rows
  for (int blocks = 8; blocks >= 4; blocks -= 2) {
    if (!gemm_turns_can(M, N, K, layout, activation, blocks)) continue;
    const int outs = (activation ? 16 : 32) * blocks;
    const long tiles = (long)((N + outs - 1) / outs) * ((M + 255) / 256);
    const long rounds = (tiles + 255) / 256;
    const double cost = blocks == 8 ? 1.0 : blocks == 6 ? 1.12 : 1.39;
    const double rate = 1250.0 * work / ((double)rounds * 256 * 256 * 32 * blocks * cost);   // TFLOP/s, roughly
    if (rate > best_rate) best_rate = rate, best = blocks;
  }
  const double others = K <= 8192 ? 800.0 : 950.0;
  return best_rate >= others ? best : 0;
}

int gemm_turns_launch(const void* a, const void* w, void* c, int c_dtype, int accumulate, int M, int N, int K,
                      int activation, int blocks, hipStream_t stream) {
  BH_REQUIRE(gemm_turns_can(M, N, K, 1, activation, blocks),
             "gemm_turns: a product of M=%d N=%d K=%d with %d blocks per wave is not one this kernel takes "
             "(M >= 256, K a multiple of 128, N a multiple of 16 and at least a tile)", M, N, K, blocks);
  BH_REQUIRE(c_dtype == BH_F32 || (c_dtype == BH_BF16 && !accumulate),
             "gemm_turns: output float32, or bfloat16 without accumulation");
  BH_REQUIRE(!activation || c_dtype == BH_BF16, "gemm_turns: SwiGLU writes bfloat16");
  BH_REQUIRE(((uintptr_t)a | (uintptr_t)w | (uintptr_t)c) % 16 == 0 && (c_dtype == BH_F32 || N % 4 == 0),
             "gemm_turns: operands and output must be 16-byte aligned");
  if (activation) launch<2>(a, w, c, blocks, M, N, K, 0, stream);
  else if (c_dtype == BH_F32) launch<1>(a, w, c, blocks, M, N, K, accumulate, stream);
  else launch<0>(a, w, c, blocks, M, N, K, 0, stream);
  return bh_check_launch("gemm_turns");
}

// For tests and measurements: the kernel at a given tile width, whatever gemm_turns_blocks would choose.
extern "C" int bh_gemm_bf16_turns(const void* a, const void* w, void* c, int c_dtype, int accumulate, int M, int N,
                                  int K, int activation, int blocks, hipStream_t stream) {
  return gemm_turns_launch(a, w, c, c_dtype, accumulate, M, N, K, activation, blocks, stream);
}
extern "C" int bh_gemm_bf16_turns_blocks(int M, int N, int K, int layout, int activation) {
  return gemm_turns_blocks(M, N, K, layout, activation);
}
