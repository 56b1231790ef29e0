// Plain host twins of the kernels: every hand-written kernel of this library beside a plain C++ function that
// takes the same arguments (but for the stream) and computes the same thing one element at a time, with the
// sums that the reference keeps in double kept in double.  The reference's rule: a GPU path with no plain
// counterpart is a GPU path nobody can debug (crates/beholdd-backend/src/cpu.rs:3-5).  Nothing on the product
// path calls these; tests compare the kernels with them, and a self-test built with the host sanitizers
// (-DBH_TWINS_SELFTEST) checks them against the reference's own test vectors and walks every index function
// over whole pages.  Compiles with the host compiler alone.
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <vector>

#include "layout.h"

namespace {

float load(const void* p, int dtype, size_t at) {
  return dtype == BH_F32 ? static_cast<const float*>(p)[at] : bf16_bits_to_f32(static_cast<const uint16_t*>(p)[at]);
}
void store(void* p, int dtype, size_t at, float v) {
  if (dtype == BH_F32) static_cast<float*>(p)[at] = v;
  else static_cast<uint16_t*>(p)[at] = f32_to_bf16_bits(v);
}
size_t width_of(int dtype) { return dtype == BH_F32 ? 4 : 2; }
bool known(int dtype) { return dtype == BH_F32 || dtype == BH_BF16; }

}  // namespace

extern "C" {

// hidden[row, :] = table[token[row], :] widened to float32 (generic.hip: bh_embed without fed tokens)
int bhp_embed(const int32_t* tokens, const void* table, int table_dtype, float* out, int n_rows, int width, int vocab) {
  if (!known(table_dtype) || n_rows <= 0 || width <= 0 || vocab <= 0) return 1;
  for (int r = 0; r < n_rows; ++r) {
    if (tokens[r] < 0 || tokens[r] >= vocab) return 2;
    for (int i = 0; i < width; ++i) out[(size_t)r * width + i] = load(table, table_dtype, (size_t)tokens[r] * width + i);
  }
  return 0;
}

// out[r] = (x[rows ? rows[r] : r] * inv) * weight, inv = 1 / sqrt(mean(x^2) + eps) (generic.hip: bh_rmsnorm;
// crates/beholdd-kernel/src/vecops.rs:54-64: the sum of squares and the inverse in double, the inverse rounded)
int bhp_rmsnorm(const float* x, const int32_t* rows, const void* weight, int w_dtype, void* out, int out_dtype,
                int n_rows, int width, float eps) {
  if (!known(out_dtype) || (weight && !known(w_dtype)) || n_rows <= 0 || width <= 0) return 1;
  for (int r = 0; r < n_rows; ++r) {
    const float* src = x + (size_t)(rows ? rows[r] : r) * width;
    double ss = 0.0;
    for (int i = 0; i < width; ++i) ss += (double)src[i] * (double)src[i];
    const float inv = (float)(1.0 / sqrt(ss / width + (double)eps));
    for (int i = 0; i < width; ++i) {
      float v = src[i] * inv;
      if (weight) v *= load(weight, w_dtype, i);
      store(out, out_dtype, (size_t)r * width + i, v);
    }
  }
  return 0;
}

// c[M, N] (+)= a[M, K] w[N, K]^T (generic.hip: bh_gemm_generic; gemm_bf16*.hip for bfloat16 operands)
int bhp_gemm(const void* a, int a_dtype, const void* w, int w_dtype, void* c, int c_dtype, int accumulate, int M,
             int N, int K) {
  if (!known(a_dtype) || !known(w_dtype) || !known(c_dtype) || M <= 0 || N <= 0 || K <= 0) return 1;
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      double sum = 0.0;
      for (int k = 0; k < K; ++k) sum += (double)load(a, a_dtype, (size_t)m * K + k) * (double)load(w, w_dtype, (size_t)n * K + k);
      const size_t at = (size_t)m * N + n;
      store(c, c_dtype, at, (float)(accumulate ? (double)load(c, c_dtype, at) + sum : sum));
    }
  return 0;
}

// out[r, i] = silu(gu[r, i]) * gu[r, F + i] (generic.hip: bh_swiglu; crates/beholdd-kernel/src/vecops.rs:91-110)
int bhp_swiglu(const void* gu, void* out, int dtype, int n_rows, int F) {
  if (!known(dtype) || n_rows <= 0 || F <= 0) return 1;
  for (int r = 0; r < n_rows; ++r)
    for (int i = 0; i < F; ++i) {
      const float g = load(gu, dtype, (size_t)r * 2 * F + i), u = load(gu, dtype, (size_t)r * 2 * F + F + i);
      store(out, dtype, (size_t)r * F + i, g / (1.0f + expf(-g)) * u);
    }
  return 0;
}

// Per head of the fused [q | k | v] projection rows: RMSNorm (weights may be null), split-half rotation over the
// first `rot` elements at the row's position (tables may be null), q to q_out, k and v into the cache page of
// (sequence, position) in the given order (generic.hip: bh_qk_norm_rope_cache;
// crates/beholdd-model/src/qwen3moe/forward.rs:1130-1196).  `pages`: how many pages the cache tensors hold.
int bhp_qk_norm_rope_cache(const void* qkv, int dtype, void* q_out, const void* q_weight, const void* k_weight, int w_dtype,
                           float eps, const float* cos_table, const float* sin_table, int table_positions, int rot,
                           const int32_t* positions, const int32_t* row_seq, void* k_pages, void* v_pages,
                           const int32_t* page_table, int table_stride, int n_rows, int H, int KVH, int hd,
                           int write_kv, int kv_order, int pages) {
  if (!known(dtype) || n_rows <= 0 || H <= 0 || KVH <= 0 || hd <= 0 || rot < 0 || rot > hd || rot % 2) return 1;
  if ((q_weight == nullptr) != (k_weight == nullptr) || (q_weight && !known(w_dtype))) return 1;
  if (kv_order == BH_KV_PIECES && hd % 32) return 1;
  if (!cos_table) rot = 0;
  const int fused = (H + 2 * KVH) * hd, half = rot / 2;
  std::vector<float> head(hd);
  for (int r = 0; r < n_rows; ++r) {
    const int pos = positions[r];
    if (pos < 0 || (rot && pos >= table_positions)) return 2;
    const int heads = write_kv ? H + 2 * KVH : H;
    for (int h = 0; h < heads; ++h) {
      const bool is_q = h < H, is_value = h >= H + KVH;
      for (int i = 0; i < hd; ++i) head[i] = load(qkv, dtype, (size_t)r * fused + (size_t)h * hd + i);
      if (!is_value) {
        const void* weight = is_q ? q_weight : k_weight;
        if (weight) {
          double ss = 0.0;
          for (int i = 0; i < hd; ++i) ss += (double)head[i] * (double)head[i];
          const float inv = (float)(1.0 / sqrt(ss / hd + (double)eps));
          for (int i = 0; i < hd; ++i) head[i] = head[i] * inv * load(weight, w_dtype, i);
        }
        for (int i = 0; i < half; ++i) {
          const float c = cos_table[(size_t)pos * half + i], s = sin_table[(size_t)pos * half + i];
          const float lo = head[i], hi = head[i + half];
          head[i] = lo * c - hi * s;
          head[i + half] = lo * s + hi * c;
        }
      }
      if (is_q) {
        for (int i = 0; i < hd; ++i) store(q_out, dtype, ((size_t)r * H + h) * hd + i, head[i]);
        continue;
      }
      if (pos / BH_PAGE >= table_stride) return 3;
      const int page = page_table[(size_t)row_seq[r] * table_stride + pos / BH_PAGE];
      if (page < 0 || page >= pages) return 4;
      const int kv_head = (h - H) % KVH, token = pos % BH_PAGE;
      const size_t base = ((size_t)page * KVH + kv_head) * BH_PAGE * hd;
      for (int i = 0; i < hd; ++i) {
        if (is_value) store(v_pages, dtype, base + bh_value_index(kv_order, token, i, hd), head[i]);
        else store(k_pages, dtype, base + bh_key_index(kv_order, token, i, hd), head[i]);
      }
    }
  }
  return 0;
}

// out[row, head] = softmax(q . K * scale) V over the keys max(0, p - window + 1) .. p of the row's sequence
// (generic.hip: bh_attention_generic; attention_bf16.hip and attention_prefill_bf16.hip for bfloat16;
// crates/beholdd-backend/src/cpu.rs:693-837: dots and value sums in double, softmax in float32)
int bhp_attention(const void* q, void* out, int dtype, const void* k_pages, const void* v_pages,
                  const int32_t* page_table, int table_stride, const int32_t* row_seq, const int32_t* positions,
                  int n_rows, int H, int KVH, int hd, float scale, int window, int kv_order, int pages) {
  if (!known(dtype) || n_rows <= 0 || H <= 0 || KVH <= 0 || H % KVH || hd <= 0 || window < 0) return 1;
  const int G = H / KVH;
  std::vector<float> score;
  std::vector<double> value(hd);
  for (int r = 0; r < n_rows; ++r) {
    const int pos = positions[r], first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    if (pos < 0 || pos / BH_PAGE >= table_stride) return 2;
    score.assign(pos + 1 - first, 0.f);
    for (int h = 0; h < H; ++h) {
      const int kv_head = h / G;
      float top = -INFINITY;
      for (int key = first; key <= pos; ++key) {
        const int page = page_table[(size_t)row_seq[r] * table_stride + key / BH_PAGE];
        if (page < 0 || page >= pages) return 4;
        const size_t base = ((size_t)page * KVH + kv_head) * BH_PAGE * hd;
        double dot = 0.0;
        for (int d = 0; d < hd; ++d)
          dot += (double)load(q, dtype, ((size_t)r * H + h) * hd + d) *
                 (double)load(k_pages, dtype, base + bh_key_index(kv_order, key % BH_PAGE, d, hd));
        score[key - first] = (float)(dot * (double)scale);
        top = fmaxf(top, score[key - first]);
      }
      float sum = 0.f;
      for (float& s : score) {
        s = expf(s - top);
        sum += s;
      }
      const float inv = 1.0f / sum;
      for (int d = 0; d < hd; ++d) value[d] = 0.0;
      for (int key = first; key <= pos; ++key) {
        const int page = page_table[(size_t)row_seq[r] * table_stride + key / BH_PAGE];
        const size_t base = ((size_t)page * KVH + kv_head) * BH_PAGE * hd;
        const double p = (double)(score[key - first] * inv);
        for (int d = 0; d < hd; ++d) value[d] += p * (double)load(v_pages, dtype, base + bh_value_index(kv_order, key % BH_PAGE, d, hd));
      }
      for (int d = 0; d < hd; ++d) store(out, dtype, ((size_t)r * H + h) * hd + d, (float)value[d]);
    }
  }
  return 0;
}

// tokens[row] = the largest logit's index, ties to the lowest; a row with a logit that is not finite: token -1,
// bad 1 (sampling.hip: bh_sample without a temperature; crates/beholdd-model/src/qwen3moe/forward.rs:1822-1842)
int bhp_argmax(const float* logits, int32_t* tokens, int32_t* bad, int n_rows, int vocab) {
  if (n_rows <= 0 || vocab <= 0) return 1;
  for (int r = 0; r < n_rows; ++r) {
    int best = 0;
    bool finite = true;
    for (int i = 0; i < vocab; ++i) {
      const float v = logits[(size_t)r * vocab + i];
      if (!isfinite(v)) finite = false;
      if (v > logits[(size_t)r * vocab + best]) best = i;
    }
    tokens[r] = finite ? best : -1;
    bad[r] = finite ? 0 : 1;
  }
  return 0;
}

// tokens[row] = a draw from softmax(logits / temperature) restricted to the top_k largest logits (0: all) and then to the
// smallest set of most likely tokens whose mass reaches top_p of what is left (ties at a threshold are kept), by the
// inverse CDF over the kept tokens in index order at uniform[row] in [0, 1); temperature <= 0: the argmax (sampling.hip:
// bh_sample with temperatures).  Sums in double.  margin[row] (may be null): how far the draw's target lies from the
// nearer end of the chosen token's interval, as a fraction of the kept mass: a kernel that sums in float32 may choose
// a neighbour when that is within its rounding.
int bhp_sample(const float* logits, const float* temperature, const int32_t* top_k, const float* top_p, const float* uniform,
               int32_t* tokens, int32_t* bad, double* margin, int n_rows, int vocab) {
  if (n_rows <= 0 || vocab <= 0 || !temperature || !uniform) return 1;
  for (int r = 0; r < n_rows; ++r) {
    const float* x = logits + (size_t)r * vocab;
    if (margin) margin[r] = 1.0;
    int best = 0;
    bool finite = true;
    for (int i = 0; i < vocab; ++i) {
      if (!isfinite(x[i])) finite = false;
      if (x[i] > x[best]) best = i;
    }
    bad[r] = finite ? 0 : 1;
    tokens[r] = finite ? best : -1;
    if (!finite || !(temperature[r] > 0.f)) continue;
    std::vector<float> sorted(x, x + vocab);
    std::sort(sorted.begin(), sorted.end(), [](float a, float b) { return a > b; });
    const int k = top_k ? top_k[r] : 0;
    float floor_value = (k > 0 && k < vocab) ? sorted[k - 1] : sorted[vocab - 1];   // ties at the k-th value are kept
    auto weight = [&](float v) { return exp(((double)v - (double)x[best]) / (double)temperature[r]); };
    const float p = top_p ? top_p[r] : 1.f;
    if (p > 0.f && p < 1.f) {
      double total = 0.0;
      for (int i = 0; i < vocab; ++i)
        if (x[i] >= floor_value) total += weight(x[i]);
      double mass = 0.0;
      for (int i = 0; i < vocab && sorted[i] >= floor_value; ++i) {   // most likely first; a value's ties all count
        mass += weight(sorted[i]);
        if ((i + 1 == vocab || sorted[i + 1] != sorted[i]) && mass >= (double)p * total) {
          floor_value = sorted[i];
          break;
        }
      }
    }
    double kept = 0.0;
    for (int i = 0; i < vocab; ++i)
      if (x[i] >= floor_value) kept += weight(x[i]);
    const double target = (double)uniform[r] * kept;
    double running = 0.0;
    int pick = -1, last = -1;
    for (int i = 0; i < vocab && pick < 0; ++i) {
      if (x[i] < floor_value) continue;
      last = i;
      const double before = running;
      running += weight(x[i]);
      if (running > target) {
        pick = i;
        if (margin) margin[r] = fmin(target - before, running - target) / kept;
      }
    }
    tokens[r] = pick >= 0 ? pick : last;
  }
  return 0;
}

int bhp_page_size() { return BH_PAGE; }
int bhp_key_index(int order, int token, int dim, int hd) { return bh_key_index(order, token, dim, hd); }
int bhp_value_index(int order, int token, int dim, int hd) { return bh_value_index(order, token, dim, hd); }
long bhp_rows_index(int block_rows, int row, int column, int width) { return bh_rows_index(block_rows, row, column, width); }

}  // extern "C"

#ifdef BH_TWINS_SELFTEST
// The reference's own vectors, and every index function over whole pages.  Built with the host sanitizers, so
// an index that leaves its page, or an uninitialised read, ends the run.
#define EXPECT(cond)                                                        \
  do {                                                                      \
    if (!(cond)) {                                                          \
      fprintf(stderr, "plain_twins self-test failed: %s (line %d)\n", #cond, __LINE__); \
      return 1;                                                             \
    }                                                                       \
  } while (0)

static bool near(float a, float b, float tol = 1e-6f) { return fabsf(a - b) <= tol; }

int main() {
  // every (token, dim) of a page has a place of its own inside the page, in both orders, for every head size
  for (int order = 0; order < 2; ++order)
    for (int hd = 16; hd <= 256; hd += 16) {
      if (order == BH_KV_PIECES && hd % 32) continue;
      std::vector<int> seen_k(BH_PAGE * hd, 0), seen_v(BH_PAGE * hd, 0);
      for (int token = 0; token < BH_PAGE; ++token)
        for (int dim = 0; dim < hd; ++dim) {
          const int k = bh_key_index(order, token, dim, hd), v = bh_value_index(order, token, dim, hd);
          EXPECT(k >= 0 && k < BH_PAGE * hd && v >= 0 && v < BH_PAGE * hd);
          seen_k[k]++;
          seen_v[v]++;
        }
      for (int i = 0; i < BH_PAGE * hd; ++i) EXPECT(seen_k[i] == 1 && seen_v[i] == 1);
    }
  // every element of a matrix whose rows lie in blocks of 8 or 16 has a place of its own within the whole blocks
  for (int block_rows = 8; block_rows <= 16; block_rows += 8)
    for (int rows = 1; rows <= 40; rows += 13) {
      const int width = 96, padded = (rows + block_rows - 1) / block_rows * block_rows;
      std::vector<int> seen(padded * width, 0);
      for (int row = 0; row < rows; ++row)
        for (int column = 0; column < width; ++column) {
          const long at = bh_rows_index(block_rows, row, column, width);
          EXPECT(at >= 0 && at < (long)padded * width);
          seen[at]++;
          EXPECT(bh_rows_index(0, row, column, width) == (long)row * width + column);
        }
      for (int i = 0; i < padded * width; ++i) EXPECT(seen[i] <= 1);
    }
  // bfloat16: widening is exact, narrowing rounds to nearest even (crates/beholdd-core/src/quant.rs:486-502)
  EXPECT(bf16_bits_to_f32(0x3F80) == 1.0f && bf16_bits_to_f32(0xC000) == -2.0f);
  EXPECT(f32_to_bf16_bits(1.0f) == 0x3F80 && f32_to_bf16_bits(1.00390625f) == 0x3F80 && f32_to_bf16_bits(1.01171875f) == 0x3F82);
  EXPECT(f32_to_bf16_bits(INFINITY) == 0x7F80 && (f32_to_bf16_bits(NAN) & 0x7FC0) == 0x7FC0);
  // rmsnorm: x = 1, eps = 0 gives the weight (crates/beholdd-kernel/src/vecops.rs:213-220)
  {
    const float x[4] = {1, 1, 1, 1}, w[4] = {2, 3, 4, 5};
    float y[4];
    EXPECT(bhp_rmsnorm(x, nullptr, w, BH_F32, y, BH_F32, 1, 4, 0.f) == 0);
    EXPECT(y[0] == 2 && y[1] == 3 && y[2] == 4 && y[3] == 5);
  }
  // split-half rotation: [1, 2, 3, 4] with cos 0, sin 1 gives [-3, -4, 1, 2] (crates/beholdd-kernel/src/vecops.rs:278-289),
  // and the attention vector q = [1, 0], keys [0, 0], [ln 3, 0], values [2, 4], [6, 8], scale 1: [2, 4] then [5, 7]
  // (crates/beholdd-backend/src/cpu.rs:1389-1411); one page, both orders where the head size allows
  {
    const float qkv[12] = {1, 2, 3, 4, 1, 2, 3, 4, 9, 8, 7, 6};   // one q head, one k head, one v head of 4
    const float cos_t[2] = {0, 0}, sin_t[2] = {1, 1};
    const int32_t positions[1] = {0}, row_seq[1] = {0}, table[1] = {0};
    float q_out[4];
    std::vector<float> k_pages(BH_PAGE * 4, 0.f), v_pages(BH_PAGE * 4, 0.f);
    EXPECT(bhp_qk_norm_rope_cache(qkv, BH_F32, q_out, nullptr, nullptr, BH_F32, 0.f, cos_t, sin_t, 1, 4, positions, row_seq,
                                  k_pages.data(), v_pages.data(), table, 1, 1, 1, 1, 4, 1, BH_KV_ROWS, 1) == 0);
    EXPECT(q_out[0] == -3 && q_out[1] == -4 && q_out[2] == 1 && q_out[3] == 2);
    EXPECT(k_pages[0] == -3 && k_pages[3] == 2 && v_pages[0 * BH_PAGE] == 9 && v_pages[3 * BH_PAGE] == 6);
  }
  {
    const float q[4] = {1, 0, 1, 0};   // two rows of one head of 2
    std::vector<float> k_pages(BH_PAGE * 2, 0.f), v_pages(BH_PAGE * 2, 0.f);
    k_pages[bh_key_index(0, 1, 0, 2)] = logf(3.0f);
    v_pages[bh_value_index(0, 0, 0, 2)] = 2; v_pages[bh_value_index(0, 0, 1, 2)] = 4;
    v_pages[bh_value_index(0, 1, 0, 2)] = 6; v_pages[bh_value_index(0, 1, 1, 2)] = 8;
    const int32_t positions[2] = {0, 1}, row_seq[2] = {0, 0}, table[1] = {0};
    float out[4];
    EXPECT(bhp_attention(q, out, BH_F32, k_pages.data(), v_pages.data(), table, 1, row_seq, positions, 2, 1, 1, 2, 1.0f, 0,
                         BH_KV_ROWS, 1) == 0);
    EXPECT(near(out[0], 2) && near(out[1], 4) && near(out[2], 5) && near(out[3], 7));
    // a page outside the cache is refused, not read
    const int32_t beyond[1] = {1};
    EXPECT(bhp_attention(q, out, BH_F32, k_pages.data(), v_pages.data(), beyond, 1, row_seq, positions, 2, 1, 1, 2, 1.0f, 0,
                         BH_KV_ROWS, 1) == 4);
  }
  // grouped heads: 4 query heads on 2 kv heads, zero keys, values [1, 10], [3, 30] (crates/beholdd-backend/src/cpu.rs:1414-1440)
  {
    const float q[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    std::vector<float> k_pages(2 * BH_PAGE, 0.f), v_pages(2 * BH_PAGE, 0.f);
    v_pages[0 * BH_PAGE + 0] = 1; v_pages[1 * BH_PAGE + 0] = 10; v_pages[0 * BH_PAGE + 1] = 3; v_pages[1 * BH_PAGE + 1] = 30;
    const int32_t positions[2] = {0, 1}, row_seq[2] = {0, 0}, table[1] = {0};
    float out[8];
    EXPECT(bhp_attention(q, out, BH_F32, k_pages.data(), v_pages.data(), table, 1, row_seq, positions, 2, 4, 2, 1, 1.0f, 0,
                         BH_KV_ROWS, 1) == 0);
    const float want[8] = {1, 1, 10, 10, 2, 2, 20, 20};
    for (int i = 0; i < 8; ++i) EXPECT(near(out[i], want[i]));
  }
  // linear: w = [1, 2, -0.5, 4], x = [3, 5, 8, 0.25] gives 10 (crates/beholdd-kernel/src/bf16.rs:181-190), bfloat16 weights
  {
    const float x[4] = {3, 5, 8, 0.25f};
    const uint16_t w[4] = {f32_to_bf16_bits(1), f32_to_bf16_bits(2), f32_to_bf16_bits(-0.5f), f32_to_bf16_bits(4)};
    float y[1] = {100};
    EXPECT(bhp_gemm(x, BH_F32, w, BH_BF16, y, BH_F32, 0, 1, 1, 4) == 0 && y[0] == 10);
    EXPECT(bhp_gemm(x, BH_F32, w, BH_BF16, y, BH_F32, 1, 1, 1, 4) == 0 && y[0] == 20);
  }
  // greedy: [-1, 3, 3, 2] gives 1; a NaN or an infinity is refused (crates/beholdd-model/src/qwen3moe/forward.rs:2257-2262)
  {
    const float rows[8] = {-1, 3, 3, 2, 0, NAN, INFINITY, 0};
    int32_t tokens[2], bad[2];
    EXPECT(bhp_argmax(rows, tokens, bad, 2, 4) == 0 && tokens[0] == 1 && bad[0] == 0 && tokens[1] == -1 && bad[1] == 1);
  }
  // a draw: logits ln 1, ln 2, ln 5 at temperature 1 are the masses 1/8, 2/8, 5/8; top_k 2 leaves 2/7, 5/7; top_p 0.5 the last alone
  {
    const float row[3] = {0.f, logf(2.f), logf(5.f)};
    const float one = 1.f, half = 0.5f;
    const int32_t two = 2;
    int32_t token, flag;
    double margin;
    const float draws[4] = {0.1f, 0.2f, 0.374f, 0.376f};
    const int want_all[4] = {0, 1, 1, 2}, want_two[4] = {1, 1, 2, 2};
    for (int i = 0; i < 4; ++i) {
      EXPECT(bhp_sample(row, &one, nullptr, nullptr, &draws[i], &token, &flag, &margin, 1, 3) == 0 && token == want_all[i] && flag == 0);
      EXPECT(bhp_sample(row, &one, &two, nullptr, &draws[i], &token, &flag, &margin, 1, 3) == 0 && token == want_two[i]);
      EXPECT(bhp_sample(row, &one, nullptr, &half, &draws[i], &token, &flag, &margin, 1, 3) == 0 && token == 2);
    }
    const float zero = 0.f;
    EXPECT(bhp_sample(row, &zero, nullptr, nullptr, &draws[0], &token, &flag, nullptr, 1, 3) == 0 && token == 2);
  }
  // swiglu: silu(0) = 0, silu(x) -> x for large x, no clamp
  {
    const float gu[4] = {0, 30, 5, 7};
    float out[2];
    EXPECT(bhp_swiglu(gu, out, BH_F32, 1, 2) == 0 && out[0] == 0 && near(out[1], 210.0f, 1e-3f));
  }
  // embedding refuses a token outside the table
  {
    const float table[4] = {1, 2, 3, 4};
    const int32_t tokens[2] = {1, 2};
    float out[4];
    EXPECT(bhp_embed(tokens, table, BH_F32, out, 1, 2, 2) == 0 && out[0] == 3 && out[1] == 4);
    EXPECT(bhp_embed(tokens, table, BH_F32, out, 2, 2, 2) == 2);
  }
  printf("plain_twins self-test ok\n");
  return 0;
}
#endif
