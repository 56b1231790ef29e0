// Entry points of sampling.hip.
#pragma once
#include "common.h"

extern "C" {

// Float-sized words of scratch that bh_sample wants for these rows when every row is greedy (0: none).
int bh_sample_scratch(int n_rows, int vocab);

// Words of scratch for a draw at a temperature without top-k and top-p (0: none is used).
int bh_sample_draw_scratch(int n_rows, int vocab);

// Words of scratch for draws with a top-k (0: none is used).
int bh_sample_top_k_scratch(int n_rows, int vocab);

// One token per row of float32 logits [n_rows, vocab]: argmax where `temperature` is null or <= 0, else
// a draw (see sampling.hip).  `scratch` (bh_sample_scratch words for greedy rows, bh_sample_draw_scratch words
// for a draw at a temperature alone, bh_sample_top_k_scratch words for draws with a top-k, or null) is the caller's.
int bh_sample(const float* logits, const float* temperature, const int32_t* top_k, const float* top_p,
              const float* uniform, int32_t* tokens, int32_t* bad, void* scratch, int n_rows, int vocab,
              hipStream_t stream);

// Greedy selection that allocates nothing.  This entry point has no counterpart in the reference.  It is
// for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops and
// harnesses that forbid hipMalloc.  It computes what bh_sample computes for greedy rows (the largest logit,
// ties to the lowest id; a row with a non-finite logit gets token -1 and bad = 1) with the same two
// kernels, and keeps the per-chunk maxima between them in a fixed array in device memory that the
// library owns (BH_GREEDY_STATIC_WORDS floats, 128 KB, held on every GPU the library runs on until the
// process ends) instead of a buffer of the caller's.  It refuses sizes whose partial results do not fit:
// 2 * n_rows * ceil(vocab / 2048) must not exceed BH_GREEDY_STATIC_WORDS.  Nothing in the array has to
// start at zero: the first kernel writes every word that the second reads.  All calls on one GPU share the
// array, so two calls that overlap there (different streams, or different threads) race; calls on one
// stream are ordered and safe.
#define BH_GREEDY_STATIC_WORDS 32768
int bh_sample_greedy_static(const float* logits, int32_t* tokens, int32_t* bad, int n_rows, int vocab,
                            hipStream_t stream);
}
