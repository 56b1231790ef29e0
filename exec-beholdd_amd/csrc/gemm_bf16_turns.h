// Matrix products of many rows in which two groups of waves take turns: see gemm_bf16_turns.hip.
#pragma once
#include "common.h"

// How many blocks of 16 weight rows a wave takes (8, 6 or 4: tiles of 256 rows x 256, 192 or 128 weight
// rows) if this way is the faster one for a product of these sizes, else 0.
int gemm_turns_blocks(int M, int N, int K, int layout, int activation);
// Whether the kernel can run these sizes at all with `blocks` blocks per wave.
bool gemm_turns_can(int M, int N, int K, int layout, int activation, int blocks);
// c_dtype BH_F32 (accumulate allowed) or BH_BF16 (no accumulate); activation 1 = SwiGLU, bfloat16 output only.
// a_blocked: A in blocks of 16 rows x 32 columns (bh_blocked_index), in a buffer of whole tiles of 256 rows;
// c_blocked: a SwiGLU's output likewise.
int gemm_turns_launch(const void* a, const void* w, void* c, int c_dtype, int accumulate, int M, int N, int K,
                      int activation, int blocks, int a_blocked, int c_blocked, hipStream_t stream);
// In how many parts of K the widest tile multiplies a product that would otherwise leave compute units idle
// (1: not this way), and that multiplication: bare sums [part][M][N] for gemm_parts_finish_kernel.
int gemm_turns_parts(int M, int N, int K, int layout, int activation);
int gemm_turns_launch_parts(const void* a, const void* w, float* sums, int M, int N, int K, int parts, int a_blocked,
                            hipStream_t stream);
