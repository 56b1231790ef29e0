// Products of 33 to 128 rows whose activations the waves of a workgroup share through LDS: see gemm_bf16_slices.hip.
#pragma once
#include "common.h"

// Whether the kernel takes a product of these sizes (W in the tiles layout, activations in blocks of 16 rows).
bool gemm_slices_takes(int M, int N, int K, int layout, int activation);
// In how many parts it cuts K (always through scratch memory and the finishing kernel, also with one part),
// and how many slices of 512 k each part has.
int gemm_slices_parts(int M, int N, int K, int activation, int* slices_per_part);
// The multiplication: bare sums [part][M][N, or 2 N weight rows for SwiGLU] for gemm_parts_finish_kernel.
int gemm_slices_launch(const void* a, const void* w, float* sums, int M, int N, int K, int activation,
                       hipStream_t stream);
// A SwiGLU with so many outputs that no parts are needed is finished by the kernel itself (gemm_slices_gated says
// which): gated[M][N] = bfloat16(silu(a Wg^T) * (a Wu^T)), in blocks of gated_block_rows rows (0: rows), times the row
// factors of a norm ahead when its partial sums are given.
bool gemm_slices_gated(int M, int N, int K, int activation);
int gemm_slices_launch_gated(const void* a, const void* w, void* gated, int gated_block_rows, int M, int N, int K,
                             const float* ahead_ss, int ahead_blocks, float ahead_eps, hipStream_t stream);
