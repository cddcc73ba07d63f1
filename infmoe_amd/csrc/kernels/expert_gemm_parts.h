// The matrix-core expert kernels are instantiated in six translation units (one kernel each - one-expert or
// grouped launch, times the three epilogues - so that they compile side by side); these are their launch stubs.  `lds` is the dynamic LDS of the launch.
#pragma once

#include "kernels.h"

namespace infmoe {

constexpr int kGemmThreads = 256;     // 4 waves
constexpr int kGemmColumns = 128;     // weight rows (output columns) per workgroup
constexpr int kGemmMaxUnits64 = 10;   // tallest tile (in 16-row units) that takes 64-float K steps: 160 rows
constexpr size_t kLdsPerCu = 160 * 1024;  // the limit is raised once, to all there is; launches ask for what they use

// tile_rows: height of every row tile but the last (grid.y of them)
hipError_t expert_gemm_launch_one(const GemmProblem& p, int rows, int tile_rows, int a_alloc_rows, dim3 grid,
                                  size_t lds, hipStream_t stream);
hipError_t expert_gemm_launch_one_relu(const GemmProblem& p, int rows, int tile_rows, int a_alloc_rows, dim3 grid,
                                       size_t lds, hipStream_t stream);
hipError_t expert_gemm_launch_one_gated(const GemmProblem& p, int rows, int tile_rows, int a_alloc_rows, dim3 grid,
                                        size_t lds, hipStream_t stream);
hipError_t expert_gemm_launch_grouped(const GemmProblem& p, size_t weight_stride, const RowTile* tiles,
                                      const int* sched, int n_col_tiles, dim3 grid, size_t lds, hipStream_t stream);
hipError_t expert_gemm_launch_grouped_relu(const GemmProblem& p, size_t weight_stride, const RowTile* tiles,
                                           const int* sched, int n_col_tiles, dim3 grid, size_t lds,
                                           hipStream_t stream);
// the few-rows-per-expert form (two workgroups per compute unit)
hipError_t expert_gemm_launch_small_one(const GemmProblem& p, int rows, int tile_rows, int a_alloc_rows, dim3 grid,
                                        size_t lds, hipStream_t stream);
hipError_t expert_gemm_launch_small_one_relu(const GemmProblem& p, int rows, int tile_rows, int a_alloc_rows, dim3 grid,
                                             size_t lds, hipStream_t stream);
hipError_t expert_gemm_launch_small_grouped(const GemmProblem& p, size_t weight_stride, const RowTile* tiles,
                                            const int* sched, int n_col_tiles, dim3 grid, size_t lds,
                                            hipStream_t stream);
hipError_t expert_gemm_launch_small_grouped_relu(const GemmProblem& p, size_t weight_stride, const RowTile* tiles,
                                                 const int* sched, int n_col_tiles, dim3 grid, size_t lds,
                                                 hipStream_t stream);
hipError_t expert_gemm_launch_grouped_gated(const GemmProblem& p, size_t weight_stride, const RowTile* tiles,
                                            const int* sched, int n_col_tiles, dim3 grid, size_t lds,
                                            hipStream_t stream);

}  // namespace infmoe
