// One of the instantiations of the matrix-core expert kernel for calls with few rows per expert (see expert_gemm_parts.h).
#include "expert_gemm_parts.h"
#include "expert_gemm_tile.h"

namespace infmoe {

hipError_t expert_gemm_launch_small_grouped(const GemmProblem& p, size_t weight_stride, const RowTile* tiles, const int* sched,
        int n_col_tiles, dim3 grid, size_t lds, hipStream_t stream) {
    const hipError_t err = allow_lds_once<expert_gemm_grouped_small_kernel<kGemmColumns, EPI_RESIDUAL>>(kLdsPerCu / 2);
    if (err != hipSuccess) return err;
    expert_gemm_grouped_small_kernel<kGemmColumns, EPI_RESIDUAL><<<grid, kGemmThreads, lds, stream>>>(p, weight_stride, tiles, sched, n_col_tiles);
    return hipGetLastError();
}

}  // namespace infmoe
