// One of the six instantiations of the matrix-core expert kernel (see expert_gemm_parts.h).
#include "expert_gemm_parts.h"
#include "expert_gemm_tile.h"

namespace infmoe {

hipError_t expert_gemm_launch_grouped_gated(const GemmProblem& p, size_t weight_stride, const RowTile* tiles, const int* sched,
                                            int n_col_tiles, dim3 grid, size_t lds, hipStream_t stream) {
    const hipError_t err = allow_lds_once<expert_gemm_grouped_kernel<kGemmColumns, EPI_GATED_GELU>>(kLdsPerCu);
    if (err != hipSuccess) return err;
    expert_gemm_grouped_kernel<kGemmColumns, EPI_GATED_GELU><<<grid, kGemmThreads, lds, stream>>>(p, weight_stride, tiles, sched, n_col_tiles);
    return hipGetLastError();
}

}  // namespace infmoe
