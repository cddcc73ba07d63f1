// One of the instantiations of the matrix-core expert kernel for calls with few rows per expert (see expert_gemm_parts.h).
#include "expert_gemm_parts.h"
#include "expert_gemm_tile.h"

namespace infmoe {

hipError_t expert_gemm_launch_small_one_relu(const GemmProblem& p, int rows, int tile_rows, int a_alloc_rows, dim3 grid, size_t lds,
        hipStream_t stream) {
    const hipError_t err = allow_lds_once<expert_gemm_small_kernel<kGemmColumns, EPI_RELU>>(kLdsPerCu / 2);
    if (err != hipSuccess) return err;
    expert_gemm_small_kernel<kGemmColumns, EPI_RELU><<<grid, kGemmThreads, lds, stream>>>(p, rows, tile_rows, a_alloc_rows);
    return hipGetLastError();
}

}  // namespace infmoe
