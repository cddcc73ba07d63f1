// Host side of the FP32 matrix-core expert GEMM (device code: expert_gemm_tile.h), and the
// one-thread-per-element kernel for shapes the matrix-core kernels do not take.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "device_math.h"
#include "expert_gemm_parts.h"
#include "kernels.h"

namespace infmoe {
namespace {

// Shapes the matrix-core kernel does not take (K not a multiple of 32, or operands that are not
// 16-byte aligned): one thread per output element.  Only small or odd shapes come here.
// row_expert == nullptr: one expert; else row r uses the weights of expert row_expert[r].
__global__ void expert_gemm_generic_kernel(GemmProblem p, int rows, size_t weight_stride,
                                           const int* __restrict__ row_expert) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)rows * p.N) return;
    const int row = idx / p.N, col = idx % p.N;
    int owner = row_expert ? row_expert[row] : 0;
    if (row_expert && p.expert_slot) owner = p.expert_slot[owner];
    const size_t w0 = (size_t)owner * weight_stride;
    const float* a = p.A + (size_t)row * p.K;
    const float* b0 = p.B + w0 + (size_t)col * p.K;
    float s0 = 0.f, s1 = 0.f;
    for (int k = 0; k < p.K; ++k) s0 += a[k] * b0[k];
    if (p.epilogue == EPI_RESIDUAL) {
        s0 += p.R[idx];
    } else {
        const float rstd = p.row_stats ? p.row_stats[2 * (size_t)row + 1] : 1.f;
        s0 *= rstd;
        if (p.epilogue == EPI_GATED_GELU) {
            const float* b1 = p.B1 + w0 + (size_t)col * p.K;
            for (int k = 0; k < p.K; ++k) s1 += a[k] * b1[k];
            s1 *= rstd;
            s0 = gelu_dot(s0, s1);
        } else {
            s0 = fmaxf(s0, 0.f);
        }
    }
    p.C[idx] = s0;
}

// LDS the kernel may touch for tiles of up to a_alloc_rows rows: the larger of the two step widths
// (32-float steps: rows of 36 floats; 64-float steps, tiles of up to 160 rows and one weight matrix:
// rows of 68 floats).
size_t lds_bytes(bool gated, int a_alloc_rows, int K) {
    const size_t nb = gated ? 2 : 1;
    size_t bytes = (2 * (size_t)a_alloc_rows * 36 + 2 * nb * kGemmColumns * 36) * sizeof(float);
    if (!gated && K % 64 == 0) {
        const size_t rows64 = (size_t)std::min(a_alloc_rows, 16 * kGemmMaxUnits64);
        bytes = std::max(bytes, (2 * rows64 * 68 + 2 * nb * kGemmColumns * 68) * sizeof(float));
    }
    return bytes;
}

bool fast_path_ok(const GemmProblem& p) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B) |
                           reinterpret_cast<uintptr_t>(p.B1);
    return p.K % 32 == 0 && (bits & 15) == 0 && (reinterpret_cast<uintptr_t>(p.row_stats) & 7) == 0;
}

// the second product needs its residual, the two-matrix form its second matrix (and its tall tiles)
bool operands_ok(const GemmProblem& p) {
    if (p.epilogue == EPI_RESIDUAL) return p.R != nullptr;
    return p.epilogue != EPI_GATED_GELU || (p.B1 != nullptr && !p.small_tiles);
}

// LDS of the few-rows-per-expert form: 32-float steps (rows of 36 floats), one weight matrix
size_t lds_bytes_small(int a_alloc_rows) {
    return 2 * ((size_t)a_alloc_rows + kGemmColumns) * 36 * sizeof(float);
}

}  // namespace

bool expert_gemm_grouped_ok(const GemmProblem& p, size_t weight_stride) {
    return fast_path_ok(p) && weight_stride % 4 == 0;
}

hipError_t launch_expert_gemm_any_shape_grouped(const GemmProblem& p, size_t weight_stride, const int* row_expert,
                                                int rows, hipStream_t stream) {
    if (rows <= 0) return hipSuccess;
    if (!operands_ok(p)) return hipErrorInvalidValue;
    const size_t n = (size_t)rows * p.N;
    expert_gemm_generic_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(p, rows, weight_stride, row_expert);
    return hipGetLastError();
}

hipError_t launch_expert_gemm(const GemmProblem& p, int rows, int tile_rows, hipStream_t stream) {
    if (rows <= 0) return hipSuccess;
    if (tile_rows <= 0 || tile_rows % 16 != 0 || tile_rows > gemm_tile_rows(p.epilogue, p.small_tiles != 0))
        return hipErrorInvalidValue;
    if (!operands_ok(p)) return hipErrorInvalidValue;
    if (!fast_path_ok(p)) {
        const size_t n = (size_t)rows * p.N;
        expert_gemm_generic_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(p, rows, 0, nullptr);
        return hipGetLastError();
    }
    const int tile = std::min(row_tile_height(rows, tile_rows), ((rows + 15) / 16) * 16);
    const int a_alloc = ((tile + 31) / 32) * 32;  // whole 32-row slabs
    const dim3 grid((rows + tile - 1) / tile, (p.N + kGemmColumns - 1) / kGemmColumns);  // x: row tiles, y: column tiles
    if (p.small_tiles) {
        // (LDS for the tallest tile of this form whatever this expert's height: the two-workgroups-per-unit
        // residency is the same for every launch of the form)
        const size_t lds = lds_bytes_small(kGemmTileRowsSmall);
        return p.epilogue == EPI_RELU ? expert_gemm_launch_small_one_relu(p, rows, tile, kGemmTileRowsSmall, grid, lds, stream)
                                      : expert_gemm_launch_small_one(p, rows, tile, kGemmTileRowsSmall, grid, lds, stream);
    }
    const bool gated = p.epilogue == EPI_GATED_GELU;
    const size_t lds = lds_bytes(gated, a_alloc, p.K);
    return gated ? expert_gemm_launch_one_gated(p, rows, tile, a_alloc, grid, lds, stream)
           : p.epilogue == EPI_RELU ? expert_gemm_launch_one_relu(p, rows, tile, a_alloc, grid, lds, stream)
                                    : expert_gemm_launch_one(p, rows, tile, a_alloc, grid, lds, stream);
}

hipError_t launch_expert_gemm_grouped(const GemmProblem& p, size_t weight_stride, const RowTile* tiles,
                                      const int* sched, int max_tiles, hipStream_t stream) {
    if (max_tiles <= 0) return hipSuccess;
    if (!expert_gemm_grouped_ok(p, weight_stride) || !operands_ok(p)) return hipErrorInvalidValue;  // see launch_expert_gemm_any_shape_grouped
    const int n_col_tiles = (p.N + kGemmColumns - 1) / kGemmColumns;
    const dim3 grid((unsigned)kXcdCount * (unsigned)xcd_tile_capacity(max_tiles) * (unsigned)n_col_tiles);
    if (p.small_tiles) {
        const size_t lds = lds_bytes_small(kGemmTileRowsSmall);
        return p.epilogue == EPI_RELU
                   ? expert_gemm_launch_small_grouped_relu(p, weight_stride, tiles, sched, n_col_tiles, grid, lds, stream)
                   : expert_gemm_launch_small_grouped(p, weight_stride, tiles, sched, n_col_tiles, grid, lds, stream);
    }
    const bool gated = p.epilogue == EPI_GATED_GELU;
    const size_t lds = lds_bytes(gated, gated ? kGemmTileRowsGated : kGemmTileRows, p.K);
    return gated ? expert_gemm_launch_grouped_gated(p, weight_stride, tiles, sched, n_col_tiles, grid, lds, stream)
           : p.epilogue == EPI_RELU
               ? expert_gemm_launch_grouped_relu(p, weight_stride, tiles, sched, n_col_tiles, grid, lds, stream)
               : expert_gemm_launch_grouped(p, weight_stride, tiles, sched, n_col_tiles, grid, lds, stream);
}

}  // namespace infmoe
