// FP32 matrix-core GEMM of the T5 feed-forward expert for gfx950.
//
// Replaces the three cublasSgemm_v2 calls, the thrust gelu*mul pass and the device-to-device
// residual copy of T5FFLayer::run (plugin/sublayers/T5FFLayer.cc:112-138, plugin/cuda/ops/gelu.cu:7-25):
//     C[rows][N] = epilogue(A[rows][K] * B[N][K]^T)
// with both operands K-contiguous (activations row-major, weights in torch Linear layout), which
// is the "TN" form v_mfma_f32_16x16x4_f32 wants: a lane feeds one float of an A row and one float
// of a B row per instruction.
//
// Tiling.  The weights are the big operand (335 MB per expert at d=4096, h=10240) and each weight
// element is reused only `rows` times, so a workgroup covers ALL rows of its expert (up to 256) x
// BN weight rows: every weight byte is fetched from HBM once.  Token counts per expert vary, so the
// tile height is a run-time multiple of 16 rows (NMB row blocks); the body is instantiated for
// NMB = 1..16 and selected per workgroup, which wastes at most 15 padded rows per expert instead of
// up to a whole fixed-height tile.  The 4 waves of a workgroup split the BN columns; each keeps
// NMB x (BN/64) accumulator blocks in registers.
//
// Pipeline.  K advances in steps of 32 floats.  Global loads of step s+2 are issued into registers
// before the matrix-core work of step s; the registers holding step s+1 are written to the other
// half of a double-buffered LDS tile afterwards; one barrier per step.  LDS rows are padded to 36 floats so that the 16-byte
// operand reads of the 16 lanes of a block hit distinct banks.  Inside a 16-float chunk the k order
// is permuted identically for A and B (lane q supplies floats 4q..4q+3 over four instructions),
// which a dot product does not see and which lets every operand read be a ds_read_b128.
//
// Grouped launch.  One launch covers every expert: row tiles come from the device-side table built
// by the dispatch scan, so no token count ever travels to the host.  Workgroup ids are dealt
// round-robin to the 8 XCDs by the hardware; the id -> tile map undoes that so each XCD works
// through a contiguous run of (expert, column tile) pairs and the activations of an expert stay
// in one XCD's L2.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "kernels.h"

namespace infmoe {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int BK = 32;            // k floats per pipeline step
constexpr int LDK = BK + 4;       // padded LDS row (floats)
constexpr int kThreads = 256;     // 4 waves

__device__ __forceinline__ float gelu_dot(float a, float b) {
    // plugin/cuda/ops/gelu.cu:8-15
    const float cdf = 0.5f * (1.0f + tanhf(a * (0.035677408136300125f * a * a + 0.7978845608028654f)));
    return a * cdf * b;
}

// One output tile: `rows` (<= 16*NMB) rows of A against BN rows of B (and of B1 when GATED).
template <int NMB, int BN, bool GATED>
__device__ __forceinline__ void gemm_tile(const float* __restrict__ A, const float* __restrict__ R,
                                          float* __restrict__ C, int rows, const float* __restrict__ B0,
                                          const float* __restrict__ B1, int n0, int N, int K, int epilogue,
                                          float* __restrict__ smem, int a_alloc_rows) {
    constexpr int NBW = BN / 64;              // 16-column blocks per wave
    constexpr int NB = GATED ? 2 : 1;         // weight matrices
    constexpr int A_ROWS = NMB * 16;
    constexpr int A_LOADS = (A_ROWS * 8 + kThreads - 1) / kThreads;  // float4 per thread per step
    constexpr int B_LOADS = (BN * 8) / kThreads;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int i = lane & 15, kq = lane >> 4;
    const int ld_row = tid >> 3, ld_c4 = tid & 7;  // this thread's (row, float4) inside a 32-row slab

    float* As = smem;                                   // [2][a_alloc_rows][LDK]
    float* Bs = smem + 2 * (size_t)a_alloc_rows * LDK;  // [2][NB*BN][LDK]
    const size_t a_buf = (size_t)a_alloc_rows * LDK, b_buf = (size_t)NB * BN * LDK;

    v4f acc[NB][NMB][NBW];
#pragma unroll
    for (int m = 0; m < NB; ++m)
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb) acc[m][mb][nb] = v4f{0.f, 0.f, 0.f, 0.f};

    // row pointers of this thread's global loads (rows past the end are clamped: their products
    // land in accumulator rows / columns that are never stored)
    const float* a_ptr[A_LOADS];
#pragma unroll
    for (int p = 0; p < A_LOADS; ++p) a_ptr[p] = A + (size_t)min(p * 32 + ld_row, rows - 1) * K + 4 * ld_c4;
    const float* b_ptr[NB][B_LOADS];
#pragma unroll
    for (int p = 0; p < B_LOADS; ++p) {
        const size_t off = (size_t)min(n0 + p * 32 + ld_row, N - 1) * K + 4 * ld_c4;
        b_ptr[0][p] = B0 + off;
        if (GATED) b_ptr[NB - 1][p] = B1 + off;
    }

    // Two register sets: global loads run two K steps ahead of the matrix core, which covers the
    // latency of an HBM miss (every weight load is one) with two steps of MFMA work.
    v4f ra[2][A_LOADS], rb[2][NB][B_LOADS];
    auto load_global = [&](auto setc, int k0) {
        constexpr int P = decltype(setc)::value;
        const bool kin = (k0 + 4 * ld_c4) < K;  // K % 4 == 0: a float4 is inside or outside as a whole
#pragma unroll
        for (int p = 0; p < A_LOADS; ++p) {
            ra[P][p] = v4f{0.f, 0.f, 0.f, 0.f};
            if (kin && (A_ROWS % 32 == 0 || p * 32 + ld_row < A_ROWS))
                ra[P][p] = *reinterpret_cast<const v4f*>(a_ptr[p] + k0);
        }
#pragma unroll
        for (int m = 0; m < NB; ++m)
#pragma unroll
            for (int p = 0; p < B_LOADS; ++p) {
                rb[P][m][p] = v4f{0.f, 0.f, 0.f, 0.f};
                if (kin) rb[P][m][p] = *reinterpret_cast<const v4f*>(b_ptr[m][p] + k0);
            }
    };
    auto store_lds = [&](auto setc, int buf) {
        constexpr int P = decltype(setc)::value;
        float* a = As + buf * a_buf;
        float* b = Bs + buf * b_buf;
#pragma unroll
        for (int p = 0; p < A_LOADS; ++p)
            if (A_ROWS % 32 == 0 || p * 32 + ld_row < A_ROWS)
                *reinterpret_cast<v4f*>(a + (p * 32 + ld_row) * LDK + 4 * ld_c4) = ra[P][p];
#pragma unroll
        for (int m = 0; m < NB; ++m)
#pragma unroll
            for (int p = 0; p < B_LOADS; ++p)
                *reinterpret_cast<v4f*>(b + (m * BN + p * 32 + ld_row) * LDK + 4 * ld_c4) = rb[P][m][p];
    };
    auto compute = [&](int buf) {
        const float* a = As + buf * a_buf + i * LDK + 4 * kq;
        const float* b = Bs + buf * b_buf + (wave * (BN / 4) + i) * LDK + 4 * kq;
#pragma unroll
        for (int g = 0; g < BK / 16; ++g) {
            v4f bf[NB][NBW];
#pragma unroll
            for (int m = 0; m < NB; ++m)
#pragma unroll
                for (int nb = 0; nb < NBW; ++nb)
                    bf[m][nb] = *reinterpret_cast<const v4f*>(b + (m * BN + 16 * nb) * LDK + 16 * g);
#pragma unroll
            for (int mb = 0; mb < NMB; ++mb) {
                const v4f af = *reinterpret_cast<const v4f*>(a + 16 * mb * LDK + 16 * g);
#pragma unroll
                for (int m = 0; m < NB; ++m)
#pragma unroll
                    for (int nb = 0; nb < NBW; ++nb) {
                        v4f c = acc[m][mb][nb];
                        c = __builtin_amdgcn_mfma_f32_16x16x4f32(af.x, bf[m][nb].x, c, 0, 0, 0);
                        c = __builtin_amdgcn_mfma_f32_16x16x4f32(af.y, bf[m][nb].y, c, 0, 0, 0);
                        c = __builtin_amdgcn_mfma_f32_16x16x4f32(af.z, bf[m][nb].z, c, 0, 0, 0);
                        c = __builtin_amdgcn_mfma_f32_16x16x4f32(af.w, bf[m][nb].w, c, 0, 0, 0);
                        acc[m][mb][nb] = c;
                    }
            }
        }
    };
    // Step s computes from LDS buffer s & 1 while register set P holds step s + 1 and the other
    // set receives step s + 2; the loop is unrolled by two so that P is a compile-time constant.
    const int nk = (K + BK - 1) / BK;
    auto step = [&](auto setc, int s) {
        constexpr int P = decltype(setc)::value;
        if (s + 2 < nk) load_global(std::integral_constant<int, 1 - P>{}, (s + 2) * BK);
        compute(s & 1);
        if (s + 1 < nk) store_lds(setc, (s + 1) & 1);
        __syncthreads();
    };
    const std::integral_constant<int, 0> set0{};
    const std::integral_constant<int, 1> set1{};
    load_global(set1, 0);
    store_lds(set1, 0);
    if (nk > 1) load_global(set0, BK);
    __syncthreads();
    for (int s = 0; s < nk; s += 2) {
        step(set0, s);
        if (s + 1 < nk) step(set1, s + 1);
    }

    // epilogue: accumulator register r of block (mb, nb) is C[16*mb + 4*kq + r][16*nb + i]
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) {
            const int col = n0 + wave * (BN / 4) + 16 * nb + i;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = 16 * mb + 4 * kq + r;
                if (row < rows && col < N) {
                    const size_t o = (size_t)row * N + col;
                    float v = acc[0][mb][nb][r];
                    if (GATED) {
                        v = gelu_dot(v, acc[NB - 1][mb][nb][r]);
                    } else if (epilogue == EPI_RELU) {
                        v = fmaxf(v, 0.f);
                    } else {
                        v += R[o];
                    }
                    C[o] = v;
                }
            }
        }
}

template <int BN, bool GATED>
__device__ __forceinline__ void gemm_dispatch(int nmb, const float* A, const float* R, float* C, int rows,
                                              const float* B0, const float* B1, int n0, int N, int K, int epilogue,
                                              float* smem, int a_alloc_rows) {
    // the gated form keeps two accumulator sets, so its tiles are half as tall
    constexpr int kMaxMb = (GATED ? kGemmTileRowsGated : kGemmTileRows) / 16;
#define INFMOE_CASE(n)                                                                                       \
    case n:                                                                                                  \
        if constexpr (n <= kMaxMb)                                                                           \
            gemm_tile<n, BN, GATED>(A, R, C, rows, B0, B1, n0, N, K, epilogue, smem, a_alloc_rows);          \
        break;
    switch (nmb) {
        INFMOE_CASE(1) INFMOE_CASE(2) INFMOE_CASE(3) INFMOE_CASE(4) INFMOE_CASE(5) INFMOE_CASE(6) INFMOE_CASE(7)
        INFMOE_CASE(8) INFMOE_CASE(9) INFMOE_CASE(10) INFMOE_CASE(11) INFMOE_CASE(12) INFMOE_CASE(13)
        INFMOE_CASE(14) INFMOE_CASE(15) INFMOE_CASE(16)
        default: break;
    }
#undef INFMOE_CASE
}

// One expert: grid.x = column tiles, grid.y = row tiles of kGemmTileRows.
template <int BN, bool GATED>
__global__ __launch_bounds__(kThreads) void expert_gemm_kernel(GemmProblem p, int rows_total, int a_alloc_rows) {
    extern __shared__ __align__(16) float smem[];
    constexpr int kTile = GATED ? kGemmTileRowsGated : kGemmTileRows;
    const int row0 = blockIdx.y * kTile;
    const int rows = min(kTile, rows_total - row0);
    const int n0 = blockIdx.x * BN;
    gemm_dispatch<BN, GATED>((rows + 15) >> 4, p.A + (size_t)row0 * p.K, p.R ? p.R + (size_t)row0 * p.N : nullptr,
                             p.C + (size_t)row0 * p.N, rows, p.B, p.B1, n0, p.N, p.K, p.epilogue, smem,
                             a_alloc_rows);
}

// All experts: 1-D grid of 8 * (row-tile capacity of an XCD) * n_col_tiles workgroups.  Workgroup id
// b runs on XCD b % 8 and takes slot b / 8 of that XCD's share of the schedule: the share's row
// tiles in descending height, all column tiles of a row tile in a row (they share its activations).
template <int BN, bool GATED>
__global__ __launch_bounds__(kThreads) void expert_gemm_grouped_kernel(GemmProblem p, size_t weight_stride,
                                                                       const RowTile* __restrict__ tiles,
                                                                       const int* __restrict__ sched,
                                                                       int n_col_tiles) {
    extern __shared__ __align__(16) float smem[];
    const int xcd = blockIdx.x % kXcdCount, slot = blockIdx.x / kXcdCount;
    const int first = sched[1 + xcd], share = sched[2 + xcd] - first;
    if (slot >= share * n_col_tiles) return;
    const RowTile rt = tiles[first + slot / n_col_tiles];
    const int n0 = (slot % n_col_tiles) * BN;
    const float* B0 = p.B + (size_t)rt.expert * weight_stride;
    const float* B1 = GATED ? p.B1 + (size_t)rt.expert * weight_stride : nullptr;
    gemm_dispatch<BN, GATED>((rt.rows + 15) >> 4, p.A + (size_t)rt.row0 * p.K,
                             p.R ? p.R + (size_t)rt.row0 * p.N : nullptr, p.C + (size_t)rt.row0 * p.N, rt.rows, B0,
                             B1, n0, p.N, p.K, p.epilogue, smem, GATED ? kGemmTileRowsGated : kGemmTileRows);
}

// Shapes the matrix-core kernel does not take (K not a multiple of 4, or operands that are not
// 16-byte aligned): one thread per output element.  Only tiny debug shapes come here.
__global__ void expert_gemm_generic_kernel(GemmProblem p, int rows) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)rows * p.N) return;
    const int row = idx / p.N, col = idx % p.N;
    const float* a = p.A + (size_t)row * p.K;
    const float* b0 = p.B + (size_t)col * p.K;
    float s0 = 0.f, s1 = 0.f;
    for (int k = 0; k < p.K; ++k) s0 += a[k] * b0[k];
    if (p.epilogue == EPI_GATED_GELU) {
        const float* b1 = p.B1 + (size_t)col * p.K;
        for (int k = 0; k < p.K; ++k) s1 += a[k] * b1[k];
        s0 = gelu_dot(s0, s1);
    } else if (p.epilogue == EPI_RELU) {
        s0 = fmaxf(s0, 0.f);
    } else {
        s0 += p.R[idx];
    }
    p.C[idx] = s0;
}

template <int BN, bool GATED>
size_t lds_bytes(int a_alloc_rows) {
    return (2 * (size_t)a_alloc_rows * LDK + 2 * (size_t)(GATED ? 2 : 1) * BN * LDK) * sizeof(float);
}

template <typename Kern>
hipError_t allow_lds(Kern kern, size_t bytes) {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)bytes);
}

bool fast_path_ok(const GemmProblem& p) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B) |
                           reinterpret_cast<uintptr_t>(p.B1);
    return p.K % 4 == 0 && (bits & 15) == 0;
}

constexpr int kBN = 128;

}  // namespace

hipError_t launch_expert_gemm(const GemmProblem& p, int rows, hipStream_t stream) {
    if (rows <= 0) return hipSuccess;
    if (!fast_path_ok(p)) {
        const size_t n = (size_t)rows * p.N;
        expert_gemm_generic_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(p, rows);
        return hipGetLastError();
    }
    const int tile = gemm_tile_rows(p.epilogue);
    const int a_alloc = min(tile, ((rows + 15) / 16) * 16);
    const dim3 grid((p.N + kBN - 1) / kBN, (rows + tile - 1) / tile);
    hipError_t err;
    if (p.epilogue == EPI_GATED_GELU) {
        const size_t lds = lds_bytes<kBN, true>(a_alloc);
        if ((err = allow_lds(expert_gemm_kernel<kBN, true>, lds_bytes<kBN, true>(kGemmTileRowsGated))) != hipSuccess) return err;
        expert_gemm_kernel<kBN, true><<<grid, kThreads, lds, stream>>>(p, rows, a_alloc);
    } else {
        const size_t lds = lds_bytes<kBN, false>(a_alloc);
        if ((err = allow_lds(expert_gemm_kernel<kBN, false>, lds_bytes<kBN, false>(kGemmTileRows))) != hipSuccess) return err;
        expert_gemm_kernel<kBN, false><<<grid, kThreads, lds, stream>>>(p, rows, a_alloc);
    }
    return hipGetLastError();
}

hipError_t launch_expert_gemm_grouped(const GemmProblem& p, size_t weight_stride, const RowTile* tiles,
                                      const int* sched, int max_tiles, hipStream_t stream) {
    if (max_tiles <= 0) return hipSuccess;
    if (!fast_path_ok(p) || weight_stride % 4 != 0) return hipErrorInvalidValue;  // callers fall back per expert
    const int n_col_tiles = (p.N + kBN - 1) / kBN;
    const dim3 grid((unsigned)kXcdCount * (unsigned)xcd_tile_capacity(max_tiles) * (unsigned)n_col_tiles);
    hipError_t err;
    if (p.epilogue == EPI_GATED_GELU) {
        const size_t lds = lds_bytes<kBN, true>(kGemmTileRowsGated);
        if ((err = allow_lds(expert_gemm_grouped_kernel<kBN, true>, lds)) != hipSuccess) return err;
        expert_gemm_grouped_kernel<kBN, true><<<grid, kThreads, lds, stream>>>(p, weight_stride, tiles, sched, n_col_tiles);
    } else {
        const size_t lds = lds_bytes<kBN, false>(kGemmTileRows);
        if ((err = allow_lds(expert_gemm_grouped_kernel<kBN, false>, lds)) != hipSuccess) return err;
        expert_gemm_grouped_kernel<kBN, false><<<grid, kThreads, lds, stream>>>(p, weight_stride, tiles, sched, n_col_tiles);
    }
    return hipGetLastError();
}

}  // namespace infmoe
