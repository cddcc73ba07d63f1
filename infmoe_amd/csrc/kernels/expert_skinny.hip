// Few-row expert GEMM for gfx950 (decode shapes: one to eight tokens per expert).
//
// Same contract as the matrix-core kernel (C = epilogue(A * B^T), replacing the cublasSgemm_v2
// calls of plugin/sublayers/T5FFLayer.cc:112-138), but with so few activation rows the work is a
// stream of the expert's weights through the chip: 2*d*h*4 bytes per expert, each byte used once
// per row.  The kernel is therefore built around bytes in flight, not around the matrix core:
//   * a workgroup owns 32 weight rows (8 per wave) and walks K in chunks of 2048 floats;
//   * the activation chunk (M x 2048 floats) is staged in LDS once per chunk and shared by all
//     32 weight rows, so activations cost L2/LDS bandwidth only;
//   * every lane keeps 16 independent 16-byte weight loads in flight (two weight rows x eight
//     1-KB wave-wide segments), and several workgroups are resident per CU;
//   * partial dot products stay in registers across chunks and are reduced across the wave once.
// Experts outside 1..kSkinnyMaxRows rows are skipped, so the grouped launch can run next to the
// matrix-core launch: each expert is processed by exactly one of the two.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace infmoe {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int KC = 2048;            // K floats per staged chunk
constexpr int KC4 = KC / 4;
constexpr int RW = 8;               // weight rows per wave
constexpr int kRowsPerWg = RW * (kThreads / 64);
constexpr int kSeg = KC / 256;      // 16-byte loads per lane per weight row per chunk

__device__ __forceinline__ float gelu_dot(float a, float b) {
    // plugin/cuda/ops/gelu.cu:8-15
    const float cdf = 0.5f * (1.0f + tanhf(a * (0.035677408136300125f * a * a + 0.7978845608028654f)));
    return a * cdf * b;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

template <int M, bool GATED>
__device__ __forceinline__ void skinny_body(const float* __restrict__ A, const float* __restrict__ R,
                                            float* __restrict__ C, int rows, const float* __restrict__ B0,
                                            const float* __restrict__ B1, int N, int K, int epilogue,
                                            float* __restrict__ smem) {
    constexpr int NB = GATED ? 2 : 1;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_base = blockIdx.x * kRowsPerWg + wave * RW;
    v4f* As4 = reinterpret_cast<v4f*>(smem);  // [M][KC4]

    float acc[NB][RW][M];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < RW; ++r)
#pragma unroll
            for (int m = 0; m < M; ++m) acc[b][r][m] = 0.f;

    for (int kc0 = 0; kc0 < K; kc0 += KC) {
        __syncthreads();  // everyone is done with the previous chunk
        for (int idx = tid; idx < M * KC4; idx += kThreads) {
            const int m = idx / KC4, c = idx - m * KC4;
            const int k = kc0 + 4 * c;
            v4f v = {0.f, 0.f, 0.f, 0.f};
            if (k < K) v = *reinterpret_cast<const v4f*>(A + (size_t)min(m, rows - 1) * K + k);
            As4[idx] = v;
        }
        __syncthreads();

#pragma unroll
        for (int rp = 0; rp < RW; rp += 2) {
            v4f w[NB][2][kSeg];
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const size_t roff = (size_t)min(n_base + rp + q, N - 1) * K;
#pragma unroll
                for (int j = 0; j < kSeg; ++j) {
                    const int k = kc0 + 4 * (lane + 64 * j);
                    w[0][q][j] = v4f{0.f, 0.f, 0.f, 0.f};
                    if (GATED) w[NB - 1][q][j] = v4f{0.f, 0.f, 0.f, 0.f};
                    if (k < K) {
                        w[0][q][j] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(B0 + roff + k));
                        if (GATED) w[NB - 1][q][j] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(B1 + roff + k));
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < kSeg; ++j) {
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    const v4f a = As4[m * KC4 + lane + 64 * j];
#pragma unroll
                    for (int b = 0; b < NB; ++b)
#pragma unroll
                        for (int q = 0; q < 2; ++q) {
                            const v4f x = w[b][q][j];
                            acc[b][rp + q][m] += (x.x * a.x + x.y * a.y) + (x.z * a.z + x.w * a.w);
                        }
                }
            }
        }
    }

#pragma unroll
    for (int r = 0; r < RW; ++r) {
        const int n = n_base + r;
#pragma unroll
        for (int m = 0; m < M; ++m) {
            float v = wave_sum(acc[0][r][m]);
            float v1 = 0.f;
            if (GATED) v1 = wave_sum(acc[NB - 1][r][m]);
            if (lane == 0 && n < N && m < rows) {
                const size_t o = (size_t)m * N + n;
                if (GATED)
                    v = gelu_dot(v, v1);
                else if (epilogue == EPI_RELU)
                    v = fmaxf(v, 0.f);
                else
                    v += R[o];
                C[o] = v;
            }
        }
    }
}

// count == nullptr: one expert with `rows_fixed` rows at row 0; else blockIdx.y is the expert.
template <bool GATED>
__global__ __launch_bounds__(kThreads) void expert_skinny_kernel(GemmProblem p, size_t weight_stride,
                                                                 const int* __restrict__ count,
                                                                 const int* __restrict__ offset, int rows_fixed) {
    extern __shared__ __align__(16) float smem[];
    int rows = rows_fixed, row0 = 0;
    const float* B0 = p.B;
    const float* B1 = p.B1;
    if (count != nullptr) {
        const int e = blockIdx.y;
        rows = count[e];
        row0 = offset[e];
        B0 += (size_t)e * weight_stride;
        if (GATED) B1 += (size_t)e * weight_stride;
    }
    if (rows <= 0 || rows > kSkinnyMaxRows) return;
    const float* A = p.A + (size_t)row0 * p.K;
    const float* R = p.R ? p.R + (size_t)row0 * p.N : nullptr;
    float* C = p.C + (size_t)row0 * p.N;
    if (rows == 1)
        skinny_body<1, GATED>(A, R, C, rows, B0, B1, p.N, p.K, p.epilogue, smem);
    else if (rows == 2)
        skinny_body<2, GATED>(A, R, C, rows, B0, B1, p.N, p.K, p.epilogue, smem);
    else if (rows <= 4)
        skinny_body<4, GATED>(A, R, C, rows, B0, B1, p.N, p.K, p.epilogue, smem);
    else
        skinny_body<8, GATED>(A, R, C, rows, B0, B1, p.N, p.K, p.epilogue, smem);
}

inline size_t lds_for_rows(int rows) {
    const int m = rows <= 1 ? 1 : rows <= 2 ? 2 : rows <= 4 ? 4 : 8;
    return (size_t)m * KC * sizeof(float);
}

bool fast_path_ok(const GemmProblem& p) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B) |
                           reinterpret_cast<uintptr_t>(p.B1);
    return p.K % 4 == 0 && (bits & 15) == 0;
}

}  // namespace

hipError_t launch_expert_skinny(const GemmProblem& p, int rows, hipStream_t stream) {
    if (rows <= 0) return hipSuccess;
    if (rows > kSkinnyMaxRows || !fast_path_ok(p)) return hipErrorInvalidValue;
    const dim3 grid((p.N + kRowsPerWg - 1) / kRowsPerWg, 1);
    const size_t lds = lds_for_rows(rows);
    if (p.epilogue == EPI_GATED_GELU)
        expert_skinny_kernel<true><<<grid, kThreads, lds, stream>>>(p, 0, nullptr, nullptr, rows);
    else
        expert_skinny_kernel<false><<<grid, kThreads, lds, stream>>>(p, 0, nullptr, nullptr, rows);
    return hipGetLastError();
}

hipError_t launch_expert_skinny_grouped(const GemmProblem& p, size_t weight_stride, const int* count,
                                        const int* offset, int E, hipStream_t stream) {
    if (E <= 0) return hipSuccess;
    if (!fast_path_ok(p) || weight_stride % 4 != 0) return hipErrorInvalidValue;
    const dim3 grid((p.N + kRowsPerWg - 1) / kRowsPerWg, E);
    const size_t lds = lds_for_rows(kSkinnyMaxRows);
    if (p.epilogue == EPI_GATED_GELU)
        expert_skinny_kernel<true><<<grid, kThreads, lds, stream>>>(p, weight_stride, count, offset, 0);
    else
        expert_skinny_kernel<false><<<grid, kThreads, lds, stream>>>(p, weight_stride, count, offset, 0);
    return hipGetLastError();
}

}  // namespace infmoe
