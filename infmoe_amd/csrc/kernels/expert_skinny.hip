// Few-row expert GEMM for gfx950 (decode shapes: one to eight tokens per expert).
//
// Same contract as the matrix-core kernel (C = epilogue(A * B^T), replacing the cublasSgemm_v2
// calls of plugin/sublayers/T5FFLayer.cc:112-138), but with so few activation rows the work is a
// stream of the expert's weights through the chip: 2*d*h*4 bytes per expert, each byte used once
// per row.  The kernel is therefore built around bytes in flight, not around the matrix core:
//   * a wave owns 8 weight rows and walks K in chunks; no LDS and no barrier, so waves never wait
//     for each other and occupancy is bounded by registers only;
//   * the activation chunk (M rows) lives in registers, loaded once per chunk from L2 and reused
//     for the wave's 8 weight rows;
//   * every lane keeps 8-16 independent 16-byte weight loads in flight (whole 1-KB wave-wide
//     segments of 2-8 weight rows), marked non-temporal: each weight byte is used once, and the
//     register budget is capped so that three waves share a SIMD (12 waves x 16 KB per CU);
//   * partial dot products stay in registers across chunks and are reduced across the wave once.
//   * a wave takes 1, 2 or 4 such 8-row blocks in turn so that it streams about 256 KB: starting a
//     wave costs a few microseconds in which it has nothing in flight (K = 4096: 6.1 TB/s with one
//     block per wave, 6.6 TB/s with two).
// The chunk length shrinks as M grows (2048, 2048, 512, 256 floats for M = 1, 2, 4, 8) so that
// activations + loads in flight + accumulators stay within 168 registers.
// An expert with more than kSkinnyMaxRows rows is done in runs of kSkinnyMaxRows rows (the last run takes what is
// left), each a pass over the expert's weights: in a decode call (at most two tokens per expert) such an expert is
// rare and its rows are rows that other experts did not get, so the passes cost no more than the experts they
// replace, and the call needs no launch of the matrix-core kernel whose grid would have to be sized for it.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "device_math.h"
#include "kernels.h"

namespace infmoe {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int RW = 8;               // weight rows per wave
constexpr int kWaves = kThreads / 64;

// v + (v of the lane that the data-parallel-primitive control CTRL names): a register-to-register move
// inside a row of 16 lanes, no trip through the LDS crossbar as a shuffle by lane index takes
template <int CTRL>
__device__ __forceinline__ float add_dpp(float v) {
    return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
// Sum over the wave, the same value in every lane: four steps inside the rows of 16 lanes (lane ^ 1,
// lane ^ 2, mirror in 8, mirror in 16), then the four row sums read as scalars.
__device__ __forceinline__ float wave_sum(float v) {
    v = add_dpp<0xB1>(v);   // quad_perm [1, 0, 3, 2]
    v = add_dpp<0x4E>(v);   // quad_perm [2, 3, 0, 1]
    v = add_dpp<0x141>(v);  // row_half_mirror
    v = add_dpp<0x140>(v);  // row_mirror
    const int bits = __float_as_int(v);
    const float s0 = __int_as_float(__builtin_amdgcn_readlane(bits, 0)), s1 = __int_as_float(__builtin_amdgcn_readlane(bits, 16));
    const float s2 = __int_as_float(__builtin_amdgcn_readlane(bits, 32)), s3 = __int_as_float(__builtin_amdgcn_readlane(bits, 48));
    return (s0 + s1) + (s2 + s3);
}

// SEG: 16-byte loads per lane per weight row per chunk; RPN: weight rows loaded together
// EPI: as in the matrix-core kernel - EPI_RESIDUAL adds R to the product; EPI_RELU and EPI_GATED_GELU carry the
// block's RMS row norm with them when `stats` is given: the weights then have gamma multiplied in, and a sum
// becomes rstd_row * sum before the activation (stats: [row][2], of which [1] = rstd_row is used).
template <int M, int SEG, int RPN, int EPI>
__device__ __forceinline__ void skinny_body(const float* __restrict__ A, const float* __restrict__ R,
                                            float* __restrict__ C, int rows, const float* __restrict__ B0,
                                            const float* __restrict__ B1, int N, int K,
                                            const float* __restrict__ stats, int row_blocks) {
    constexpr bool GATED = EPI == EPI_GATED_GELU;
    constexpr bool NORM = EPI != EPI_RESIDUAL;
    constexpr int NB = GATED ? 2 : 1;
    constexpr int KC = SEG * 256;                   // k floats per chunk
    constexpr int RP = RPN / NB > 0 ? RPN / NB : 1;
    static_assert(RW % RP == 0, "bad chunking");
    // the wave index is uniform: as a scalar it lets every row base live in SGPRs, so a load needs
    // only the lane's 32-bit offset instead of a 64-bit address per (row, segment)
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    float rstd[M];
#pragma unroll
    for (int m = 0; m < M; ++m) rstd[m] = NORM && stats != nullptr ? stats[2 * min(m, rows - 1) + 1] : 1.f;
#pragma unroll 1
    for (int rb = 0; rb < row_blocks; ++rb) {
    const int n_base = ((blockIdx.x * kWaves + wave) * row_blocks + rb) * RW;
    if (n_base >= N) return;  // no barriers in this kernel: a wave may leave early

    float acc[NB][RW][M];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < RW; ++r)
#pragma unroll
            for (int m = 0; m < M; ++m) acc[b][r][m] = 0.f;

    // Whole chunks of K: every load is unconditional and issued back to back.
    auto chunk = [&](int kc0) {
        v4f a[M][SEG];
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const v4f* pa = reinterpret_cast<const v4f*>(A + (size_t)min(m, rows - 1) * K + kc0) + lane;
#pragma unroll
            for (int j = 0; j < SEG; ++j) a[m][j] = pa[64 * j];
        }
#pragma unroll
        for (int rp = 0; rp < RW; rp += RP) {
            v4f w[NB][RP][SEG];
#pragma unroll
            for (int q = 0; q < RP; ++q) {
                const size_t roff = (size_t)min(n_base + rp + q, N - 1) * K + kc0;
                const v4f* pb0 = reinterpret_cast<const v4f*>(B0 + roff) + lane;
                const v4f* pb1 = GATED ? reinterpret_cast<const v4f*>(B1 + roff) + lane : nullptr;
#pragma unroll
                for (int j = 0; j < SEG; ++j) {
                    w[0][q][j] = __builtin_nontemporal_load(pb0 + 64 * j);
                    if (GATED) w[NB - 1][q][j] = __builtin_nontemporal_load(pb1 + 64 * j);
                }
            }
#pragma unroll
            for (int q = 0; q < RP; ++q)
#pragma unroll
                for (int j = 0; j < SEG; ++j)
#pragma unroll
                    for (int b = 0; b < NB; ++b) {
                        const v4f x = w[b][q][j];
#pragma unroll
                        for (int m = 0; m < M; ++m)
                            acc[b][rp + q][m] += (x.x * a[m][j].x + x.y * a[m][j].y) + (x.z * a[m][j].z + x.w * a[m][j].w);
                    }
            // keep the next group's loads behind this group's arithmetic: hoisting them all to the
            // top of the chunk would need four times the registers and cost occupancy
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    int kc0 = 0;
    for (; kc0 + KC <= K; kc0 += KC) chunk(kc0);
    // what is left of an odd K (K % 4 == 0): one float4 per lane and step, kept deliberately small
#pragma unroll 1
    for (int k = kc0 + 4 * lane; k < K; k += 256) {
        v4f a[M];
#pragma unroll
        for (int m = 0; m < M; ++m) a[m] = *reinterpret_cast<const v4f*>(A + (size_t)min(m, rows - 1) * K + k);
#pragma unroll
        for (int r = 0; r < RW; ++r) {
            const size_t roff = (size_t)min(n_base + r, N - 1) * K + k;
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const v4f x = *reinterpret_cast<const v4f*>((b == 0 ? B0 : B1) + roff);
#pragma unroll
                for (int m = 0; m < M; ++m)
                    acc[b][r][m] += (x.x * a[m].x + x.y * a[m].y) + (x.z * a[m].z + x.w * a[m].w);
            }
        }
    }

    // Lane m * RW + r stores output (row m, column n_base + r) and fetches its residual value before
    // the reductions start (from a clamped, always valid address): loaded next to its store, each of
    // the RW * M values would be waited for by itself.
    static_assert(RW * M <= 64, "one lane per output");
    constexpr bool residual = EPI == EPI_RESIDUAL;
    const int my_m = lane / RW, my_n = n_base + lane % RW;
    float res = 0.f;
    if (residual) res = R[(size_t)min(my_m, rows - 1) * N + min(my_n, N - 1)];
#pragma unroll
    for (int r = 0; r < RW; ++r) {
#pragma unroll
        for (int m = 0; m < M; ++m) {
            float v = wave_sum(acc[0][r][m]);
            if (NORM) v *= rstd[m];
            if (GATED)
                v = gelu_dot(v, rstd[m] * wave_sum(acc[NB - 1][r][m]));
            else if (residual)
                v += res;
            else
                v = fmaxf(v, 0.f);
            if (lane == m * RW + r && my_n < N && m < rows) C[(size_t)m * N + my_n] = v;
        }
    }
    }  // row blocks
}

// count == nullptr: one expert with `rows_fixed` rows at row 0; else blockIdx.y is the expert.
template <int EPI>
__global__ __launch_bounds__(kThreads, EPI == EPI_GATED_GELU ? 2 : 3) void expert_skinny_kernel(GemmProblem p, size_t weight_stride,
                                                                 const int* __restrict__ count,
                                                                 const int* __restrict__ offset, int rows_fixed,
                                                                 int row_blocks) {
    constexpr bool GATED = EPI == EPI_GATED_GELU;
    int rows = rows_fixed, row0 = 0;
    const float* B0 = p.B;
    const float* B1 = p.B1;
    if (count != nullptr) {
        const int e = blockIdx.y;
        rows = count[e];
        row0 = offset[e];
        const int owner = p.expert_slot ? p.expert_slot[e] : e;
        B0 += (size_t)owner * weight_stride;
        if (GATED) B1 += (size_t)owner * weight_stride;
    }
    if (rows <= 0) return;
    // The last run of up to kSkinnyMaxRows rows - for nearly every expert of a decode call the only one - is
    // straight-line code; the full runs of a taller expert go before it in a loop of the 8-row body.  (One loop
    // over all runs around the switch cost the second product's kernel four spilled registers.)
    const int last = ((rows - 1) / kSkinnyMaxRows) * kSkinnyMaxRows;  // first row of the last run
#pragma unroll 1
    for (int r0 = 0; r0 < last; r0 += kSkinnyMaxRows) {  // (a body returns when its wave has no weight rows left)
        const int at = row0 + r0;
        skinny_body<8, 1, 8, EPI>(p.A + (size_t)at * p.K, p.R ? p.R + (size_t)at * p.N : nullptr, p.C + (size_t)at * p.N, 8,
                                  B0, B1, p.N, p.K,
                                  EPI != EPI_RESIDUAL && p.row_stats != nullptr ? p.row_stats + 2 * (size_t)at : nullptr,
                                  row_blocks);
    }
    row0 += last;
    rows -= last;
    const float* A = p.A + (size_t)row0 * p.K;
    const float* R = p.R ? p.R + (size_t)row0 * p.N : nullptr;
    float* C = p.C + (size_t)row0 * p.N;
    const float* stats = EPI != EPI_RESIDUAL && p.row_stats != nullptr ? p.row_stats + 2 * (size_t)row0 : nullptr;
    // One body per row count: a row more than needed would cost its loads of the activation chunk
    // again for every block of weight rows (with 5 rows in the 8-row body, 60 % more of them).
    switch (rows) {
        case 1: skinny_body<1, 8, 2, EPI>(A, R, C, rows, B0, B1, p.N, p.K, stats, row_blocks); break;
        case 2: skinny_body<2, 8, 2, EPI>(A, R, C, rows, B0, B1, p.N, p.K, stats, row_blocks); break;
        case 3: skinny_body<3, 2, 8, EPI>(A, R, C, rows, B0, B1, p.N, p.K, stats, row_blocks); break;
        case 4: skinny_body<4, 2, 8, EPI>(A, R, C, rows, B0, B1, p.N, p.K, stats, row_blocks); break;
        case 5: skinny_body<5, 1, 8, EPI>(A, R, C, rows, B0, B1, p.N, p.K, stats, row_blocks); break;
        case 6: skinny_body<6, 1, 8, EPI>(A, R, C, rows, B0, B1, p.N, p.K, stats, row_blocks); break;
        case 7: skinny_body<7, 1, 8, EPI>(A, R, C, rows, B0, B1, p.N, p.K, stats, row_blocks); break;
        default: skinny_body<8, 1, 8, EPI>(A, R, C, rows, B0, B1, p.N, p.K, stats, row_blocks); break;
    }
}

bool fast_path_ok(const GemmProblem& p) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B) |
                           reinterpret_cast<uintptr_t>(p.B1);
    if (p.epilogue == EPI_RESIDUAL && p.R == nullptr) return false;
    return p.K % 4 == 0 && (bits & 15) == 0;
}

// 8-row blocks per wave: about 256 KB of weights
int row_blocks_for(int K) {
    const size_t block_bytes = (size_t)RW * K * sizeof(float);
    return block_bytes <= 80 * 1024 ? 4 : (block_bytes <= 200 * 1024 ? 2 : 1);
}

}  // namespace

hipError_t launch_expert_skinny(const GemmProblem& p, int rows, hipStream_t stream) {
    if (rows <= 0) return hipSuccess;
    if (!fast_path_ok(p)) return hipErrorInvalidValue;
    const int rb = row_blocks_for(p.K), rows_per_wg = RW * kWaves * rb;
    const dim3 grid((p.N + rows_per_wg - 1) / rows_per_wg, 1);
    if (p.epilogue == EPI_GATED_GELU)
        expert_skinny_kernel<EPI_GATED_GELU><<<grid, kThreads, 0, stream>>>(p, 0, nullptr, nullptr, rows, rb);
    else if (p.epilogue == EPI_RELU)
        expert_skinny_kernel<EPI_RELU><<<grid, kThreads, 0, stream>>>(p, 0, nullptr, nullptr, rows, rb);
    else
        expert_skinny_kernel<EPI_RESIDUAL><<<grid, kThreads, 0, stream>>>(p, 0, nullptr, nullptr, rows, rb);
    return hipGetLastError();
}

hipError_t launch_expert_skinny_grouped(const GemmProblem& p, size_t weight_stride, const int* count,
                                        const int* offset, int E, hipStream_t stream) {
    if (E <= 0) return hipSuccess;
    if (!fast_path_ok(p) || weight_stride % 4 != 0) return hipErrorInvalidValue;
    const int rb = row_blocks_for(p.K), rows_per_wg = RW * kWaves * rb;
    const dim3 grid((p.N + rows_per_wg - 1) / rows_per_wg, E);
    if (p.epilogue == EPI_GATED_GELU)
        expert_skinny_kernel<EPI_GATED_GELU><<<grid, kThreads, 0, stream>>>(p, weight_stride, count, offset, 0, rb);
    else if (p.epilogue == EPI_RELU)
        expert_skinny_kernel<EPI_RELU><<<grid, kThreads, 0, stream>>>(p, weight_stride, count, offset, 0, rb);
    else
        expert_skinny_kernel<EPI_RESIDUAL><<<grid, kThreads, 0, stream>>>(p, weight_stride, count, offset, 0, rb);
    return hipGetLastError();
}

}  // namespace infmoe
