// FP32 matrix-core GEMM of the T5 feed-forward expert for gfx950.
//
// Replaces the three cublasSgemm_v2 calls, the thrust gelu*mul pass and the device-to-device
// residual copy of T5FFLayer::run (plugin/sublayers/T5FFLayer.cc:112-138, plugin/cuda/ops/gelu.cu:7-25):
//     C[rows][N] = epilogue(A[rows][K] * B[N][K]^T)
// with both operands K-contiguous (activations row-major, weights in torch Linear layout), which
// is the "TN" form the FP32 matrix-core instructions want: a lane feeds one float of an A row and
// one float of a B row per instruction.  The work is done by v_mfma_f32_32x32x2_f32, which on this
// part sustains 99% of the 157 TFLOP/s peak from one wave per SIMD where v_mfma_f32_16x16x4_f32
// tops out at 79% (measured with register-only loops); the 16x16x4 form is kept for one 16-row
// block at the bottom of a tile so that row counts are padded to 16, not 32.
//
// Tiling.  The weights are the big operand (335 MB per expert at d=4096, h=10240) and each weight
// element is reused only `rows` times, so a workgroup covers ALL rows of its expert (up to 256) x
// BN weight rows: every weight byte is fetched from HBM once.  Token counts per expert vary, so the
// tile height is a run-time multiple of 16 rows (NMB of them: NMB/2 blocks of 32 rows plus one of
// 16 when NMB is odd); the body is instantiated for NMB = 1..16 and selected per workgroup, which
// wastes at most 15 padded rows per expert instead of up to a whole fixed-height tile.  The 4
// waves of a workgroup split the BN = 128 columns, 32 each, and keep the accumulators of all row
// blocks in registers.
//
// Pipeline.  K advances in steps of 32 floats.  While the matrix core works on step s from one half
// of a double-buffered LDS tile, the global loads of step s+2 go into registers and the registers
// holding step s+1 are written to the other half; one barrier per step.  These memory operations
// are not issued in bursts before and after the MFMAs (that left the matrix core idle a quarter of
// the time) but dealt out a few at a time between small groups of MFMAs.  LDS rows are padded to 36 floats so that the 16-byte
// operand reads of the lanes of a block hit distinct banks.  Inside an 8-float (32x32x2) or 16-float
// (16x16x4) chunk the k order is permuted identically for A and B (lane group q supplies floats
// 4q..4q+3 over four instructions), which a dot product does not see and which lets every operand
// read be a ds_read_b128.
//
// Grouped launch.  One launch covers every expert: row tiles come from the device-side table built
// by the dispatch scan, so no token count ever travels to the host.  Workgroup ids are dealt
// round-robin to the 8 XCDs by the hardware; the id -> tile map undoes that so each XCD works
// through a contiguous run of (expert, column tile) pairs and the activations of an expert stay
// in one XCD's L2.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <type_traits>

#include "kernels.h"

namespace infmoe {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kMaxMb64 = 10;      // tallest tile (in 16-row units) that takes 64-float K steps: 160 rows
constexpr int kThreads = 256;     // 4 waves

__device__ __forceinline__ float gelu_dot(float a, float b) {
    // plugin/cuda/ops/gelu.cu:8-15
    const float cdf = 0.5f * (1.0f + tanhf(a * (0.035677408136300125f * a * a + 0.7978845608028654f)));
    return a * cdf * b;
}

// f(integral_constant<int, I>) for I in [I0, N): an unrolled loop whose index is a constant expression
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// One output tile: `rows` (<= 16*NMB) rows of A against BN rows of B (and of B1 when GATED).
// BK: floats of K per pipeline step (32 or 64).
template <int NMB, int BN, bool GATED, int BK>
__device__ __forceinline__ void gemm_tile(const float* __restrict__ A, const float* __restrict__ R,
                                          float* __restrict__ C, int rows, const float* __restrict__ B0,
                                          const float* __restrict__ B1, int n0, int N, int K, int epilogue,
                                          float* __restrict__ smem, int a_alloc_rows) {
    static_assert(BN == 128, "each of the 4 waves owns one 32-column block");
    constexpr int NB = GATED ? 2 : 1;         // weight matrices
    constexpr int N32 = NMB / 2;              // 32-row blocks (v_mfma_f32_32x32x2_f32)
    constexpr bool T16 = (NMB & 1) != 0;      // one trailing 16-row block (v_mfma_f32_16x16x4_f32)
    constexpr int LDK = BK + 4;               // padded LDS row (floats)
    constexpr int KH = BK / 32;               // 32-float halves of a step's row
    constexpr int A_ROWS = NMB * 16;
    constexpr int A_LOADS = ((A_ROWS + 31) / 32) * KH;  // float4 per thread per step: KH per 32-row slab
    constexpr int B_LOADS = (BN / 32) * KH;
    constexpr int NV = A_LOADS + NB * B_LOADS;   // global loads (and LDS writes) per thread per step

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int i32 = lane & 31, kh = lane >> 5;  // 32x32x2: row / column fed, which float4 of 8 k
    const int i16 = lane & 15, kq = lane >> 4;  // 16x16x4: row / column fed, which float4 of 16 k
    const int ld_row = tid >> 3, ld_c4 = tid & 7;  // this thread's (row, float4) inside a 32-row slab

    float* As = smem;                                   // [2][a_alloc_rows][LDK]
    float* Bs = smem + 2 * (size_t)a_alloc_rows * LDK;  // [2][NB*BN][LDK]
    const size_t a_buf = (size_t)a_alloc_rows * LDK, b_buf = (size_t)NB * BN * LDK;

    v16f acc32[NB][N32 > 0 ? N32 : 1];
    v4f acc16[NB][2];
#pragma unroll
    for (int m = 0; m < NB; ++m) {
#pragma unroll
        for (int mb = 0; mb < (N32 > 0 ? N32 : 1); ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc32[m][mb][r] = 0.f;
        acc16[m][0] = v4f{0.f, 0.f, 0.f, 0.f};
        acc16[m][1] = v4f{0.f, 0.f, 0.f, 0.f};
    }

    // Global addresses are a wave-uniform base (kept in scalar registers and advanced along K) plus a
    // 32-bit per-thread byte offset, so a load needs no 64-bit vector arithmetic.  Rows past the end
    // are clamped: their products land in accumulator rows / columns that are never stored.
    const char* a_base = reinterpret_cast<const char*>(A);
    const char* b_base[NB];
    b_base[0] = reinterpret_cast<const char*>(B0 + (size_t)n0 * K);
    if (GATED) b_base[NB - 1] = reinterpret_cast<const char*>(B1 + (size_t)n0 * K);
    unsigned a_off[A_LOADS], b_off[B_LOADS];
#pragma unroll
    for (int p = 0; p < A_LOADS; ++p)  // item p: slab p / KH, half p % KH
        a_off[p] = ((unsigned)min((p / KH) * 32 + ld_row, rows - 1) * (unsigned)K + 32u * (p % KH) + 4u * ld_c4) * 4u;
#pragma unroll
    for (int p = 0; p < B_LOADS; ++p)
        b_off[p] = ((unsigned)min((p / KH) * 32 + ld_row, N - 1 - n0) * (unsigned)K + 32u * (p % KH) + 4u * ld_c4) * 4u;

    // Two register sets: global loads run two K steps ahead of the matrix core, which covers the
    // latency of an HBM miss (every weight load is one) with two steps of MFMA work.
    v4f ra[2][A_LOADS], rb[2][NB][B_LOADS];
    // item L of the global loads of the step starting at k0 (K % BK == 0 on this path), into set P
    auto gload = [&](auto setc, auto lc, int k0) {
        constexpr int P = decltype(setc)::value, L = decltype(lc)::value;
        if constexpr (L < A_LOADS) {
            ra[P][L] = *reinterpret_cast<const v4f*>(a_base + (size_t)k0 * 4 + a_off[L]);
        } else {
            constexpr int M = (L - A_LOADS) / B_LOADS, Q = (L - A_LOADS) % B_LOADS;
            rb[P][M][Q] = *reinterpret_cast<const v4f*>(b_base[M] + (size_t)k0 * 4 + b_off[Q]);
        }
    };
    // item L of register set P into LDS buffer BUF
    auto lstore = [&](auto setc, auto lc, auto bufc) {
        constexpr int P = decltype(setc)::value, L = decltype(lc)::value, BUF = decltype(bufc)::value;
        if constexpr (L < A_LOADS) {
            *reinterpret_cast<v4f*>(As + BUF * a_buf + ((L / KH) * 32 + ld_row) * LDK + 32 * (L % KH) + 4 * ld_c4) = ra[P][L];
        } else {
            constexpr int M = (L - A_LOADS) / B_LOADS, Q = (L - A_LOADS) % B_LOADS;
            *reinterpret_cast<v4f*>(Bs + BUF * b_buf + (M * BN + (Q / KH) * 32 + ld_row) * LDK + 32 * (Q % KH) + 4 * ld_c4) =
                rb[P][M][Q];
        }
    };

    // MFMA operands, double-buffered by k group so that the reads of group g+1 fly under the MFMAs of g
    v4f af32[2][N32 > 0 ? N32 : 1], bf32[2][NB];  // 32x32x2: 8-k groups
    v4f af16[2], bf16[2][NB][2];                  // 16x16x4: 16-k groups
    const float* a32 = As + i32 * LDK + 4 * kh;
    const float* b32 = Bs + (wave * 32 + i32) * LDK + 4 * kh;
    const float* a16 = As + (32 * N32 + i16) * LDK + 4 * kq;
    const float* b16 = Bs + (wave * 32 + i16) * LDK + 4 * kq;
    auto read32 = [&](auto bufc, auto gc, auto qc) {  // operand q of 8-k group g: q < NB weights, else row block q - NB
        constexpr int BUF = decltype(bufc)::value, G = decltype(gc)::value, Q = decltype(qc)::value;
        if constexpr (Q < NB)
            bf32[G & 1][Q] = *reinterpret_cast<const v4f*>(b32 + BUF * b_buf + Q * BN * LDK + 8 * G);
        else
            af32[G & 1][Q - NB] = *reinterpret_cast<const v4f*>(a32 + BUF * a_buf + 32 * (Q - NB) * LDK + 8 * G);
    };
    auto read16 = [&](auto bufc, auto gc, auto qc) {  // operand q of 16-k group g: 0 = rows, then weights (m, nb)
        constexpr int BUF = decltype(bufc)::value, G = decltype(gc)::value, Q = decltype(qc)::value;
        if constexpr (Q == 0)
            af16[G & 1] = *reinterpret_cast<const v4f*>(a16 + BUF * a_buf + 16 * G);
        else
            bf16[G & 1][(Q - 1) / 2][(Q - 1) % 2] = *reinterpret_cast<const v4f*>(
                b16 + BUF * b_buf + (((Q - 1) / 2) * BN + 16 * ((Q - 1) % 2)) * LDK + 16 * G);
    };

    // One K step = S slots.  A slot issues a few memory operations and then a handful of MFMAs,
    // and nothing may be moved across a slot boundary, so the matrix core is fed continuously:
    //   * the first half of the slots carries the global loads of step s + 2 (register set 1 - P),
    //   * the second half writes register set P (step s + 1) into LDS buffer 1 - P,
    //   * every slot group carries the LDS operand reads of the next k group.
    // The loop over steps is unrolled by two so that P, and with it every LDS address offset and
    // register index, is a compile-time constant.
    constexpr int G32 = BK / 8, G16 = BK / 16;  // k groups of a step
    constexpr int S32 = N32 > 0 ? 4 * G32 : 0, S16 = T16 ? 4 * G16 : 0, S = S32 + S16, SV = S / 2;
    constexpr int R32 = NB + N32, R16 = 1 + 2 * NB;
    const int nk = K / BK;
    auto step = [&](auto setc, int s) {
        constexpr int P = decltype(setc)::value;
        const std::integral_constant<int, P> cur{};
        const std::integral_constant<int, 1 - P> other{};
        const int kload = min(s + 2, nk - 1) * BK;  // the surplus loads of the last two steps are discarded
        if constexpr (N32 > 0)
            static_for<0, R32>([&](auto qc) { read32(cur, std::integral_constant<int, 0>{}, qc); });
        else
            static_for<0, R16>([&](auto qc) { read16(cur, std::integral_constant<int, 0>{}, qc); });
        static_for<0, S>([&](auto tc) {
            constexpr int t = decltype(tc)::value;
            if constexpr (t < SV)
                static_for<(t * NV) / SV, ((t + 1) * NV) / SV>([&](auto lc) { gload(other, lc, kload); });
            else
                static_for<((t - SV) * NV) / (S - SV), ((t - SV + 1) * NV) / (S - SV)>(
                    [&](auto lc) { lstore(cur, lc, other); });
            if constexpr (t < S32) {
                constexpr int g = t / 4, j = t % 4;
                if constexpr (g < G32 - 1 && j < 3)  // a third of the next group's operands per slot
                    static_for<0, R32>([&](auto qc) {
                        if constexpr (decltype(qc)::value % 3 == j) read32(cur, std::integral_constant<int, g + 1>{}, qc);
                    });
                if constexpr (g == G32 - 1 && j < 3 && T16)
                    static_for<0, R16>([&](auto qc) {
                        if constexpr (decltype(qc)::value % 3 == j) read16(cur, std::integral_constant<int, 0>{}, qc);
                    });
#pragma unroll
                for (int mb = 0; mb < N32; ++mb)
#pragma unroll
                    for (int m = 0; m < NB; ++m)
                        acc32[m][mb] = __builtin_amdgcn_mfma_f32_32x32x2f32(af32[g & 1][mb][j], bf32[g & 1][m][j],
                                                                             acc32[m][mb], 0, 0, 0);
            } else {
                constexpr int g = (t - S32) / 4, j = (t - S32) % 4;
                if constexpr (g < G16 - 1 && j < 3)
                    static_for<0, R16>([&](auto qc) {
                        if constexpr (decltype(qc)::value % 3 == j) read16(cur, std::integral_constant<int, g + 1>{}, qc);
                    });
#pragma unroll
                for (int m = 0; m < NB; ++m)
#pragma unroll
                    for (int nb = 0; nb < 2; ++nb)
                        acc16[m][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(af16[g & 1][j], bf16[g & 1][m][nb][j],
                                                                             acc16[m][nb], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        __syncthreads();
    };
    const std::integral_constant<int, 0> set0{};
    const std::integral_constant<int, 1> set1{};
    static_for<0, NV>([&](auto lc) { gload(set1, lc, 0); });
    static_for<0, NV>([&](auto lc) { lstore(set1, lc, set0); });
    static_for<0, NV>([&](auto lc) { gload(set0, lc, min(1, nk - 1) * BK); });
    __syncthreads();
    for (int s = 0; s < nk; s += 2) {
        step(set0, s);
        if (s + 1 < nk) step(set1, s + 1);
    }

    // epilogue
    auto emit = [&](int row, int col, float v, float v1) {
        if (row < rows && col < N) {
            const size_t o = (size_t)row * N + col;
            if (GATED) {
                v = gelu_dot(v, v1);
            } else if (epilogue == EPI_RELU) {
                v = fmaxf(v, 0.f);
            } else {
                v += R[o];
            }
            C[o] = v;
        }
    };
    // 32x32 block: register r holds row 8*(r/4) + 4*(lane/32) + r%4, column lane%32
#pragma unroll
    for (int mb = 0; mb < N32; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            emit(32 * mb + 8 * (r / 4) + 4 * kh + (r % 4), n0 + wave * 32 + i32, acc32[0][mb][r], acc32[NB - 1][mb][r]);
    // 16x16 block: register r holds row 4*(lane/16) + r, column lane%16
    if (T16) {
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                emit(32 * N32 + 4 * kq + r, n0 + wave * 32 + 16 * nb + i16, acc16[0][nb][r], acc16[NB - 1][nb][r]);
    }
}

template <int BN, bool GATED>
__device__ __forceinline__ void gemm_dispatch(int nmb, const float* A, const float* R, float* C, int rows,
                                              const float* B0, const float* B1, int n0, int N, int K, int epilogue,
                                              float* smem, int a_alloc_rows) {
    // the gated form keeps two accumulator sets, so its tiles are half as tall
    constexpr int kMaxMb = (GATED ? kGemmTileRowsGated : kGemmTileRows) / 16;
    // Tiles of up to 160 rows take K in steps of 64 floats (half as many barriers per flop); the LDS
    // cannot hold two such stages of a taller tile or of two weight matrices, which take steps of 32.
    const bool wide = !GATED && (K & 63) == 0;
#define INFMOE_CASE(n)                                                                                       \
    case n:                                                                                                  \
        if constexpr (n <= kMaxMb) {                                                                         \
            if constexpr (!GATED && n <= kMaxMb64) {                                                         \
                if (wide) {                                                                                  \
                    gemm_tile<n, BN, GATED, 64>(A, R, C, rows, B0, B1, n0, N, K, epilogue, smem,             \
                                                min(a_alloc_rows, 16 * kMaxMb64));                           \
                    break;                                                                                   \
                }                                                                                            \
            }                                                                                                \
            gemm_tile<n, BN, GATED, 32>(A, R, C, rows, B0, B1, n0, N, K, epilogue, smem, a_alloc_rows);      \
        }                                                                                                    \
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

// Shapes the matrix-core kernel does not take (K not a multiple of 32, or operands that are not
// 16-byte aligned): one thread per output element.  Only small or odd shapes come here.
// row_expert == nullptr: one expert; else row r uses the weights of expert row_expert[r].
__global__ void expert_gemm_generic_kernel(GemmProblem p, int rows, size_t weight_stride,
                                           const int* __restrict__ row_expert) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)rows * p.N) return;
    const int row = idx / p.N, col = idx % p.N;
    const size_t w0 = row_expert ? (size_t)row_expert[row] * weight_stride : 0;
    const float* a = p.A + (size_t)row * p.K;
    const float* b0 = p.B + w0 + (size_t)col * p.K;
    float s0 = 0.f, s1 = 0.f;
    for (int k = 0; k < p.K; ++k) s0 += a[k] * b0[k];
    if (p.epilogue == EPI_GATED_GELU) {
        const float* b1 = p.B1 + w0 + (size_t)col * p.K;
        for (int k = 0; k < p.K; ++k) s1 += a[k] * b1[k];
        s0 = gelu_dot(s0, s1);
    } else if (p.epilogue == EPI_RELU) {
        s0 = fmaxf(s0, 0.f);
    } else {
        s0 += p.R[idx];
    }
    p.C[idx] = s0;
}

// LDS the kernel may touch for tiles of up to a_alloc_rows rows: the larger of the two step widths.
template <int BN, bool GATED>
size_t lds_bytes(int a_alloc_rows, int K) {
    const size_t nb = GATED ? 2 : 1;
    size_t bytes = (2 * (size_t)a_alloc_rows * 36 + 2 * nb * BN * 36) * sizeof(float);
    if (!GATED && K % 64 == 0) {
        const size_t rows64 = (size_t)std::min(a_alloc_rows, 16 * kMaxMb64);
        bytes = std::max(bytes, (2 * rows64 * 68 + 2 * nb * BN * 68) * sizeof(float));
    }
    return bytes;
}

bool fast_path_ok(const GemmProblem& p) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B) |
                           reinterpret_cast<uintptr_t>(p.B1);
    return p.K % 32 == 0 && (bits & 15) == 0;
}

}  // namespace

bool expert_gemm_grouped_ok(const GemmProblem& p, size_t weight_stride) {
    return fast_path_ok(p) && weight_stride % 4 == 0;
}

hipError_t launch_expert_gemm_any_shape_grouped(const GemmProblem& p, size_t weight_stride, const int* row_expert,
                                                int rows, hipStream_t stream) {
    if (rows <= 0) return hipSuccess;
    const size_t n = (size_t)rows * p.N;
    expert_gemm_generic_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(p, rows, weight_stride, row_expert);
    return hipGetLastError();
}

namespace {

constexpr int kBN = 128;
constexpr size_t kLdsPerCu = 160 * 1024;  // the limit is raised once, to all there is; launches ask for what they use

}  // namespace

hipError_t launch_expert_gemm(const GemmProblem& p, int rows, hipStream_t stream) {
    if (rows <= 0) return hipSuccess;
    if (!fast_path_ok(p)) {
        const size_t n = (size_t)rows * p.N;
        expert_gemm_generic_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(p, rows, 0, nullptr);
        return hipGetLastError();
    }
    const int tile = gemm_tile_rows(p.epilogue);
    const int a_alloc = min(tile, ((rows + 31) / 32) * 32);  // whole 32-row slabs
    const dim3 grid((p.N + kBN - 1) / kBN, (rows + tile - 1) / tile);
    hipError_t err;
    if (p.epilogue == EPI_GATED_GELU) {
        const size_t lds = lds_bytes<kBN, true>(a_alloc, p.K);
        if ((err = allow_lds_once<expert_gemm_kernel<kBN, true>>(kLdsPerCu)) != hipSuccess) return err;
        expert_gemm_kernel<kBN, true><<<grid, kThreads, lds, stream>>>(p, rows, a_alloc);
    } else {
        const size_t lds = lds_bytes<kBN, false>(a_alloc, p.K);
        if ((err = allow_lds_once<expert_gemm_kernel<kBN, false>>(kLdsPerCu)) != hipSuccess) return err;
        expert_gemm_kernel<kBN, false><<<grid, kThreads, lds, stream>>>(p, rows, a_alloc);
    }
    return hipGetLastError();
}

hipError_t launch_expert_gemm_grouped(const GemmProblem& p, size_t weight_stride, const RowTile* tiles,
                                      const int* sched, int max_tiles, hipStream_t stream) {
    if (max_tiles <= 0) return hipSuccess;
    if (!expert_gemm_grouped_ok(p, weight_stride)) return hipErrorInvalidValue;  // see launch_expert_gemm_any_shape_grouped
    const int n_col_tiles = (p.N + kBN - 1) / kBN;
    const dim3 grid((unsigned)kXcdCount * (unsigned)xcd_tile_capacity(max_tiles) * (unsigned)n_col_tiles);
    hipError_t err;
    if (p.epilogue == EPI_GATED_GELU) {
        const size_t lds = lds_bytes<kBN, true>(kGemmTileRowsGated, p.K);
        if ((err = allow_lds_once<expert_gemm_grouped_kernel<kBN, true>>(kLdsPerCu)) != hipSuccess) return err;
        expert_gemm_grouped_kernel<kBN, true><<<grid, kThreads, lds, stream>>>(p, weight_stride, tiles, sched, n_col_tiles);
    } else {
        const size_t lds = lds_bytes<kBN, false>(kGemmTileRows, p.K);
        if ((err = allow_lds_once<expert_gemm_grouped_kernel<kBN, false>>(kLdsPerCu)) != hipSuccess) return err;
        expert_gemm_grouped_kernel<kBN, false><<<grid, kThreads, lds, stream>>>(p, weight_stride, tiles, sched, n_col_tiles);
    }
    return hipGetLastError();
}

}  // namespace infmoe
