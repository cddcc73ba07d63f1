// FP32 matrix-core GEMM of the T5 feed-forward expert for gfx950: device code.
// Included by the translation units that instantiate one kernel each (the tile body exists in some
// sixty shapes per one-matrix kernel, so they compile side by side).
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
// element is reused only `rows` times, so a workgroup covers ALL rows of its expert (up to 256, or
// 192 with two weight matrices; a taller expert is cut into equal tiles, see row_tile_height) x BN
// weight rows: every weight byte is fetched from HBM once.  Token counts per expert vary, so the
// tile height is a run-time multiple of 16 rows (NMB of them: NMB/2 blocks of 32 rows plus one of
// 16 when NMB is odd) plus up to two groups of 4 rows; the body is instantiated for NMB = 1..16 and
// selected per workgroup, which wastes at most 3 padded rows per expert (15 where the groups are
// not used) instead of up to a whole fixed-height tile.  The 4 waves of a workgroup split the
// BN = 128 columns, 32 each, and keep the accumulators of all row blocks in registers.
//
// Pipeline.  K advances in steps of BK = 32 or 64 floats.  While the matrix core works on step s from one half
// of a double-buffered LDS tile, the global loads of step s+2 go into registers and the registers
// holding step s+1 are written to the other half; one barrier per step.  These memory operations
// are not issued in bursts before and after the MFMAs (that left the matrix core idle a quarter of
// the time) but dealt out a few at a time between small groups of MFMAs.  LDS rows are padded to
// BK + 4 floats so that the 16-byte operand reads of the lanes of a block hit distinct banks.  Inside an 8-float (32x32x2) or 16-float
// (16x16x4) chunk the k order is permuted identically for A and B (lane group q supplies floats
// 4q..4q+3 over four instructions), which a dot product does not see and which lets every operand
// read be a ds_read_b128.
//
// Grouped launch.  One launch covers every expert: row tiles come from the device-side table built
// by the dispatch scan, so no token count ever travels to the host.  Workgroup ids are dealt
// round-robin to the 8 XCDs by the hardware; the id -> tile map undoes that so each XCD works
// through a contiguous run of (expert, column tile) pairs and the activations of an expert stay
// in one XCD's L2.
#pragma once

#include <hip/hip_runtime.h>

#include <algorithm>
#include <type_traits>

#include "device_math.h"
#include "expert_gemm_parts.h"
#include "kernels.h"

namespace infmoe {
namespace {


typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kMaxMb64 = kGemmMaxUnits64;
constexpr int kThreads = kGemmThreads;

// f(integral_constant<int, I>) for I in [I0, N): an unrolled loop whose index is a constant expression
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// One output tile: `rows` (<= 16*NMB + 4*G4) rows of A against BN rows of B (and of B1 when GATED).
// BK: floats of K per pipeline step (32 or 64).
// G4: groups of 4 rows below the 16-row units, on v_mfma_f32_4x4x1_16b_f32 (16 blocks of 4x4 per
// instruction: 8 blocks cover the wave's 32 columns, the two halves of the wave take the two float4 of
// an 8-k group and their sums meet in the epilogue).  The instruction takes the B operand exactly as
// the 32x32x2 form holds it (lane -> column lane % 32, float4 lane / 32), so a group costs one more
// LDS read per k group and four short instructions: rows are padded to 4, not to 16.
// EPI: the epilogue.  EPI_RESIDUAL adds R to the product.  EPI_RELU / EPI_GATED_GELU can carry the RMS row
// norm of the T5 feed-forward block (README.md:115, plugin/sublayers/T5FFLayer.cc:98-103) with them: when
// `stats` is given, A holds the raw rows, B holds weights whose columns were multiplied by the norm's gamma
// beforehand, and the product becomes rstd_r * acc before the activation, which is the product of the
// normed rows with the plain weights (stats: [row][2], of which [1] = rstd_r is used).  The inner loop does
// not know of any of it.
// D: register sets of the global loads, i.e. how many K steps they run ahead of the matrix core (2 or 4).
template <int NMB, int G4, int BN, int EPI, int BK, int D, bool STREAM_B = false>
__device__ __forceinline__ void gemm_tile(const float* __restrict__ A, const float* __restrict__ R,
                                          float* __restrict__ C, int rows, const float* __restrict__ B0,
                                          const float* __restrict__ B1, int n0, int N, int K,
                                          const float* __restrict__ stats, float* __restrict__ smem,
                                          int a_alloc_rows) {
    static_assert(BN == 128, "each of the 4 waves owns one 32-column block");
    constexpr bool GATED = EPI == EPI_GATED_GELU;
    constexpr bool NORM = EPI != EPI_RESIDUAL;
    constexpr int NB = GATED ? 2 : 1;         // weight matrices
    constexpr int N32 = NMB / 2;              // 32-row blocks (v_mfma_f32_32x32x2_f32)
    constexpr bool T16 = (NMB & 1) != 0;      // one trailing 16-row block (v_mfma_f32_16x16x4_f32)
    constexpr int LDK = BK + 4;               // padded LDS row (floats)
    constexpr int KH = BK / 32;               // 32-float halves of a step's row
    static_assert(G4 == 0 || (!GATED && NMB >= 2), "row groups of 4 ride on the 32x32x2 slots");
    constexpr int TAIL0 = NMB * 16;           // first row of the 4-row groups
    constexpr int A_ROWS = NMB * 16 + 4 * G4;
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
    v4f acc4[G4 > 0 ? G4 : 1];
#pragma unroll
    for (int q = 0; q < (G4 > 0 ? G4 : 1); ++q) acc4[q] = v4f{0.f, 0.f, 0.f, 0.f};
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

    // D register sets: global loads run D K steps ahead of the matrix core.  Two steps of MFMA work cover the
    // latency of an HBM miss (every weight load is one) when a tile has a hundred rows or more.  A tile of a few
    // dozen rows has little arithmetic per step; near the point where the weights' arrival and the arithmetic
    // take equally long (about 40 rows) a wait for a load stalls the matrix core, and four sets take 2-3 % off
    // calls with 50-77 rows per expert.  (For taller tiles they cost more registers than they save waits: with
    // four sets up to 128 rows the same calls ran 3 % slower.  Where the weights alone set the pace, below 32
    // rows, the depth makes no difference.)
    static_assert(D == 2 || D == 4, "the step loop is unrolled by D");
    v4f ra[D][A_LOADS], rb[D][NB][B_LOADS];
    // item L of the global loads of the step starting at k0 (K % BK == 0 on this path), into set P
    auto gload = [&](auto setc, auto lc, int k0) {
        constexpr int P = decltype(setc)::value, L = decltype(lc)::value;
        if constexpr (L < A_LOADS) {
            ra[P][L] = *reinterpret_cast<const v4f*>(a_base + (size_t)k0 * 4 + a_off[L]);
        } else {
            constexpr int M = (L - A_LOADS) / B_LOADS, Q = (L - A_LOADS) % B_LOADS;
            // STREAM_B (calls with few rows per expert): a weight byte is read by one workgroup, once: streamed past
            // the caches, which is worth 3-6 % where the weights' arrival sets the pace (256-512 tokens over 32
            // experts).  Tall tiles: plain loads - the row tiles of an expert with several are scheduled side by
            // side to share their weight rows through the L2, and a line marked as streaming does not stay for that.
            const v4f* src = reinterpret_cast<const v4f*>(b_base[M] + (size_t)k0 * 4 + b_off[Q]);
            rb[P][M][Q] = STREAM_B ? __builtin_nontemporal_load(src) : *src;
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
    v4f af4[2][G4 > 0 ? G4 : 1];                  // 4x4x1: the 8-k groups of the 32x32x2 form, row lane % 4
    const float* a4 = As + (TAIL0 + (lane & 3)) * LDK + 4 * kh;
    const float* a32 = As + i32 * LDK + 4 * kh;
    const float* b32 = Bs + (wave * 32 + i32) * LDK + 4 * kh;
    const float* a16 = As + (32 * N32 + i16) * LDK + 4 * kq;
    const float* b16 = Bs + (wave * 32 + i16) * LDK + 4 * kq;
    // operand q of 8-k group g: q < NB weights, then the 32-row blocks, then the 4-row groups
    auto read32 = [&](auto bufc, auto gc, auto qc) {
        constexpr int BUF = decltype(bufc)::value, G = decltype(gc)::value, Q = decltype(qc)::value;
        if constexpr (Q < NB)
            bf32[G & 1][Q] = *reinterpret_cast<const v4f*>(b32 + BUF * b_buf + Q * BN * LDK + 8 * G);
        else if constexpr (Q < NB + N32)
            af32[G & 1][Q - NB] = *reinterpret_cast<const v4f*>(a32 + BUF * a_buf + 32 * (Q - NB) * LDK + 8 * G);
        else
            af4[G & 1][Q - NB - N32] = *reinterpret_cast<const v4f*>(a4 + BUF * a_buf + 4 * (Q - NB - N32) * LDK + 8 * G);
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
    //   * the first half of the slots carries the global loads of step s + D, into register set s % D (whose
    //     previous content, step s, went to LDS during step s - 1),
    //   * the second half, but for its last two slots, writes register set (s + 1) % D (step s + 1) into LDS
    //     buffer (s + 1) % 2; then the workgroup's one barrier of the step,
    //   * every slot group carries the LDS operand reads of the next k group (from LDS buffer s % 2), and the
    //     last two slots, behind the barrier, those of the first k group of step s + 1 from the buffer just
    //     filled: the next step's first matrix instructions find their operands there instead of waiting for
    //     them at the top of the step with nothing else to do (worth 1 % on calls with 50-77 rows per expert,
    //     nothing on tall tiles: the wait was shorter than it looks in the source).
    // The loop over steps is unrolled by D so that P = s % D, and with it every LDS address offset and
    // register index, is a compile-time constant.
    constexpr int G32 = BK / 8, G16 = BK / 16;  // k groups of a step
    constexpr int S32 = N32 > 0 ? 4 * G32 : 0, S16 = T16 ? 4 * G16 : 0, S = S32 + S16, SV = S / 2, SB = S - 2;
    constexpr int R32 = NB + N32 + G4, R16 = 1 + 2 * NB;
    const int nk = K / BK;
    auto step = [&](auto pc, int s) {
        constexpr int P = decltype(pc)::value;
        const std::integral_constant<int, P % 2> cur{};          // LDS buffer the matrix core reads
        const std::integral_constant<int, 1 - P % 2> other{};    // LDS buffer being filled
        const std::integral_constant<int, P> lset{};             // register set being loaded
        const std::integral_constant<int, (P + 1) % D> sset{};   // register set written to LDS
        const int kload = min(s + D, nk - 1) * BK;  // the surplus loads of the last D steps are discarded
        static_for<0, S>([&](auto tc) {
            constexpr int t = decltype(tc)::value;
            if constexpr (t < SV) {
                static_for<(t * NV) / SV, ((t + 1) * NV) / SV>([&](auto lc) { gload(lset, lc, kload); });
            } else if constexpr (t < SB) {
                static_for<((t - SV) * NV) / (SB - SV), ((t - SV + 1) * NV) / (SB - SV)>(
                    [&](auto lc) { lstore(sset, lc, other); });
            } else {
                // every wave's share of step s + 1 is in LDS; nobody reads buffer `cur` any more (the last k
                // group's operands were waited for two slots ago)
                if constexpr (t == SB) __syncthreads();
                if constexpr (N32 > 0)
                    static_for<0, R32>([&](auto qc) {
                        if constexpr (decltype(qc)::value % 2 == t - SB) read32(other, std::integral_constant<int, 0>{}, qc);
                    });
                else
                    static_for<0, R16>([&](auto qc) {
                        if constexpr (decltype(qc)::value % 2 == t - SB) read16(other, std::integral_constant<int, 0>{}, qc);
                    });
            }
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
#pragma unroll
                for (int q = 0; q < G4; ++q)
                    acc4[q] = __builtin_amdgcn_mfma_f32_4x4x1f32(af4[g & 1][q][j], bf32[g & 1][0][j], acc4[q], 0, 0, 0);
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
    };
    // step 0 into set 0 and on into LDS buffer 0, steps 1 .. D-1 into their sets
    const std::integral_constant<int, 0> zero{};
    static_for<0, NV>([&](auto lc) { gload(zero, lc, 0); });
    static_for<1, D>([&](auto jc) {
        static_for<0, NV>([&](auto lc) { gload(jc, lc, min((int)decltype(jc)::value, nk - 1) * BK); });
    });
    static_for<0, NV>([&](auto lc) { lstore(zero, lc, zero); });
    __syncthreads();
    // the first step's first operands (every later step's are read in the last slots of the step before)
    if constexpr (N32 > 0)
        static_for<0, R32>([&](auto qc) { read32(zero, zero, qc); });
    else
        static_for<0, R16>([&](auto qc) { read16(zero, zero, qc); });
    for (int s = 0; s < nk; s += D)
        static_for<0, D>([&](auto pc) {
            if (s + decltype(pc)::value < nk) step(pc, s + decltype(pc)::value);
        });

    // epilogue
    // 32x32 block: register r holds row 8*(r/4) + 4*(lane/32) + r%4, column lane%32
    // 16x16 block: register r holds row 4*(lane/16) + r, column lane%16
    // 4x4 blocks: register r holds row r of the group, column lane % 32; the upper half of the wave
    // holds the other float4 of every 8-k group
#pragma unroll
    for (int q = 0; q < G4; ++q)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc4[q][r] += __shfl_xor(acc4[q][r], 32);
    constexpr bool residual = EPI == EPI_RESIDUAL;
    if constexpr (NORM) {
        if (stats != nullptr) {
            // rstd of every row this lane holds, fetched together (clamped, always valid addresses)
            auto st = [&](int row) { return stats[2 * min(row, rows - 1) + 1]; };
#pragma unroll
            for (int mb = 0; mb < N32; ++mb) {
                float f[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) f[r] = st(32 * mb + 8 * (r / 4) + 4 * kh + (r % 4));
#pragma unroll
                for (int m = 0; m < NB; ++m)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc32[m][mb][r] *= f[r];
            }
            if (T16) {
                float f[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) f[r] = st(32 * N32 + 4 * kq + r);
#pragma unroll
                for (int m = 0; m < NB; ++m)
#pragma unroll
                    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc16[m][nb][r] *= f[r];
            }
#pragma unroll
            for (int q = 0; q < G4; ++q)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc4[q][r] *= st(TAIL0 + 4 * q + r);
        }
    }
    if constexpr (residual) {
        // The residual values of a block are fetched together before the first is used (from clamped,
        // always valid addresses) and added to the accumulators: loaded next to its store inside the
        // bounds check, every value would be waited for by itself, and the second GEMM of the
        // sublayer then ran 3 % longer than the first.
        const float* rcol = R + min(n0 + wave * 32 + i32, N - 1);
        auto at = [&](const float* col, int row) { return col[(size_t)min(row, rows - 1) * N]; };
#pragma unroll
        for (int mb = 0; mb < N32; ++mb) {
            float res[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) res[r] = at(rcol, 32 * mb + 8 * (r / 4) + 4 * kh + (r % 4));
#pragma unroll
            for (int r = 0; r < 16; ++r) acc32[0][mb][r] += res[r];
        }
        if (T16) {
            float res[2][4];
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    res[nb][r] = at(R + min(n0 + wave * 32 + 16 * nb + i16, N - 1), 32 * N32 + 4 * kq + r);
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc16[0][nb][r] += res[nb][r];
        }
        if (G4 > 0) {
            float res[G4 > 0 ? G4 : 1][4];
#pragma unroll
            for (int q = 0; q < G4; ++q)
#pragma unroll
                for (int r = 0; r < 4; ++r) res[q][r] = at(rcol, TAIL0 + 4 * q + r);
#pragma unroll
            for (int q = 0; q < G4; ++q)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc4[q][r] += res[q][r];
        }
    }
    auto emit = [&](int row, int col, float v, float v1) {
        if (row < rows && col < N) {
            if (GATED)
                v = gelu_dot(v, v1);
            else if (!residual)
                v = fmaxf(v, 0.f);
            C[(size_t)row * N + col] = v;
        }
    };
#pragma unroll
    for (int mb = 0; mb < N32; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            emit(32 * mb + 8 * (r / 4) + 4 * kh + (r % 4), n0 + wave * 32 + i32, acc32[0][mb][r], acc32[NB - 1][mb][r]);
    if (T16) {
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                emit(32 * N32 + 4 * kq + r, n0 + wave * 32 + 16 * nb + i16, acc16[0][nb][r], acc16[NB - 1][nb][r]);
    }
#pragma unroll
    for (int q = 0; q < G4; ++q)
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (kh == 0) emit(TAIL0 + 4 * q + r, n0 + wave * 32 + i32, acc4[q][r], 0.f);
}

// How `rows` rows are cut into 16-row units (two make a 32x32x2 block, an odd one a 16x16x4 block)
// and 4-row groups: whole units, then one or two groups for a remainder of up to 8 rows when there
// are at least two units to ride on; otherwise one more unit.  Measured on 32 uniform experts of
// 128 + r rows: one group costs 44 % of a further unit, two 60 %, three 95 % (so three are not used);
// on 4096 tokens over 32 experts (108..147 rows each) the layer gains 1.3 %.
struct TileShape {
    int nmb, g4;
};
// (Tiles of up to 160 rows carry groups only in their 64-float-step form, which K % 64 == 0 selects:
// the 32-float-step form of those heights is instantiated without groups to keep the build short.)
template <bool GATED>
__device__ __forceinline__ TileShape tile_shape(int rows, bool wide) {
    const int full = rows >> 4, rem = rows & 15;
    const TileShape units{(rows + 15) >> 4, 0};
    if (GATED || rem == 0 || rem > 8 || full < 2) return units;
    const TileShape groups{full, (rem + 3) >> 2};
    if (!wide && 16 * groups.nmb + 4 * groups.g4 <= 16 * kMaxMb64) return units;
    return groups;
}

// Register sets of the global loads (gemm_tile's D) for a tile of 16 * nmb + 4 * g4 rows: tiles of up to 64
// rows keep four steps in flight, taller ones two.
constexpr int depth_of(int nmb, int g4) { return 16 * nmb + 4 * g4 <= 64 ? 4 : 2; }

template <int BN, int EPI>
__device__ __forceinline__ void gemm_dispatch(const float* A, const float* R, float* C, int rows, const float* B0,
                                              const float* B1, int n0, int N, int K, const float* stats,
                                              float* smem, int a_alloc_rows) {
    constexpr bool GATED = EPI == EPI_GATED_GELU;
    // the gated form keeps two accumulator sets, so its tiles are half as tall
    constexpr int kMaxMb = (GATED ? kGemmTileRowsGated : kGemmTileRows) / 16;
    // Tiles of up to 160 rows take K in steps of 64 floats (half as many barriers per flop); the LDS
    // cannot hold two such stages of a taller tile or of two weight matrices, which take steps of 32.
    const bool wide = !GATED && (K & 63) == 0;
    const TileShape shape = tile_shape<GATED>(rows, wide);
#define INFMOE_CASE_G(n, g)                                                                                     \
    case 4 * (n) + (g):                                                                                         \
        if constexpr ((n) <= kMaxMb && ((g) == 0 || (!GATED && (n) >= 2 && (n) < kMaxMb))) {                    \
            if constexpr (!GATED && 16 * (n) + 4 * (g) <= 16 * kMaxMb64) {                                      \
                if (wide) {                                                                                     \
                    gemm_tile<n, g, BN, EPI, 64, depth_of(n, g)>(A, R, C, rows, B0, B1, n0, N, K, stats, smem,  \
                                                                 min(a_alloc_rows, 16 * kMaxMb64));             \
                    break;                                                                                      \
                }                                                                                               \
            }                                                                                                   \
            if constexpr ((g) == 0 || 16 * (n) + 4 * (g) > 16 * kMaxMb64)                                       \
                gemm_tile<n, g, BN, EPI, 32, depth_of(n, g)>(A, R, C, rows, B0, B1, n0, N, K, stats, smem,      \
                                                             a_alloc_rows);                                     \
        }                                                                                                       \
        break;
#define INFMOE_CASE(n) INFMOE_CASE_G(n, 0) INFMOE_CASE_G(n, 1) INFMOE_CASE_G(n, 2)
    switch (4 * shape.nmb + shape.g4) {
        INFMOE_CASE(1) INFMOE_CASE(2) INFMOE_CASE(3) INFMOE_CASE(4) INFMOE_CASE(5) INFMOE_CASE(6) INFMOE_CASE(7)
        INFMOE_CASE(8) INFMOE_CASE(9) INFMOE_CASE(10) INFMOE_CASE(11) INFMOE_CASE(12) INFMOE_CASE(13)
        INFMOE_CASE(14) INFMOE_CASE(15) INFMOE_CASE(16)
        default: break;
    }
#undef INFMOE_CASE
#undef INFMOE_CASE_G
}

// One expert: grid.x = row tiles of tile_rows rows (the last may be shorter), grid.y = column tiles: the row tiles
// of a column tile are dispatched side by side and share its weight rows through the caches.
template <int BN, int EPI>
__global__ __launch_bounds__(kThreads) void expert_gemm_kernel(GemmProblem p, int rows_total, int tile_rows,
                                                               int a_alloc_rows) {
    extern __shared__ __align__(16) float smem[];
    const int row0 = blockIdx.x * tile_rows;
    const int rows = min(tile_rows, rows_total - row0);
    const int n0 = blockIdx.y * BN;
    gemm_dispatch<BN, EPI>(p.A + (size_t)row0 * p.K, p.R ? p.R + (size_t)row0 * p.N : nullptr,
                           p.C + (size_t)row0 * p.N, rows, p.B, p.B1, n0, p.N, p.K,
                           p.row_stats ? p.row_stats + 2 * (size_t)row0 : nullptr, smem, a_alloc_rows);
}

// All experts: 1-D grid of 8 * (row-tile capacity of an XCD) * n_col_tiles workgroups.  Workgroup id
// b runs on XCD b % 8 and takes slot b / 8 of that XCD's share of the schedule.  The share is a list of runs
// of row tiles (RowTile::pad = place in the run | run length << 16; a run is 1..4 row tiles of one expert, the
// dispatch scan makes them): a run of L tiles owns L * n_col_tiles consecutive slots, column tile by column
// tile with the run's L row tiles side by side, so workgroups that start together read the same weight rows
// (one fetch from memory, L - 1 hits in the XCD's L2) and the column tiles of a row tile, which share its
// activations, follow each other at a distance of L.
// Returns false for a slot beyond the share.
__device__ __forceinline__ bool grouped_slot(const RowTile* __restrict__ tiles, const int* __restrict__ sched,
                                             int n_col_tiles, RowTile* rt, int* col_tile) {
    const int xcd = blockIdx.x % kXcdCount, slot = blockIdx.x / kXcdCount;
    const int first = sched[1 + xcd], share = sched[2 + xcd] - first;
    if (slot >= share * n_col_tiles) return false;
    const int i = slot / n_col_tiles;  // some tile of the run the slot belongs to
    const int pad = tiles[first + i].pad;
    const int L = max(pad >> 16, 1), i0 = i - (pad & 0xffff);
    const int local = slot - i0 * n_col_tiles;
    *rt = tiles[first + i0 + local % L];
    *col_tile = local / L;
    return true;
}

template <int BN, int EPI>
__global__ __launch_bounds__(kThreads) void expert_gemm_grouped_kernel(GemmProblem p, size_t weight_stride,
                                                                       const RowTile* __restrict__ tiles,
                                                                       const int* __restrict__ sched,
                                                                       int n_col_tiles) {
    extern __shared__ __align__(16) float smem[];
    RowTile rt;
    int col_tile;
    if (!grouped_slot(tiles, sched, n_col_tiles, &rt, &col_tile)) return;
    const int n0 = col_tile * BN;
    const int owner = p.expert_slot ? p.expert_slot[rt.expert] : rt.expert;
    constexpr bool GATED = EPI == EPI_GATED_GELU;
    const float* B0 = p.B + (size_t)owner * weight_stride;
    const float* B1 = GATED ? p.B1 + (size_t)owner * weight_stride : nullptr;
    gemm_dispatch<BN, EPI>(p.A + (size_t)rt.row0 * p.K, p.R ? p.R + (size_t)rt.row0 * p.N : nullptr,
                           p.C + (size_t)rt.row0 * p.N, rt.rows, B0, B1, n0, p.N, p.K,
                           p.row_stats ? p.row_stats + 2 * (size_t)rt.row0 : nullptr, smem,
                           GATED ? kGemmTileRowsGated : kGemmTileRows);
}

// ---- Calls with few rows per expert (gemm_small_tiles(): tokens <= 64 * experts).
// The kernels above keep one workgroup per compute unit: their registers and LDS are sized for tiles of 256
// rows.  A tile of a few dozen rows has little arithmetic per byte of weights; what it needs is bytes in
// flight and no dead time, and a workgroup by itself has dead time: its start (nothing computes until the
// first loads are back), its end (nothing loads while the last tile is stored) and the turn of every barrier.
// Here the same tile body is instantiated for tiles of up to kGemmTileRowsSmall rows only - 32-float steps,
// few accumulators, half the LDS - so that TWO workgroups share a compute unit and each fills the other's gaps
// (the second launch bound below asks the compiler to stay within the registers of two waves per SIMD).
// Row counts are padded to 4 (whole 16-row units plus one or two 4-row groups) from 32 rows on, to 16 below.
// Which path a call takes depends on (tokens, experts) only, so every schedule of a layer agrees on it.
template <int BN, int EPI>
__device__ __forceinline__ void gemm_dispatch_small(const float* A, const float* R, float* C, int rows, const float* B0,
                                                    int n0, int N, int K, const float* stats, float* smem,
                                                    int a_alloc_rows) {
    static_assert(EPI != EPI_GATED_GELU, "the two-matrix form keeps its tall tiles");
    constexpr int kMaxMb = kGemmTileRowsSmall / 16;
    const int full = rows >> 4, rem = rows & 15;
    int nmb = (rows + 15) >> 4, g4 = 0;
    if (rem != 0 && rem <= 8 && full >= 2) nmb = full, g4 = (rem + 3) >> 2;
#define INFMOE_SMALL_G(n, g)                                                                                          \
    case 4 * (n) + (g):                                                                                               \
        if constexpr ((n) <= kMaxMb && ((g) == 0 || ((n) >= 2 && (n) < kMaxMb)))                                      \
            gemm_tile<n, g, BN, EPI, 32, depth_of(n, g), true>(A, R, C, rows, B0, nullptr, n0, N, K, stats, smem,     \
                                                               a_alloc_rows);                                        \
        break;
#define INFMOE_SMALL(n) INFMOE_SMALL_G(n, 0) INFMOE_SMALL_G(n, 1) INFMOE_SMALL_G(n, 2)
    switch (4 * nmb + g4) {
        INFMOE_SMALL(1) INFMOE_SMALL(2) INFMOE_SMALL(3) INFMOE_SMALL(4) INFMOE_SMALL(5) INFMOE_SMALL(6)
        default: break;
    }
#undef INFMOE_SMALL
#undef INFMOE_SMALL_G
}

template <int BN, int EPI>
__global__ __launch_bounds__(kThreads, 2) void expert_gemm_small_kernel(GemmProblem p, int rows_total, int tile_rows,
                                                                        int a_alloc_rows) {
    extern __shared__ __align__(16) float smem[];
    const int row0 = blockIdx.x * tile_rows;  // (x = row tile, y = column tile, as in expert_gemm_kernel)
    const int rows = min(tile_rows, rows_total - row0);
    const int n0 = blockIdx.y * BN;
    gemm_dispatch_small<BN, EPI>(p.A + (size_t)row0 * p.K, p.R ? p.R + (size_t)row0 * p.N : nullptr,
                                 p.C + (size_t)row0 * p.N, rows, p.B, n0, p.N, p.K,
                                 p.row_stats ? p.row_stats + 2 * (size_t)row0 : nullptr, smem, a_alloc_rows);
}

// (the same map from workgroup id to (row tile, column tile) as expert_gemm_grouped_kernel)
template <int BN, int EPI>
__global__ __launch_bounds__(kThreads, 2) void expert_gemm_grouped_small_kernel(GemmProblem p, size_t weight_stride,
                                                                                const RowTile* __restrict__ tiles,
                                                                                const int* __restrict__ sched,
                                                                                int n_col_tiles) {
    extern __shared__ __align__(16) float smem[];
    RowTile rt;
    int col_tile;
    if (!grouped_slot(tiles, sched, n_col_tiles, &rt, &col_tile)) return;
    const int n0 = col_tile * BN;
    const int owner = p.expert_slot ? p.expert_slot[rt.expert] : rt.expert;
    gemm_dispatch_small<BN, EPI>(p.A + (size_t)rt.row0 * p.K, p.R ? p.R + (size_t)rt.row0 * p.N : nullptr,
                                 p.C + (size_t)rt.row0 * p.N, rt.rows, p.B + (size_t)owner * weight_stride, n0, p.N, p.K,
                                 p.row_stats ? p.row_stats + 2 * (size_t)rt.row0 : nullptr, smem, kGemmTileRowsSmall);
}

}  // namespace
}  // namespace infmoe
