// Gating, first of two launches, for calls with many tokens: partial scores of one slice of the
// embedding dimension with that slice of the (gamma-folded) centroids resident in LDS.
//
// Replaces, together with the combine launch of gating.hip, the chain layernorm_gpu -> cublasSgemm_v2
// -> expert_select_top1_kernel (plugin/MoELayerPlugin.cc:315-345).
//
// Why this shape.  The input is read once (T*d*4 bytes: the bound of the whole gating), the centroids
// are tiny (E*d*4) but every token needs all of them.  A workgroup that walks all of d for its tokens
// re-reads every centroid through the first-level cache, two bytes of centroid per byte of input at 16
// tokens x 32 experts, and the rate a compute unit sustains through that cache is what bounded the
// one-launch kernel.  Here the embedding dimension is cut into S slices of ks floats.  Workgroup
// (g, j) copies slice j of all centroids into LDS once (EP x ks floats: 66 KB at 32 experts x 512) and
// then streams the slice-j part of its tokens past it: no barrier after the fill, no centroid traffic
// in the loop.  Slice j = workgroup id mod S, and workgroup ids are dealt round-robin to the 8 XCDs,
// so with S = 8 every XCD's L2 holds one slice only.
//
// A wave owns 16 tokens at a time (v_mfma_f32_16x16x4_f32: tokens are the A rows, 16 experts per B
// block).  Its loads go straight into the matrix operand layout - lane (i, q) reads floats
// 16*g + 4*q .. +3 of token i, so 8 consecutive loads of a lane cover 512 contiguous bytes of a row -
// in two register sets of 8 KB per wave, one being consumed while the other is in flight.  The k order
// inside a 16-float group is permuted identically for both operands (instruction c multiplies element c
// of every lane's float4), which a dot product does not see.  The row sums of x and x^2 that the norm
// needs come from the same registers.
//
// Output: partials[j][t][0..E) = sum over slice j of x[t][k] * cf[e][k]; [E] = sum x; [E+1] = sum x^2
// - the layout the combine launch of gating.hip adds up in slice order before it selects.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cfloat>
#include <cmath>
#include <type_traits>

#include "kernels.h"

namespace infmoe {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kGroupsPerChunk = 8;                  // 16-float groups per register set
constexpr int kChunk = 16 * kGroupsPerChunk;        // floats of K per register set: 128
constexpr size_t kSlabLdsLimit = 150 * 1024;        // of the 160 KB a compute unit has

// f(integral_constant<int, I>) for I in [I, N)
template <int I, int N, typename F>
__device__ __forceinline__ void static_for_sets(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for_sets<I + 1, N>(f);
    }
}

template <int NBLK, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void gate_slab_kernel(const float* __restrict__ X, const float* __restrict__ Cf,
                                                               float* __restrict__ partials, int T, int d, int E,
                                                               int ks, int S, int tiles_per_wave,
                                                               int* __restrict__ zero_stats,
                                                               int* __restrict__ zero_hist, int n_hist) {
    extern __shared__ __align__(16) float slab[];  // [16 * NBLK][ks + 4]
    constexpr int EP = 16 * NBLK;
    const int LDK = ks + 4, W = E + 2;
    const int j = blockIdx.x % S, g = blockIdx.x / S;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int i16 = lane & 15, kq = lane >> 4;
    const int nch = ks / kChunk;
    const size_t k0 = (size_t)j * ks;
    // the routing statistics the combine launch counts into start at zero (saves a fill launch)
    if (zero_stats != nullptr && blockIdx.x == 0 && tid < 4) zero_stats[tid] = 0;
    // ... and so does the per-block histogram of the assignment that it adds into (saves the histogram launch)
    if (zero_hist != nullptr)
        for (int q = blockIdx.x * (64 * WAVES) + tid; q < n_hist; q += gridDim.x * (64 * WAVES)) zero_hist[q] = 0;

    // Tiles of this workgroup: (g * tiles_per_wave + it) * WAVES + wave, it = 0 .. tiles_per_wave - 1.
    // The wave walks the chunks of all its tiles as one sequence: chunk n sits in register set n & 1,
    // and while it is consumed the other set receives chunk n + 1, across tile boundaries too.
    const int first_tile = (g * tiles_per_wave) * WAVES + wave;
    const int all_tiles = (T + 15) / 16;
    const int my_tiles = first_tile >= all_tiles ? 0 : min(tiles_per_wave, (all_tiles - first_tile + WAVES - 1) / WAVES);
    const int total = my_tiles * nch;

    // Register sets of 8 KB per wave: chunk n sits in set n % SETS, and SETS - 1 chunks are in flight while one
    // is consumed.  Two sets.  More, which the registers would allow, make the launch slower, not faster (4096
    // tokens x 4096 x 32 experts: 19.1 us with two, 21.0 with three, 23.3 with four; 16384 x 2048 x 64: 49.5 /
    // 54.1 / 55.3), also with the slab's loads issued ahead of the tokens' so that they are not waited for
    // together.  The launch is not short of bytes in flight: between 2048 and 4096 tokens of 4096 floats it
    // takes 5.5 us more for 33.6 MB more (6.1 TB/s); the rest, 8 us, is what a launch, the slab's fill and the
    // last tiles' stores cost once.  (Non-temporal loads of the tokens change nothing.)
    constexpr int SETS = 2;
    v4f xa[SETS][kGroupsPerChunk];
    int ltile = first_tile, lchunk = 0;  // load cursor
    auto load_into = [&](auto setc) {
        constexpr int P = decltype(setc)::value;
        // rows beyond T are clamped (their results are never stored)
        const float* src = X + (size_t)min(min(ltile, all_tiles - 1) * 16 + i16, T - 1) * d + k0 + 4 * kq + lchunk * kChunk;
#pragma unroll
        for (int gg = 0; gg < kGroupsPerChunk; ++gg) xa[P][gg] = *reinterpret_cast<const v4f*>(src + 16 * gg);
        if (++lchunk == nch) {
            lchunk = 0;
            ltile += WAVES;
        }
    };
    {   // slice j of every centroid row -> LDS (rows beyond E are zero: their columns are never stored).
        // ks is a power of two times 128, so (row, float4) of item idx are a shift and a mask; every pass has eight
        // loads per thread in flight before the first is stored.  The wave's first SETS - 1 chunks of tokens go out
        // between the loads and the stores of the last pass: loads complete in the order they were issued, so the
        // slab's are waited for alone, with the tokens' still on their way.
        const int n4 = ks / 4, sh = 31 - __clz(n4);
        const int items = EP * n4;
#pragma unroll 1
        for (int base = 0; base < items; base += 8 * 64 * WAVES) {
            v4f v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int idx = min(base + u * 64 * WAVES + tid, items - 1);
                const int e = idx >> sh, c = idx & (n4 - 1);
                v[u] = *reinterpret_cast<const v4f*>(Cf + (size_t)min(e, E - 1) * d + k0 + 4 * c);
            }
            if (base + 8 * 64 * WAVES >= items) {
                static_for_sets<0, SETS - 1>([&](auto uc) {
                    if (decltype(uc)::value < total) load_into(uc);
                });
                __builtin_amdgcn_sched_barrier(0);  // the tokens' loads stay in front of the slab's stores
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int idx = base + u * 64 * WAVES + tid;
                const int e = idx >> sh, c = idx & (n4 - 1);
                if (idx < items) *reinterpret_cast<v4f*>(slab + e * LDK + 4 * c) = e < E ? v[u] : v4f{0.f, 0.f, 0.f, 0.f};
            }
        }
    }
    __syncthreads();  // the only barrier: from here on the waves run independently
    if (total == 0) return;

    const float* crow = slab + i16 * LDK + 4 * kq;
    float* part = partials + (size_t)j * T * W;

    v4f acc[2][NBLK];
    float s1 = 0.f, s2 = 0.f;
    auto reset = [&]() {
#pragma unroll
        for (int nb = 0; nb < NBLK; ++nb) {
            acc[0][nb] = v4f{0.f, 0.f, 0.f, 0.f};
            acc[1][nb] = v4f{0.f, 0.f, 0.f, 0.f};
        }
        s1 = 0.f, s2 = 0.f;
    };
    reset();
    int ctile = first_tile, cchunk = 0;  // compute cursor
    auto flush = [&]() {
        const int t0 = ctile * 16;
        // lanes i, i+16, i+32, i+48 hold the four float4 slots of one row
        s1 += __shfl_xor(s1, 16);
        s1 += __shfl_xor(s1, 32);
        s2 += __shfl_xor(s2, 16);
        s2 += __shfl_xor(s2, 32);
        // D layout of 16x16x4: lane holds column (lane & 15), rows 4 * (lane >> 4) + r
#pragma unroll
        for (int nb = 0; nb < NBLK; ++nb) {
            const v4f sum = acc[0][nb] + acc[1][nb];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int t = t0 + 4 * kq + r, e = 16 * nb + i16;
                if (t < T && e < E) part[(size_t)t * W + e] = sum[r];
            }
        }
        if (kq == 0 && t0 + i16 < T) {
            part[(size_t)(t0 + i16) * W + E] = s1;
            part[(size_t)(t0 + i16) * W + E + 1] = s2;
        }
    };
    auto compute = [&](auto setc) {
        constexpr int P = decltype(setc)::value;
#pragma unroll
        for (int gg = 0; gg < kGroupsPerChunk; ++gg) {
            const v4f x = xa[P][gg];
            s1 += (x.x + x.y) + (x.z + x.w);
            s2 += (x.x * x.x + x.y * x.y) + (x.z * x.z + x.w * x.w);
            v4f cb[NBLK];
#pragma unroll
            for (int nb = 0; nb < NBLK; ++nb)
                cb[nb] = *reinterpret_cast<const v4f*>(crow + 16 * nb * LDK + (cchunk * kGroupsPerChunk + gg) * 16);
            // consecutive instructions go to different accumulators so that none waits for its predecessor
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int nb = 0; nb < NBLK; ++nb)
                    acc[gg & 1][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(x[q], cb[nb][q], acc[gg & 1][nb], 0, 0, 0);
        }
        if (++cchunk == nch) {  // the tile is done (wave-uniform)
            flush();
            reset();
            cchunk = 0;
            ctile += WAVES;
        }
    };
    // (no loads beyond the wave's last chunk: with four chunks per wave a surplus one is a quarter more traffic)
    for (int n = 0; n < total; n += SETS) {
        static_for_sets<0, SETS>([&](auto uc) {
            constexpr int U = decltype(uc)::value;
            if (n + U < total) {
                if (n + U + SETS - 1 < total) load_into(std::integral_constant<int, (U + SETS - 1) % SETS>{});
                __builtin_amdgcn_sched_barrier(0);  // the loads go out before the arithmetic, not next to their use
                compute(uc);
            }
        });
    }
}


// ---------------------------------------------------------------------------------------------
// Second launch: add the slices' partial scores in slice order, apply the norm to the score tile,
// select the best expert per token with the reference's tie rule (lowest index wins,
// plugin/cuda/moe.cu:62-68), and re-score in float64 the rare token whose two best FP32 scores are
// closer than FP32 accumulation can order.  Sixteen lanes own one token (lane i the experts i, i + 16,
// ...), a wave four tokens; the waves of a workgroup meet once, to learn whether any token needs the
// re-scoring, which the whole workgroup then does together.
struct CombineArgs {
    int T, d, E, S;
    const float* partials;  // [S][T][E + 2]
    const float* cstats;    // [2E]: per expert the sum and the Euclidean norm of centroid * gamma
    const float* X;         // for the float64 re-scoring
    const float* C;         // plain centroids [E][d]
    const float* gamma;     // [d] or null
    const float* bias;      // [E] or null
    int norm_kind;
    int* sel;
    float* coeff;
    int* stats;     // or null
    int* nan_flag;  // null, or an int (host memory the device can write) set to nan_value when a token has no orderable score
    int nan_value;
    float err_depth;  // n of the error bound of a score (gate_err_depth)
    // null, or [ceil(T / hist_block)][E] ints, zero on entry, that receive the number of tokens of every block
    // of hist_block consecutive tokens that chose each expert: what the first pass of the counting sort
    // (hist_kernel) would compute from sel in a launch of its own
    int* block_hist;
    int hist_block;
};

__device__ __forceinline__ double wave_sum64(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

constexpr int kCand = 4;  // experts re-scored by one sweep over the embedding dimension

// Float64 scores of up to kCand experts for token t, computed by the whole workgroup in one sweep over d
// (every thread of the workgroup calls this; s_part is LDS scratch of [4][2 + 2 * kCand] doubles).
// Returns, in every thread, sc[c] = rstd * (x.g.c - mu * sum g.c) + bias for the experts cand[0..kCand).
// With 256 threads a row of 4096 floats is four float4 per thread, and the unrolled loop has the loads of
// all rows in flight at once: the sweep costs one memory round trip, not one per piece of the row.
// NC: how many of the kCand candidates are looked at (2 when only the best two are close, the usual case: half
// the loads and half the double-precision arithmetic); sc[c] for c >= NC is not set.
template <int NC>
__device__ __forceinline__ void rescore(const CombineArgs& a, int t, const int (&cand)[kCand], double (&sc)[kCand],
                                        double (*s_part)[2 + 2 * kCand]) {
    const int tid = threadIdx.x, d = a.d;
    const float* xr = a.X + (size_t)t * d;
    const float* cr[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) cr[c] = a.C + (size_t)cand[c] * d;
    const bool use_gamma = a.norm_kind != NORM_NONE && a.gamma != nullptr;
    const bool centered = a.norm_kind == NORM_CENTERED;
    double r[2 + 2 * kCand];
#pragma unroll
    for (int q = 0; q < 2 + 2 * kCand; ++q) r[q] = 0.0;
    // Blocks of 4096 floats, four float4 per thread of each of the six rows: all 24 loads are issued (from
    // clamped, always valid addresses; a piece beyond the row is masked out of the sums) before the first is
    // used, so a block costs one trip to memory, not one per piece.  (As a loop with the loads next to their
    // use the sweep took 11 us of the launch's critical path.)
    for (int kb = 0; kb < d; kb += 4096) {
        v4f xv[4], gv[4], cv[NC][4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int k = min(kb + 1024 * u + 4 * tid, d - 4);
            xv[u] = *reinterpret_cast<const v4f*>(xr + k);
            gv[u] = use_gamma ? *reinterpret_cast<const v4f*>(a.gamma + k) : v4f{1.f, 1.f, 1.f, 1.f};
#pragma unroll
            for (int c = 0; c < NC; ++c) cv[c][u] = *reinterpret_cast<const v4f*>(cr[c] + k);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (kb + 1024 * u + 4 * tid >= d) continue;
            const double x0 = xv[u].x, x1 = xv[u].y, x2 = xv[u].z, x3 = xv[u].w;
            r[0] += (x0 + x1) + (x2 + x3);
            r[1] += (x0 * x0 + x1 * x1) + (x2 * x2 + x3 * x3);
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const double g0 = (double)gv[u].x * (double)cv[c][u].x, g1 = (double)gv[u].y * (double)cv[c][u].y;
                const double g2 = (double)gv[u].z * (double)cv[c][u].z, g3 = (double)gv[u].w * (double)cv[c][u].w;
                r[2 + c] += (x0 * g0 + x1 * g1) + (x2 * g2 + x3 * g3);
                if (centered) r[2 + kCand + c] += (g0 + g1) + (g2 + g3);  // (only the centered norm wants sum g c)
            }
        }
    }
#pragma unroll
    for (int q = 0; q < 2 + 2 * kCand; ++q) {
        if ((q >= 2 + NC && q < 2 + kCand) || q >= 2 + kCand + NC) continue;  // sums of candidates not looked at
        r[q] = wave_sum64(r[q]);
        if ((tid & 63) == 0) s_part[tid >> 6][q] = r[q];
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < 2 + 2 * kCand; ++q) r[q] = (s_part[0][q] + s_part[1][q]) + (s_part[2][q] + s_part[3][q]);
    __syncthreads();  // s_part may be written again by the next call
    double mu = 0.0, rstd = 1.0;
    if (a.norm_kind == NORM_RMS) {
        rstd = 1.0 / sqrt(r[1] / d + 1e-6);
    } else if (a.norm_kind == NORM_CENTERED) {
        mu = r[0] / d;
        rstd = 1.0 / sqrt(fmax(r[1] / d - mu * mu, 0.0) + 1e-6);
    }
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        sc[c] = rstd * (r[2 + c] - mu * r[2 + kCand + c]);
        if (a.bias != nullptr) sc[c] += (double)a.bias[cand[c]];
    }
}

template <int NBLK>
__global__ __launch_bounds__(256) void gate_combine_kernel(const CombineArgs a) {
    // slices whose loads are in flight together
    constexpr int JU = NBLK <= 2 ? 8 : (NBLK == 4 ? 4 : 2);
    const int T = a.T, E = a.E, S = a.S, W = E + 2;
    const int lane = threadIdx.x & 63;
    const int i = lane & 15, grp = lane >> 4;
    const int t = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 4 + grp;
    const bool live = t < T;
    const size_t slice = (size_t)T * W;
    const float* src = a.partials + (size_t)min(t, T - 1) * W;

    float dot[NBLK], st = 0.f;
    int eidx[NBLK];
#pragma unroll
    for (int nb = 0; nb < NBLK; ++nb) dot[nb] = 0.f, eidx[nb] = min(16 * nb + i, E - 1);  // clamped: masked below
    for (int j0 = 0; j0 < S; j0 += JU) {
        float v[JU][NBLK], sv[JU];
#pragma unroll
        for (int jj = 0; jj < JU; ++jj) {
            const float* p = src + (size_t)min(j0 + jj, S - 1) * slice;
#pragma unroll
            for (int nb = 0; nb < NBLK; ++nb) v[jj][nb] = p[eidx[nb]];
            sv[jj] = p[E + (i & 1)];  // lane 0 of the group: sum x, lane 1: sum x^2
        }
#pragma unroll
        for (int jj = 0; jj < JU; ++jj) {  // in slice order
            const bool on = j0 + jj < S;
#pragma unroll
            for (int nb = 0; nb < NBLK; ++nb) dot[nb] += on ? v[jj][nb] : 0.f;
            st += on ? sv[jj] : 0.f;
        }
    }
    const float a1 = __shfl(st, lane & 48), a2 = __shfl(st, (lane & 48) + 1);
    float mu = 0.f, rstd = 1.f;
    if (a.norm_kind == NORM_RMS) {
        rstd = 1.0f / sqrtf(a2 / (float)a.d + kNormEps);
    } else if (a.norm_kind == NORM_CENTERED) {
        mu = a1 / (float)a.d;
        rstd = 1.0f / sqrtf(fmaxf(a2 / (float)a.d - mu * mu, 0.f) + kNormEps);
    }
    // scores of this lane's experts; an expert beyond E never wins (NaN: no comparison with it holds)
    float score[NBLK], cnmax = 0.f;
#pragma unroll
    for (int nb = 0; nb < NBLK; ++nb) {
        const bool valid = 16 * nb + i < E;
        float sc = rstd * (dot[nb] - mu * a.cstats[eidx[nb]]);
        if (a.bias != nullptr) sc += a.bias[eidx[nb]];
        score[nb] = valid ? sc : __builtin_nanf("");
        cnmax = fmaxf(cnmax, valid ? a.cstats[E + eidx[nb]] : 0.f);
    }
    float best = -FLT_MAX;  // plugin/cuda/moe.cu:26-27
    int besti = -1;
#pragma unroll
    for (int nb = 0; nb < NBLK; ++nb)
        if (score[nb] > best) best = score[nb], besti = 16 * nb + i;  // strict: the lowest index keeps a tie
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off);
        const int oi = __shfl_xor(besti, off);
        if (ov > best || (ov == best && (unsigned)oi < (unsigned)besti)) best = ov, besti = oi;
        cnmax = fmaxf(cnmax, __shfl_xor(cnmax, off));
    }
    float second = -FLT_MAX;
#pragma unroll
    for (int nb = 0; nb < NBLK; ++nb)
        if (16 * nb + i != besti && score[nb] > second) second = score[nb];
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) second = fmaxf(second, __shfl_xor(second, off));

    // FP32 accumulation over d terms cannot order two scores closer than twice its own rounding error (gate_err_depth)
    const float bound = a.err_depth * FLT_EPSILON * rstd * sqrtf(a2) * cnmax;
    const float thr = fmaxf(bound, 4e-6f * fabsf(best));
    const bool flagged = live && besti >= 0 && E > 1 && (best - second) < thr;
    __shared__ int s_sel[16];  // the 16 tokens' experts, as last decided
    if (i == 0) s_sel[threadIdx.x >> 4] = live ? max(besti, 0) : -1;
    if (live && i == 0) {
        a.sel[t] = besti < 0 ? 0 : besti;  // no orderable score: the reference asserts (plugin/cuda/moe.cu:70)
        a.coeff[t] = besti < 0 ? __builtin_nanf("") : best;  // NaN marks the row: the combine step writes NaN for it
        if (besti < 0) {
            if (a.stats != nullptr) atomicAdd(&a.stats[1], 1);
            if (a.nan_flag != nullptr) *reinterpret_cast<volatile int*>(a.nan_flag) = a.nan_value;
        }
    }

    // ---- float64 re-scoring, token by token, by the whole workgroup (rare: about one token in a few
    // thousand for Gaussian scores, so almost every workgroup leaves after the one barrier below)
    __shared__ unsigned long long s_todo[4];
    __shared__ int s_cand[kCand], s_nc, s_tt;
    __shared__ double s_part[4][2 + 2 * kCand];
    const int wave = threadIdx.x >> 6;
    {
        const unsigned long long mine = __ballot(flagged && i == 0);
        if (lane == 0) s_todo[wave] = mine;
    }
    __syncthreads();
    for (int w = 0; w < 4; ++w) {
        unsigned long long todo = s_todo[w];  // the same in every thread of the workgroup
        while (todo != 0) {
            const int L = __ffsll((long long)todo) - 1;  // lane 0 of the token's group, in wave w
            todo &= todo - 1;
            if (wave == w) {
                // candidates: the experts within the bound of the best, in ascending index
                const float floor_ = __shfl(best - thr, L);
                int nc = 0;
#pragma unroll
                for (int nb = 0; nb < NBLK; ++nb) {
                    const bool in = (lane >> 4) == (L >> 4) && 16 * nb + i < E && score[nb] >= floor_;
                    unsigned bits = (unsigned)((__ballot(in) >> (L & 48)) & 0xffffu);
                    while (bits != 0) {
                        const int e = 16 * nb + __ffs((int)bits) - 1;
                        bits &= bits - 1;
                        if (nc < kCand && lane == 0) s_cand[nc] = e;
                        ++nc;
                    }
                }
                const int tt = __shfl(t, L);
                if (lane == 0) s_nc = nc, s_tt = tt;
            }
            __syncthreads();
            const int nc = s_nc, tt = s_tt;
            int cand[kCand];
#pragma unroll
            for (int c = 0; c < kCand; ++c) cand[c] = s_cand[c < nc ? c : 0];  // spare slots repeat candidate 0
            double top = -DBL_MAX, runner = -DBL_MAX;
            int topi = -1;
            auto offer = [&](double sc, int e) {  // offered in ascending index, strict '>': lowest index wins ties
                if (sc > top) {
                    runner = top;
                    top = sc;
                    topi = e;
                } else if (sc > runner) {
                    runner = sc;
                }
            };
            double sc[kCand];
            if (nc <= 2) {
                rescore<2>(a, tt, cand, sc, s_part);
                offer(sc[0], cand[0]);
                if (nc == 2) offer(sc[1], cand[1]);
            } else if (nc <= kCand) {
                rescore<kCand>(a, tt, cand, sc, s_part);
#pragma unroll
                for (int c = 0; c < kCand; ++c)
                    if (c < nc) offer(sc[c], cand[c]);
            } else {  // many experts that close: every expert is re-scored
                for (int e0 = 0; e0 < E; e0 += kCand) {
#pragma unroll
                    for (int c = 0; c < kCand; ++c) cand[c] = min(e0 + c, E - 1);
                    rescore<kCand>(a, tt, cand, sc, s_part);
#pragma unroll
                    for (int c = 0; c < kCand; ++c)
                        if (e0 + c < E) offer(sc[c], e0 + c);
                }
            }
            if (threadIdx.x == 0) {
                if (topi >= 0) {
                    a.sel[tt] = topi;
                    a.coeff[tt] = (float)top;
                    s_sel[tt - blockIdx.x * 16] = topi;
                }
                if (a.stats != nullptr) {
                    atomicAdd(&a.stats[2], 1);
                    if (nc > 1 && topi >= 0 && (top - runner) < 1e-6 * fmax(fabs(top), DBL_MIN)) atomicAdd(&a.stats[0], 1);
                }
            }
            // rescore() ends with a barrier, so s_cand / s_nc may be rewritten by the next token's owner
        }
    }
    if (a.block_hist != nullptr) {  // integer sums: the order the additions arrive in does not matter
        __syncthreads();
        const int tk = blockIdx.x * 16 + threadIdx.x;
        if (threadIdx.x < 16 && s_sel[threadIdx.x] >= 0)
            atomicAdd(&a.block_hist[(size_t)(tk / a.hist_block) * E + s_sel[threadIdx.x]], 1);
    }
}

template <int NBLK, int WAVES>
hipError_t launch_one(const GateSlabPlan& p, int T, int d, int E, const float* x, const float* cf, float* partials,
                      int* zero_stats, int* zero_hist, int n_hist, hipStream_t stream) {
    const size_t lds = (size_t)16 * NBLK * (p.ks + 4) * sizeof(float);
    const hipError_t err = allow_lds_once<gate_slab_kernel<NBLK, WAVES>>(kSlabLdsLimit);
    if (err != hipSuccess) return err;
    gate_slab_kernel<NBLK, WAVES><<<dim3(p.groups * p.slices), 64 * WAVES, lds, stream>>>(x, cf, partials, T, d, E, p.ks,
                                                                                         p.slices, p.tiles_per_wave, zero_stats, zero_hist, n_hist);
    return hipGetLastError();
}

constexpr int nblk_of(int E) { return E <= 16 ? 1 : (E <= 32 ? 2 : (E <= 64 ? 4 : 8)); }

}  // namespace

bool gate_slab_plan(int T, int d, int E, size_t scratch_floats, GateSlabPlan* plan) {
    if (E > 128 || T < kGateSlabMinTokens || d % kChunk != 0) return false;
    // (slices of 128 << n floats: the kernel takes (row, column) of a slab element by shift and mask)
    const int EP = 16 * nblk_of(E);
    const size_t W = (size_t)E + 2;
    const int tiles = (T + 15) / 16;
    // Slices: as few as give every compute unit eight waves of 16 tokens (a wave keeps 16 KB of loads in
    // flight), no more than the combine launch adds (16), and so that the partial scores stay below a
    // quarter of the input's bytes; the slice has to fit the LDS.
    int best = 0;
    for (int ks = 1024; ks >= kChunk; ks >>= 1) {
        if (d % ks != 0) continue;
        const int S = d / ks;
        if (S < 2) continue;  // one slice needs no second launch: the one-kernel path does that
        if ((size_t)EP * (ks + 4) * sizeof(float) > kSlabLdsLimit) continue;
        if (S > kGateMaxSlices || (size_t)S * W * 4 > (size_t)d) break;
        best = ks;
        if ((long long)tiles * S >= 8 * 256) break;
    }
    if (best == 0) return false;
    GateSlabPlan p{};
    p.ks = best;
    p.slices = d / best;
    if ((size_t)p.slices * T * W > scratch_floats) return false;
    // 8 waves per workgroup (128 tokens share one fill of the slab) unless that leaves compute units idle
    p.waves = (long long)((tiles + 7) / 8) * p.slices >= 256 ? 8 : 4;
    int per_group = p.waves;
    p.tiles_per_wave = 1;
    // with tokens to spare a wave takes several tiles in turn: fewer fills of the slab per token
    while (p.tiles_per_wave < 8 && (long long)((tiles + 2 * per_group - 1) / (2 * per_group)) * p.slices >= 256) {
        per_group *= 2;
        p.tiles_per_wave *= 2;
    }
    p.groups = (tiles + per_group - 1) / per_group;
    *plan = p;
    return true;
}

// Enough for every call of up to T tokens, not only for one of exactly T: the plan cuts d into MORE slices when
// there are fewer tokens (until tiles * slices reaches 8 * 256), so slices(T') * T' is not monotone in T', and a
// caller sizes one workspace for its largest batch and then calls with any smaller one.  slices(T') never grows
// with T', so the largest product on [1, T] sits at the right end of a stretch of constant slice count: at T
// itself or at the last token count before some slice count s makes the plan stop, 16 * (ceil(8 * 256 / s) - 1).
size_t gate_slab_scratch_floats(int T, int d, int E) {
    size_t most = 0;
    auto at = [&](int t) {
        GateSlabPlan p{};
        if (t >= 1 && t <= T && gate_slab_plan(t, d, E, (size_t)-1, &p)) most = std::max(most, (size_t)p.slices * t);
    };
    at(T);
    for (int s = 2; s <= kGateMaxSlices; ++s) at(16 * ((8 * 256 + s - 1) / s - 1));
    return most * ((size_t)E + 2);
}

hipError_t launch_gate_slab(const GateSlabPlan& p, int T, int d, int E, const float* x, const float* folded_centroids,
                            float* partials, hipStream_t stream, int* zero_stats, int* zero_hist, int n_hist) {
    if (p.ks < kChunk || (p.ks & (p.ks - 1)) != 0 || p.slices * p.ks != d || p.groups <= 0 || p.tiles_per_wave <= 0)
        return hipErrorInvalidValue;
    if ((long long)p.groups * p.tiles_per_wave * p.waves * 16 < T) return hipErrorInvalidValue;  // tokens not covered
    if ((size_t)16 * nblk_of(E) * (p.ks + 4) * sizeof(float) > kSlabLdsLimit) return hipErrorInvalidValue;
    if (((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(folded_centroids)) & 15) != 0) return hipErrorInvalidValue;
#define INFMOE_SLAB(NB)                                                                                     \
    return p.waves == 8 ? launch_one<NB, 8>(p, T, d, E, x, folded_centroids, partials, zero_stats, zero_hist, n_hist, stream) \
           : (p.waves == 4 ? launch_one<NB, 4>(p, T, d, E, x, folded_centroids, partials, zero_stats, zero_hist, n_hist, stream) \
                           : hipErrorInvalidValue)
    switch (nblk_of(E)) {
        case 1: INFMOE_SLAB(1);
        case 2: INFMOE_SLAB(2);
        case 4: INFMOE_SLAB(4);
        case 8: INFMOE_SLAB(8);
        default: return hipErrorInvalidValue;
    }
#undef INFMOE_SLAB
}

}  // namespace infmoe

namespace infmoe {

bool gate_combine_ok(int d, int E) { return E <= 128 && d % 4 == 0; }

hipError_t launch_gate_combine(int T, int d, int E, int slices, const float* partials, const float* centroid_stats,
                               const float* x, const float* centroids, const float* gamma, int norm_kind,
                               const float* score_bias, int* sel, float* coeff, int* stats, int* nan_flag,
                               hipStream_t stream, int nan_value, float err_depth, int* block_hist) {
    if (T <= 0) return hipSuccess;
    if (!gate_combine_ok(d, E) || slices < 1 || slices > kGateMaxSlices) return hipErrorInvalidValue;
    CombineArgs a{};
    a.T = T, a.d = d, a.E = E, a.S = slices;
    a.partials = partials, a.cstats = centroid_stats, a.X = x, a.C = centroids, a.gamma = gamma, a.bias = score_bias;
    a.norm_kind = norm_kind, a.sel = sel, a.coeff = coeff, a.stats = stats, a.nan_flag = nan_flag, a.nan_value = nan_value, a.err_depth = err_depth;
    a.block_hist = block_hist, a.hist_block = kCountBlockTokens;
    const dim3 grid((T + 15) / 16);
    switch (nblk_of(E)) {
        case 1: gate_combine_kernel<1><<<grid, 256, 0, stream>>>(a); break;
        case 2: gate_combine_kernel<2><<<grid, 256, 0, stream>>>(a); break;
        case 4: gate_combine_kernel<4><<<grid, 256, 0, stream>>>(a); break;
        default: gate_combine_kernel<8><<<grid, 256, 0, stream>>>(a); break;
    }
    return hipGetLastError();
}

}  // namespace infmoe
