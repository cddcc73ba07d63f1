// Fused gating for gfx950: optional row norm, token x centroid scoring and top-1 selection in
// one pass over the input.  Replaces the chain layernorm_gpu -> cublasSgemm_v2 ->
// expert_select_top1_kernel of the reference (plugin/MoELayerPlugin.cc:315-345,
// plugin/cuda/ops/layernorm.cu:136-188, plugin/cuda/moe.cu:13-76) and removes the
// normalised-input and score-matrix round trips through memory.
//
// Work split: one workgroup (4 waves) owns 16 or 64 tokens and a slice of the embedding dimension,
// which it walks in chunks that are staged through LDS with row-contiguous global loads; each wave
// takes a quarter of every chunk and runs v_mfma_f32_16x16x4_f32 with the tokens as the A rows and
// up to 128 experts (8 column blocks) as the B columns.  The row statistics of the norm are
// accumulated from the same registers that feed the matrix core, and the norm is applied to the
// score tile instead of to the input:
//     rms:      score = rstd * sum_k x_k g_k c_ek
//     centered: score = rstd * (sum_k x_k g_k c_ek - mu * sum_k g_k c_ek)
// Partial tiles of the 4 waves meet in LDS, then 16 lanes reduce one token to
// (best, index, runner-up) with the reference's tie rule (lowest index wins,
// plugin/cuda/moe.cu:62-68).
//
// A compute unit can keep only about its first-level cache's worth of loads in flight, and every
// workgroup reads all centroids, so what bounds the kernel is the traffic through that cache per
// token: 64-token workgroups read a quarter of the centroid bytes per token that 16-token ones do.
// To still fill the chip when there are few tokens, the embedding dimension is split over up to
// 16 workgroups per token group; each writes its partial dot products and row sums to scratch
// memory, and a second launch of the kernel adds them in slice order and does the selection.  (A
// single launch in which the last workgroup to arrive combines the partial sums needs device-wide
// fences, and those cost more here - about 8 us each with the chip busy - than the second launch.)
//
// FP32 accumulation over d terms cannot order two scores closer than its own rounding error,
// so a token whose top-2 gap is below a Cauchy-Schwarz error bound is re-scored by the whole
// workgroup in float64.  Such tokens are rare (about one in a few thousand for Gaussian
// scores); they are counted in stats[2], and those whose float64 gap is below 1e-6 relative
// (no arithmetic can be expected to order them) in stats[0].
#include <hip/hip_runtime.h>

#include <cfloat>
#include <algorithm>
#include <cmath>
#include <type_traits>

#include "kernels.h"

namespace infmoe {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kWaves = 4;  // waves per workgroup; each takes a quarter of every staged K chunk
constexpr int kThreads = 64 * kWaves;
constexpr int kMaxCand = 4;          // near-tied experts the quick float64 re-scoring handles
constexpr int kMaxSlices = 16;       // most workgroups that share one token group's embedding dimension
constexpr int kTargetGroups = 256;   // workgroups wanted per launch: one per compute unit

enum GateMode : int {
    GATE_WHOLE = 0,    // one launch: scores, selection
    GATE_SLICES = 1,   // first of two launches: partial scores of one slice of the embedding dimension
    GATE_COMBINE = 2,  // second launch: add the slices' partial scores, selection
};

// Floats of K staged per step, by tile height (token rows + expert rows + gamma row): two buffers
// of rows x (KC + 4) floats stay below 106 KB.
constexpr int gate_kc(int nblk, int mb) {
    const int rows = 16 * mb + 16 * nblk + 1;
    return rows <= 49 ? 256 : (rows <= 97 ? 128 : 64);
}

struct GateArgs {
    int T, d, E;
    const float* X;
    const float* C;
    const float* gamma;
    const float* Cf;      // centroids * gamma, or null
    const float* cstats;  // [2E] sum and norm of the rows of Cf, or null
    int norm_kind;
    const float* bias;
    int* sel;
    float* coeff;
    int* stats;
    int mode;       // GateMode
    int slices;     // workgroups per token group
    int steps_per;  // K chunks per slice
    int* nan_flag;    // null, or an int (host memory the device can write) set to nan_value when a token has no orderable score
    int nan_value;
    float err_depth;  // n of the error bound of a score (see gate_err_depth)
    float* partials;  // [slices][T][E + 2]: dot products, row sum, row sum of squares
    float* gpart;     // [groups][slices][2E]: sum and sum of squares of the folded centroid slice
    int* zero_stats;  // GATE_SLICES only: null, or the 4 ints the later combine launch counts into, set to zero here
};

// Four floats of a row starting at k.  With VEC (d % 4 == 0, 16-byte aligned rows) the load is
// unconditional: a k beyond the row is clamped to the last float4 and the caller discards the value
// when it uses it, so that no load sits inside a branch and many can be in flight.
template <bool VEC>
__device__ __forceinline__ v4f load4(const float* __restrict__ row, int k, int d) {
    v4f v = {0.f, 0.f, 0.f, 0.f};
    if (VEC) {
        v = *reinterpret_cast<const v4f*>(row + min(k, d - 4));
    } else {
        if (k + 0 < d) v.x = row[k + 0];
        if (k + 1 < d) v.y = row[k + 1];
        if (k + 2 < d) v.z = row[k + 2];
        if (k + 3 < d) v.w = row[k + 3];
    }
    return v;
}

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

// NBLK: 16-expert column blocks handled per pass (experts per pass = 16*NBLK).
// MB: 16-token row blocks per workgroup.  With MB = 1 the four waves split every K chunk and their
// partial tiles meet in LDS; with MB = 4 each wave owns 16 tokens and walks the whole chunk.
// PRE: the caller supplies the centroids already multiplied by gamma (Cf) and, per expert, the sum
// and the Euclidean norm of that product (cstats[0..E) and cstats[E..2E)): they depend on the layer's
// parameters only, so the layer computes them once instead of every workgroup of every call.
template <int NBLK, int MB, bool VEC, bool GAMMA, bool PRE>
__global__ __launch_bounds__(kThreads) void gate_top1_kernel(const GateArgs arg) {
    constexpr int EP = 16 * NBLK;
    constexpr int TM = 16 * MB;
    constexpr bool SPLITK = MB == 1;  // the waves split K (and meet in s_part) rather than the tokens
    __shared__ float s_score[TM][EP + 1];
    __shared__ float s_part[SPLITK ? kWaves : 1][SPLITK ? 16 : 1][SPLITK ? EP + 1 : 1];
    __shared__ float s_s1[kWaves][16], s_s2[kWaves][16];
    __shared__ float s_g1[kWaves][EP], s_g2[kWaves][EP];
    __shared__ float s_a1[TM], s_a2[TM];
    __shared__ float s_mu[TM], s_rstd[TM], s_xnorm[TM];
    __shared__ float s_G[EP], s_cn[EP];
    __shared__ float s_best[TM], s_second[TM], s_thr[TM], s_cnmax;
    __shared__ int s_besti[TM], s_rescue[TM];
    __shared__ double s_red[kWaves][2];
    __shared__ double s_sc64[EP];
    __shared__ double s_bcast[2];
    __shared__ int s_cand[kMaxCand], s_ncand;
    __shared__ double s_red2[kWaves][2 + 2 * kMaxCand];

    const int T = arg.T, d = arg.d, E = arg.E, norm_kind = arg.norm_kind;
    const float* __restrict__ X = arg.X;
    const float* __restrict__ C = arg.C;
    const float* __restrict__ gamma = arg.gamma;
    const float* __restrict__ bias = arg.bias;
    int* __restrict__ sel = arg.sel;
    float* __restrict__ coeff = arg.coeff;
    int* __restrict__ stats = arg.stats;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int i = lane & 15;   // A row (token) / B column (expert) this lane feeds
    const int kq = lane >> 4;  // which float4 of the 16-float chunk this lane feeds
    constexpr bool use_gamma = GAMMA;  // the norm's gamma is folded into the centroids as they are loaded

    // Token group g, slice j of the embedding dimension.
    const int S = arg.slices, mode = arg.mode;
    const int g = mode == GATE_SLICES ? blockIdx.x / S : blockIdx.x;
    const int j = mode == GATE_SLICES ? blockIdx.x % S : 0;
    const int t0 = g * TM;
    // the routing statistics the combine launch counts into start at zero (saves a fill launch)
    if (mode == GATE_SLICES && arg.zero_stats != nullptr && blockIdx.x == 0 && tid < 4) arg.zero_stats[tid] = 0;

    if (tid < TM) {
        s_best[tid] = -FLT_MAX;  // plugin/cuda/moe.cu:26-27
        s_second[tid] = -FLT_MAX;
        s_besti[tid] = -1;
        s_rescue[tid] = 0;
    }
    if (tid == 0) s_cnmax = 0.f;

    // Staging tile in LDS, two buffers of ROWS x (KC + 4) floats: the token rows, EP centroid rows and
    // (with a norm) the gamma row, KC floats of K at a time.  Every wave-wide global load reads whole
    // 512-byte or 1-KB stretches of one or two rows, which is what DRAM serves best; the MFMA operand
    // layout (a lane needs 16 bytes of "its" row) is produced by the LDS reads, not by the global loads.
    constexpr int KC = gate_kc(NBLK, MB);
    constexpr int KC4 = KC / 4, LD = KC + 4;
    constexpr bool GROW = GAMMA && !PRE;  // stage a gamma row and fold it into the centroids here
    constexpr int ROWS = TM + EP + (GROW ? 1 : 0);
    constexpr int NL = (ROWS * KC4 + kThreads - 1) / kThreads;  // 16-byte loads per thread per step
    extern __shared__ __align__(16) float s_tile[];
    const int nsteps = (d + KC - 1) / KC;
    const int s_begin = j * arg.steps_per;
    const int nst = min(nsteps - s_begin, arg.steps_per);  // >= 1 by the launcher's choice of slices
    const int k_lo = s_begin * KC, k_hi = min(d, (s_begin + nst) * KC);
    const int W = E + 2;  // floats per token and slice in `partials`

    // Scores of the pass over experts e0 .. e0+EP from what is in LDS: raw dot products in s_score, raw
    // row sums in s_a1 / s_a2, and (without PRE) the centroid sums in s_G and sums of squares in s_cn.
    auto finish_pass = [&](int e0) {
        if (tid < TM) {
            const float a1 = s_a1[tid], a2 = s_a2[tid];
            float mu = 0.f, rstd = 1.f;
            if (norm_kind == NORM_RMS) {
                rstd = 1.0f / sqrtf(a2 / (float)d + kNormEps);
            } else if (norm_kind == NORM_CENTERED) {
                mu = a1 / (float)d;
                rstd = 1.0f / sqrtf(fmaxf(a2 / (float)d - mu * mu, 0.f) + kNormEps);
            }
            s_mu[tid] = mu;
            s_rstd[tid] = rstd;
            s_xnorm[tid] = sqrtf(a2);
        } else if (tid >= 64 && tid < 64 + EP) {
            const int e = tid - 64;
            if (PRE) {
                const int ee = min(e0 + e, E - 1);
                s_G[e] = arg.cstats[ee];
                s_cn[e] = arg.cstats[E + ee];
            } else {
                s_cn[e] = sqrtf(s_cn[e]);
            }
        }
        __syncthreads();
        for (int idx = tid; idx < TM * EP; idx += kThreads) {
            const int tok = idx / EP, e = idx - tok * EP;
            float sc = s_rstd[tok] * (s_score[tok][e] - s_mu[tok] * s_G[e]);
            if (bias != nullptr && e0 + e < E) sc += bias[e0 + e];
            s_score[tok][e] = sc;
        }
        __syncthreads();

        const int nvalid = min(E - e0, EP);
        float cmax = 0.f;
        for (int e = lane; e < nvalid; e += 64) cmax = fmaxf(cmax, s_cn[e]);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) cmax = fmaxf(cmax, __shfl_xor(cmax, off));
        if (tid == 0) s_cnmax = fmaxf(s_cnmax, cmax);
        // 16 lanes reduce one token; a wave takes four tokens at a time
#pragma unroll 1
        for (int q = 0; q < MB; ++q) {
            const int tok = (TM / kWaves) * wave + 4 * q + kq;
            float v = -FLT_MAX;
            int vi = -1;
            for (int e = i; e < nvalid; e += 16) {
                const float s = s_score[tok][e];
                if (s > v) {
                    v = s;
                    vi = e0 + e;
                }
            }
#pragma unroll
            for (int off = 8; off > 0; off >>= 1) {
                const float ov = __shfl_xor(v, off);
                const int oi = __shfl_xor(vi, off);
                if (ov > v || (ov == v && (unsigned)oi < (unsigned)vi)) {
                    v = ov;
                    vi = oi;
                }
            }
            float v2 = -FLT_MAX;
            for (int e = i; e < nvalid; e += 16) {
                const float s = s_score[tok][e];
                if (e0 + e != vi && s > v2) v2 = s;
            }
#pragma unroll
            for (int off = 8; off > 0; off >>= 1) v2 = fmaxf(v2, __shfl_xor(v2, off));
            if (i == 0) {
                const float B = s_best[tok];
                if (v > B) {
                    s_second[tok] = fmaxf(B, v2);
                    s_best[tok] = v;
                    s_besti[tok] = vi;
                } else {
                    s_second[tok] = fmaxf(s_second[tok], v);
                }
            }
        }
        __syncthreads();
    };

    for (int e0 = 0; mode != GATE_COMBINE && e0 < E; e0 += EP) {
        v4f acc[2][NBLK];  // two sets, for even and odd 16-float groups: twice as many independent chains
        float gs[NBLK], cn[NBLK], s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int nb = 0; nb < NBLK; ++nb) {
            acc[0][nb] = v4f{0.f, 0.f, 0.f, 0.f};
            acc[1][nb] = v4f{0.f, 0.f, 0.f, 0.f};
            gs[nb] = 0.f;
            cn[nb] = 0.f;
        }

        // item l of this thread: float4 c4 of tile row `row`; rows beyond T / E are clamped (their
        // scores are never used), items beyond the tile repeat its last one
        const float* rptr[NL];
        int lds_off[NL], kcol[NL];
#pragma unroll
        for (int l = 0; l < NL; ++l) {
            const int idx = min(tid + l * kThreads, ROWS * KC4 - 1);
            const int row = idx / KC4, c4 = idx % KC4;
            rptr[l] = row < TM ? X + (size_t)min(t0 + row, T - 1) * d
                      : row < TM + EP ? (PRE ? arg.Cf : C) + (size_t)min(e0 + row - TM, E - 1) * d
                                      : gamma;
            lds_off[l] = row * LD + 4 * c4;
            kcol[l] = 4 * c4;
        }
        // Two register sets: the loads of step s + 2 are issued before the arithmetic of step s and
        // written to LDS one step later, so about two steps' worth of bytes is in flight per CU - the
        // arithmetic of one step is shorter than a memory round trip and would not cover it.
        v4f rg[2][NL];
        auto load_step = [&](auto setc, int sl) {
            constexpr int P = decltype(setc)::value;
            const int k0 = k_lo + min(sl, nst - 1) * KC;
#pragma unroll
            for (int l = 0; l < NL; ++l) rg[P][l] = load4<VEC>(rptr[l], k0 + kcol[l], d);
        };
        auto store_step = [&](auto setc, int buf, int sl) {
            constexpr int P = decltype(setc)::value;
            const int k0 = k_lo + sl * KC;
            const v4f zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int l = 0; l < NL; ++l)  // k beyond the slice was read from a clamped address: store zeros
                *reinterpret_cast<v4f*>(s_tile + buf * (ROWS * LD) + lds_off[l]) = (k0 + kcol[l] < k_hi) ? rg[P][l] : zero;
        };
        auto compute_step = [&](int buf) {
            // SPLITK: this wave's quarter of the chunk, token rows 0..15; otherwise the whole chunk and
            // token rows 16*wave .. 16*wave+15
            constexpr int NG = (SPLITK ? KC / kWaves : KC) / 16;
            const float* tile = s_tile + buf * (ROWS * LD) + (SPLITK ? wave * (KC / kWaves) : 0) + 4 * kq;
            const float* xrow = tile + ((SPLITK ? 0 : 16 * wave) + i) * LD;
#pragma unroll
            for (int gq = 0; gq < NG; ++gq) {
                const v4f xv = *reinterpret_cast<const v4f*>(xrow + 16 * gq);
                v4f gv = {1.f, 1.f, 1.f, 1.f};
                if (GROW) gv = *reinterpret_cast<const v4f*>(tile + (TM + EP) * LD + 16 * gq);
                s1 += (xv.x + xv.y) + (xv.z + xv.w);
                s2 += (xv.x * xv.x + xv.y * xv.y) + (xv.z * xv.z + xv.w * xv.w);
                v4f cv[NBLK];
#pragma unroll
                for (int nb = 0; nb < NBLK; ++nb) {
                    cv[nb] = *reinterpret_cast<const v4f*>(tile + (TM + 16 * nb + i) * LD + 16 * gq);
                    if (!PRE) {
                        cv[nb] *= gv;
                        gs[nb] += (cv[nb].x + cv[nb].y) + (cv[nb].z + cv[nb].w);
                        cn[nb] += (cv[nb].x * cv[nb].x + cv[nb].y * cv[nb].y) + (cv[nb].z * cv[nb].z + cv[nb].w * cv[nb].w);
                    }
                }
                // The k order inside a 16-float group is permuted identically for A and B, which a dot
                // product does not see: step c multiplies element c of every lane's float4.  Consecutive
                // instructions go to different accumulators so that none waits for its predecessor.
#pragma unroll
                for (int c = 0; c < 4; ++c)
#pragma unroll
                    for (int nb = 0; nb < NBLK; ++nb)
                        acc[gq & 1][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[c], cv[nb][c], acc[gq & 1][nb], 0, 0, 0);
            }
        };
        // step sl computes from buffer sl & 1; set P holds step sl + 1, the other set receives step sl + 2
        auto step = [&](auto setc, int sl) {
            constexpr int P = decltype(setc)::value;
            load_step(std::integral_constant<int, 1 - P>{}, sl + 2);
            __builtin_amdgcn_sched_barrier(0);  // the loads go out before the arithmetic, not next to their use
            compute_step(sl & 1);
            store_step(setc, (sl + 1) & 1, sl + 1);
            __syncthreads();
        };
        const std::integral_constant<int, 0> set0{};
        const std::integral_constant<int, 1> set1{};
        __syncthreads();  // the previous pass is done with the tile
        load_step(set1, 0);
        store_step(set1, 0, 0);
        load_step(set0, 1);
        __syncthreads();
        // Steps go in pairs without a branch between them: a conditional second step is a block of its
        // own, and the compiler then moves the first step's loads down into it, next to the LDS stores
        // that use them, which exposes a full memory round trip per pair.  With an odd number of
        // chunks the last step works on a tile of zeros (its predecessor stored k >= k_hi as zeros).
        for (int sl = 0; sl < nst; sl += 2) {
            step(set0, sl);
            step(set1, sl + 1);
        }

        // lanes i, i+16, i+32, i+48 hold the four float4 slots of one row
        s1 += __shfl_xor(s1, 16);
        s1 += __shfl_xor(s1, 32);
        s2 += __shfl_xor(s2, 16);
        s2 += __shfl_xor(s2, 32);
        if (kq == 0) {
            s_s1[wave][i] = s1;
            s_s2[wave][i] = s2;
        }
#pragma unroll
        for (int nb = 0; nb < NBLK; ++nb) {
            float gsum = gs[nb], n2 = cn[nb];
            gsum += __shfl_xor(gsum, 16);
            gsum += __shfl_xor(gsum, 32);
            n2 += __shfl_xor(n2, 16);
            n2 += __shfl_xor(n2, 32);
            if (kq == 0) {
                s_g1[wave][16 * nb + i] = gsum;
                s_g2[wave][16 * nb + i] = n2;
            }
            // D layout of 16x16x4: lane holds column (lane & 15), rows 4*(lane >> 4) + r
            const v4f sum = acc[0][nb] + acc[1][nb];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if (SPLITK) s_part[wave][4 * kq + r][16 * nb + i] = sum[r];
                else s_score[16 * wave + 4 * kq + r][16 * nb + i] = sum[r];
            }
        }
        __syncthreads();
        if (SPLITK) {  // the four waves hold partial sums over K of the same 16 tokens
            for (int idx = tid; idx < 16 * EP; idx += kThreads) {
                const int tok = idx / EP, e = idx - tok * EP;
                float dot = 0.f;
#pragma unroll
                for (int w = 0; w < kWaves; ++w) dot += s_part[SPLITK ? w : 0][SPLITK ? tok : 0][SPLITK ? e : 0];
                s_score[tok][e] = dot;
            }
        }
        if (tid < TM) {
            float a1 = 0.f, a2 = 0.f;
            if (SPLITK) {
#pragma unroll
                for (int w = 0; w < kWaves; ++w) a1 += s_s1[w][tid], a2 += s_s2[w][tid];
            } else {  // wave tid / 16 owns this token
                a1 = s_s1[tid >> 4][tid & 15], a2 = s_s2[tid >> 4][tid & 15];
            }
            s_a1[tid] = a1;
            s_a2[tid] = a2;
        } else if (!PRE && tid >= 64 && tid < 64 + EP) {
            const int e = tid - 64;
            float g1 = 0.f, g2 = 0.f;
            if (SPLITK) {
#pragma unroll
                for (int w = 0; w < kWaves; ++w) g1 += s_g1[w][e], g2 += s_g2[w][e];
            } else {  // every wave saw all of K
                g1 = s_g1[0][e], g2 = s_g2[0][e];
            }
            s_G[e] = g1;
            s_cn[e] = g2;
        }
        __syncthreads();

        if (mode == GATE_WHOLE) {
            finish_pass(e0);
        } else {
            // this slice's share of the pass goes to scratch memory
            float* part = arg.partials + (size_t)j * T * W;
            for (int idx = tid; idx < TM * EP; idx += kThreads) {
                const int tok = idx / EP, e = idx - tok * EP;
                if (t0 + tok < T && e0 + e < E) part[(size_t)(t0 + tok) * W + e0 + e] = s_score[tok][e];
            }
            if (e0 == 0 && tid < TM && t0 + tid < T) {
                part[(size_t)(t0 + tid) * W + E] = s_a1[tid];
                part[(size_t)(t0 + tid) * W + E + 1] = s_a2[tid];
            }
            if (!PRE && tid >= 64 && tid < 64 + EP && e0 + tid - 64 < E) {
                float* gp = arg.gpart + ((size_t)g * S + j) * 2 * E;
                gp[e0 + tid - 64] = s_G[tid - 64];
                gp[E + e0 + tid - 64] = s_cn[tid - 64];
            }
            if (e0 + EP < E) __syncthreads();  // the next pass overwrites what is being read here
        }
    }

    if (mode == GATE_SLICES) return;
    if (mode == GATE_COMBINE) {
        for (int e0 = 0; e0 < E; e0 += EP) {
            for (int idx = tid; idx < TM * EP; idx += kThreads) {
                const int tok = idx / EP, e = idx - tok * EP;
                float sum = 0.f;
                if (t0 + tok < T && e0 + e < E) {
                    // all slices' loads go out together (a loop over a run-time count waits for each
                    // in turn); the sum is taken in slice order
                    const float* src = arg.partials + (size_t)(t0 + tok) * W + e0 + e;
                    float v[kMaxSlices];
#pragma unroll
                    for (int jj = 0; jj < kMaxSlices; ++jj) v[jj] = src[(size_t)min(jj, S - 1) * T * W];
#pragma unroll
                    for (int jj = 0; jj < kMaxSlices; ++jj) sum += jj < S ? v[jj] : 0.f;
                }
                s_score[tok][e] = sum;
            }
            if (tid < TM) {
                float a1 = 0.f, a2 = 0.f;
                if (t0 + tid < T) {
                    const float* src = arg.partials + (size_t)(t0 + tid) * W + E;
                    float v1[kMaxSlices], v2[kMaxSlices];
#pragma unroll
                    for (int jj = 0; jj < kMaxSlices; ++jj) {
                        v1[jj] = src[(size_t)min(jj, S - 1) * T * W];
                        v2[jj] = src[(size_t)min(jj, S - 1) * T * W + 1];
                    }
#pragma unroll
                    for (int jj = 0; jj < kMaxSlices; ++jj) a1 += jj < S ? v1[jj] : 0.f, a2 += jj < S ? v2[jj] : 0.f;
                }
                s_a1[tid] = a1;
                s_a2[tid] = a2;
            } else if (!PRE && tid >= 64 && tid < 64 + EP) {
                const int e = tid - 64;
                float g1 = 0.f, g2 = 0.f;
                if (e0 + e < E) {
                    const float* src = arg.gpart + (size_t)g * S * 2 * E + e0 + e;
                    for (int jj = 0; jj < S; ++jj) g1 += src[(size_t)jj * 2 * E], g2 += src[(size_t)jj * 2 * E + E];
                }
                s_G[e] = g1;
                s_cn[e] = g2;
            }
            __syncthreads();
            finish_pass(e0);
        }
    }

    // ---- decide, per token, whether FP32 ordered the top two safely
    if (tid < TM) {
        const int t = t0 + tid;
        if (t < T) {
            const float B = s_best[tid], S2 = s_second[tid];
            const int I = s_besti[tid];
            if (I < 0) {  // no orderable score: the reference asserts (plugin/cuda/moe.cu:70)
                sel[t] = 0;
                coeff[t] = __builtin_nanf("");  // marks the row: the combine step writes NaN for it
                if (stats) atomicAdd(&stats[1], 1);
                if (arg.nan_flag) *reinterpret_cast<volatile int*>(arg.nan_flag) = arg.nan_value;
            } else {
                sel[t] = I;
                coeff[t] = B;
                const float bound = arg.err_depth * FLT_EPSILON * s_rstd[tid] * s_xnorm[tid] * s_cnmax;  // see gate_err_depth
                s_thr[tid] = fmaxf(bound, 4e-6f * fabsf(B));
                if (E > 1 && (B - S2) < s_thr[tid]) s_rescue[tid] = 1;
            }
        }
    }
    __syncthreads();

    // ---- float64 re-scoring of the flagged tokens by the whole workgroup: the waves share the
    // row statistics, then each wave takes every kWaves-th expert and the scores meet in LDS
    for (int tok = 0; tok < TM; ++tok) {
        if (!s_rescue[tok]) continue;  // uniform: read from LDS after the barrier
        // Quick path (one pass over experts, at most kMaxCand experts within the bound of the best):
        // only those candidates can win, so one sweep over d computes, in float64, the row statistics
        // and the candidates' dot products together - a single round of loads instead of one per
        // expert group.
        if (E <= EP) {
            if (tid == 0) {
                int n = 0;
                const float floor_ = s_best[tok] - s_thr[tok];
                for (int e = 0; e < E; ++e)
                    if (s_score[tok][e] >= floor_) {
                        if (n < kMaxCand) s_cand[n] = e;
                        ++n;
                    }
                s_ncand = n;
            }
            __syncthreads();
            const int nc = s_ncand;
            if (nc <= kMaxCand) {
                const int t = t0 + tok;
                const float* xr = X + (size_t)t * d;
                const float* cr[kMaxCand];
#pragma unroll
                for (int c = 0; c < kMaxCand; ++c) cr[c] = C + (size_t)s_cand[c < nc ? c : 0] * d;  // spare slots repeat candidate 0
                double a1 = 0.0, a2 = 0.0, dx[kMaxCand], dg[kMaxCand];
#pragma unroll
                for (int c = 0; c < kMaxCand; ++c) dx[c] = 0.0, dg[c] = 0.0;
                if (VEC) {
#pragma unroll 4
                    for (int k = 4 * tid; k < d; k += 4 * kThreads) {
                        const v4f xv = *reinterpret_cast<const v4f*>(xr + k);
                        v4f gv = {1.f, 1.f, 1.f, 1.f};
                        if (use_gamma) gv = *reinterpret_cast<const v4f*>(gamma + k);
                        const double x0 = xv.x, x1 = xv.y, x2 = xv.z, x3 = xv.w;
                        a1 += (x0 + x1) + (x2 + x3);
                        a2 += (x0 * x0 + x1 * x1) + (x2 * x2 + x3 * x3);
#pragma unroll
                        for (int c = 0; c < kMaxCand; ++c) {
                            const v4f cv = *reinterpret_cast<const v4f*>(cr[c] + k);
                            const double g0 = (double)gv.x * (double)cv.x, g1 = (double)gv.y * (double)cv.y;
                            const double g2 = (double)gv.z * (double)cv.z, g3 = (double)gv.w * (double)cv.w;
                            dx[c] += (x0 * g0 + x1 * g1) + (x2 * g2 + x3 * g3);
                            dg[c] += (g0 + g1) + (g2 + g3);
                        }
                    }
                } else {
                    for (int k = tid; k < d; k += kThreads) {
                        const double xv = xr[k], gv = use_gamma ? (double)gamma[k] : 1.0;
                        a1 += xv;
                        a2 += xv * xv;
#pragma unroll
                        for (int c = 0; c < kMaxCand; ++c) {
                            const double gc = gv * (double)cr[c][k];
                            dx[c] += xv * gc;
                            dg[c] += gc;
                        }
                    }
                }
                a1 = wave_sum(a1);
                a2 = wave_sum(a2);
#pragma unroll
                for (int c = 0; c < kMaxCand; ++c) dx[c] = wave_sum(dx[c]), dg[c] = wave_sum(dg[c]);
                if (lane == 0) {
                    s_red2[wave][0] = a1;
                    s_red2[wave][1] = a2;
#pragma unroll
                    for (int c = 0; c < kMaxCand; ++c) s_red2[wave][2 + c] = dx[c], s_red2[wave][2 + kMaxCand + c] = dg[c];
                }
                __syncthreads();
                if (tid == 0) {
                    double r[2 + 2 * kMaxCand];
                    for (int q = 0; q < 2 + 2 * kMaxCand; ++q) {
                        r[q] = 0.0;
                        for (int w = 0; w < kWaves; ++w) r[q] += s_red2[w][q];
                    }
                    double mu = 0.0, rstd = 1.0;
                    if (norm_kind == NORM_RMS) {
                        rstd = 1.0 / sqrt(r[1] / d + 1e-6);
                    } else if (norm_kind == NORM_CENTERED) {
                        mu = r[0] / d;
                        rstd = 1.0 / sqrt(fmax(r[1] / d - mu * mu, 0.0) + 1e-6);
                    }
                    double best = -DBL_MAX, second = -DBL_MAX;
                    int besti = -1;
                    for (int c = 0; c < nc; ++c) {  // candidates are in ascending expert order: lowest index wins ties
                        double sc = rstd * (r[2 + c] - mu * r[2 + kMaxCand + c]);
                        if (bias != nullptr) sc += (double)bias[s_cand[c]];
                        if (sc > best) {
                            second = best;
                            best = sc;
                            besti = s_cand[c];
                        } else if (sc > second) {
                            second = sc;
                        }
                    }
                    if (besti >= 0) {
                        sel[t] = besti;
                        coeff[t] = (float)best;
                    }
                    if (stats) {
                        atomicAdd(&stats[2], 1);
                        if (nc > 1 && besti >= 0 && (best - second) < 1e-6 * fmax(fabs(best), DBL_MIN)) atomicAdd(&stats[0], 1);
                    }
                }
                __syncthreads();
                continue;
            }
        }
        // General path: every expert is re-scored.
        const int t = t0 + tok;
        const float* xr = X + (size_t)t * d;
        double a1 = 0.0, a2 = 0.0;
        for (int k = tid; k < d; k += kThreads) {
            const double v = xr[k];
            a1 += v;
            a2 += v * v;
        }
        a1 = wave_sum(a1);
        a2 = wave_sum(a2);
        if (lane == 0) {
            s_red[wave][0] = a1;
            s_red[wave][1] = a2;
        }
        __syncthreads();
        if (tid == 0) {
            double t1 = 0.0, t2 = 0.0;
            for (int w = 0; w < kWaves; ++w) t1 += s_red[w][0], t2 += s_red[w][1];
            double mu = 0.0, rstd = 1.0;
            if (norm_kind == NORM_RMS) {
                rstd = 1.0 / sqrt(t2 / d + 1e-6);
            } else if (norm_kind == NORM_CENTERED) {
                mu = t1 / d;
                rstd = 1.0 / sqrt(fmax(t2 / d - mu * mu, 0.0) + 1e-6);
            }
            s_bcast[0] = mu;
            s_bcast[1] = rstd;
        }
        __syncthreads();
        const double mu = s_bcast[0], rstd = s_bcast[1];
        double best = -DBL_MAX, second = -DBL_MAX;
        int besti = -1;
        for (int e0 = 0; e0 < E; e0 += EP) {
            const int nvalid = min(E - e0, EP);
            // wave w scores experts w, w + kWaves, ... of this pass; the k loop is outside so that
            // x and gamma are loaded once per slice and all of the wave's centroid loads fly together
            constexpr int EPW = EP / kWaves;
            double a[EPW];
            const float* cr[EPW];
#pragma unroll
            for (int j = 0; j < EPW; ++j) {
                a[j] = 0.0;
                cr[j] = C + (size_t)(e0 + min(wave + j * kWaves, nvalid - 1)) * d;  // clamped: extra results are dropped
            }
            if (VEC) {
#pragma unroll 4
                for (int k = 4 * lane; k < d; k += 256) {
                    const v4f xv = *reinterpret_cast<const v4f*>(xr + k);
                    v4f gv = {1.f, 1.f, 1.f, 1.f};
                    if (use_gamma) gv = *reinterpret_cast<const v4f*>(gamma + k);
                    const double x0 = ((double)xv.x - mu) * (double)gv.x, x1 = ((double)xv.y - mu) * (double)gv.y;
                    const double x2 = ((double)xv.z - mu) * (double)gv.z, x3 = ((double)xv.w - mu) * (double)gv.w;
#pragma unroll
                    for (int j = 0; j < EPW; ++j) {
                        const v4f cv = *reinterpret_cast<const v4f*>(cr[j] + k);
                        a[j] += (x0 * (double)cv.x + x1 * (double)cv.y) + (x2 * (double)cv.z + x3 * (double)cv.w);
                    }
                }
            } else {
                for (int k = lane; k < d; k += 64) {
                    const double xg = ((double)xr[k] - mu) * (use_gamma ? (double)gamma[k] : 1.0);
#pragma unroll
                    for (int j = 0; j < EPW; ++j) a[j] += xg * (double)cr[j][k];
                }
            }
#pragma unroll
            for (int j = 0; j < EPW; ++j) {
                const double sum = wave_sum(a[j]);
                if (lane == 0 && wave + j * kWaves < nvalid) s_sc64[wave + j * kWaves] = sum;
            }
            __syncthreads();
            if (tid == 0) {
                for (int e = 0; e < nvalid; ++e) {  // ascending index, strict '>': lowest index wins ties
                    double sc = rstd * s_sc64[e];
                    if (bias != nullptr) sc += (double)bias[e0 + e];
                    if (sc > best) {
                        second = best;
                        best = sc;
                        besti = e0 + e;
                    } else if (sc > second) {
                        second = sc;
                    }
                }
            }
            __syncthreads();
        }
        if (tid == 0) {
            if (besti >= 0) {
                sel[t] = besti;
                coeff[t] = (float)best;
            }
            if (stats) {
                atomicAdd(&stats[2], 1);
                if (besti >= 0 && (best - second) < 1e-6 * fmax(fabs(best), DBL_MIN)) atomicAdd(&stats[0], 1);
            }
        }
    }
}

// centroids * gamma and, per expert, the sum and the Euclidean norm of that product: what
// fold_centroids_host computes, for callers that hand over the plain centroids on every call.
__global__ __launch_bounds__(kThreads) void fold_centroids_kernel(int d, int E, const float* __restrict__ C,
                                                                  const float* __restrict__ gamma,
                                                                  float* __restrict__ folded, float* __restrict__ cstats) {
    __shared__ double s_red[kWaves][2];
    const int e = blockIdx.x, tid = threadIdx.x;
    double sum = 0.0, sq = 0.0;
    for (int k = tid; k < d; k += kThreads) {
        const float v = gamma != nullptr ? C[(size_t)e * d + k] * gamma[k] : C[(size_t)e * d + k];
        folded[(size_t)e * d + k] = v;
        sum += v;
        sq += (double)v * v;
    }
    sum = wave_sum(sum);
    sq = wave_sum(sq);
    if ((tid & 63) == 0) s_red[tid >> 6][0] = sum, s_red[tid >> 6][1] = sq;
    __syncthreads();
    if (tid == 0) {
        double a = 0.0, b = 0.0;
        for (int w = 0; w < kWaves; ++w) a += s_red[w][0], b += s_red[w][1];
        cstats[e] = (float)a;
        cstats[E + e] = (float)sqrt(b);
    }
}

// floats at the end of the scratch that hold the folded centroids and their statistics
size_t gate_fold_floats(int d, int E) { return (((size_t)E * d + 3) & ~(size_t)3) + (((size_t)2 * E + 3) & ~(size_t)3); }

// How a call is split into workgroups.
struct GatePlan {
    int mb;         // 16-token blocks per workgroup: 1 or 4
    int groups;     // token groups
    int slices;     // workgroups per token group
    int steps_per;  // K chunks per slice
};

constexpr int nblk_for(int E) { return E <= 16 ? 1 : (E <= 32 ? 2 : (E <= 64 ? 4 : 8)); }

}  // namespace

// Which two scores FP32 can order.  A score is rstd * (sum_k x_k (g c)_k [- mu * sum_k (g c)_k]); every path here
// forms the sum as chains of matrix-core accumulations (one instruction adds four products to a running sum),
// two chains per slice added once, then the slices (and, in one form, the four waves' quarters) in a fixed
// order.  For a summation of that shape the standard bound is |computed - exact| <= n u sum_k |x_k (g c)_k|
// with u = 2^-24 and n the longest chain of roundings a term passes through: the chain's length (slice / 8
// instructions), three roundings inside an instruction, one for the product g c held in FP32, one for the two
// chains, the slices, the waves.  By Cauchy-Schwarz sum_k |x_k (g c)_k| <= |x| |g c|, so each score is within
// n u rstd |x| max_e |g c_e| of its exact value, and two scores further apart than twice that - n eps rstd |x|
// max|g c|, eps = 2 u = FLT_EPSILON - are ordered as the exact ones.  The centered norm subtracts mu * sum (g c):
// the error of mu, at most n u |x| / sqrt(d), times |sum g c| <= sqrt(d) |g c| has the same form once more, so n
// doubles.  n comes from the launch plan (`err_depth`).  This is a worst-case bound: a token inside it (about
// one in 400 for Gaussian scores at d = 4096) is re-scored in float64, which costs its workgroup one sweep over
// the row.  (The factor was 8 before, an empirical value a tenth of the bound.)
float gate_err_depth(int slice_floats, int slices, int norm_kind) {
    const float n = (float)(slice_floats / 8 + slices + 3 + 1 + 1 + 3);
    return norm_kind == NORM_CENTERED ? 2.f * n : n;
}

namespace {

GatePlan gate_plan(int T, int d, int E, bool vec, size_t scratch_floats) {
    const int nblk = nblk_for(E);
    const int W = E + 2;
    auto slices_for = [&](int mb, GatePlan* p) {
        const int kc = gate_kc(nblk, mb);
        const int nsteps = (d + kc - 1) / kc;
        const int groups = (T + 16 * mb - 1) / (16 * mb);
        int want = (kTargetGroups + groups - 1) / groups;
        want = std::min(want, std::min(kMaxSlices, nsteps));
        want = std::min(want, std::max(1, d / (2 * W)));  // partial sums stay a fraction of the input's bytes
        const int per = (nsteps + want - 1) / want;
        p->mb = mb, p->groups = groups, p->steps_per = per, p->slices = (nsteps + per - 1) / per;
        if (p->slices > 1 && (size_t)p->slices * T * W + (size_t)groups * p->slices * 2 * E > scratch_floats) {
            p->slices = 1;
            p->steps_per = nsteps;
        }
    };
    GatePlan wide{}, narrow{};
    slices_for(1, &narrow);
    if (!vec || T < 64 * kTargetGroups) return narrow;
    // 64-token workgroups move a quarter of the centroid bytes per token; take them when they give
    // every compute unit a workgroup without slicing (measured at 4096 tokens x 4096 x 32 experts:
    // 64 tokens x 4 slices 46 us, 16 tokens unsliced 32 us)
    slices_for(4, &wide);
    wide.slices = 1;
    wide.steps_per = (d + gate_kc(nblk, 4) - 1) / gate_kc(nblk, 4);
    return wide;
}

// Which launches of a sliced call are issued here: the slices' partial scores may already be in a.partials
// (written by the slab launch), and the combine may be left to the wave-per-four-tokens kernel.
enum : int { kLaunchSlices = 1, kLaunchCombine = 2 };
template <int NBLK>
hipError_t launch_nblk(GateArgs a, bool vec, bool pre, bool use_gamma, const GatePlan& plan, hipStream_t stream,
                       int what = kLaunchSlices | kLaunchCombine) {
    a.slices = plan.slices, a.steps_per = plan.steps_per;
    if (plan.steps_per > 0)  // (the slab launch has set the depth of its own slices)
        a.err_depth = gate_err_depth(std::min(a.d, plan.steps_per * gate_kc(NBLK, plan.mb)), plan.slices, a.norm_kind);
    const dim3 block(kThreads);
    hipError_t err = hipSuccess;
#define INFMOE_GATE(M, V, G, P)                                                                                   \
    do {                                                                                                          \
        constexpr int KC = gate_kc(NBLK, M);                                                                      \
        const size_t lds = 2 * (size_t)(16 * (M) + 16 * NBLK + ((G) && !(P) ? 1 : 0)) * (KC + 4) * sizeof(float); \
        err = allow_lds_once<gate_top1_kernel<NBLK, M, V, G, P>>(lds);                                            \
        if (err != hipSuccess) return err;                                                                        \
        if (plan.slices == 1) {                                                                                   \
            a.mode = GATE_WHOLE;                                                                                  \
            gate_top1_kernel<NBLK, M, V, G, P><<<dim3(plan.groups), block, lds, stream>>>(a);                     \
        } else {                                                                                                  \
            a.mode = GATE_SLICES;                                                                                 \
            if (what & kLaunchSlices)                                                                             \
                gate_top1_kernel<NBLK, M, V, G, P><<<dim3(plan.groups * plan.slices), block, lds, stream>>>(a);   \
            a.mode = GATE_COMBINE; /* does not touch the staging tile */                                          \
            if (what & kLaunchCombine)                                                                            \
                gate_top1_kernel<NBLK, M, V, G, P><<<dim3(plan.groups), block, 0, stream>>>(a);                   \
        }                                                                                                         \
    } while (0)
#define INFMOE_GATE_M(V, G, P)                     \
    do {                                           \
        if (plan.mb == 4) INFMOE_GATE(4, V, G, P); \
        else INFMOE_GATE(1, V, G, P);              \
    } while (0)
    if (vec && pre) {  // the layer's path: 16-byte rows and precomputed centroid data
        if (use_gamma) INFMOE_GATE_M(true, true, true);
        else INFMOE_GATE_M(true, false, true);
    } else if (vec) {
        if (use_gamma) INFMOE_GATE_M(true, true, false);
        else INFMOE_GATE_M(true, false, false);
    } else {  // rows that are not 16-byte aligned: 16-token workgroups only
        if (use_gamma) INFMOE_GATE(1, false, true, false);
        else INFMOE_GATE(1, false, false, false);
    }
#undef INFMOE_GATE_M
#undef INFMOE_GATE
    return hipGetLastError();
}

}  // namespace

// Scratch of the sliced one-kernel path: enough for every call of up to T tokens.  Only 16-token workgroups
// are sliced, and only while there are fewer than kTargetGroups token groups: slices * tokens <=
// (kTargetGroups / groups + 1) * groups * 16 <= 16 * kTargetGroups + tokens + 16, and groups * slices <=
// 2 * kTargetGroups.
static size_t sliced_scratch_floats(int T, int d, int E) {
    const int kc = gate_kc(nblk_for(E), 1);
    const size_t W = (size_t)E + 2;
    const size_t max_slices = std::min<size_t>(std::min(kMaxSlices, (d + kc - 1) / kc), std::max<size_t>(1, (size_t)d / (2 * W)));
    if (max_slices <= 1 || T <= 0) return 0;
    const size_t tokens = std::min(T, 16 * kTargetGroups);
    const size_t rows = std::min(max_slices * tokens, (size_t)16 * kTargetGroups + tokens + 16);
    return rows * W + (size_t)2 * kTargetGroups * 2 * (size_t)E;
}

// [partial scores of either path | folded centroids and their statistics (used when the caller did not fold)]
size_t gate_scratch_floats(int T, int d, int E) {
    if (T <= 0) return 0;
    const size_t partial = std::max(sliced_scratch_floats(T, d, E), gate_slab_scratch_floats(T, d, E));
    return ((partial + 3) & ~(size_t)3) + gate_fold_floats(d, E);
}

hipError_t launch_gate_top1(int T, int d, int E, const float* x, const float* centroids, const float* gamma,
                            int norm_kind, const float* score_bias, int* sel, float* coeff, int* stats,
                            hipStream_t stream, const float* folded_centroids, const float* centroid_stats,
                            float* scratch, size_t scratch_floats, bool zero_stats, int* nan_flag, int nan_value,
                            int* block_hist, bool* block_hist_done) {
    if (block_hist_done != nullptr) *block_hist_done = false;
    if (T <= 0) return zero_stats && stats ? launch_fill_i32(stats, 4, 0, stream) : hipSuccess;
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(centroids) |
                           reinterpret_cast<uintptr_t>(gamma) | reinterpret_cast<uintptr_t>(folded_centroids)) & 15) == 0;
    bool pre = folded_centroids != nullptr && centroid_stats != nullptr;
    const bool vec = d % 4 == 0 && aligned;
    const bool use_gamma = norm_kind != NORM_NONE && gamma != nullptr;
    // the end of the scratch is set aside for the folded centroids; the partial scores get the rest
    const size_t fold_floats = gate_fold_floats(d, E);
    size_t partial_floats = 0;
    if (scratch != nullptr && scratch_floats >= fold_floats) {
        partial_floats = scratch_floats - fold_floats;
        if (!pre && vec) {  // the caller holds plain centroids: fold them here, once per call
            float* folded = scratch + partial_floats;
            float* cstats = folded + (((size_t)E * d + 3) & ~(size_t)3);
            fold_centroids_kernel<<<E, kThreads, 0, stream>>>(d, E, centroids, use_gamma ? gamma : nullptr, folded, cstats);
            folded_centroids = folded, centroid_stats = cstats;
            pre = true;
        }
    }
    GateArgs a{};
    a.T = T, a.d = d, a.E = E;
    a.X = x, a.C = centroids, a.gamma = gamma, a.Cf = folded_centroids, a.cstats = centroid_stats;
    a.norm_kind = norm_kind, a.bias = score_bias, a.sel = sel, a.coeff = coeff, a.stats = stats;
    a.nan_flag = nan_flag, a.nan_value = nan_value;
    a.partials = scratch;
    GatePlan plan{};
    GateSlabPlan slab{};
    const bool use_slab = pre && vec && gate_slab_plan(T, d, E, partial_floats, &slab);
    if (use_slab) {
        // many tokens: partial scores per slice with the centroid slice resident in LDS, then the combine
        // (one block of tokens: the counting sort does all its passes in one launch and wants no histogram)
        if (T <= kCountBlockTokens) block_hist = nullptr;
        const int n_hist = block_hist ? ((T + kCountBlockTokens - 1) / kCountBlockTokens) * E : 0;
        const hipError_t err = launch_gate_slab(slab, T, d, E, x, folded_centroids, scratch, stream,
                                                zero_stats ? stats : nullptr, block_hist, n_hist);
        if (err != hipSuccess) return err;
        plan.mb = T < 64 * kTargetGroups ? 1 : 4;
        plan.groups = (T + 16 * plan.mb - 1) / (16 * plan.mb);
        plan.slices = slab.slices;
        plan.steps_per = 0;  // the combine does not walk the embedding dimension
        a.err_depth = gate_err_depth(slab.ks, slab.slices, norm_kind);
    } else {
        plan = gate_plan(T, d, E, vec, partial_floats);
        if (zero_stats && stats != nullptr) {
            if (plan.slices > 1) {  // two launches: the first clears what the second counts into
                a.zero_stats = stats;
            } else {
                const hipError_t err = launch_fill_i32(stats, 4, 0, stream);
                if (err != hipSuccess) return err;
            }
        }
    }
    a.gpart = scratch ? scratch + (size_t)plan.slices * T * (E + 2) : nullptr;
    // a sliced call whose centroids are folded leaves the second launch to the lean combine kernel
    const bool lean = plan.slices > 1 && pre && vec && gate_combine_ok(d, E);
    const int what = (use_slab ? 0 : kLaunchSlices) | (lean ? 0 : kLaunchCombine);
    hipError_t err = hipSuccess;
    if (what != 0) {
        switch (nblk_for(E)) {
            case 1: err = launch_nblk<1>(a, vec, pre, use_gamma, plan, stream, what); break;
            case 2: err = launch_nblk<2>(a, vec, pre, use_gamma, plan, stream, what); break;
            case 4: err = launch_nblk<4>(a, vec, pre, use_gamma, plan, stream, what); break;
            default: err = launch_nblk<8>(a, vec, pre, use_gamma, plan, stream, what); break;
        }
    }
    if (err != hipSuccess || !lean) return err;
    if (use_slab && block_hist != nullptr && block_hist_done != nullptr) *block_hist_done = true;
    const float depth = use_slab ? a.err_depth
                                 : gate_err_depth(std::min(d, plan.steps_per * gate_kc(nblk_for(E), plan.mb)), plan.slices, norm_kind);
    return launch_gate_combine(T, d, E, plan.slices, scratch, centroid_stats, x, centroids, use_gamma ? gamma : nullptr,
                               norm_kind, score_bias, sel, coeff, stats, nan_flag, stream, nan_value, depth,
                               use_slab ? block_hist : nullptr);
}

void fold_centroids_host(int d, int E, const float* centroids, const float* gamma, float* folded, float* cstats) {
    for (int e = 0; e < E; ++e) {
        double sum = 0.0, sq = 0.0;
        for (int k = 0; k < d; ++k) {
            const float v = gamma ? centroids[(size_t)e * d + k] * gamma[k] : centroids[(size_t)e * d + k];
            folded[(size_t)e * d + k] = v;
            sum += v;
            sq += (double)v * v;
        }
        cstats[e] = (float)sum;
        cstats[E + e] = (float)sqrt(sq);
    }
}

}  // namespace infmoe
