// Fused gating for gfx950: optional row norm, token x centroid scoring and top-1 selection in
// one pass over the input.  Replaces the chain layernorm_gpu -> cublasSgemm_v2 ->
// expert_select_top1_kernel of the reference (plugin/MoELayerPlugin.cc:315-345,
// plugin/cuda/ops/layernorm.cu:136-188, plugin/cuda/moe.cu:13-76) and removes the
// normalised-input and score-matrix round trips through memory.
//
// Work split: one workgroup (4 waves) owns 16 tokens and walks the embedding dimension in chunks
// that are staged through LDS with row-contiguous global loads; each wave takes a quarter of every
// chunk and runs v_mfma_f32_16x16x4_f32 with the tokens as the A rows and up to 128 experts
// (8 column blocks) as the B columns.  The row
// statistics of the norm are accumulated from the same registers that feed the matrix core,
// and the norm is applied to the 16xE score tile instead of to the 16xd input:
//     rms:      score = rstd * sum_k x_k g_k c_ek
//     centered: score = rstd * (sum_k x_k g_k c_ek - mu * sum_k g_k c_ek)
// Partial tiles of the 4 waves meet in LDS, then each wave reduces 4 tokens to
// (best, index, runner-up) with the reference's tie rule (lowest index wins,
// plugin/cuda/moe.cu:62-68).
//
// FP32 accumulation over d terms cannot order two scores closer than its own rounding error,
// so a token whose top-2 gap is below a Cauchy-Schwarz error bound is re-scored by the whole
// workgroup in float64.  Such tokens are rare (about one in a few thousand for Gaussian
// scores); they are counted in stats[2], and those whose float64 gap is below 1e-6 relative
// (no arithmetic can be expected to order them) in stats[0].
#include <hip/hip_runtime.h>

#include <cfloat>
#include <cmath>
#include <type_traits>

#include "kernels.h"

namespace infmoe {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kTokens = 16;   // tokens per workgroup (MFMA M)
constexpr int kWaves = 4;     // waves per workgroup; each takes a quarter of every staged K chunk
constexpr int kThreads = 64 * kWaves;
constexpr int kMaxCand = 4;   // near-tied experts the quick float64 re-scoring handles

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
// PRE: the caller supplies the centroids already multiplied by gamma (Cf) and, per expert, the sum
// and the Euclidean norm of that product (cstats[0..E) and cstats[E..2E)): they depend on the layer's
// parameters only, so the layer computes them once instead of every workgroup of every call.
template <int NBLK, bool VEC, bool GAMMA, bool PRE>
__global__ __launch_bounds__(kThreads) void gate_top1_kernel(int T, int d, int E, const float* __restrict__ X,
                                                             const float* __restrict__ C,
                                                             const float* __restrict__ gamma,
                                                             const float* __restrict__ Cf,
                                                             const float* __restrict__ cstats, int norm_kind,
                                                             const float* __restrict__ bias, int* __restrict__ sel,
                                                             float* __restrict__ coeff, int* __restrict__ stats) {
    constexpr int EP = 16 * NBLK;
    __shared__ float s_part[kWaves][kTokens][EP + 1];
    __shared__ float s_score[kTokens][EP + 1];
    __shared__ float s_s1[kWaves][kTokens], s_s2[kWaves][kTokens];
    __shared__ float s_g1[kWaves][EP], s_g2[kWaves][EP];
    __shared__ float s_mu[kTokens], s_rstd[kTokens], s_xnorm[kTokens];
    __shared__ float s_G[EP], s_cn[EP];
    __shared__ float s_best[kTokens], s_second[kTokens], s_cnmax;
    __shared__ int s_besti[kTokens], s_rescue[kTokens];
    __shared__ double s_red[kWaves][2];
    __shared__ double s_sc64[EP];
    __shared__ double s_bcast[2];
    __shared__ float s_thr[kTokens];
    __shared__ int s_cand[kMaxCand], s_ncand;
    __shared__ double s_red2[kWaves][2 + 2 * kMaxCand];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int i = lane & 15;   // A row (token) / B column (expert) this lane feeds
    const int kq = lane >> 4;  // which float4 of the 16-float chunk this lane feeds
    const int t0 = blockIdx.x * kTokens;
    constexpr bool use_gamma = GAMMA;  // the norm's gamma is folded into the centroids as they are loaded

    if (tid < kTokens) {
        s_best[tid] = -FLT_MAX;  // plugin/cuda/moe.cu:26-27
        s_second[tid] = -FLT_MAX;
        s_besti[tid] = -1;
        s_rescue[tid] = 0;
    }
    if (tid == 0) s_cnmax = 0.f;

    // Staging tile in LDS, two buffers of ROWS x (KC + 4) floats: 16 token rows, EP centroid rows and
    // (with a norm) the gamma row, KC floats of K at a time.  Every wave-wide global load reads whole
    // 512-byte or 1-KB stretches of one or two rows, which is what DRAM serves best; the MFMA operand
    // layout (a lane needs 16 bytes of "its" row) is produced by the LDS reads, not by the global loads.
    constexpr int KC = NBLK <= 2 ? 256 : (NBLK == 4 ? 128 : 64);
    constexpr int KC4 = KC / 4, LD = KC + 4;
    constexpr bool GROW = GAMMA && !PRE;  // stage a gamma row and fold it into the centroids here
    constexpr int ROWS = kTokens + EP + (GROW ? 1 : 0);
    constexpr int NL = (ROWS * KC4 + kThreads - 1) / kThreads;  // 16-byte loads per thread per step
    extern __shared__ __align__(16) float s_tile[];
    const int nsteps = (d + KC - 1) / KC;

    for (int e0 = 0; e0 < E; e0 += EP) {
        v4f acc[NBLK];
        float gs[NBLK], cn[NBLK];
#pragma unroll
        for (int nb = 0; nb < NBLK; ++nb) {
            acc[nb] = v4f{0.f, 0.f, 0.f, 0.f};
            gs[nb] = 0.f;
            cn[nb] = 0.f;
        }
        float s1 = 0.f, s2 = 0.f;

        // item l of this thread: float4 c4 of tile row `row`; rows beyond T / E are clamped (their
        // scores are never used), items beyond the tile repeat its last one
        const float* rptr[NL];
        int lds_off[NL], kcol[NL];
#pragma unroll
        for (int l = 0; l < NL; ++l) {
            const int idx = min(tid + l * kThreads, ROWS * KC4 - 1);
            const int row = idx / KC4, c4 = idx % KC4;
            rptr[l] = row < kTokens ? X + (size_t)min(t0 + row, T - 1) * d
                      : row < kTokens + EP ? (PRE ? Cf : C) + (size_t)min(e0 + row - kTokens, E - 1) * d
                                           : gamma;
            lds_off[l] = row * LD + 4 * c4;
            kcol[l] = 4 * c4;
        }
        // Two register sets: the loads of step s + 2 are issued before the arithmetic of step s and
        // written to LDS one step later, so about two steps' worth of bytes (2 x 49 KB for 32
        // experts) is in flight per CU - the arithmetic of one step is far shorter than a memory
        // round trip and would not cover it.
        v4f rg[2][NL];
        auto load_step = [&](auto setc, int k0) {
            constexpr int P = decltype(setc)::value;
#pragma unroll
            for (int l = 0; l < NL; ++l) rg[P][l] = load4<VEC>(rptr[l], k0 + kcol[l], d);
        };
        auto store_step = [&](auto setc, int buf, int k0) {
            constexpr int P = decltype(setc)::value;
            const v4f zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int l = 0; l < NL; ++l)  // k beyond the row was read from a clamped address: store zeros
                *reinterpret_cast<v4f*>(s_tile + buf * (ROWS * LD) + lds_off[l]) = (k0 + kcol[l] < d) ? rg[P][l] : zero;
        };
        auto compute_step = [&](int buf) {
            const float* tile = s_tile + buf * (ROWS * LD) + wave * (KC / kWaves) + 4 * kq;
#pragma unroll
            for (int g = 0; g < KC / kWaves / 16; ++g) {
                const v4f xv = *reinterpret_cast<const v4f*>(tile + i * LD + 16 * g);
                v4f gv = {1.f, 1.f, 1.f, 1.f};
                if (GROW) gv = *reinterpret_cast<const v4f*>(tile + (kTokens + EP) * LD + 16 * g);
                s1 += (xv.x + xv.y) + (xv.z + xv.w);
                s2 += (xv.x * xv.x + xv.y * xv.y) + (xv.z * xv.z + xv.w * xv.w);
#pragma unroll
                for (int nb = 0; nb < NBLK; ++nb) {
                    v4f cv = *reinterpret_cast<const v4f*>(tile + (kTokens + 16 * nb + i) * LD + 16 * g);
                    if (!PRE) {
                        cv *= gv;
                        gs[nb] += (cv.x + cv.y) + (cv.z + cv.w);
                        cn[nb] += (cv.x * cv.x + cv.y * cv.y) + (cv.z * cv.z + cv.w * cv.w);
                    }
                    // The k order inside a 16-float group is permuted identically for A and B, which
                    // a dot product does not see: step j multiplies element j of every lane's float4.
                    acc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv.x, cv.x, acc[nb], 0, 0, 0);
                    acc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv.y, cv.y, acc[nb], 0, 0, 0);
                    acc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv.z, cv.z, acc[nb], 0, 0, 0);
                    acc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv.w, cv.w, acc[nb], 0, 0, 0);
                }
            }
        };
        // step s computes from buffer s & 1; set P holds step s + 1, the other set receives step s + 2
        auto step = [&](auto setc, int s) {
            constexpr int P = decltype(setc)::value;
            load_step(std::integral_constant<int, 1 - P>{}, min(s + 2, nsteps - 1) * KC);
            compute_step(s & 1);
            store_step(setc, (s + 1) & 1, (s + 1) * KC);
            __syncthreads();
        };
        const std::integral_constant<int, 0> set0{};
        const std::integral_constant<int, 1> set1{};
        __syncthreads();  // the previous pass is done with the tile
        load_step(set1, 0);
        store_step(set1, 0, 0);
        load_step(set0, min(1, nsteps - 1) * KC);
        __syncthreads();
        for (int s = 0; s < nsteps; s += 2) {
            step(set0, s);
            if (s + 1 < nsteps) step(set1, s + 1);
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
            float g = gs[nb], n2 = cn[nb];
            g += __shfl_xor(g, 16);
            g += __shfl_xor(g, 32);
            n2 += __shfl_xor(n2, 16);
            n2 += __shfl_xor(n2, 32);
            if (kq == 0) {
                s_g1[wave][16 * nb + i] = g;
                s_g2[wave][16 * nb + i] = n2;
            }
            // D layout of 16x16x4: lane holds column (lane & 15), rows 4*(lane >> 4) + r
#pragma unroll
            for (int r = 0; r < 4; ++r) s_part[wave][4 * kq + r][16 * nb + i] = acc[nb][r];
        }
        __syncthreads();

        if (tid < kTokens) {
            float a1 = 0.f, a2 = 0.f;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) a1 += s_s1[w][tid], a2 += s_s2[w][tid];
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
                s_G[e] = cstats[ee];
                s_cn[e] = cstats[E + ee];
            } else {
                float g1 = 0.f, g2 = 0.f;
#pragma unroll
                for (int w = 0; w < kWaves; ++w) g1 += s_g1[w][e], g2 += s_g2[w][e];
                s_G[e] = g1;
                s_cn[e] = sqrtf(g2);
            }
        }
        __syncthreads();

        for (int idx = tid; idx < kTokens * EP; idx += kThreads) {
            const int tok = idx / EP, e = idx - tok * EP;
            float dot = 0.f;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) dot += s_part[w][tok][e];
            float sc = s_rstd[tok] * (dot - s_mu[tok] * s_G[e]);
            if (bias != nullptr && e0 + e < E) sc += bias[e0 + e];
            s_score[tok][e] = sc;
        }
        __syncthreads();

        // each wave reduces kTokens / kWaves tokens
        const int nvalid = min(E - e0, EP);
        float cmax = 0.f;
        for (int e = lane; e < nvalid; e += 64) cmax = fmaxf(cmax, s_cn[e]);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) cmax = fmaxf(cmax, __shfl_xor(cmax, off));
        if (tid == 0) s_cnmax = fmaxf(s_cnmax, cmax);
        for (int q = 0; q < kTokens / kWaves; ++q) {
            const int tok = (kTokens / kWaves) * wave + q;
            float v = -FLT_MAX;
            int vi = -1;
            for (int e = lane; e < nvalid; e += 64) {
                const float s = s_score[tok][e];
                if (s > v) {
                    v = s;
                    vi = e0 + e;
                }
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const float ov = __shfl_xor(v, off);
                const int oi = __shfl_xor(vi, off);
                if (ov > v || (ov == v && (unsigned)oi < (unsigned)vi)) {
                    v = ov;
                    vi = oi;
                }
            }
            float v2 = -FLT_MAX;
            for (int e = lane; e < nvalid; e += 64) {
                const float s = s_score[tok][e];
                if (e0 + e != vi && s > v2) v2 = s;
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) v2 = fmaxf(v2, __shfl_xor(v2, off));
            if (lane == 0) {
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
    }

    // ---- decide, per token, whether FP32 ordered the top two safely
    if (tid < kTokens) {
        const int t = t0 + tid;
        if (t < T) {
            const float B = s_best[tid], S = s_second[tid];
            const int I = s_besti[tid];
            if (I < 0) {  // no orderable score: the reference asserts (plugin/cuda/moe.cu:70)
                sel[t] = 0;
                coeff[t] = B;
                if (stats) atomicAdd(&stats[1], 1);
            } else {
                sel[t] = I;
                coeff[t] = B;
                const float bound = 8.f * FLT_EPSILON * s_rstd[tid] * s_xnorm[tid] * s_cnmax;
                s_thr[tid] = fmaxf(bound, 4e-6f * fabsf(B));
                if (E > 1 && (B - S) < s_thr[tid]) s_rescue[tid] = 1;
            }
        }
    }
    __syncthreads();

    // ---- float64 re-scoring of the flagged tokens by the whole workgroup: the waves share the
    // row statistics, then each wave takes every kWaves-th expert and the scores meet in LDS
    for (int tok = 0; tok < kTokens; ++tok) {
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

template <int NBLK>
hipError_t launch_nblk(int T, int d, int E, const float* x, const float* c, const float* gamma, const float* cf,
                       const float* cstats, int norm_kind, const float* bias, int* sel, float* coeff, int* stats,
                       hipStream_t stream) {
    const dim3 grid((T + kTokens - 1) / kTokens), block(kThreads);
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(c) |
                           reinterpret_cast<uintptr_t>(gamma) | reinterpret_cast<uintptr_t>(cf)) & 15) == 0;
    const bool pre = cf != nullptr && cstats != nullptr;
    const bool vec = d % 4 == 0 && aligned;
    const bool use_gamma = norm_kind != NORM_NONE && gamma != nullptr;
    constexpr int KC = NBLK <= 2 ? 256 : (NBLK == 4 ? 128 : 64);
    hipError_t err = hipSuccess;
#define INFMOE_GATE(V, G, P)                                                                                       \
    do {                                                                                                           \
        const size_t lds = 2 * (size_t)(kTokens + 16 * NBLK + ((G) && !(P) ? 1 : 0)) * (KC + 4) * sizeof(float);   \
        err = allow_lds_once<gate_top1_kernel<NBLK, V, G, P>>(lds);                                                \
        if (err != hipSuccess) return err;                                                                         \
        gate_top1_kernel<NBLK, V, G, P><<<grid, block, lds, stream>>>(T, d, E, x, c, gamma, cf, cstats, norm_kind, \
                                                                      bias, sel, coeff, stats);                    \
    } while (0)
    if (vec && pre) {  // the layer's path: 16-byte rows and precomputed centroid data
        if (use_gamma) INFMOE_GATE(true, true, true);
        else INFMOE_GATE(true, false, true);
    } else if (vec) {
        if (use_gamma) INFMOE_GATE(true, true, false);
        else INFMOE_GATE(true, false, false);
    } else {
        if (use_gamma) INFMOE_GATE(false, true, false);
        else INFMOE_GATE(false, false, false);
    }
#undef INFMOE_GATE
    return hipGetLastError();
}

}  // namespace

hipError_t launch_gate_top1(int T, int d, int E, const float* x, const float* centroids, const float* gamma,
                            int norm_kind, const float* score_bias, int* sel, float* coeff, int* stats,
                            hipStream_t stream, const float* folded_centroids, const float* centroid_stats) {
    if (T <= 0) return hipSuccess;
#define INFMOE_NBLK(n) \
    return launch_nblk<n>(T, d, E, x, centroids, gamma, folded_centroids, centroid_stats, norm_kind, score_bias, sel, coeff, stats, stream)
    if (E <= 16) INFMOE_NBLK(1);
    if (E <= 32) INFMOE_NBLK(2);
    if (E <= 64) INFMOE_NBLK(4);
    INFMOE_NBLK(8);
#undef INFMOE_NBLK
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
