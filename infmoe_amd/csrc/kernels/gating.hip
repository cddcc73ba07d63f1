// Fused gating for gfx950: optional row norm, token x centroid scoring and top-1 selection in
// one pass over the input.  Replaces the chain layernorm_gpu -> cublasSgemm_v2 ->
// expert_select_top1_kernel of the reference (plugin/MoELayerPlugin.cc:315-345,
// plugin/cuda/ops/layernorm.cu:136-188, plugin/cuda/moe.cu:13-76) and removes the
// normalised-input and score-matrix round trips through memory.
//
// Work split: one workgroup (4 waves) owns 16 tokens; the 4 waves split the embedding
// dimension in interleaved 16-float chunks and each runs v_mfma_f32_16x16x4_f32 with the
// tokens as the A rows and up to 128 experts (8 column blocks) as the B columns.  The row
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

#include "kernels.h"

namespace infmoe {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kTokens = 16;   // tokens per workgroup (MFMA M)
constexpr int kWaves = 4;     // waves per workgroup, each takes every 4th 16-float chunk
constexpr int kThreads = 64 * kWaves;

template <bool VEC>
__device__ __forceinline__ v4f load4(const float* __restrict__ row, int k, int d) {
    v4f v = {0.f, 0.f, 0.f, 0.f};
    if (VEC) {
        if (k < d) v = *reinterpret_cast<const v4f*>(row + k);
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
template <int NBLK, bool VEC>
__global__ __launch_bounds__(kThreads) void gate_top1_kernel(int T, int d, int E, const float* __restrict__ X,
                                                             const float* __restrict__ C,
                                                             const float* __restrict__ gamma, int norm_kind,
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
    __shared__ double s_red[kWaves][8];
    __shared__ double s_bcast[2];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int i = lane & 15;   // A row (token) / B column (expert) this lane feeds
    const int kq = lane >> 4;  // which float4 of the 16-float chunk this lane feeds
    const int t0 = blockIdx.x * kTokens;
    const int nchunks = (d + 15) >> 4;
    const bool use_gamma = (norm_kind != NORM_NONE) && gamma != nullptr;

    if (tid < kTokens) {
        s_best[tid] = -FLT_MAX;  // plugin/cuda/moe.cu:26-27
        s_second[tid] = -FLT_MAX;
        s_besti[tid] = -1;
        s_rescue[tid] = 0;
    }
    if (tid == 0) s_cnmax = 0.f;

    const float* xrow = X + (size_t)min(t0 + i, T - 1) * d;

    for (int e0 = 0; e0 < E; e0 += EP) {
        const float* crow[NBLK];
        v4f acc[NBLK];
        float gs[NBLK], cn[NBLK];
#pragma unroll
        for (int nb = 0; nb < NBLK; ++nb) {
            crow[nb] = C + (size_t)min(e0 + 16 * nb + i, E - 1) * d;
            acc[nb] = v4f{0.f, 0.f, 0.f, 0.f};
            gs[nb] = 0.f;
            cn[nb] = 0.f;
        }
        float s1 = 0.f, s2 = 0.f;

        for (int c = wave; c < nchunks; c += kWaves) {
            const int k = c * 16 + 4 * kq;
            const v4f xv = load4<VEC>(xrow, k, d);
            v4f gv = {1.f, 1.f, 1.f, 1.f};
            if (use_gamma) gv = load4<VEC>(gamma, k, d);
            s1 += (xv.x + xv.y) + (xv.z + xv.w);
            s2 += (xv.x * xv.x + xv.y * xv.y) + (xv.z * xv.z + xv.w * xv.w);
#pragma unroll
            for (int nb = 0; nb < NBLK; ++nb) {
                v4f cv = load4<VEC>(crow[nb], k, d);
                cv *= gv;
                gs[nb] += (cv.x + cv.y) + (cv.z + cv.w);
                cn[nb] += (cv.x * cv.x + cv.y * cv.y) + (cv.z * cv.z + cv.w * cv.w);
                // The k order inside a chunk is permuted identically for A and B, which a dot
                // product does not see: step j multiplies element j of every lane's float4.
                acc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv.x, cv.x, acc[nb], 0, 0, 0);
                acc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv.y, cv.y, acc[nb], 0, 0, 0);
                acc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv.z, cv.z, acc[nb], 0, 0, 0);
                acc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv.w, cv.w, acc[nb], 0, 0, 0);
            }
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
            const float a1 = (s_s1[0][tid] + s_s1[1][tid]) + (s_s1[2][tid] + s_s1[3][tid]);
            const float a2 = (s_s2[0][tid] + s_s2[1][tid]) + (s_s2[2][tid] + s_s2[3][tid]);
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
            s_G[e] = (s_g1[0][e] + s_g1[1][e]) + (s_g1[2][e] + s_g1[3][e]);
            s_cn[e] = sqrtf((s_g2[0][e] + s_g2[1][e]) + (s_g2[2][e] + s_g2[3][e]));
        }
        __syncthreads();

        for (int idx = tid; idx < kTokens * EP; idx += kThreads) {
            const int tok = idx / EP, e = idx - tok * EP;
            float dot = (s_part[0][tok][e] + s_part[1][tok][e]) + (s_part[2][tok][e] + s_part[3][tok][e]);
            float sc = s_rstd[tok] * (dot - s_mu[tok] * s_G[e]);
            if (bias != nullptr && e0 + e < E) sc += bias[e0 + e];
            s_score[tok][e] = sc;
        }
        __syncthreads();

        // each wave reduces 4 tokens
        const int nvalid = min(E - e0, EP);
        float cmax = 0.f;
        for (int e = lane; e < nvalid; e += 64) cmax = fmaxf(cmax, s_cn[e]);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) cmax = fmaxf(cmax, __shfl_xor(cmax, off));
        if (tid == 0) s_cnmax = fmaxf(s_cnmax, cmax);
        for (int q = 0; q < 4; ++q) {
            const int tok = 4 * wave + q;
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
                const float bound = 16.f * FLT_EPSILON * s_rstd[tid] * s_xnorm[tid] * s_cnmax;
                if (E > 1 && (B - S) < fmaxf(bound, 4e-6f * fabsf(B))) s_rescue[tid] = 1;
            }
        }
    }
    __syncthreads();

    // ---- float64 re-scoring of the flagged tokens by the whole workgroup
    for (int tok = 0; tok < kTokens; ++tok) {
        if (!s_rescue[tok]) continue;  // uniform: read from LDS after the barrier
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
            const double t1 = (s_red[0][0] + s_red[1][0]) + (s_red[2][0] + s_red[3][0]);
            const double t2 = (s_red[0][1] + s_red[1][1]) + (s_red[2][1] + s_red[3][1]);
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
        for (int e0 = 0; e0 < E; e0 += 8) {
            double a[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (int k = tid; k < d; k += kThreads) {
                const double xv = ((double)xr[k] - mu) * (use_gamma ? (double)gamma[k] : 1.0);
#pragma unroll
                for (int j = 0; j < 8; ++j) a[j] += xv * (double)C[(size_t)min(e0 + j, E - 1) * d + k];
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                a[j] = wave_sum(a[j]);
                if (lane == 0) s_red[wave][j] = a[j];
            }
            __syncthreads();
            if (tid == 0) {
                for (int j = 0; j < 8 && e0 + j < E; ++j) {
                    double sc = rstd * ((s_red[0][j] + s_red[1][j]) + (s_red[2][j] + s_red[3][j]));
                    if (bias != nullptr) sc += (double)bias[e0 + j];
                    if (sc > best) {
                        second = best;
                        best = sc;
                        besti = e0 + j;
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
hipError_t launch_nblk(int T, int d, int E, const float* x, const float* c, const float* gamma, int norm_kind,
                       const float* bias, int* sel, float* coeff, int* stats, hipStream_t stream) {
    const dim3 grid((T + kTokens - 1) / kTokens), block(kThreads);
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(c) |
                           reinterpret_cast<uintptr_t>(gamma)) & 15) == 0;
    if (d % 4 == 0 && aligned)
        gate_top1_kernel<NBLK, true><<<grid, block, 0, stream>>>(T, d, E, x, c, gamma, norm_kind, bias, sel, coeff, stats);
    else
        gate_top1_kernel<NBLK, false><<<grid, block, 0, stream>>>(T, d, E, x, c, gamma, norm_kind, bias, sel, coeff, stats);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_gate_top1(int T, int d, int E, const float* x, const float* centroids, const float* gamma,
                            int norm_kind, const float* score_bias, int* sel, float* coeff, int* stats,
                            hipStream_t stream) {
    if (T <= 0) return hipSuccess;
    if (E <= 16) return launch_nblk<1>(T, d, E, x, centroids, gamma, norm_kind, score_bias, sel, coeff, stats, stream);
    if (E <= 32) return launch_nblk<2>(T, d, E, x, centroids, gamma, norm_kind, score_bias, sel, coeff, stats, stream);
    if (E <= 64) return launch_nblk<4>(T, d, E, x, centroids, gamma, norm_kind, score_bias, sel, coeff, stats, stream);
    return launch_nblk<8>(T, d, E, x, centroids, gamma, norm_kind, score_bias, sel, coeff, stats, stream);
}

}  // namespace infmoe
