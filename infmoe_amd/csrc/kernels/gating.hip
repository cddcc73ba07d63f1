// Fused gating for gfx950: optional row norm, token x centroid scoring and top-1 selection in
// one pass over the input.  Replaces the chain layernorm_gpu -> cublasSgemm_v2 ->
// expert_select_top1_kernel of the reference (plugin/MoELayerPlugin.cc:315-345,
// plugin/cuda/ops/layernorm.cu:136-188, plugin/cuda/moe.cu:13-76) and removes the
// normalised-input and score-matrix round trips through memory.
//
// Work split: one workgroup (8 waves) owns 16 tokens; the 8 waves split the embedding
// dimension in interleaved 16-float chunks and each runs v_mfma_f32_16x16x4_f32 with the
// tokens as the A rows and up to 128 experts (8 column blocks) as the B columns.  The row
// statistics of the norm are accumulated from the same registers that feed the matrix core,
// and the norm is applied to the 16xE score tile instead of to the 16xd input:
//     rms:      score = rstd * sum_k x_k g_k c_ek
//     centered: score = rstd * (sum_k x_k g_k c_ek - mu * sum_k g_k c_ek)
// Partial tiles of the 8 waves meet in LDS, then each wave reduces 2 tokens to
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
#include <type_traits>

#include "kernels.h"

namespace infmoe {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kTokens = 16;   // tokens per workgroup (MFMA M)
constexpr int kWaves = 8;     // waves per workgroup, each takes every 8th 16-float chunk
constexpr int kThreads = 64 * kWaves;

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
template <int NBLK, bool VEC, bool GAMMA>
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
    __shared__ double s_red[kWaves][2];
    __shared__ double s_sc64[EP];
    __shared__ double s_bcast[2];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int i = lane & 15;   // A row (token) / B column (expert) this lane feeds
    const int kq = lane >> 4;  // which float4 of the 16-float chunk this lane feeds
    const int t0 = blockIdx.x * kTokens;
    const int nchunks = (d + 15) >> 4;
    constexpr bool use_gamma = GAMMA;  // the norm's gamma is folded into the centroids as they are loaded

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

        // The wave's chunks are taken U at a time, and the loads of the next batch are issued
        // before the arithmetic of the current one (two register sets, loop unrolled by two):
        // without that every chunk would wait out a full memory latency.
        constexpr int U = NBLK <= 2 ? 4 : (NBLK == 4 ? 2 : 1);
        v4f xr[2][U], gr[2][U], cr[2][U][NBLK];
        auto load_batch = [&](auto setc, int c0) {
            constexpr int P = decltype(setc)::value;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int k = (c0 + u * kWaves) * 16 + 4 * kq;
                xr[P][u] = load4<VEC>(xrow, k, d);
                gr[P][u] = v4f{1.f, 1.f, 1.f, 1.f};
                if (use_gamma) gr[P][u] = load4<VEC>(gamma, k, d);
#pragma unroll
                for (int nb = 0; nb < NBLK; ++nb) cr[P][u][nb] = load4<VEC>(crow[nb], k, d);
            }
        };
        auto compute_batch = [&](auto setc, int c0) {
            constexpr int P = decltype(setc)::value;
            const v4f zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const bool inside = (c0 + u * kWaves) * 16 + 4 * kq < d;  // beyond the row: contributes nothing
                const v4f xv = inside ? xr[P][u] : zero, gv = gr[P][u];
                s1 += (xv.x + xv.y) + (xv.z + xv.w);
                s2 += (xv.x * xv.x + xv.y * xv.y) + (xv.z * xv.z + xv.w * xv.w);
#pragma unroll
                for (int nb = 0; nb < NBLK; ++nb) {
                    const v4f cv = inside ? cr[P][u][nb] * gv : zero;
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
        };
        const std::integral_constant<int, 0> set0{};
        const std::integral_constant<int, 1> set1{};
        constexpr int kStride = U * kWaves;  // chunks between two batches of one wave
        load_batch(set0, wave);
        for (int c = wave; c < nchunks; c += 2 * kStride) {
            if (c + kStride < nchunks) load_batch(set1, c + kStride);
            compute_batch(set0, c);
            if (c + kStride < nchunks) {
                if (c + 2 * kStride < nchunks) load_batch(set0, c + 2 * kStride);
                compute_batch(set1, c + kStride);
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
            float g1 = 0.f, g2 = 0.f;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) g1 += s_g1[w][e], g2 += s_g2[w][e];
            s_G[e] = g1;
            s_cn[e] = sqrtf(g2);
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
                if (E > 1 && (B - S) < fmaxf(bound, 4e-6f * fabsf(B))) s_rescue[tid] = 1;
            }
        }
    }
    __syncthreads();

    // ---- float64 re-scoring of the flagged tokens by the whole workgroup: the waves share the
    // row statistics, then each wave takes every kWaves-th expert and the scores meet in LDS
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
hipError_t launch_nblk(int T, int d, int E, const float* x, const float* c, const float* gamma, int norm_kind,
                       const float* bias, int* sel, float* coeff, int* stats, hipStream_t stream) {
    const dim3 grid((T + kTokens - 1) / kTokens), block(kThreads);
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(c) |
                           reinterpret_cast<uintptr_t>(gamma)) & 15) == 0;
    const bool vec = d % 4 == 0 && aligned;
    const bool use_gamma = norm_kind != NORM_NONE && gamma != nullptr;
#define INFMOE_GATE(V, G) \
    gate_top1_kernel<NBLK, V, G><<<grid, block, 0, stream>>>(T, d, E, x, c, gamma, norm_kind, bias, sel, coeff, stats)
    if (vec && use_gamma) INFMOE_GATE(true, true);
    else if (vec) INFMOE_GATE(true, false);
    else if (use_gamma) INFMOE_GATE(false, true);
    else INFMOE_GATE(false, false);
#undef INFMOE_GATE
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
