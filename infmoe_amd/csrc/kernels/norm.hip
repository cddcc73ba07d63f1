// Row norm with gamma only (the reference calls layernorm_gpu with beta == nullptr at both sites,
// plugin/MoELayerPlugin.cc:324-325 and plugin/sublayers/T5FFLayer.cc:102-103).
//   centered: gamma * (x - mu) * rsqrt(var + eps), biased variance  (plugin/cuda/ops/layernorm.cu:149-161)
//   rms:      gamma * x * rsqrt(mean(x^2) + eps)                    (README.md:115)
// One wave per row.  The row is read once into registers when it is at most 8192 floats (two
// exact passes for the centered form: mean, then variance about the mean, instead of the
// reference's Welford merge) and re-read from cache otherwise.  The register array is sized for the
// row (2048, 4096 or 8192 floats): with the largest size for every row only three waves fit a SIMD,
// and 4096 rows then run as one full generation of workgroups plus a third of one.  For the grouped expert launch
// every routed row picks the gamma of its own expert.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace infmoe {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
constexpr int kThreads = 256;
constexpr int kMaxRegVec = 32;  // float4 per lane held in registers -> rows up to 64*32*4 = 8192 floats

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

// RV: float4 per lane held in registers (rows of up to 256 * RV floats take the one-pass form)
template <bool VEC, int RV>
__global__ __launch_bounds__(kThreads) void row_norm_kernel(float* __restrict__ out, const float* __restrict__ in,
                                                            int rows, int d, const float* __restrict__ gamma_base,
                                                            size_t gamma_stride, const int* __restrict__ row_expert,
                                                            int norm_kind, const int* __restrict__ expert_slot) {
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    if (r >= rows) return;
    const float* x = in + (size_t)r * d;
    float* y = out + (size_t)r * d;
    int owner = row_expert ? row_expert[r] : 0;
    if (row_expert && expert_slot) owner = expert_slot[owner];
    const float* g = gamma_base + (size_t)owner * gamma_stride;
    const float inv_d = 1.0f / (float)d;

    if (VEC && d <= 64 * 4 * RV) {
        const int n4 = d >> 2;
        v4f v[RV];
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < RV; ++j) {
            const int k = lane + 64 * j;
            v[j] = (k < n4) ? reinterpret_cast<const v4f*>(x)[k] : v4f{0.f, 0.f, 0.f, 0.f};
        }
        float mu = 0.f;
        if (norm_kind == NORM_CENTERED) {
#pragma unroll
            for (int j = 0; j < RV; ++j) s += (v[j].x + v[j].y) + (v[j].z + v[j].w);
            mu = wave_sum(s) * inv_d;
        }
        float q = 0.f;
#pragma unroll
        for (int j = 0; j < RV; ++j) {
            const int k = lane + 64 * j;
            if (k < n4) {
                const v4f c = v[j] - mu;
                q += (c.x * c.x + c.y * c.y) + (c.z * c.z + c.w * c.w);
            }
        }
        const float rstd = 1.0f / sqrtf(wave_sum(q) * inv_d + kNormEps);
#pragma unroll
        for (int j = 0; j < RV; ++j) {
            const int k = lane + 64 * j;
            if (k < n4) reinterpret_cast<v4f*>(y)[k] = reinterpret_cast<const v4f*>(g)[k] * ((v[j] - mu) * rstd);
        }
    } else {
        float mu = 0.f;
        if (norm_kind == NORM_CENTERED) {
            float s = 0.f;
            for (int k = lane; k < d; k += 64) s += x[k];
            mu = wave_sum(s) * inv_d;
        }
        float q = 0.f;
        for (int k = lane; k < d; k += 64) {
            const float c = x[k] - mu;
            q += c * c;
        }
        const float rstd = 1.0f / sqrtf(wave_sum(q) * inv_d + kNormEps);
        for (int k = lane; k < d; k += 64) y[k] = g[k] * ((x[k] - mu) * rstd);
    }
}

// One wave per weight row: the row times gamma, in place.
template <bool VEC>
__global__ __launch_bounds__(kThreads) void fold_gamma_kernel(float* __restrict__ w, const float* __restrict__ gamma,
                                                              int n_rows, int d) {
    const int lane = threadIdx.x & 63;
    const int n = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    if (n >= n_rows) return;
    float* row = w + (size_t)n * d;
    if (VEC) {
        const int n4 = d >> 2;
        v4f* r4 = reinterpret_cast<v4f*>(row);
        const v4f* g4 = reinterpret_cast<const v4f*>(gamma);
        for (int k = lane; k < n4; k += 64) r4[k] = r4[k] * g4[k];
    } else {
        for (int k = lane; k < d; k += 64) row[k] = row[k] * gamma[k];
    }
}

}  // namespace

hipError_t launch_fold_gamma(float* w, const float* gamma, int n_rows, int d, hipStream_t stream) {
    if (n_rows <= 0) return hipSuccess;
    const dim3 grid((n_rows + kThreads / 64 - 1) / (kThreads / 64));
    const bool aligned = ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(gamma)) & 15) == 0;
    if (d % 4 == 0 && aligned)
        fold_gamma_kernel<true><<<grid, kThreads, 0, stream>>>(w, gamma, n_rows, d);
    else
        fold_gamma_kernel<false><<<grid, kThreads, 0, stream>>>(w, gamma, n_rows, d);
    return hipGetLastError();
}

hipError_t launch_row_norm(float* out, const float* in, int rows, int d, const float* gamma_base,
                           size_t gamma_stride, const int* row_expert, int norm_kind, hipStream_t stream,
                           const int* expert_slot) {
    if (rows <= 0) return hipSuccess;
    const dim3 grid((rows + kThreads / 64 - 1) / (kThreads / 64));
    const bool aligned = ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(in) |
                           reinterpret_cast<uintptr_t>(gamma_base)) & 15) == 0 &&
                         (gamma_stride % 4 == 0);
#define INFMOE_NORM(V, RV)                                                                                        \
    row_norm_kernel<V, RV><<<grid, kThreads, 0, stream>>>(out, in, rows, d, gamma_base, gamma_stride, row_expert, \
                                                          norm_kind, expert_slot)
    if (d % 4 == 0 && aligned) {
        if (d <= 2048) INFMOE_NORM(true, 8);
        else if (d <= 4096) INFMOE_NORM(true, 16);
        else INFMOE_NORM(true, kMaxRegVec);
    } else {
        INFMOE_NORM(false, 1);
    }
#undef INFMOE_NORM
    return hipGetLastError();
}

}  // namespace infmoe
