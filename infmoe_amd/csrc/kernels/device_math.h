// Small device functions shared by kernels that must agree bit for bit.
#pragma once

#include <hip/hip_runtime.h>

namespace infmoe {

// plugin/cuda/ops/gelu.cu:8-15
__device__ __forceinline__ float gelu_dot(float a, float b) {
    const float cdf = 0.5f * (1.0f + tanhf(a * (0.035677408136300125f * a * a + 0.7978845608028654f)));
    return a * cdf * b;
}

// plugin/cuda/common.cuh:24-27
__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

// base_layer output mix, plugin/cuda/moe.cu:120-126: a * post + (1 - a) * routed with b = 1 - a.
// Written with explicit roundings so that the stand-alone mix kernel and the fused GEMM epilogue
// give the same bits whatever the compiler contracts elsewhere.
__device__ __forceinline__ float mix_value(float a, float b, float post, float routed) {
    return __fmaf_rn(a, post, __fmul_rn(b, routed));
}

}  // namespace infmoe
