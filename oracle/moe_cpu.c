/*
 * CPU restatement (C, FP32, OpenMP) of InfMoE's MoELayerPlugin hot path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE: it is the reported CPU baseline of the
 * benchmark and is itself checked against the float64 numpy oracle (oracle/moe_oracle.py) by
 * tests/test_oracle_cpu.py.  The shipped library never links or calls it.
 *
 * Steps and the reference lines they restate (paths relative to the Harry-Chen/InfMoE tree),
 * with the intended math (row stride applied, post-expert rows gathered):
 *   norm            plugin/cuda/ops/layernorm.cu:136-174 (centered) / README.md:115 (rms)
 *   scoring         plugin/MoELayerPlugin.cc:332-337
 *   top-1           plugin/cuda/moe.cu:60-75
 *   count + sort    plugin/cuda/moe.cu:181-199
 *   scatter         plugin/cuda/moe.cu:98-113
 *   expert FFN      plugin/sublayers/T5FFLayer.cc:90-141, plugin/cuda/ops/gelu.cu:7-16
 *   gather / mix    plugin/cuda/moe.cu:89-96,115-127, plugin/cuda/common.cuh:24-27
 *
 * Build: gcc -O3 -march=x86-64-v3 -fopenmp -shared -fPIC oracle/moe_cpu.c -o oracle/libmoe_cpu.so -lm
 */
#include <math.h>
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { NORM_NONE = 0, NORM_RMS = 1, NORM_CENTERED = 2 };
enum { FFN_RELU = 0, FFN_GATED_GELU = 1 };
#define EPS 1e-6f

typedef float v8 __attribute__((vector_size(32), aligned(4)));

static inline float hsum(v8 v) { return ((v[0] + v[4]) + (v[1] + v[5])) + ((v[2] + v[6]) + (v[3] + v[7])); }

int moe_cpu_threads(void) { return omp_get_max_threads(); }

/* out[r,:] = gamma * norm(x[r,:]) */
void moe_cpu_layernorm(float* out, const float* x, int rows, int d, const float* gamma, int kind) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r) {
        const float* xr = x + (size_t)r * d;
        float* o = out + (size_t)r * d;
        float mu = 0.f;
        if (kind == NORM_CENTERED) {
            float s = 0.f;
#pragma omp simd reduction(+ : s)
            for (int k = 0; k < d; ++k) s += xr[k];
            mu = s / (float)d;
        }
        float q = 0.f;
#pragma omp simd reduction(+ : q)
        for (int k = 0; k < d; ++k) q += (xr[k] - mu) * (xr[k] - mu);
        const float rstd = 1.0f / sqrtf(q / (float)d + EPS);
        for (int k = 0; k < d; ++k) o[k] = gamma[k] * ((xr[k] - mu) * rstd);
    }
}

/* C[M][N] (+)= A[M][K] * B[N][K]^T, both operands K-contiguous; 3x4 register tile, 8-wide over k.
 * epilogue: 0 store, 1 relu, 2 add residual R[M][N] */
static void gemm_tn(float* C, const float* A, const float* B, int M, int N, int K, int epilogue, const float* R) {
    const int K8 = K & ~7;
#pragma omp parallel for collapse(2) schedule(dynamic, 4)
    for (int m0 = 0; m0 < M; m0 += 3) {
        for (int n0 = 0; n0 < N; n0 += 4) {
            const int mr = M - m0 < 3 ? M - m0 : 3, nr = N - n0 < 4 ? N - n0 : 4;
            float acc[3][4] = {{0}};
            if (mr == 3 && nr == 4) {
                v8 s[3][4];
                for (int i = 0; i < 3; ++i)
                    for (int j = 0; j < 4; ++j) s[i][j] = (v8){0, 0, 0, 0, 0, 0, 0, 0};
                const float *a0 = A + (size_t)m0 * K, *a1 = a0 + K, *a2 = a1 + K;
                const float *b0 = B + (size_t)n0 * K, *b1 = b0 + K, *b2 = b1 + K, *b3 = b2 + K;
                for (int k = 0; k < K8; k += 8) {
                    const v8 x0 = *(const v8*)(a0 + k), x1 = *(const v8*)(a1 + k), x2 = *(const v8*)(a2 + k);
                    v8 y = *(const v8*)(b0 + k);
                    s[0][0] += x0 * y, s[1][0] += x1 * y, s[2][0] += x2 * y;
                    y = *(const v8*)(b1 + k);
                    s[0][1] += x0 * y, s[1][1] += x1 * y, s[2][1] += x2 * y;
                    y = *(const v8*)(b2 + k);
                    s[0][2] += x0 * y, s[1][2] += x1 * y, s[2][2] += x2 * y;
                    y = *(const v8*)(b3 + k);
                    s[0][3] += x0 * y, s[1][3] += x1 * y, s[2][3] += x2 * y;
                }
                for (int i = 0; i < 3; ++i)
                    for (int j = 0; j < 4; ++j) acc[i][j] = hsum(s[i][j]);
                for (int k = K8; k < K; ++k)
                    for (int i = 0; i < 3; ++i)
                        for (int j = 0; j < 4; ++j) acc[i][j] += A[(size_t)(m0 + i) * K + k] * B[(size_t)(n0 + j) * K + k];
            } else {
                for (int i = 0; i < mr; ++i)
                    for (int j = 0; j < nr; ++j) {
                        const float *a = A + (size_t)(m0 + i) * K, *b = B + (size_t)(n0 + j) * K;
                        float s = 0.f;
#pragma omp simd reduction(+ : s)
                        for (int k = 0; k < K; ++k) s += a[k] * b[k];
                        acc[i][j] = s;
                    }
            }
            for (int i = 0; i < mr; ++i)
                for (int j = 0; j < nr; ++j) {
                    const size_t o = (size_t)(m0 + i) * N + n0 + j;
                    float v = acc[i][j];
                    if (epilogue == 1) v = v > 0.f ? v : 0.f;
                    if (epilogue == 2) v += R[o];
                    C[o] = v;
                }
        }
    }
}

static inline float gelu_dot(float a, float b) {
    const float cdf = 0.5f * (1.0f + tanhf(a * (0.035677408136300125f * a * a + 0.7978845608028654f)));
    return a * cdf * b;
}

/* one expert: out = in + FFN(norm(in)); weights = [gamma d | wi h*d | wo d*h] or
 * [gamma d | wi_0 | wi_1 | wo]; ws holds rows*(d + 2h) floats */
void moe_cpu_t5ff(int rows, int d, int h, int norm_kind, int ffn_kind, const float* w, const float* in, float* out,
                  float* ws) {
    if (rows <= 0) return;
    const size_t dh = (size_t)d * h;
    float* ln = ws;
    float* h0 = ln + (size_t)rows * d;
    moe_cpu_layernorm(ln, in, rows, d, w, norm_kind);
    if (ffn_kind == FFN_GATED_GELU) {
        float* h1 = h0 + (size_t)rows * h;
        gemm_tn(h0, ln, w + d, rows, h, d, 0, NULL);
        gemm_tn(h1, ln, w + d + dh, rows, h, d, 0, NULL);
        const size_t n = (size_t)rows * h;
#pragma omp parallel for schedule(static)
        for (size_t i = 0; i < n; ++i) h0[i] = gelu_dot(h0[i], h1[i]);
        gemm_tn(out, h0, w + d + 2 * dh, rows, d, h, 2, in);
    } else {
        gemm_tn(h0, ln, w + d, rows, h, d, 1, NULL);
        gemm_tn(out, h0, w + d + dh, rows, d, h, 2, in);
    }
}

/*
 * Whole layer.  x [T][d]; centroids [E][d]; gamma [d] (cpm_2) or NULL; bias [E] or NULL;
 * weights: E pointers to expert slots (NULL array = Identity sub-layer); variant flags as
 * plugin/MoELayerPlugin.cc:44-58.  Outputs: y [T][d], sel[T], count[E].  Returns 0, or -1 when a
 * row has no orderable score.
 */
int moe_cpu_layer(int T, int d, int h, int E, const float* x, const float* centroids, const float* gamma,
                  const float* bias, int ln_before_score, int base_layer_mix, int norm_kind, int ffn_kind,
                  const float* const* weights, float* y, int32_t* sel, int32_t* count) {
    float* xaff = NULL;
    const float* xa = x;
    if (ln_before_score) {
        xaff = (float*)malloc(sizeof(float) * (size_t)T * d);
        moe_cpu_layernorm(xaff, x, T, d, gamma, norm_kind);
        xa = xaff;
    }
    float* coeff = (float*)malloc(sizeof(float) * (size_t)T);
    float* aff = (float*)malloc(sizeof(float) * (size_t)T * E);
    gemm_tn(aff, xa, centroids, T, E, d, 0, NULL);
    int bad = 0;
#pragma omp parallel for schedule(static) reduction(+ : bad)
    for (int t = 0; t < T; ++t) {
        float best = -3.402823466e+38f;
        int pos = -1;
        for (int e = 0; e < E; ++e) {
            const float s = aff[(size_t)t * E + e] + (bias ? bias[e] : 0.f);
            if (s > best) best = s, pos = e;
        }
        if (pos < 0) bad++, pos = 0;
        sel[t] = pos;
        coeff[t] = best;
    }
    free(aff);
    free(xaff);
    if (bad) {
        free(coeff);
        return -1;
    }
    int32_t* offset = (int32_t*)calloc((size_t)E + 1, sizeof(int32_t));
    int32_t* cursor = (int32_t*)malloc(sizeof(int32_t) * (size_t)E);
    int32_t* pos = (int32_t*)malloc(sizeof(int32_t) * (size_t)T);
    memset(count, 0, sizeof(int32_t) * (size_t)E);
    for (int t = 0; t < T; ++t) count[sel[t]]++;
    for (int e = 1; e <= E; ++e) offset[e] = offset[e - 1] + count[e - 1];
    memcpy(cursor, offset, sizeof(int32_t) * (size_t)E);
    for (int t = 0; t < T; ++t) pos[cursor[sel[t]]++] = t;

    float* routed = (float*)malloc(sizeof(float) * (size_t)T * d);
    float* post = (float*)malloc(sizeof(float) * (size_t)T * d);
#pragma omp parallel for schedule(static)
    for (int r = 0; r < T; ++r) memcpy(routed + (size_t)r * d, x + (size_t)pos[r] * d, sizeof(float) * d);

    if (weights == NULL) {
        memcpy(post, routed, sizeof(float) * (size_t)T * d);
    } else {
        int maxrows = 0;
        for (int e = 0; e < E; ++e) maxrows = count[e] > maxrows ? count[e] : maxrows;
        float* ws = (float*)malloc(sizeof(float) * (size_t)maxrows * ((size_t)d + 2 * (size_t)h));
        for (int e = 0; e < E; ++e)
            moe_cpu_t5ff(count[e], d, h, norm_kind, ffn_kind, weights[e], routed + (size_t)offset[e] * d,
                         post + (size_t)offset[e] * d, ws);
        free(ws);
    }
#pragma omp parallel for schedule(static)
    for (int r = 0; r < T; ++r) {
        float* o = y + (size_t)pos[r] * d;
        const float* p = post + (size_t)r * d;
        if (base_layer_mix) {
            const float a = 1.0f / (1.0f + expf(-coeff[pos[r]]));
            const float* q = routed + (size_t)r * d;
            for (int k = 0; k < d; ++k) o[k] = a * p[k] + (1.0f - a) * q[k];
        } else {
            memcpy(o, p, sizeof(float) * d);
        }
    }
    free(routed), free(post), free(pos), free(cursor), free(offset), free(coeff);
    return 0;
}
