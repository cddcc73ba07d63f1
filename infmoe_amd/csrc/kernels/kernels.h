// Host-side launchers of the gfx950 kernels.  Plain C++ signatures (no HIP kernel syntax) so
// the host code of the layer and of the sub-layers can be read without the device code.
// Every launcher is asynchronous on `stream` and returns the hipError_t of the launch.
#pragma once

#include <hip/hip_runtime_api.h>

#include <atomic>
#include <cstddef>
#include <cstdint>

#include "../../../include/infmoe_sublayer.h"  // RowTile

namespace infmoe {

enum NormKind : int32_t { NORM_NONE = 0, NORM_RMS = 1, NORM_CENTERED = 2 };
enum FfnKind : int32_t { FFN_RELU = 0, FFN_GATED_GELU = 1 };

constexpr float kNormEps = 1e-6f;  // plugin/MoELayerPlugin.cc:324, plugin/sublayers/T5FFLayer.cc:102

// ---- gating (replaces layernorm_gpu + cublasSgemm + expert_select_top1_kernel,
//      plugin/MoELayerPlugin.cc:315-345)
// Optional: folded_centroids [E][d] = centroids * gamma (device) and centroid_stats [2E] = per expert
// the sum and the Euclidean norm of that product (device), both made by fold_centroids_host; with
// them the kernel skips work that depends on the layer's parameters only.
// Optional: scratch (gate_scratch_floats(T, d, E) floats, any contents): with it the embedding dimension
// of a call with few tokens is split over several workgroups per token group, and a second launch adds
// their partial scores and selects.
// zero_stats: `stats` (4 ints) is set to zero before anything is counted into it, by the first of two
// launches where there are two, else by a small fill launch; without it the caller has cleared them.
// A token without an orderable score (a NaN in its row; the reference asserts, plugin/cuda/moe.cu:70) gets
// expert 0 and the coefficient NaN, is counted in stats[1], and sets *nan_flag (an int the device can
// write, e.g. page-locked host memory) to nan_value (say, a number that names the call) when that pointer is given.
// Optional: block_hist, the scratch of launch_expert_count for the same T and E.  A call that takes the two-launch
// path for many tokens leaves the first pass of the counting sort in it (tokens per expert of every block of
// kCountBlockTokens tokens) and sets *block_hist_done; launch_expert_count is then told to skip that pass.
size_t gate_scratch_floats(int T, int d, int E);
hipError_t launch_gate_top1(int T, int d, int E, const float* x, const float* centroids, const float* gamma,
                            int norm_kind, const float* score_bias, int* sel, float* coeff, int* stats,
                            hipStream_t stream, const float* folded_centroids = nullptr,
                            const float* centroid_stats = nullptr, float* scratch = nullptr,
                            size_t scratch_floats = 0, bool zero_stats = false, int* nan_flag = nullptr,
                            int nan_value = 1, int* block_hist = nullptr, bool* block_hist_done = nullptr);
// Calls with many tokens: the first of two launches writes partial scores per slice of the embedding
// dimension with that slice of the folded centroids resident in LDS (gating_slab.hip); the combine launch
// of the gating kernel adds the slices and selects.  The plan says how a call is cut; gate_slab_plan
// returns false for shapes this path does not take (more than 128 experts, d not a multiple of 128, few tokens,
// scratch too small).
struct GateSlabPlan {
    int ks;              // floats of the embedding dimension per slice (a multiple of 128)
    int slices;          // d / ks, at most kGateMaxSlices
    int waves;           // waves per workgroup: 4 or 8, each 16 tokens at a time
    int tiles_per_wave;  // 16-token tiles a wave takes in turn
    int groups;          // workgroups per slice
};
constexpr int kGateMaxSlices = 16;
constexpr int kGateSlabMinTokens = 1024;
bool gate_slab_plan(int T, int d, int E, size_t scratch_floats, GateSlabPlan* plan);
size_t gate_slab_scratch_floats(int T, int d, int E);
// partials: [slices][T][E + 2] floats (dot products, row sum, row sum of squares)
// zero_stats: null, or 4 ints that the launch sets to zero (the combine launch counts into them)
// zero_hist: null, or n_hist ints that the launch sets to zero (the block histogram the combine launch adds into)
hipError_t launch_gate_slab(const GateSlabPlan& plan, int T, int d, int E, const float* x,
                            const float* folded_centroids, float* partials, hipStream_t stream,
                            int* zero_stats = nullptr, int* zero_hist = nullptr, int n_hist = 0);
// The second launch of a sliced gating call: adds the slices' partial scores ([slices][T][E + 2]), selects,
// and re-scores near ties in float64 from x, the plain centroids and gamma.  Takes up to 128 experts and
// rows of 16-byte-aligned float4 (gate_combine_ok); centroid_stats as fold_centroids_host makes them.
bool gate_combine_ok(int d, int E);
hipError_t launch_gate_combine(int T, int d, int E, int slices, const float* partials, const float* centroid_stats,
                               const float* x, const float* centroids, const float* gamma, int norm_kind,
                               const float* score_bias, int* sel, float* coeff, int* stats, int* nan_flag,
                               hipStream_t stream, int nan_value, float err_depth, int* block_hist = nullptr);
// n of the rounding-error bound n * FLT_EPSILON * rstd * |x| * max|g c| under which two FP32 scores are not
// trusted to be in the exact order (such a token is re-scored in float64): slices of `slice_floats` floats of the
// embedding dimension, `slices` of them.
float gate_err_depth(int slice_floats, int slices, int norm_kind);
void fold_centroids_host(int d, int E, const float* centroids, const float* gamma, float* folded, float* cstats);

// ---- dispatch (replaces moe_expert_count, plugin/cuda/moe.cu:161-212)
// (RowTile, the unit of work of the grouped expert GEMM - `rows` consecutive routed rows of one expert -
// is declared in the public plug-in header.)
constexpr int kCountBlockTokens = 1024;  // tokens ranked by one workgroup
size_t expert_count_scratch_bytes(int T, int E);
constexpr int kXcdCount = 8;    // accelerator dies of an MI355X; workgroup ids are dealt to them round-robin
constexpr int kSchedInts = 16;  // [0] number of row tiles, [1..9] first tile of each XCD's share
inline int max_row_tiles(int T, int E, int tile_rows) { return (T + tile_rows - 1) / tile_rows + E; }
// Height of the row tiles an expert's `rows` rows are cut into when no tile may exceed `tile_rows` (a
// multiple of 16): as few tiles as that allows, all of one height (a multiple of 16; the last tile
// takes what is left), so that 300 rows become 160 + 140 rather than 256 + 44.  The grouped and the
// one-expert launches both cut by this rule: which matrix instruction a row meets depends on its
// place in its tile, and the two schedules have to agree bit for bit.
#if defined(__HIPCC__)
__host__ __device__
#endif
inline int row_tile_height(int rows, int tile_rows) {
    const int n = (rows + tile_rows - 1) / tile_rows;
    return n <= 1 ? tile_rows : ((rows + n - 1) / n + 15) / 16 * 16;
}
// Most row tiles one XCD may be given (bounds the grid of the grouped launch).
inline int xcd_tile_capacity(int max_tiles) {
    const int cap = 2 * ((max_tiles + kXcdCount - 1) / kXcdCount) + 8;
    return cap < max_tiles ? cap : max_tiles;
}
// Optional outputs for the grouped expert launch (all may be null):
//   tiles (2*max_row_tiles entries) / sched (kSchedInts ints): row tiles of height <= tile_rows
//     over the experts with more than `skinny_max` rows, dealt to the 8 XCDs so that the padded
//     row counts balance, each XCD's share in descending height
//   row_expert[T]: expert of every routed row
// hist_ready: the scratch already holds the per-block histogram of sel (launch_gate_top1 left it there).
hipError_t launch_expert_count(int T, int E, const int* sel, int* pos, int* count, int* offset, void* scratch,
                               RowTile* tiles, int* sched, int tile_rows, int skinny_max, int* row_expert,
                               hipStream_t stream, bool hist_ready = false);

// The same with the scratch in a device array owned by the library (kExpertCountStaticInts ints per GPU,
// held until the process ends): no allocation and no caller-supplied scratch.  Calls on one GPU share
// the array, so calls that overlap there race.  hipErrorInvalidValue when the scratch would not fit.
constexpr size_t kExpertCountStaticInts = 64 * 1024;
hipError_t launch_expert_count_static(int T, int E, const int* sel, int* pos, int* count, int* offset,
                                      hipStream_t stream);

// Small fill kernel (used instead of hipMemsetAsync so that callers may capture the layer in a graph).
hipError_t launch_fill_i32(int* dst, int n, int value, hipStream_t stream);

// ---- scatter / gather / mix (replaces plugin/cuda/moe.cu:214-258)
// row_stats: null, or [T][2] that receives launch_row_stats' numbers (norm_kind) for every routed row
hipError_t launch_scatter(int T, int d, const float* x, const float* coeff, const int* pos, float* routed,
                          float* routed_coeff, hipStream_t stream, float* row_stats = nullptr,
                          int norm_kind = NORM_NONE);
// routed_coeff: null, or [T]; a routed row whose coefficient is NaN (a token the gating could not score) is
// written as NaN in full
hipError_t launch_gather(int T, int d, const float* buf, const int* pos, float* out, hipStream_t stream,
                         const float* routed_coeff = nullptr);
hipError_t launch_mix_gather(int T, int d, const int* pos, const float* routed, const float* post,
                             const float* routed_coeff, float* out, hipStream_t stream);

// ---- row norm (replaces layernorm_gpu, plugin/cuda/ops/layernorm.cu:176-188)
// gamma of row r is gamma_base + slot(row_expert[r]) * gamma_stride (row_expert null -> gamma_base), where
// slot(e) = expert_slot[e], or e when expert_slot is null.
hipError_t launch_row_norm(float* out, const float* in, int rows, int d, const float* gamma_base,
                           size_t gamma_stride, const int* row_expert, int norm_kind, hipStream_t stream,
                           const int* expert_slot = nullptr);

// Row statistics of the norm: stats[r] = (mu_r, rstd_r) with mu_r = 0 and rstd_r = rsqrt(mean(x^2) + eps) for
// the rms form, the mean and rsqrt(biased variance + eps) for the centered one (two exact passes).  The
// scatter of the layer computes the same numbers, by the same device code, while it copies the rows.
hipError_t launch_row_stats(float* stats, const float* in, int rows, int d, int norm_kind, hipStream_t stream);

// In place: w[n][k] *= gamma[k] for the n_rows rows of a [n_rows][d] weight matrix (what the norm-carrying
// first product wants of an expert's input-side weights).
hipError_t launch_fold_gamma(float* w, const float* gamma, int n_rows, int d, hipStream_t stream);

// ---- expert GEMMs (replace the three cublasSgemm_v2 calls, fused_gelu_dot_gpu and the D2D
//      residual copy of plugin/sublayers/T5FFLayer.cc:112-138)
// The first product of the feed-forward block can carry the block's RMS row norm with it (plugin/sublayers/
// T5FFLayer.cc:99-103 runs the norm as a launch of its own and keeps the normed rows in memory): with weights
// whose columns were multiplied by gamma (launch_fold_gamma) and the rows' rstd_r from launch_row_stats, the
// product of the normed rows with the plain weights is P = rstd_r * (A*B^T) on the raw rows A.  Without row
// statistics P = A*B^T.  (The centered norm is not carried this way: rstd_r * (A*B^T - mu_r * sum_k B_nk)
// subtracts two large numbers when a row's mean is large against its deviation, and then loses to the
// reference's order of operations - norm first - by orders of magnitude.  It stays a launch of its own.)
enum Epilogue : int32_t {
    EPI_RELU = 0,        // C = max(P, 0)
    EPI_GATED_GELU = 1,  // C = gelu_tanh(P0) * P1
    EPI_RESIDUAL = 2     // C = R + A*B^T
};
struct GemmProblem {
    const float* A;    // [rows][K] activations (row stride K)
    const float* B;    // [N][K] weights, K contiguous (torch Linear layout)
    const float* B1;   // second weight matrix for EPI_GATED_GELU, else null
    const float* R;    // [rows][N] residual for EPI_RESIDUAL, else null
    float* C;          // [rows][N]
    int N, K;
    int epilogue;
    // EPI_RELU / EPI_GATED_GELU with the RMS norm carried along: row_stats [rows][2] = (-, rstd) per row of A
    // (the pairs launch_row_stats writes).  Null: the plain product.
    const float* row_stats;
    // grouped launches only: null, or [E] where expert e's weights are at B + expert_slot[e] * weight_stride
    // instead of B + e * weight_stride (experts held in slots in whatever order they arrived)
    const int* expert_slot;
    // nonzero: the call has few rows per expert (gemm_small_tiles()) and its tiles, of at most kGemmTileRowsSmall
    // rows, go to the kernels that run two workgroups per compute unit.  Not with EPI_GATED_GELU.
    int small_tiles;
};
// One expert, `rows` known on the host, cut into row tiles of at most `tile_rows` rows (a multiple of
// 16 no larger than gemm_tile_rows(p.epilogue); both launches of a sub-layer pass the same value so
// that they cut the rows as the grouped launch does).
hipError_t launch_expert_gemm(const GemmProblem& p, int rows, int tile_rows, hipStream_t stream);
// All experts in one launch: A, R, C address routed rows globally; expert e's weights are at
// B + e*weight_stride (floats).  Row tiles and their number come from launch_expert_count.
hipError_t launch_expert_gemm_grouped(const GemmProblem& p, size_t weight_stride, const RowTile* tiles,
                                      const int* sched, int max_tiles, hipStream_t stream);
// Whether the grouped matrix-core launch takes this problem (K a multiple of 32, 16-byte aligned
// operands); if not, the launch below does every routed row (row r with the weights of expert
// row_expert[r]) one output element per thread.
bool expert_gemm_grouped_ok(const GemmProblem& p, size_t weight_stride);
hipError_t launch_expert_gemm_any_shape_grouped(const GemmProblem& p, size_t weight_stride, const int* row_expert,
                                                int rows, hipStream_t stream);
constexpr int kGemmTileRows = 256;       // tallest row tile of the GEMM kernel
constexpr int kGemmTileRowsGated = 192;  // ... of its two-matrix (gated) form (two accumulator sets)
constexpr int kGemmTileRowsSmall = 96;   // ... of the form for calls with few rows per expert
inline int gemm_tile_rows(int epilogue, bool small_tiles = false) {
    return epilogue == EPI_GATED_GELU ? kGemmTileRowsGated : (small_tiles ? kGemmTileRowsSmall : kGemmTileRows);
}
// Whether a layer call of `tokens` tokens over `experts` experts takes the few-rows-per-expert form of the
// matrix-core kernels (on average at most 64 rows per expert; an expert with more than kGemmTileRowsSmall is
// cut into several tiles).  A function of the call's shape only: the grouped and the per-expert schedule of a
// layer have to pick the same kernel for the same expert to agree bit for bit.
inline bool gemm_small_tiles(int tokens, int experts, int ffn_kind) {
    return ffn_kind != FFN_GATED_GELU && (long long)tokens <= 64ll * experts;
}

// Few-row experts (decode): every weight row is streamed once and dotted with up to kSkinnyMaxRows activation
// rows held in registers; an expert with more rows is done in runs of kSkinnyMaxRows, one pass over its weights
// each.
constexpr int kSkinnyMaxRows = 8;
hipError_t launch_expert_skinny(const GemmProblem& p, int rows, hipStream_t stream);
hipError_t launch_expert_skinny_grouped(const GemmProblem& p, size_t weight_stride, const int* count,
                                        const int* offset, int E, hipStream_t stream);

// Kernels whose dynamic LDS exceeds 64 KB need the limit raised once per device.  Doing it on the
// first launch only keeps later launches free of runtime calls other than the launch itself, so a
// caller may capture them in a graph after one eager call.
template <auto Kern>
inline hipError_t allow_lds_once(size_t bytes) {
    static std::atomic<uint64_t> done{0};
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return err;
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    err = hipFuncSetAttribute(reinterpret_cast<const void*>(Kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (err == hipSuccess) done.fetch_or(bit, std::memory_order_release);
    return err;
}

}  // namespace infmoe
