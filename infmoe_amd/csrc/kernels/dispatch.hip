// Token dispatch and combine for gfx950.
//
// Replaces moe_expert_count, which the reference runs on the CPU between two blocking copies
// (plugin/cuda/moe.cu:161-212), by three small device kernels with no host round trip:
//   1. per-block histogram of the expert assignment,
//   2. one-workgroup exclusive scan over (block, expert) and over experts, which also emits the
//      row tiles of the grouped expert launch,
//   3. stable ranking: token t goes to row offset[e] + (tokens of e in earlier blocks) +
//      (tokens of e earlier in this block).  The rank inside a block is built from wave ballots
//      (one per bit of the expert index) in token order, so the permutation does not depend on the order atomics retire in and is
//      bit-identical to the reference's sequential counting sort.
// and the row-copy kernels batch_scatter_feature_and_weight_kernel / batch_gather_kernel /
// fused_batch_mix_and_gather_kernel (plugin/cuda/moe.cu:89-127) by wave-per-row copies with
// 16-byte accesses.
#include <hip/hip_runtime.h>

#include <initializer_list>
#include <mutex>

#include "device_math.h"
#include "kernels.h"

namespace infmoe {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
constexpr int kThreads = 256;
constexpr int kPerThread = kCountBlockTokens / kThreads;

__device__ __forceinline__ void hist_body(int T, int E, const int* __restrict__ sel, int* __restrict__ blockhist,
                                          int* s_hist) {
    for (int e = threadIdx.x; e < E; e += kThreads) s_hist[e] = 0;
    __syncthreads();
    const int base = blockIdx.x * kCountBlockTokens;
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
        const int t = base + j * kThreads + threadIdx.x;
        if (t < T) atomicAdd(&s_hist[min(max(sel[t], 0), E - 1)], 1);  // integer sums: order-free
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += kThreads) blockhist[(size_t)blockIdx.x * E + e] = s_hist[e];
}

__global__ __launch_bounds__(kThreads) void hist_kernel(int T, int E, const int* __restrict__ sel,
                                                        int* __restrict__ blockhist) {
    extern __shared__ int s_dyn[];
    hist_body(T, E, sel, blockhist, s_dyn);
}

constexpr int kMaxSortedTiles = 1024;  // row tiles the scan orders by cost; beyond that they stay in expert order
constexpr int kRunTiles = 4;           // row tiles of one expert that share their weight tiles through an XCD's L2

// `tiles` holds 2*max_tiles entries (the second half is spare), `sched` kSchedInts ints:
// [0] number of row tiles, [1 + x] first tile of XCD x (x = 0..8).
// Everything the single workgroup touches more than once lives in LDS: a chain of dependent global
// reads by one thread costs about a microsecond per link.
__device__ __forceinline__ void scan_body(int T, int E, int nblk, int* __restrict__ blockhist,
                                          int* __restrict__ count, int* __restrict__ offset,
                                          RowTile* __restrict__ tiles, int* __restrict__ sched, int max_tiles,
                                          int xcd_cap, int tile_rows, int skinny_max, int* s_dyn) {
    // s_dyn: [count E | offset E | first tile E]
    int* s_count = s_dyn;
    int* s_off = s_dyn + E;
    int* s_tile0 = s_dyn + 2 * E;
    __shared__ int s_n, s_total;
    __shared__ RowTile s_raw[kMaxSortedTiles];
    __shared__ int s_cost[kMaxSortedTiles];
    __shared__ int s_sched[kSchedInts];
    for (int e = threadIdx.x; e < E; e += kThreads) {
        int run = 0;
        for (int b = 0; b < nblk; ++b) {
            const int c = blockhist[(size_t)b * E + e];
            blockhist[(size_t)b * E + e] = run;  // tokens of e in earlier blocks
            run += c;
        }
        s_count[e] = run;
        count[e] = run;
    }
    __syncthreads();
    if (threadIdx.x == 0) {  // exclusive prefixes of rows and of row tiles (LDS only)
        int off = 0, nt = 0;
        for (int e = 0; e < E; ++e) {
            const int c = s_count[e];
            s_off[e] = off;
            s_tile0[e] = nt;
            if (c > skinny_max) nt += (c + tile_rows - 1) / tile_rows;  // tiles of row_tile_height(c, tile_rows)
            off += c;
        }
        s_total = off;
        s_n = nt;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += kThreads) offset[e] = s_off[e];
    if (threadIdx.x == 0) offset[E] = s_total;  // == T (plugin/MoELayerPlugin.cc:351)
    if (tiles == nullptr) return;
    const int n = s_n;
    const bool sorted = n <= kMaxSortedTiles;
    for (int e = threadIdx.x; e < E; e += kThreads) {
        const int c = s_count[e];
        if (c <= skinny_max) continue;
        int j = s_tile0[e];
        const int per = row_tile_height(c, tile_rows);
        // (runs: see below; an expert's nt tiles make as few runs as kRunTiles allows, of equal length)
        const int nt = (c + tile_rows - 1) / tile_rows, nruns = (nt + kRunTiles - 1) / kRunTiles;
        const int len = (nt + nruns - 1) / nruns;
        int p = 0, head = j, cost = 0;
        for (int m0 = 0; m0 < c; m0 += per, ++j) {
            RowTile rt;
            rt.expert = e;
            rt.row0 = s_off[e] + m0;
            rt.rows = min(per, c - m0);
            rt.pad = 0;
            if (sorted) {
                rt.pad = p | (min(len, nt - (head - s_tile0[e])) << 16);  // place in the run | length of the run
                s_raw[j] = rt;
                s_cost[j] = -1;  // not the head of a run (the head's entry is set when the run is complete)
                cost += (rt.rows + 15) >> 4;
                if (++p == len || m0 + per >= c) {
                    s_cost[head] = cost;  // a run is known by its first tile; its cost: the padded height of its tiles
                    p = 0, head = j + 1, cost = 0;
                }
            } else {
                tiles[j] = rt;  // many tiles balance by themselves: expert order, equal contiguous shares
            }
        }
    }
    if (!sorted) {
        if (threadIdx.x <= kXcdCount) sched[1 + threadIdx.x] = (int)(((long long)n * threadIdx.x) / kXcdCount);
        if (threadIdx.x == 0) sched[0] = n;
        return;
    }
    __shared__ int s_nruns;
    if (threadIdx.x == 0) s_nruns = 0;  // (no tiles at all: nobody counts the runs below)
    __syncthreads();
    // Runs.  The row tiles of an expert with several of them (all of one height but the last) are kept together
    // in runs of up to kRunTiles: a run goes to one XCD as a whole, and the launch takes its workgroups column tile
    // by column tile, the run's row tiles side by side, so that workgroups that start together read the same
    // weight rows and all but one find them in the XCD's L2.  (Tile by tile, an expert of 19 row tiles had its
    // weights fetched from memory 19 times.)  An expert's tiles are cut into as few runs as kRunTiles allows, of
    // equal length (made with the tiles, above); a run is the unit of the balance below.
    // Heaviest run first to the XCD with the least work so far (among those with room: the grid is sized for
    // xcd_cap tiles per XCD).  Inside an XCD the runs keep that order, so the light ones fill the tail.  The
    // assignment is sequential by nature; it is done by one wave whose lanes 0..7 each keep one XCD's work and
    // tile count in registers, 64 runs fetched from LDS at a time, the minimum found with three lane
    // exchanges inside the registers (one thread walking LDS took 0.3 us per run).
    __shared__ int s_order[kMaxSortedTiles];   // heads of runs by descending cost
    __shared__ int s_place[kMaxSortedTiles];   // per head: XCD << 16 | position inside the XCD's share
    for (int j = threadIdx.x; j < n; j += kThreads) {
        const int cj = s_cost[j];
        int rank = 0, heads = 0;
        for (int i = 0; i < n; ++i) {
            const int ci = s_cost[i];
            rank += (ci > cj) || (ci == cj && i < j);
            heads += ci >= 0;
        }
        if (cj >= 0) s_order[rank] = j;
        if (j == 0) s_nruns = heads;
    }
    __syncthreads();
    if (threadIdx.x < 64) {
        static_assert(kXcdCount == 8, "the minimum below is taken over eight lanes");
        const int lane = threadIdx.x;
        int load = 0, held = 0;  // lanes 0..7: work (padded 16-row units) and row tiles given to XCD `lane` so far
        const int nruns = s_nruns;
        auto lane_min = [](int v) {  // the minimum over each group of eight lanes, in all of them
            v = min(v, __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, false));   // lane ^ 1
            v = min(v, __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, false));   // lane ^ 2
            return min(v, __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, false));  // lane <-> 7 - lane
        };
        for (int r0 = 0; r0 < nruns; r0 += 64) {
            const int mine = r0 + lane < nruns ? s_order[r0 + lane] : 0;  // lane q: run r0 + q
            const int my_len = s_raw[mine].pad >> 16, my_cost = s_cost[mine];
            const int cnt = min(64, nruns - r0);
            for (int q = 0; q < cnt; ++q) {
                const int head = __builtin_amdgcn_readlane(mine, q), L = __builtin_amdgcn_readlane(my_len, q);
                const int cost = __builtin_amdgcn_readlane(my_cost, q);
                // (work << 3 | lane: the least work wins, the lower XCD on a tie; work stays far below 2^27)
                const int key = lane < kXcdCount && held + L <= xcd_cap ? (load << 3) | lane : 0x7fffffff;
                const int won = __builtin_amdgcn_readfirstlane(lane_min(key));
                // (no XCD with room cannot happen: the capacities add up to more than twice the tiles)
                const int best = won == 0x7fffffff ? 0 : won & 7;
                if (lane == best) {
                    s_place[head] = (best << 16) | held;
                    load += cost;
                    held += L;
                }
            }
        }
        int start = 0;
        for (int x = 0; x < kXcdCount; ++x) {
            if (lane == 0) s_sched[1 + x] = start;
            start += __builtin_amdgcn_readlane(held, x);
        }
        if (lane == 0) s_sched[1 + kXcdCount] = start, s_sched[0] = n;
    }
    __syncthreads();
    for (int j = threadIdx.x; j < n; j += kThreads) {
        const int p = s_raw[j].pad & 0xffff, head = j - p;
        const int place = s_place[head];
        tiles[s_sched[1 + (place >> 16)] + (place & 0xffff) + p] = s_raw[j];
    }
    if (threadIdx.x < 2 + kXcdCount) sched[threadIdx.x] = s_sched[threadIdx.x];
    (void)T;
    (void)max_tiles;
}

__global__ __launch_bounds__(kThreads) void scan_kernel(int T, int E, int nblk, int* __restrict__ blockhist,
                                                        int* __restrict__ count, int* __restrict__ offset,
                                                        RowTile* __restrict__ tiles, int* __restrict__ sched,
                                                        int max_tiles, int xcd_cap, int tile_rows, int skinny_max) {
    extern __shared__ int s_dyn[];
    scan_body(T, E, nblk, blockhist, count, offset, tiles, sched, max_tiles, xcd_cap, tile_rows, skinny_max, s_dyn);
}

__device__ __forceinline__ void rank_body(int T, int E, const int* __restrict__ sel,
                                          const int* __restrict__ blockbase, const int* __restrict__ offset,
                                          int* __restrict__ pos, int* __restrict__ row_expert, int* s_run) {
    // s_run: tokens of each expert already ranked in this block
    for (int e = threadIdx.x; e < E; e += kThreads) s_run[e] = offset[e] + blockbase[(size_t)blockIdx.x * E + e];
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned long long below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    const int base = blockIdx.x * kCountBlockTokens;
    const int index_bits = E > 1 ? 32 - __clz(E - 1) : 0;
    // all of this thread's assignments are fetched before the first barrier: inside the loop every
    // load would cost a memory round trip of its own
    int chosen[kPerThread];
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
        const int t = base + j * kThreads + threadIdx.x;
        chosen[j] = t < T ? min(max(sel[t], 0), E - 1) : -1;
    }
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
        const int t = base + j * kThreads + threadIdx.x;  // token order == (j, wave, lane) order
        const bool valid = t < T;
        const int e = chosen[j];
        // Lanes of this wave that chose the same expert: one ballot per bit of the expert index
        // (a lane keeps the lanes that agree with it on every bit), instead of one round per distinct
        // expert in the wave.
        unsigned long long same = __ballot(valid);
        for (int bit = 0; bit < index_bits; ++bit) {
            const bool set = (e >> bit) & 1;
            const unsigned long long m = __ballot(valid && set);
            same &= set ? m : ~m;
        }
        const int rank = __popcll(same & below);  // earlier lanes of the group
        const int cnt = __popcll(same);
        const bool leader = valid && (same & below) == 0;
        // waves take turns so that earlier tokens get lower rows; inside a wave every lane has read
        // its expert's running count before the leaders advance it (LDS operations of one wave
        // complete in order), so one barrier per turn is enough
        for (int w = 0; w < kThreads / 64; ++w) {
            if (wave == w) {
                const int r = valid ? s_run[e] + rank : 0;
                if (valid) {
                    pos[r] = t;
                    if (row_expert != nullptr) row_expert[r] = e;
                }
                if (leader) s_run[e] = r - rank + cnt;
            }
            __syncthreads();
        }
    }
}

__global__ __launch_bounds__(kThreads) void rank_kernel(int T, int E, const int* __restrict__ sel,
                                                        const int* __restrict__ blockbase,
                                                        const int* __restrict__ offset, int* __restrict__ pos,
                                                        int* __restrict__ row_expert) {
    extern __shared__ int s_dyn[];
    rank_body(T, E, sel, blockbase, offset, pos, row_expert, s_dyn);
}

// Up to kCountBlockTokens tokens (decode shapes): the three steps in one launch of one workgroup.
// What one step writes to global memory is read by the next after a barrier of the same workgroup.
__global__ __launch_bounds__(kThreads) void count_small_kernel(int T, int E, const int* __restrict__ sel,
                                                               int* __restrict__ blockhist, int* __restrict__ pos,
                                                               int* __restrict__ count, int* __restrict__ offset,
                                                               RowTile* __restrict__ tiles, int* __restrict__ sched,
                                                               int max_tiles, int xcd_cap, int tile_rows,
                                                               int skinny_max, int* __restrict__ row_expert) {
    extern __shared__ int s_dyn[];
    hist_body(T, E, sel, blockhist, s_dyn);
    __threadfence_block();
    __syncthreads();
    scan_body(T, E, 1, blockhist, count, offset, tiles, sched, max_tiles, xcd_cap, tile_rows, skinny_max, s_dyn);
    __threadfence_block();
    __syncthreads();
    rank_body(T, E, sel, blockhist, offset, pos, row_expert, s_dyn);
}

// ---- row copies: one wave per row, 16-byte accesses when the row length allows
template <bool VEC>
__device__ __forceinline__ void copy_row(float* __restrict__ dst, const float* __restrict__ src, int d, int lane) {
    if (VEC) {
        const int n4 = d >> 2;
        const v4f* s = reinterpret_cast<const v4f*>(src);
        v4f* o = reinterpret_cast<v4f*>(dst);
        int k = lane;
        for (; k + 192 < n4; k += 256) {  // four independent loads in flight
            const v4f a = s[k], b = s[k + 64], c = s[k + 128], e = s[k + 192];
            o[k] = a;
            o[k + 64] = b;
            o[k + 128] = c;
            o[k + 192] = e;
        }
        for (; k < n4; k += 64) o[k] = s[k];
    } else {
        for (int k = lane; k < d; k += 64) dst[k] = src[k];
    }
}

template <bool VEC>
__global__ __launch_bounds__(kThreads) void scatter_kernel(int T, int d, const float* __restrict__ x,
                                                           const float* __restrict__ coeff,
                                                           const int* __restrict__ pos, float* __restrict__ routed,
                                                           float* __restrict__ routed_coeff) {
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    if (r >= T) return;
    const int t = pos[r];
    copy_row<VEC>(routed + (size_t)r * d, x + (size_t)t * d, d, lane);
    if (lane == 0 && coeff != nullptr && routed_coeff != nullptr) routed_coeff[r] = coeff[t];
}

__device__ __forceinline__ float wave_sum_f(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

// The scatter with the row statistics of the experts' norm computed on the way (COPY), or the statistics alone
// of rows where they lie (pos == nullptr, no copy): stats[r] = (mu, rstd) of routed row r, as the first expert
// product wants them (the norm itself is folded into that product).  rms: mu = 0, rstd = rsqrt(mean(x^2) +
// eps).  centered: the mean, then a second sweep over the row (it has just been read: it comes from cache)
// for the variance about the mean - the exact two-pass form (plugin/cuda/ops/layernorm.cu:30-130 merges
// Welford partials instead).  Both launches run this code, so the numbers agree bit for bit.
template <bool VEC, bool COPY>
__global__ __launch_bounds__(kThreads) void scatter_stats_kernel(int T, int d, const float* __restrict__ x,
                                                                 const float* __restrict__ coeff,
                                                                 const int* __restrict__ pos,
                                                                 float* __restrict__ routed,
                                                                 float* __restrict__ routed_coeff,
                                                                 float* __restrict__ stats, int norm_kind) {
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    if (r >= T) return;
    const int t = pos != nullptr ? pos[r] : r;
    const float* src = x + (size_t)t * d;
    float* dst = COPY ? routed + (size_t)r * d : nullptr;
    float s1 = 0.f, s2 = 0.f;
    if (VEC) {
        const int n4 = d >> 2;
        const v4f* s = reinterpret_cast<const v4f*>(src);
        v4f* o = reinterpret_cast<v4f*>(dst);
        float p1[4] = {0.f, 0.f, 0.f, 0.f}, p2[4] = {0.f, 0.f, 0.f, 0.f};
        auto take = [&](const v4f& v, int q) {
            p1[q] += (v.x + v.y) + (v.z + v.w);
            p2[q] += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
        };
        int k = lane;
        for (; k + 192 < n4; k += 256) {  // four independent loads in flight
            const v4f a = s[k], b = s[k + 64], c = s[k + 128], e = s[k + 192];
            if (COPY) o[k] = a, o[k + 64] = b, o[k + 128] = c, o[k + 192] = e;
            take(a, 0), take(b, 1), take(c, 2), take(e, 3);
        }
        for (; k < n4; k += 64) {
            const v4f a = s[k];
            if (COPY) o[k] = a;
            take(a, 0);
        }
        s1 = (p1[0] + p1[1]) + (p1[2] + p1[3]);
        s2 = (p2[0] + p2[1]) + (p2[2] + p2[3]);
    } else {
        for (int k = lane; k < d; k += 64) {
            const float v = src[k];
            if (COPY) dst[k] = v;
            s1 += v;
            s2 += v * v;
        }
    }
    const float inv_d = 1.0f / (float)d;
    float mu = 0.f, rstd = 1.f;
    if (norm_kind == NORM_RMS) {
        rstd = 1.0f / sqrtf(wave_sum_f(s2) * inv_d + kNormEps);
    } else if (norm_kind == NORM_CENTERED) {
        mu = wave_sum_f(s1) * inv_d;
        float q = 0.f;
        if (VEC) {
            const int n4 = d >> 2;
            const v4f* s = reinterpret_cast<const v4f*>(src);
            float q4[4] = {0.f, 0.f, 0.f, 0.f};
            auto take = [&](const v4f& v, int i) {
                const v4f c = v - mu;
                q4[i] += (c.x * c.x + c.y * c.y) + (c.z * c.z + c.w * c.w);
            };
            int k = lane;
            for (; k + 192 < n4; k += 256) {
                const v4f a = s[k], b = s[k + 64], c = s[k + 128], e = s[k + 192];
                take(a, 0), take(b, 1), take(c, 2), take(e, 3);
            }
            for (; k < n4; k += 64) take(s[k], 0);
            q = (q4[0] + q4[1]) + (q4[2] + q4[3]);
        } else {
            for (int k = lane; k < d; k += 64) {
                const float c = src[k] - mu;
                q += c * c;
            }
        }
        rstd = 1.0f / sqrtf(wave_sum_f(q) * inv_d + kNormEps);
    }
    if (lane == 0) {
        stats[2 * (size_t)r] = mu;
        stats[2 * (size_t)r + 1] = rstd;
        if (COPY && coeff != nullptr && routed_coeff != nullptr) routed_coeff[r] = coeff[t];
    }
}

template <bool VEC>
__global__ __launch_bounds__(kThreads) void gather_kernel(int T, int d, const float* __restrict__ buf,
                                                          const int* __restrict__ pos, float* __restrict__ out,
                                                          const float* __restrict__ routed_coeff) {
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    if (r >= T) return;
    float* dst = out + (size_t)pos[r] * d;
    if (routed_coeff != nullptr && isnan(routed_coeff[r])) {  // a token the gating could not score: NaN out
        for (int k = lane; k < d; k += 64) dst[k] = __builtin_nanf("");
        return;
    }
    copy_row<VEC>(dst, buf + (size_t)r * d, d, lane);
}

template <bool VEC>
__global__ __launch_bounds__(kThreads) void mix_gather_kernel(int T, int d, const int* __restrict__ pos,
                                                              const float* __restrict__ routed,
                                                              const float* __restrict__ post,
                                                              const float* __restrict__ routed_coeff,
                                                              float* __restrict__ out) {
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    if (r >= T) return;
    // plugin/cuda/common.cuh:24-27 and plugin/cuda/moe.cu:120-126
    const float a = sigmoid_f(routed_coeff[r]);
    const float b = 1.0f - a;
    auto mix4 = [&](const v4f& pv, const v4f& qv) {
        return v4f{mix_value(a, b, pv.x, qv.x), mix_value(a, b, pv.y, qv.y), mix_value(a, b, pv.z, qv.z),
                   mix_value(a, b, pv.w, qv.w)};
    };
    const float* p = post + (size_t)r * d;
    const float* q = routed + (size_t)r * d;
    float* o = out + (size_t)pos[r] * d;
    if (VEC) {
        const int n4 = d >> 2;
        const v4f* p4 = reinterpret_cast<const v4f*>(p);
        const v4f* q4 = reinterpret_cast<const v4f*>(q);
        v4f* o4 = reinterpret_cast<v4f*>(o);
        int k = lane;
        for (; k + 64 < n4; k += 128) {
            const v4f p0 = p4[k], p1 = p4[k + 64], q0 = q4[k], q1 = q4[k + 64];
            o4[k] = mix4(p0, q0);
            o4[k + 64] = mix4(p1, q1);
        }
        for (; k < n4; k += 64) o4[k] = mix4(p4[k], q4[k]);
    } else {
        for (int k = lane; k < d; k += 64) o[k] = mix_value(a, b, p[k], q[k]);
    }
}

__global__ void fill_i32_kernel(int* __restrict__ dst, int n, int value) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = value;
}

inline dim3 row_grid(int T) { return dim3((T + kThreads / 64 - 1) / (kThreads / 64)); }

// 16-byte accesses need rows that start on 16-byte boundaries
inline bool vec_ok(int d, std::initializer_list<const void*> ptrs) {
    if (d % 4 != 0) return false;
    for (const void* p : ptrs)
        if (reinterpret_cast<uintptr_t>(p) & 15) return false;
    return true;
}

}  // namespace

size_t expert_count_scratch_bytes(int T, int E) {
    const size_t nblk = (size_t)(T + kCountBlockTokens - 1) / kCountBlockTokens;
    return ((nblk * (size_t)E * sizeof(int)) + 255) & ~(size_t)255;
}

hipError_t launch_expert_count(int T, int E, const int* sel, int* pos, int* count, int* offset, void* scratch,
                               RowTile* tiles, int* sched, int tile_rows, int skinny_max, int* row_expert,
                               hipStream_t stream, bool hist_ready) {
    const int nblk = (T + kCountBlockTokens - 1) / kCountBlockTokens;
    int* blockhist = static_cast<int*>(scratch);
    const size_t lds = (size_t)E * sizeof(int);
    const int max_tiles = max_row_tiles(T, E, tile_rows);
    if (nblk == 1) {
        count_small_kernel<<<1, kThreads, 3 * lds, stream>>>(T, E, sel, blockhist, pos, count, offset, tiles, sched,
                                                             max_tiles, xcd_tile_capacity(max_tiles), tile_rows,
                                                             skinny_max, row_expert);
        return hipGetLastError();
    }
    if (nblk > 0 && !hist_ready) hist_kernel<<<nblk, kThreads, lds, stream>>>(T, E, sel, blockhist);
    scan_kernel<<<1, kThreads, 3 * lds, stream>>>(T, E, nblk, blockhist, count, offset, tiles, sched, max_tiles,
                                            xcd_tile_capacity(max_tiles), tile_rows, skinny_max);
    if (nblk > 0) rank_kernel<<<nblk, kThreads, lds, stream>>>(T, E, sel, blockhist, offset, pos, row_expert);
    return hipGetLastError();
}

// ---- the same three kernels with their block-histogram scratch in a device array of the library
// instead of in memory the caller brings.  The array exists once per GPU (each device holds its own
// copy at its own address); its address is looked up once per device, with that device current, and
// kept.  Host code never passes the array's name to a kernel: the name is a host-side handle of the
// symbol, not a device address.
namespace {
static __device__ __align__(256) int g_count_scratch[kExpertCountStaticInts];
constexpr int kMaxDevices = 64;

hipError_t static_count_scratch(int** out) {
    static std::mutex lock;
    static int* ptrs[kMaxDevices] = {};
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return err;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> guard(lock);
    if (ptrs[dev] == nullptr) {
        void* p = nullptr;
        err = hipGetSymbolAddress(&p, HIP_SYMBOL(g_count_scratch));
        if (err != hipSuccess) return err;
        if (p == nullptr) return hipErrorInvalidSymbol;
        ptrs[dev] = static_cast<int*>(p);
    }
    *out = ptrs[dev];
    return hipSuccess;
}
}  // namespace

hipError_t launch_expert_count_static(int T, int E, const int* sel, int* pos, int* count, int* offset,
                                      hipStream_t stream) {
    if (expert_count_scratch_bytes(T, E) > sizeof(int) * kExpertCountStaticInts) return hipErrorInvalidValue;
    int* blockhist = nullptr;
    const hipError_t err = static_count_scratch(&blockhist);
    if (err != hipSuccess) return err;
    // every entry the scan and the ranking read is written by the histogram of the same call, so
    // nothing of an earlier call's contents has to be cleared
    return launch_expert_count(T, E, sel, pos, count, offset, blockhist, nullptr, nullptr, kGemmTileRows, 0, nullptr,
                               stream);
}

hipError_t launch_fill_i32(int* dst, int n, int value, hipStream_t stream) {
    if (n <= 0) return hipSuccess;
    fill_i32_kernel<<<(n + 255) / 256, 256, 0, stream>>>(dst, n, value);
    return hipGetLastError();
}

hipError_t launch_row_stats(float* stats, const float* in, int rows, int d, int norm_kind, hipStream_t stream) {
    if (rows <= 0) return hipSuccess;
    if (vec_ok(d, {in}))
        scatter_stats_kernel<true, false><<<row_grid(rows), kThreads, 0, stream>>>(rows, d, in, nullptr, nullptr, nullptr,
                                                                                   nullptr, stats, norm_kind);
    else
        scatter_stats_kernel<false, false><<<row_grid(rows), kThreads, 0, stream>>>(rows, d, in, nullptr, nullptr, nullptr,
                                                                                    nullptr, stats, norm_kind);
    return hipGetLastError();
}

hipError_t launch_scatter(int T, int d, const float* x, const float* coeff, const int* pos, float* routed,
                          float* routed_coeff, hipStream_t stream, float* row_stats, int norm_kind) {
    if (T <= 0) return hipSuccess;
    if (row_stats != nullptr) {
        if (vec_ok(d, {x, routed}))
            scatter_stats_kernel<true, true><<<row_grid(T), kThreads, 0, stream>>>(T, d, x, coeff, pos, routed, routed_coeff,
                                                                                   row_stats, norm_kind);
        else
            scatter_stats_kernel<false, true><<<row_grid(T), kThreads, 0, stream>>>(T, d, x, coeff, pos, routed, routed_coeff,
                                                                                    row_stats, norm_kind);
        return hipGetLastError();
    }
    if (vec_ok(d, {x, routed}))
        scatter_kernel<true><<<row_grid(T), kThreads, 0, stream>>>(T, d, x, coeff, pos, routed, routed_coeff);
    else
        scatter_kernel<false><<<row_grid(T), kThreads, 0, stream>>>(T, d, x, coeff, pos, routed, routed_coeff);
    return hipGetLastError();
}

hipError_t launch_gather(int T, int d, const float* buf, const int* pos, float* out, hipStream_t stream,
                         const float* routed_coeff) {
    if (T <= 0) return hipSuccess;
    if (vec_ok(d, {buf, out}))
        gather_kernel<true><<<row_grid(T), kThreads, 0, stream>>>(T, d, buf, pos, out, routed_coeff);
    else
        gather_kernel<false><<<row_grid(T), kThreads, 0, stream>>>(T, d, buf, pos, out, routed_coeff);
    return hipGetLastError();
}

hipError_t launch_mix_gather(int T, int d, const int* pos, const float* routed, const float* post,
                             const float* routed_coeff, float* out, hipStream_t stream) {
    if (T <= 0) return hipSuccess;
    if (vec_ok(d, {routed, post, out}))
        mix_gather_kernel<true><<<row_grid(T), kThreads, 0, stream>>>(T, d, pos, routed, post, routed_coeff, out);
    else
        mix_gather_kernel<false><<<row_grid(T), kThreads, 0, stream>>>(T, d, pos, routed, post, routed_coeff, out);
    return hipGetLastError();
}

}  // namespace infmoe
