/*
 * infmoe.h - C ABI of the MI355X (gfx950) MoE layer: a drop-in for the math of
 * InfMoE's MoELayerPlugin hot path.
 *
 * Plain C types only: device and host buffers are `void*` / `float*`, the HIP
 * stream is passed as `void*` (a hipStream_t).  Every function returns an
 * infmoe_status (0 = OK) and never aborts or throws; the message of the last
 * failure on the calling thread is available from infmoe_last_error().
 * Citations are file:line in the Harry-Chen/InfMoE tree.
 *
 * Call order (mirrors the TensorRT lifecycle the reference is driven by,
 * plugin/MoELayerPlugin.h:91-133):
 *   infmoe_create -> [infmoe_set_expert_weights ...] -> infmoe_configure ->
 *   infmoe_workspace_size -> infmoe_initialize -> infmoe_enqueue ... ->
 *   infmoe_terminate -> infmoe_destroy
 *
 * Threading: one infmoe_enqueue in flight per handle.  Work is ordered after
 * prior work on the caller's stream; on return everything the call launched is
 * either on that stream or joined back into it by events, so the output is
 * ready when the caller's stream reaches that point.  The host is blocked once
 * per call only when experts are streamed (max_concurrency < expert_count).
 */
#ifndef INFMOE_H
#define INFMOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum infmoe_status {
    INFMOE_OK = 0,
    INFMOE_ERR_INVALID_ARGUMENT = 1, /* bad pointer, size or shape */
    INFMOE_ERR_UNKNOWN_FIELD = 2,    /* plugin/MoELayerPluginCreator.cc:111-114 */
    INFMOE_ERR_MISSING_FIELD = 3,    /* plugin/MoELayerPluginCreator.cc:118-125, plugin/MoELayerPlugin.cc:76-79 */
    INFMOE_ERR_UNSUPPORTED = 4,      /* unknown variant / sub-layer: plugin/MoELayerPlugin.cc:37-40,53-56 */
    INFMOE_ERR_IO = 5,               /* weight file missing / malformed: plugin/MoELayerPluginCreator.cc:132-140 */
    INFMOE_ERR_STATE = 6,            /* call order violated (e.g. enqueue before initialize) */
    INFMOE_ERR_HIP = 7,              /* a HIP runtime call failed (plugin/utility.h:13-21 exits instead) */
    INFMOE_ERR_NAN = 8               /* a token had no orderable score (plugin/cuda/moe.cu:70,184 assert instead);
                                        see infmoe_enqueue for when it is reported */
} infmoe_status;

/* Same numeric values as nvinfer1::PluginFieldType so a caller can pass fields through. */
typedef enum infmoe_field_type {
    INFMOE_FIELD_FLOAT32 = 1,
    INFMOE_FIELD_INT32 = 5,
    INFMOE_FIELD_CHAR = 6,
    INFMOE_FIELD_UNKNOWN = 8 /* the reference passes its strings with this type (plugin/MoELayerPluginCreator.cc:39-44) */
} infmoe_field_type;

/* Mirrors nvinfer1::PluginField {name, data, type, length}. */
typedef struct infmoe_field {
    const char* name;
    const void* data;
    int32_t type;   /* infmoe_field_type */
    int32_t length; /* element count (chars for strings) */
} infmoe_field;

typedef struct infmoe_plugin infmoe_plugin; /* opaque: replaces class MoELayerPlugin */

/* ---------------------------------------------------------------- life cycle */

/*
 * Replaces MoELayerPluginCreator::createPlugin (plugin/MoELayerPluginCreator.cc:58-148).
 * Recognised fields (names, types and defaults as plugin/MoELayerPluginCreator.cc:15-47,65):
 *   expert_count, embedding_size, hidden_size, max_concurrency (INT32 x1, mc default 2)
 *   expert_centroids  FLOAT32[E*d], in-memory layout [E][d] (plugin/MoELayerPlugin.cc:334-336)
 *   expert_weight_file   chars (npz path; may be omitted when weights are given by pointer)
 *   expert_sublayer_type chars: "T5_FF" | "Identity"
 *   moe_variant          chars: "cpm_2" | "base_layer" | "default"
 *   layernorm_weight     FLOAT32[d], required iff cpm_2 (plugin/MoELayerPlugin.cc:76-79)
 * Two optional fields the reference does not have, because its code and its README
 * disagree (code: plugin/cuda/ops/layernorm.cu:149-161, plugin/sublayers/T5FFLayer.cc:105-138;
 * README.md:113-117):
 *   norm_kind  chars: "rms" (default) | "centered"
 *   ffn_kind   chars: "relu" (default; weights wi_weight, wo_weight) |
 *                     "gated_gelu" (weights wi_0_weight, wi_1_weight, wo_weight)
 * Arrays and strings are copied; the caller keeps ownership of `fields`.
 * Any positive sizes are accepted, as in the reference.  The matrix-core expert kernels take embedding_size and
 * hidden_size that are multiples of 32 (every size in the reference's examples but the README's toy one); other
 * sizes compute the same results on a plain one-output-per-thread kernel at a few percent of that speed.
 */
int32_t infmoe_create(const char* layer_name, const infmoe_field* fields, int32_t n_fields, infmoe_plugin** out);

/* Replaces MoELayerPlugin::clone (plugin/MoELayerPlugin.cc:83-102,465-468): parameters are
 * deep-copied, the sub-layer (and so the expert weights) is shared. */
int32_t infmoe_clone(const infmoe_plugin* src, infmoe_plugin** out);

/*
 * By-pointer weight provider (no counterpart in the reference, which only reads the npz
 * file: plugin/sublayers/T5FFLayer.cc:143-147).  `key` is the npz member name without the
 * "<expert>/" prefix: layer_norm_weight [d]; wi_weight [h][d] or wi_0_weight, wi_1_weight
 * [h][d]; wo_weight [d][h] (plugin/sublayers/T5FFLayer.cc:61-87, python/infmoe/config.py:46-52).
 * `host` holds `count` floats and is copied into the sub-layer's page-locked store before
 * the call returns.  Must be called before infmoe_initialize.
 */
int32_t infmoe_set_expert_weights(infmoe_plugin* p, int32_t expert, const char* key, const float* host, size_t count);

/* Harness extension: per-expert additive bias on the gating score (NULL clears it).  Not a
 * reference attribute; used to produce skewed routing.  `host` holds E floats. */
int32_t infmoe_set_score_bias(infmoe_plugin* p, const float* host);

/* Replaces configurePlugin (plugin/MoELayerPlugin.cc:170-180): dims must be [B, S, embedding_size]. */
int32_t infmoe_configure(infmoe_plugin* p, const int32_t* dims, int32_t nb_dims);

/* Replaces getWorkspaceSize (plugin/MoELayerPlugin.cc:253-273).  Bytes of caller-owned device
 * scratch infmoe_enqueue needs for an input of `dims`.  Never smaller for more tokens: a workspace sized for
 * the largest batch serves every smaller one. */
int32_t infmoe_workspace_size(const infmoe_plugin* p, const int32_t* dims, int32_t nb_dims, size_t* out_bytes);

/* Replaces initialize (plugin/MoELayerPlugin.cc:197-201 -> plugin/sublayers/T5FFLayer.cc:143-147):
 * loads expert weights into page-locked host memory, uploads centroids / gating gamma, creates
 * streams and events, and, when max_concurrency >= expert_count, uploads every expert once into
 * plugin-owned device memory (the reference re-copies on every enqueue, plugin/MoELayerPlugin.cc:365,385-387);
 * otherwise it allocates max_concurrency weight slots, which keep experts between calls (an expert
 * still in a slot is not copied again). */
int32_t infmoe_initialize(infmoe_plugin* p);

/*
 * Replaces MoELayerPlugin::enqueue (plugin/MoELayerPlugin.cc:279-416).
 * inputs[0]: device float [B,S,d]; outputs[0]: device float [B,S,d]; `workspace`: device,
 * at least infmoe_workspace_size bytes, 256-byte aligned; `hip_stream`: hipStream_t.
 * Allocates nothing, neither device nor host memory, on either schedule (the lists the streamed schedule makes
 * per call live in the layer, sized by infmoe_initialize).
 *
 * Streams: one infmoe_enqueue in flight per handle.  The weight slots of a streamed layer (max_concurrency <
 * expert_count) keep experts between calls, so there a call on another stream than the previous call's first
 * waits, on the device, for that call's end; with resident experts calls on different streams are the caller's
 * to order (the layer's routing counts are one block of device memory).
 *
 * A token whose scores cannot be ordered (a NaN in its row; the reference asserts there,
 * plugin/cuda/moe.cu:70,184) does not stop the call, whatever the schedule: the call completes, that
 * token's output row is NaN in full, every other row is computed as usual, and the token is counted
 * in stats[1] of infmoe_last_routing.  INFMOE_ERR_NAN is returned once per such call, by whichever
 * of these comes first: the call itself when it waits for the routing anyway (experts streamed,
 * max_concurrency < expert_count); the first later infmoe_enqueue on the handle that finds the
 * device's report - a DEFERRED NOTICE: that later call is queued in full, its own output is valid, and
 * the message (infmoe_last_error) names the number of the call that met the NaN (calls that queue work
 * are counted from 1 per handle since infmoe_initialize); not at all if infmoe_last_routing has reported
 * the count in between.  The host looks for the report only inside infmoe_enqueue: a caller that
 * replays a captured graph of the layer never enters it and has to poll infmoe_last_routing (stats[1])
 * if it wants to know.
 */
int32_t infmoe_enqueue(infmoe_plugin* p, const int32_t* dims, int32_t nb_dims, const void* const* inputs,
                       void* const* outputs, void* workspace, void* hip_stream);

/* Replaces terminate (plugin/MoELayerPlugin.cc:203-237): frees device and page-locked memory. */
int32_t infmoe_terminate(infmoe_plugin* p);
/* Replaces destroy (plugin/MoELayerPlugin.h:118). */
void infmoe_destroy(infmoe_plugin* p);

/*
 * Routing report of the most recent infmoe_enqueue (blocks until that call's gating is done).
 * count_host: E ints, tokens per expert (may be NULL).  stats_host: 3 ints (may be NULL):
 *   [0] tokens whose top-2 score gap is below 1e-6 relative (exempt from bit-exact assignment)
 *   [1] tokens with no orderable score (NaN rows; plugin/cuda/moe.cu:70)
 *   [2] tokens whose assignment was re-derived in float64 inside the gating kernel
 */
int32_t infmoe_last_routing(infmoe_plugin* p, int32_t* count_host, int32_t* stats_host);

/*
 * How the most recent infmoe_enqueue with streamed experts (max_concurrency < expert_count) got its
 * experts' weights: *copies = experts copied host-to-device in that call, *hits = experts that ran from a
 * slot still holding them from an earlier call (either may be NULL).  No counterpart in the reference,
 * which copies every active expert on every call (plugin/MoELayerPlugin.cc:365,385-387).  Both are 0
 * when the experts are resident.
 */
int32_t infmoe_last_streaming(infmoe_plugin* p, int32_t* copies, int32_t* hits);

/*
 * Phase timing (no counterpart in the reference, which only prints wall time from Python,
 * python/examples/stacked_moe.py:55-60).  When enabled, infmoe_enqueue records HIP events on its
 * stream at the phase boundaries; infmoe_last_timing waits for the last call and returns the
 * elapsed milliseconds of: [0] gating, [1] count+sort, [2] scatter (with the row statistics of the expert
 * norm), [3] what a sub-layer does before its first product (T5_FF: nothing with the rms norm, which rides on
 * that product; the row norm with the centered one),
 * [4] first expert GEMM (norm and activation fused), [5] second expert GEMM (residual fused),
 * [6] gather / mix.  Phases 3-5 are only separated when all experts are resident (otherwise the
 * whole streamed expert loop is reported in [4]).  `ms` holds INFMOE_N_PHASES floats.
 * `enable` is the number of most recent calls whose marks are kept (0 = off, 1 = the last call, up
 * to 4096); infmoe_timing_history returns those of the last min(max_calls, kept) calls, oldest
 * first, INFMOE_N_PHASES floats per call, and their number in *n_calls.
 */
#define INFMOE_N_PHASES 7
int32_t infmoe_set_timing(infmoe_plugin* p, int32_t enable);
int32_t infmoe_last_timing(infmoe_plugin* p, float* ms);
int32_t infmoe_timing_history(infmoe_plugin* p, float* ms, int32_t max_calls, int32_t* n_calls);

/* Replaces getSerializationSize / serialize / deserializePlugin (plugin/MoELayerPlugin.cc:104-143,418-458).
 * A versioned little-endian format of this library's own; expert weights are not serialised,
 * only the file path, as in the reference. */
int32_t infmoe_serialization_size(const infmoe_plugin* p, size_t* out_bytes);
int32_t infmoe_serialize(const infmoe_plugin* p, void* buffer, size_t buffer_bytes);
int32_t infmoe_deserialize(const char* layer_name, const void* data, size_t bytes, infmoe_plugin** out);

/*
 * Replaces cnpy::npz_load for one array (plugin/thirdparty/cnpy/cnpy.cpp:229-276, used at
 * plugin/sublayers/T5FFLayer.cc:143-147): reads float32 member `name` (e.g. "3/wo_weight",
 * README.md:121) of the .npz archive `path` into `dst_host` in C order.  The member must be
 * little-endian float32 of shape (rows, cols), or (rows,) when cols == 0; stored and deflated
 * members, zip64 archives and Fortran-ordered 2-D members are read.  Host memory only: needs no GPU.
 */
int32_t infmoe_npz_read_f32(const char* path, const char* name, float* dst_host, size_t rows, size_t cols);

const char* infmoe_last_error(void);
const char* infmoe_plugin_name(void);    /* "MoELayerPlugin", plugin/MoELayerPlugin.h:18-19 */
const char* infmoe_plugin_version(void); /* "1" */

/* ---------------------------------------------------------------- kernel-level entry points
 * One per host launcher of plugin/cuda/moe.h:9-64 and plugin/cuda/ops.h:9-21.  All pointers are
 * device pointers unless named *_host; all launches are asynchronous on `hip_stream`. */

enum { INFMOE_NORM_NONE = 0, INFMOE_NORM_RMS = 1, INFMOE_NORM_CENTERED = 2 };
enum { INFMOE_FFN_RELU = 0, INFMOE_FFN_GATED_GELU = 1 };

/*
 * Fused gating: replaces layernorm_gpu + cublasSgemm_v2 + moe_expert_select
 * (plugin/MoELayerPlugin.cc:315-345, plugin/cuda/moe.cu:147-159).
 * x [T][d]; centroids [E][d]; gamma [d] or NULL (norm_kind NONE); score_bias [E] or NULL;
 * sel int32 [T]; coeff float [T] (the winning score); stats int32[3] as infmoe_last_routing
 * (accumulated with atomics: zero it first) or NULL.
 * `scratch`: NULL, or infmoe_gate_top1_scratch_bytes(T,d,E) bytes of device memory (16-byte aligned,
 * any contents): with it the embedding dimension is cut into slices that different workgroups
 * take (the reference's cuBLAS call does the like inside the library) - for few tokens so that the
 * whole chip works, for many so that a slice of the centroids stays in on-chip memory - and a second
 * launch adds the slices' partial scores.  The result does not depend on it beyond FP32 rounding of
 * the scores.
 */
size_t infmoe_gate_top1_scratch_bytes(int32_t T, int32_t d, int32_t E);
int32_t infmoe_gate_top1(int32_t T, int32_t d, int32_t E, const float* x, const float* centroids, const float* gamma,
                         int32_t norm_kind, const float* score_bias, int32_t* sel, float* coeff, int32_t* stats,
                         void* scratch, void* hip_stream);

/*
 * Replaces moe_expert_count (plugin/cuda/moe.cu:161-212), on the device and without a host
 * round trip: histogram, exclusive prefix, stable counting sort.
 * sel int32[T] (values in [0,E)) -> pos int32[T], count int32[E], offset int32[E+1].
 * `scratch`: infmoe_expert_count_scratch_bytes(T,E) bytes of device memory.
 */
size_t infmoe_expert_count_scratch_bytes(int32_t T, int32_t E);
int32_t infmoe_expert_count(int32_t T, int32_t E, const int32_t* sel, int32_t* pos, int32_t* count, int32_t* offset,
                            void* scratch, void* hip_stream);

/*
 * The same computation as infmoe_expert_count for callers that cannot allocate device memory
 * and have no scratch to pass (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  No counterpart in the reference.  The block-histogram scratch lives
 * in a device array inside the library, INFMOE_EXPERT_COUNT_NOALLOC_MAX_INTS int32 (256 KiB)
 * on every GPU the library runs on, held until the process ends.  The call allocates nothing
 * (no hipMalloc / hipFree, on the first call neither) and returns INFMOE_ERR_INVALID_ARGUMENT
 * when ceil(T / 1024) * E (rounded up to 64) exceeds that many ints.  All calls on one GPU share
 * the array: calls that overlap there (different streams, different threads) race; calls on one
 * stream are ordered.  Nothing has to be cleared between calls.  The first call on a device
 * looks up the array's address and must not be made while a stream capture is in progress.
 */
#define INFMOE_EXPERT_COUNT_NOALLOC_MAX_INTS 65536
int32_t infmoe_expert_count_noalloc(int32_t T, int32_t E, const int32_t* sel, int32_t* pos, int32_t* count,
                                    int32_t* offset, void* hip_stream);

/* Replaces moe_expert_scatter (plugin/cuda/moe.cu:214-228): routed[r,:] = x[pos[r],:],
 * routed_coeff[r] = coeff[pos[r]] (coeff / routed_coeff may both be NULL). */
int32_t infmoe_expert_scatter(int32_t T, int32_t d, const float* x, const float* coeff, const int32_t* pos,
                              float* routed, float* routed_coeff, void* hip_stream);

/* Replaces moe_expert_gather (plugin/cuda/moe.cu:230-240): out[pos[r],:] = buf[r,:]. */
int32_t infmoe_expert_gather(int32_t T, int32_t d, const float* buf, const int32_t* pos, float* out, void* hip_stream);

/* Replaces moe_expert_base_layer_fused_mix_and_gather (plugin/cuda/moe.cu:242-258):
 * a = sigmoid(routed_coeff[r]); out[pos[r],:] = a*post[r,:] + (1-a)*routed[r,:]. */
int32_t infmoe_expert_mix_gather(int32_t T, int32_t d, const int32_t* pos, const float* routed, const float* post,
                                 const float* routed_coeff, float* out, void* hip_stream);

/* Replaces layernorm_gpu<float,float> with beta == NULL (plugin/cuda/ops.h:9-17,
 * plugin/cuda/ops/layernorm.cu:176-188); eps is fixed at 1e-6 as at both call sites. */
int32_t infmoe_layernorm(float* out, const float* in, int32_t rows, int32_t d, const float* gamma, int32_t norm_kind,
                         void* hip_stream);

/*
 * Replaces T5FFLayer::weightSize / workspaceSize / run (plugin/sublayers/T5FFLayer.cc:43-53,90-141)
 * for one expert: out = in + FFN(norm(in)).  `weights` is one device slot laid out
 * [gamma d | wi h*d | wo d*h] (relu) or [gamma d | wi_0 h*d | wi_1 h*d | wo d*h] (gated_gelu),
 * as plugin/sublayers/T5FFLayer.cc:100,112,118-119,130-131.
 */
size_t infmoe_t5ff_weight_bytes(int32_t d, int32_t h, int32_t ffn_kind);
size_t infmoe_t5ff_workspace_bytes(int32_t rows, int32_t d, int32_t h, int32_t ffn_kind);
int32_t infmoe_t5ff_run(int32_t rows, int32_t d, int32_t h, int32_t norm_kind, int32_t ffn_kind, const void* weights,
                        const float* in, float* out, void* workspace, void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* INFMOE_H */
