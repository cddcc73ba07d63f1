// extern "C" surface of the library (include/infmoe.h).  Nothing throws or aborts across it.
#include <cstring>
#include <memory>
#include <new>

#include "../../include/infmoe.h"
#include "kernels/kernels.h"
#include "moe_layer.h"
#include "npz_reader.h"
#include "sublayers/t5ff_layer.h"

using namespace infmoe;

struct infmoe_plugin {
    std::unique_ptr<MoELayer> layer;
};

namespace {

template <typename F>
int32_t guarded(F&& f) {
    try {
        return f();
    } catch (const std::bad_alloc&) {
        return fail(INFMOE_ERR_INVALID_ARGUMENT, "out of host memory");
    } catch (const std::exception& e) {
        return fail(INFMOE_ERR_INVALID_ARGUMENT, "unexpected exception: %s", e.what());
    } catch (...) {
        return fail(INFMOE_ERR_INVALID_ARGUMENT, "unexpected exception");
    }
}

Status field_int(const infmoe_field& f, int* out) {
    // plugin/MoELayerPluginCreator.cc:76-87: length == 1 and data != nullptr
    if (f.length != 1 || f.data == nullptr) return fail(INFMOE_ERR_INVALID_ARGUMENT, "field %s must hold one int32", f.name);
    *out = *static_cast<const int32_t*>(f.data);
    return INFMOE_OK;
}

Status field_floats(const infmoe_field& f, std::vector<float>* out) {
    if (f.length <= 0 || f.data == nullptr) return fail(INFMOE_ERR_INVALID_ARGUMENT, "field %s must hold float32 data", f.name);
    const float* p = static_cast<const float*>(f.data);
    out->assign(p, p + f.length);
    return INFMOE_OK;
}

Status field_string(const infmoe_field& f, std::string* out) {
    if (f.length <= 0 || f.data == nullptr) return fail(INFMOE_ERR_INVALID_ARGUMENT, "field %s must hold characters", f.name);
    const char* p = static_cast<const char*>(f.data);
    out->assign(p, strnlen(p, (size_t)f.length));  // a trailing NUL inside `length` is dropped
    return INFMOE_OK;
}

Status check(const infmoe_plugin* p) {
    if (p == nullptr || !p->layer) return fail(INFMOE_ERR_INVALID_ARGUMENT, "null plugin handle");
    return INFMOE_OK;
}

}  // namespace

extern "C" {

int32_t infmoe_create(const char* layer_name, const infmoe_field* fields, int32_t n_fields, infmoe_plugin** out) {
    return guarded([&]() -> int32_t {
        if (out == nullptr || (fields == nullptr && n_fields > 0) || n_fields < 0)
            return fail(INFMOE_ERR_INVALID_ARGUMENT, "null argument");
        *out = nullptr;
        MoEParams p;
        p.layerName = layer_name ? layer_name : "";
        for (int i = 0; i < n_fields; ++i) {
            const infmoe_field& f = fields[i];
            if (f.name == nullptr) return fail(INFMOE_ERR_INVALID_ARGUMENT, "field %d has no name", i);
            std::string s;
            if (strcmp(f.name, "expert_count") == 0) {
                INFMOE_TRY(field_int(f, &p.expertCount));
            } else if (strcmp(f.name, "embedding_size") == 0) {
                INFMOE_TRY(field_int(f, &p.embeddingSize));
            } else if (strcmp(f.name, "hidden_size") == 0) {
                INFMOE_TRY(field_int(f, &p.hiddenSize));
            } else if (strcmp(f.name, "max_concurrency") == 0) {
                INFMOE_TRY(field_int(f, &p.maxConcurrency));
            } else if (strcmp(f.name, "expert_centroids") == 0) {
                INFMOE_TRY(field_floats(f, &p.centroids));
            } else if (strcmp(f.name, "expert_weight_file") == 0) {
                INFMOE_TRY(field_string(f, &p.weightFile));
            } else if (strcmp(f.name, "expert_sublayer_type") == 0) {
                INFMOE_TRY(field_string(f, &p.sublayerType));
            } else if (strcmp(f.name, "moe_variant") == 0) {
                INFMOE_TRY(field_string(f, &p.variant));
            } else if (strcmp(f.name, "layernorm_weight") == 0) {
                INFMOE_TRY(field_floats(f, &p.layernormWeight));
            } else if (strcmp(f.name, "norm_kind") == 0) {
                INFMOE_TRY(field_string(f, &s));
                if (s == "rms") p.normKind = NORM_RMS;
                else if (s == "centered") p.normKind = NORM_CENTERED;
                else return fail(INFMOE_ERR_UNSUPPORTED, "unsupported norm_kind: %s", s.c_str());
            } else if (strcmp(f.name, "ffn_kind") == 0) {
                INFMOE_TRY(field_string(f, &s));
                if (s == "relu") p.ffnKind = FFN_RELU;
                else if (s == "gated_gelu") p.ffnKind = FFN_GATED_GELU;
                else return fail(INFMOE_ERR_UNSUPPORTED, "unsupported ffn_kind: %s", s.c_str());
            } else {
                // plugin/MoELayerPluginCreator.cc:111-114
                return fail(INFMOE_ERR_UNKNOWN_FIELD, "unknown field name in PluginFieldCollection: %s", f.name);
            }
        }
        std::unique_ptr<MoELayer> layer;
        INFMOE_TRY(MoELayer::create(std::move(p), &layer));
        *out = new infmoe_plugin{std::move(layer)};
        return INFMOE_OK;
    });
}

int32_t infmoe_clone(const infmoe_plugin* src, infmoe_plugin** out) {
    return guarded([&]() -> int32_t {
        INFMOE_TRY(check(src));
        if (out == nullptr) return fail(INFMOE_ERR_INVALID_ARGUMENT, "null output pointer");
        std::unique_ptr<MoELayer> layer;
        INFMOE_TRY(src->layer->clone(&layer));
        *out = new infmoe_plugin{std::move(layer)};
        return INFMOE_OK;
    });
}

int32_t infmoe_set_expert_weights(infmoe_plugin* p, int32_t expert, const char* key, const float* host, size_t count) {
    return guarded([&]() -> int32_t {
        INFMOE_TRY(check(p));
        return p->layer->sublayer()->setWeights(expert, key, host, count);
    });
}

int32_t infmoe_set_score_bias(infmoe_plugin* p, const float* host) {
    return guarded([&]() -> int32_t {
        INFMOE_TRY(check(p));
        return p->layer->setScoreBias(host);
    });
}

int32_t infmoe_configure(infmoe_plugin* p, const int32_t* dims, int32_t nb_dims) {
    return guarded([&]() -> int32_t {
        INFMOE_TRY(check(p));
        return p->layer->configure(dims, nb_dims);
    });
}

int32_t infmoe_workspace_size(const infmoe_plugin* p, const int32_t* dims, int32_t nb_dims, size_t* out_bytes) {
    return guarded([&]() -> int32_t {
        INFMOE_TRY(check(p));
        return p->layer->workspaceSize(dims, nb_dims, out_bytes);
    });
}

int32_t infmoe_initialize(infmoe_plugin* p) {
    return guarded([&]() -> int32_t {
        INFMOE_TRY(check(p));
        return p->layer->initialize();
    });
}

int32_t infmoe_enqueue(infmoe_plugin* p, const int32_t* dims, int32_t nb_dims, const void* const* inputs,
                       void* const* outputs, void* workspace, void* hip_stream) {
    return guarded([&]() -> int32_t {
        INFMOE_TRY(check(p));
        return p->layer->enqueue(dims, nb_dims, inputs, outputs, workspace, static_cast<hipStream_t>(hip_stream));
    });
}

int32_t infmoe_terminate(infmoe_plugin* p) {
    return guarded([&]() -> int32_t {
        INFMOE_TRY(check(p));
        return p->layer->terminate();
    });
}

void infmoe_destroy(infmoe_plugin* p) {
    try {
        delete p;
    } catch (...) {
    }
}

int32_t infmoe_last_routing(infmoe_plugin* p, int32_t* count_host, int32_t* stats_host) {
    return guarded([&]() -> int32_t {
        INFMOE_TRY(check(p));
        return p->layer->lastRouting(count_host, stats_host);
    });
}

int32_t infmoe_last_streaming(infmoe_plugin* p, int32_t* copies, int32_t* hits) {
    return guarded([&]() -> int32_t {
        INFMOE_TRY(check(p));
        return p->layer->lastStreaming(copies, hits);
    });
}

int32_t infmoe_set_timing(infmoe_plugin* p, int32_t enable) {
    return guarded([&]() -> int32_t {
        INFMOE_TRY(check(p));
        return p->layer->setTiming(enable);
    });
}

int32_t infmoe_last_timing(infmoe_plugin* p, float* ms) {
    return guarded([&]() -> int32_t {
        INFMOE_TRY(check(p));
        if (ms == nullptr) return fail(INFMOE_ERR_INVALID_ARGUMENT, "null output pointer");
        return p->layer->lastTiming(ms);
    });
}

int32_t infmoe_timing_history(infmoe_plugin* p, float* ms, int32_t max_calls, int32_t* n_calls) {
    return guarded([&]() -> int32_t {
        INFMOE_TRY(check(p));
        int n = 0;
        INFMOE_TRY(p->layer->timingHistory(ms, max_calls, &n));
        if (n_calls) *n_calls = n;
        return INFMOE_OK;
    });
}

int32_t infmoe_serialization_size(const infmoe_plugin* p, size_t* out_bytes) {
    return guarded([&]() -> int32_t {
        INFMOE_TRY(check(p));
        if (out_bytes == nullptr) return fail(INFMOE_ERR_INVALID_ARGUMENT, "null output pointer");
        return p->layer->serializationSize(out_bytes);
    });
}

int32_t infmoe_serialize(const infmoe_plugin* p, void* buffer, size_t buffer_bytes) {
    return guarded([&]() -> int32_t {
        INFMOE_TRY(check(p));
        return p->layer->serialize(buffer, buffer_bytes);
    });
}

int32_t infmoe_deserialize(const char* layer_name, const void* data, size_t bytes, infmoe_plugin** out) {
    return guarded([&]() -> int32_t {
        if (out == nullptr) return fail(INFMOE_ERR_INVALID_ARGUMENT, "null output pointer");
        *out = nullptr;
        std::unique_ptr<MoELayer> layer;
        INFMOE_TRY(MoELayer::deserialize(layer_name, data, bytes, &layer));
        *out = new infmoe_plugin{std::move(layer)};
        return INFMOE_OK;
    });
}

int32_t infmoe_npz_read_f32(const char* path, const char* name, float* dst_host, size_t rows, size_t cols) {
    return guarded([&]() -> int32_t {
        if (path == nullptr || name == nullptr || dst_host == nullptr) return fail(INFMOE_ERR_INVALID_ARGUMENT, "null argument");
        NpzReader npz;
        INFMOE_TRY(npz.open(path));
        return npz.read_f32(name, dst_host, rows, cols);
    });
}

const char* infmoe_last_error(void) { return last_error_slot().c_str(); }
const char* infmoe_plugin_name(void) { return "MoELayerPlugin"; }
const char* infmoe_plugin_version(void) { return "1"; }

// ---------------------------------------------------------------- kernel-level entry points

#define INFMOE_NEED(cond, msg) \
    if (!(cond)) return fail(INFMOE_ERR_INVALID_ARGUMENT, msg)

static_assert(kExpertCountStaticInts == INFMOE_EXPERT_COUNT_NOALLOC_MAX_INTS, "header and kernel disagree on the limit");

size_t infmoe_gate_top1_scratch_bytes(int32_t T, int32_t d, int32_t E) {
    return sizeof(float) * gate_scratch_floats(T < 0 ? 0 : T, d < 1 ? 1 : d, E < 1 ? 1 : E);
}

int32_t infmoe_gate_top1(int32_t T, int32_t d, int32_t E, const float* x, const float* centroids, const float* gamma,
                         int32_t norm_kind, const float* score_bias, int32_t* sel, float* coeff, int32_t* stats,
                         void* scratch, void* hip_stream) {
    return guarded([&]() -> int32_t {
        INFMOE_NEED(T >= 0 && d > 0 && E > 0, "gate_top1: bad sizes");
        INFMOE_NEED(T == 0 || (x && centroids && sel && coeff), "gate_top1: null pointer");
        INFMOE_NEED(norm_kind >= NORM_NONE && norm_kind <= NORM_CENTERED, "gate_top1: bad norm_kind");
        INFMOE_NEED(norm_kind == NORM_NONE || gamma != nullptr, "gate_top1: norm needs gamma");
        INFMOE_NEED((reinterpret_cast<uintptr_t>(scratch) & 15) == 0, "gate_top1: scratch must be 16-byte aligned");
        hipStream_t stream = static_cast<hipStream_t>(hip_stream);
        INFMOE_HIP(launch_gate_top1(T, d, E, x, centroids, gamma, norm_kind, score_bias, sel, coeff, stats, stream, nullptr,
                                    nullptr, static_cast<float*>(scratch), scratch ? gate_scratch_floats(T, d, E) : 0));
        return INFMOE_OK;
    });
}

size_t infmoe_expert_count_scratch_bytes(int32_t T, int32_t E) {
    return expert_count_scratch_bytes(T < 0 ? 0 : T, E < 1 ? 1 : E);
}

int32_t infmoe_expert_count(int32_t T, int32_t E, const int32_t* sel, int32_t* pos, int32_t* count, int32_t* offset,
                            void* scratch, void* hip_stream) {
    return guarded([&]() -> int32_t {
        INFMOE_NEED(T >= 0 && E > 0, "expert_count: bad sizes");
        INFMOE_NEED(count && offset && (T == 0 || (sel && pos && scratch)), "expert_count: null pointer");
        INFMOE_HIP(launch_expert_count(T, E, sel, pos, count, offset, scratch, nullptr, nullptr, kGemmTileRows, 0,
                                       nullptr, static_cast<hipStream_t>(hip_stream)));
        return INFMOE_OK;
    });
}

int32_t infmoe_expert_count_noalloc(int32_t T, int32_t E, const int32_t* sel, int32_t* pos, int32_t* count,
                                    int32_t* offset, void* hip_stream) {
    return guarded([&]() -> int32_t {
        INFMOE_NEED(T >= 0 && E > 0, "expert_count_noalloc: bad sizes");
        INFMOE_NEED(count && offset && (T == 0 || (sel && pos)), "expert_count_noalloc: null pointer");
        const size_t need = expert_count_scratch_bytes(T, E) / sizeof(int32_t);
        if (need > (size_t)INFMOE_EXPERT_COUNT_NOALLOC_MAX_INTS)
            return fail(INFMOE_ERR_INVALID_ARGUMENT,
                        "expert_count_noalloc: ceil(T/1024)*E = %zu ints of scratch exceed the built-in %d; use "
                        "infmoe_expert_count with caller-supplied scratch",
                        need, INFMOE_EXPERT_COUNT_NOALLOC_MAX_INTS);
        INFMOE_HIP(launch_expert_count_static(T, E, sel, pos, count, offset, static_cast<hipStream_t>(hip_stream)));
        return INFMOE_OK;
    });
}

int32_t infmoe_expert_scatter(int32_t T, int32_t d, const float* x, const float* coeff, const int32_t* pos,
                              float* routed, float* routed_coeff, void* hip_stream) {
    return guarded([&]() -> int32_t {
        INFMOE_NEED(T >= 0 && d > 0, "expert_scatter: bad sizes");
        INFMOE_NEED(T == 0 || (x && pos && routed), "expert_scatter: null pointer");
        INFMOE_HIP(launch_scatter(T, d, x, coeff, pos, routed, routed_coeff, static_cast<hipStream_t>(hip_stream)));
        return INFMOE_OK;
    });
}

int32_t infmoe_expert_gather(int32_t T, int32_t d, const float* buf, const int32_t* pos, float* out, void* hip_stream) {
    return guarded([&]() -> int32_t {
        INFMOE_NEED(T >= 0 && d > 0, "expert_gather: bad sizes");
        INFMOE_NEED(T == 0 || (buf && pos && out), "expert_gather: null pointer");
        INFMOE_HIP(launch_gather(T, d, buf, pos, out, static_cast<hipStream_t>(hip_stream)));
        return INFMOE_OK;
    });
}

int32_t infmoe_expert_mix_gather(int32_t T, int32_t d, const int32_t* pos, const float* routed, const float* post,
                                 const float* routed_coeff, float* out, void* hip_stream) {
    return guarded([&]() -> int32_t {
        INFMOE_NEED(T >= 0 && d > 0, "expert_mix_gather: bad sizes");
        INFMOE_NEED(T == 0 || (pos && routed && post && routed_coeff && out), "expert_mix_gather: null pointer");
        INFMOE_HIP(launch_mix_gather(T, d, pos, routed, post, routed_coeff, out, static_cast<hipStream_t>(hip_stream)));
        return INFMOE_OK;
    });
}

int32_t infmoe_layernorm(float* out, const float* in, int32_t rows, int32_t d, const float* gamma, int32_t norm_kind,
                         void* hip_stream) {
    return guarded([&]() -> int32_t {
        INFMOE_NEED(rows >= 0 && d > 0, "layernorm: bad sizes");
        INFMOE_NEED(norm_kind == NORM_RMS || norm_kind == NORM_CENTERED, "layernorm: norm_kind must be rms or centered");
        INFMOE_NEED(gamma && (rows == 0 || (out && in)), "layernorm: null pointer");
        INFMOE_HIP(launch_row_norm(out, in, rows, d, gamma, 0, nullptr, norm_kind, static_cast<hipStream_t>(hip_stream)));
        return INFMOE_OK;
    });
}

size_t infmoe_t5ff_weight_bytes(int32_t d, int32_t h, int32_t ffn_kind) { return T5FFLayer::weightBytes(d, h, ffn_kind); }

size_t infmoe_t5ff_workspace_bytes(int32_t rows, int32_t d, int32_t h, int32_t /*ffn_kind*/) {
    return T5FFLayer::workspaceBytes(rows, d, h);
}

int32_t infmoe_t5ff_run(int32_t rows, int32_t d, int32_t h, int32_t norm_kind, int32_t ffn_kind, const void* weights,
                        const float* in, float* out, void* workspace, void* hip_stream) {
    return guarded([&]() -> int32_t {
        INFMOE_NEED(rows >= 0 && d > 0 && h > 0, "t5ff_run: bad sizes");
        INFMOE_NEED(norm_kind == NORM_RMS || norm_kind == NORM_CENTERED, "t5ff_run: norm_kind must be rms or centered");
        INFMOE_NEED(ffn_kind == FFN_RELU || ffn_kind == FFN_GATED_GELU, "t5ff_run: bad ffn_kind");
        INFMOE_NEED(rows == 0 || (weights && in && out && workspace), "t5ff_run: null pointer");
        return T5FFLayer::runOne(rows, rows, 1, d, h, norm_kind, ffn_kind, weights, in, out, workspace,
                                 static_cast<hipStream_t>(hip_stream), /*folded=*/false, nullptr);
    });
}

}  // extern "C"
