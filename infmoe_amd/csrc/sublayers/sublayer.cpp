// Defaults of the plug-in point and the registry of expert types.
#include "sublayer.h"

#include <cstring>
#include <map>
#include <mutex>
#include <vector>

#include "identity_layer.h"
#include "t5ff_layer.h"

namespace infmoe {

Status MoESubLayer::makeResident() {
    if (mResident != nullptr || weightSize() == 0) return INFMOE_OK;
    mResidentStride = align_up(weightSize());
    INFMOE_HIP(hipMalloc(&mResident, mResidentStride * (size_t)mExpertCount));
    for (int e = 0; e < mExpertCount; ++e) {
        const Status s = copyWeights(static_cast<char*>(mResident) + mResidentStride * (size_t)e, e, nullptr);
        if (s != INFMOE_OK) {
            releaseResident();
            return s;
        }
    }
    INFMOE_HIP(hipStreamSynchronize(nullptr));
    return INFMOE_OK;
}

void MoESubLayer::releaseResident() {
    if (mResident) (void)hipFree(mResident);
    mResident = nullptr;
    mResidentStride = 0;
}

Status MoESubLayer::runGrouped(const GroupedRun& g) {
    // the host has to know the rows of every expert to call run() for it: one wait on the stream
    const int E = mExpertCount;
    std::vector<int32_t> host((size_t)2 * E + 1);
    INFMOE_HIP(hipMemcpyAsync(host.data(), g.count, sizeof(int32_t) * E, hipMemcpyDeviceToHost, g.stream));
    INFMOE_HIP(hipMemcpyAsync(host.data() + E, g.offset, sizeof(int32_t) * (E + 1), hipMemcpyDeviceToHost, g.stream));
    INFMOE_HIP(hipStreamSynchronize(g.stream));
    const int32_t* count = host.data();
    const int32_t* offset = host.data() + E;
    const bool slots = g.weights != nullptr;
    const char* weights = static_cast<const char*>(slots ? g.weights : residentWeights());
    const size_t stride = slots ? g.weightStride : residentStride();
    if (slots && g.expertSlotHost == nullptr) return fail(INFMOE_ERR_INVALID_ARGUMENT, "grouped run from slots without the slot table");
    const size_t d = (size_t)mEmbeddingSize;
    for (int e = 0; e < E; ++e) {  // ascending, empties skipped (plugin/MoELayerPlugin.cc:361-363,383-384)
        if (count[e] <= 0) continue;
        const size_t owner = slots ? (size_t)g.expertSlotHost[e] : (size_t)e;
        INFMOE_TRY(runInLayer(g.tokenCount, count[e], weights ? weights + stride * owner : nullptr,
                              g.input + (size_t)offset[e] * d, g.output + (size_t)offset[e] * d,
                              static_cast<char*>(g.workspace) + workspaceOffset(offset[e]), g.stream,
                              g.rowStats ? g.rowStats + 2 * (size_t)offset[e] : nullptr));
    }
    return INFMOE_OK;
}

namespace {

struct Registry {
    std::mutex lock;
    std::map<std::string, SubLayerFactory> factories;
    Registry() {
        // plugin/MoELayerPlugin.cc:28-41, names from plugin/MoELayerPlugin.h:23-26
        factories["T5_FF"] = [](const SubLayerConfig& c) -> std::shared_ptr<MoESubLayer> {
            return std::make_shared<T5FFLayer>(c.expertCount, c.embeddingSize, c.hiddenSize, c.weightFile, c.maxConcurrency,
                                               c.normKind, c.ffnKind);
        };
        factories["Identity"] = [](const SubLayerConfig&) -> std::shared_ptr<MoESubLayer> {
            return std::make_shared<IdentityLayer>();
        };
    }
};

Registry& registry() {
    static Registry r;  // built on first use: safe to call from another library's static initialisers
    return r;
}

}  // namespace

Status register_sublayer(const char* type, SubLayerFactory factory) {
    if (type == nullptr || *type == 0 || factory == nullptr) return fail(INFMOE_ERR_INVALID_ARGUMENT, "register_sublayer: null name or factory");
    Registry& r = registry();
    std::lock_guard<std::mutex> guard(r.lock);
    r.factories[type] = factory;
    return INFMOE_OK;
}

Status make_sublayer(const char* type, const SubLayerConfig& config, std::shared_ptr<MoESubLayer>* out) {
    SubLayerFactory factory = nullptr;
    if (type != nullptr) {
        Registry& r = registry();
        std::lock_guard<std::mutex> guard(r.lock);
        auto it = r.factories.find(type);
        if (it != r.factories.end()) factory = it->second;
    }
    if (factory == nullptr) return fail(INFMOE_ERR_UNSUPPORTED, "unsupported sublayer type: %s", type ? type : "(null)");
    *out = factory(config);
    if (!*out) return fail(INFMOE_ERR_UNSUPPORTED, "the factory of sublayer type %s returned nothing", type);
    return INFMOE_OK;
}

}  // namespace infmoe
