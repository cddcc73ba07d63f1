// Host side of the MoE layer: the counterpart of class MoELayerPlugin without the TensorRT
// scaffolding (plugin/MoELayerPlugin.h:45-134, plugin/MoELayerPlugin.cc).
#pragma once

#include <hip/hip_runtime_api.h>

#include <memory>
#include <string>
#include <vector>

#include "status.h"
#include "sublayers/sublayer.h"

namespace infmoe {

// plugin/MoELayerPlugin.h:36-42
struct MoEFlags {
    bool layernormOnInputBeforeScore = false;
    bool baseLayerOutputMix = false;
};

struct MoEParams {
    std::string layerName;
    int expertCount = -1, embeddingSize = -1, hiddenSize = -1, maxConcurrency = 2;
    std::vector<float> centroids;        // [E][d]
    std::vector<float> layernormWeight;  // [d] or empty
    std::string weightFile, sublayerType, variant;
    int normKind = NORM_RMS, ffnKind = FFN_RELU;
    MoEFlags flags;
};

class MoELayer {
   public:
    static Status parseFlags(const char* variant, MoEFlags* out);            // plugin/MoELayerPlugin.cc:44-58
    static Status create(MoEParams&& params, std::unique_ptr<MoELayer>* out);  // ctor checks, :60-81
    Status clone(std::unique_ptr<MoELayer>* out) const;                        // :83-102
    ~MoELayer();

    Status configure(const int32_t* dims, int32_t nbDims);                     // :170-180
    Status workspaceSize(const int32_t* dims, int32_t nbDims, size_t* bytes) const;  // :253-273
    Status initialize();                                                       // :197-201, :14-26, :182-195
    Status enqueue(const int32_t* dims, int32_t nbDims, const void* const* inputs, void* const* outputs,
                   void* workspace, hipStream_t stream);                       // :279-416
    Status terminate();                                                        // :203-237
    Status setScoreBias(const float* host);
    Status lastRouting(int32_t* countHost, int32_t* statsHost);
    Status lastStreaming(int32_t* copies, int32_t* hits) const;
    Status setTiming(int depth);  // 0: off; n: keep the phase marks of the last n calls
    Status lastTiming(float* ms);
    Status timingHistory(float* ms, int maxCalls, int* nCalls);

    Status serializationSize(size_t* bytes) const;
    Status serialize(void* buffer, size_t bytes) const;
    static Status deserialize(const char* layerName, const void* data, size_t bytes, std::unique_ptr<MoELayer>* out);

    MoESubLayer* sublayer() { return mSublayer.get(); }
    const MoEParams& params() const { return mParams; }

   private:
    MoELayer() = default;
    struct Carve;  // workspace layout
    Status carve(int T, void* workspace, Carve* c) const;
    bool resident() const;
    Status checkDims(const int32_t* dims, int32_t nbDims, int* tokens) const;
    Status runStreamed(int T, const Carve& c, hipStream_t stream, GroupedRun& g);
    Status initializeSteps();

    MoEParams mParams;
    std::shared_ptr<MoESubLayer> mSublayer;
    std::vector<float> mScoreBias;
    int mSequenceLength = -1;
    bool mInitialized = false;

    // device / runtime state, created by initialize()
    float* mCentroidsGpu = nullptr;
    float* mLayernormGpu = nullptr;
    float* mScoreBiasGpu = nullptr;
    float* mFoldedGpu = nullptr;      // centroids * gating gamma [E][d], then [sum E | norm E]
    int32_t* mRoutingGpu = nullptr;   // [count E | offset E+1 | stats 4]
    int32_t* mRoutingHost = nullptr;  // page-locked mirror
    int32_t* mNanFlagHost = nullptr;  // in the same allocation: set by the gating kernels, read by the host
    int32_t* mNanFlagDev = nullptr;   // its device address
    int mNanRowsSeen = 0;             // streamed schedule: NaN rows of the call in progress
    int32_t mCallNumber = 0;          // calls that queued work, 1-based; what the device writes into the NaN flag
    char* mSlotPool = nullptr;        // streamed experts: max_concurrency weight slots, kept between calls
    std::vector<int> mSlotExpert;     // expert held by each slot, -1 for none
    int32_t* mSlotTableGpu = nullptr;   // [E] slot of every expert, for launches over all experts from the slots
    int32_t* mSlotTableHost = nullptr;  // page-locked staging of the same
    std::vector<int> mSlotTableSent;    // what the device copy holds
    uint64_t mSlotVersion = 0;        // sub-layer weights version the slots' contents belong to
    int mLastCopies = 0, mLastHits = 0;  // of the most recent streamed call
    hipStream_t mCopyStream = nullptr;
    std::vector<hipStream_t> mComputeStreams;
    std::vector<hipEvent_t> mCopyDone, mComputeDone, mJoin;
    hipEvent_t mFork = nullptr, mRoutingDone = nullptr;
    // streamed schedule: the slots are state that outlives a call, so a call on another stream than the last one's
    // first waits for that one's end
    hipEvent_t mCallDone = nullptr;
    hipStream_t mLastStream = nullptr;
    bool mHaveCallDone = false;
    // streamed schedule: lists made per call, with room for E (or max_concurrency) entries from initialize() on, so
    // that a call touches no allocator
    std::vector<int> mNeeded, mOrder, mSlotOf, mStreamSlots, mLastUse;
    bool mTiming = false;
    int mTimingDepth = 0;            // calls whose marks are kept
    long long mTimedCalls = 0;       // timed calls since timing was switched on
    std::vector<hipEvent_t> mMarks;  // mTimingDepth sets of INFMOE_N_PHASES + 1 phase boundaries
};

}  // namespace infmoe
