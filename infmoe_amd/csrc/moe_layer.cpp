#include "moe_layer.h"

#include <sys/stat.h>

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstring>

namespace infmoe {

std::string& last_error_slot() {
    static thread_local std::string slot;
    return slot;
}

// ---------------------------------------------------------------- construction

Status MoELayer::parseFlags(const char* variant, MoEFlags* out) {
    // plugin/MoELayerPlugin.cc:44-58, names from plugin/MoELayerPlugin.h:28-32
    MoEFlags f;
    if (variant == nullptr) return fail(INFMOE_ERR_MISSING_FIELD, "moe_variant is required");
    if (strcmp(variant, "base_layer") == 0) {
        f.baseLayerOutputMix = true;
    } else if (strcmp(variant, "cpm_2") == 0) {
        f.layernormOnInputBeforeScore = true;
    } else if (strcmp(variant, "default") == 0) {
    } else {
        return fail(INFMOE_ERR_UNSUPPORTED, "unsupported moe variant: %s", variant);
    }
    *out = f;
    return INFMOE_OK;
}

Status MoELayer::create(MoEParams&& p, std::unique_ptr<MoELayer>* out) {
    // plugin/MoELayerPluginCreator.cc:117-140 and plugin/MoELayerPlugin.cc:74-80
    if (p.embeddingSize <= 0) return fail(INFMOE_ERR_MISSING_FIELD, "embedding_size must be given and positive");
    if (p.expertCount <= 0) return fail(INFMOE_ERR_MISSING_FIELD, "expert_count must be given and positive");
    if (p.hiddenSize <= 0) return fail(INFMOE_ERR_MISSING_FIELD, "hidden_size must be given and positive");
    if (p.maxConcurrency <= 0) return fail(INFMOE_ERR_INVALID_ARGUMENT, "max_concurrency must be positive");
    if (p.normKind != NORM_RMS && p.normKind != NORM_CENTERED) return fail(INFMOE_ERR_INVALID_ARGUMENT, "bad norm_kind %d", p.normKind);
    if (p.ffnKind != FFN_RELU && p.ffnKind != FFN_GATED_GELU) return fail(INFMOE_ERR_INVALID_ARGUMENT, "bad ffn_kind %d", p.ffnKind);
    if (p.centroids.empty()) return fail(INFMOE_ERR_MISSING_FIELD, "expert_centroids is required");
    if (p.centroids.size() != (size_t)p.embeddingSize * p.expertCount)
        return fail(INFMOE_ERR_INVALID_ARGUMENT, "expert_centroids has %zu floats, expected expert_count*embedding_size = %zu",
                    p.centroids.size(), (size_t)p.embeddingSize * p.expertCount);
    if (p.sublayerType.empty()) return fail(INFMOE_ERR_MISSING_FIELD, "expert_sublayer_type is required");
    if (p.variant.empty()) return fail(INFMOE_ERR_MISSING_FIELD, "moe_variant is required");
    if (!p.layernormWeight.empty() && p.layernormWeight.size() != (size_t)p.embeddingSize)
        return fail(INFMOE_ERR_INVALID_ARGUMENT, "layernorm_weight has %zu floats, expected embedding_size = %d",
                    p.layernormWeight.size(), p.embeddingSize);
    INFMOE_TRY(parseFlags(p.variant.c_str(), &p.flags));
    if (p.flags.layernormOnInputBeforeScore && p.layernormWeight.empty())
        return fail(INFMOE_ERR_MISSING_FIELD, "layernorm_weight is required for moe_variant cpm_2");
    if (!p.weightFile.empty()) {
        struct stat st {};
        if (stat(p.weightFile.c_str(), &st) != 0) return fail(INFMOE_ERR_IO, "cannot stat weight file: %s", p.weightFile.c_str());
        if (!S_ISREG(st.st_mode)) return fail(INFMOE_ERR_IO, "weight file must be a regular file: %s", p.weightFile.c_str());
    }
    std::unique_ptr<MoELayer> layer(new MoELayer());
    SubLayerConfig sc{};
    sc.expertCount = p.expertCount, sc.embeddingSize = p.embeddingSize, sc.hiddenSize = p.hiddenSize;
    sc.maxConcurrency = p.maxConcurrency, sc.weightFile = p.weightFile.empty() ? nullptr : p.weightFile.c_str();
    sc.normKind = p.normKind, sc.ffnKind = p.ffnKind;
    INFMOE_TRY(make_sublayer(p.sublayerType.c_str(), sc, &layer->mSublayer));
    layer->mParams = std::move(p);
    *out = std::move(layer);
    return INFMOE_OK;
}

Status MoELayer::clone(std::unique_ptr<MoELayer>* out) const {
    std::unique_ptr<MoELayer> layer(new MoELayer());
    layer->mParams = mParams;       // deep copy of centroids / gamma
    layer->mSublayer = mSublayer;   // shared, so stacked layers hold the expert weights once
    layer->mScoreBias = mScoreBias;
    layer->mSequenceLength = mSequenceLength;
    *out = std::move(layer);
    return INFMOE_OK;
}

MoELayer::~MoELayer() { (void)terminate(); }

Status MoELayer::setScoreBias(const float* host) {
    if (host == nullptr) {
        mScoreBias.clear();
    } else if (host != mScoreBias.data()) {  // (initialize() hands the stored values back in to upload them)
        mScoreBias.assign(host, host + mParams.expertCount);
    }
    if (mInitialized) {
        if (mScoreBias.empty()) return INFMOE_OK;
        if (mScoreBiasGpu == nullptr) INFMOE_HIP(hipMalloc(reinterpret_cast<void**>(&mScoreBiasGpu), sizeof(float) * mParams.expertCount));
        INFMOE_HIP(hipMemcpy(mScoreBiasGpu, mScoreBias.data(), sizeof(float) * mParams.expertCount, hipMemcpyHostToDevice));
    }
    return INFMOE_OK;
}

// ---------------------------------------------------------------- shapes and workspace

Status MoELayer::checkDims(const int32_t* dims, int32_t nbDims, int* tokens) const {
    // plugin/MoELayerPlugin.cc:172-177
    if (dims == nullptr || nbDims != 3) return fail(INFMOE_ERR_INVALID_ARGUMENT, "input must be 3-D [batch, seq, embedding_size]");
    if (dims[2] != mParams.embeddingSize)
        return fail(INFMOE_ERR_INVALID_ARGUMENT, "last input dimension is %d, expected embedding_size = %d", dims[2], mParams.embeddingSize);
    if (dims[0] < 0 || dims[1] < 0) return fail(INFMOE_ERR_INVALID_ARGUMENT, "negative input dimension");
    const int64_t t = (int64_t)dims[0] * dims[1];
    if (t > 0x3fffffff) return fail(INFMOE_ERR_INVALID_ARGUMENT, "too many tokens");
    *tokens = (int)t;
    return INFMOE_OK;
}

Status MoELayer::configure(const int32_t* dims, int32_t nbDims) {
    int t = 0;
    INFMOE_TRY(checkDims(dims, nbDims, &t));
    Dims in;
    in.nbDims = 3;
    for (int i = 0; i < 3; ++i) in.d[i] = dims[i];
    if (!mSublayer->configureWithFormat(&in, 1, &in, 1)) return fail(INFMOE_ERR_INVALID_ARGUMENT, "sub-layer rejected the input format");
    mSequenceLength = dims[1];
    return INFMOE_OK;
}

bool MoELayer::resident() const {
    return mSublayer->weightSize() == 0 || mParams.maxConcurrency >= mParams.expertCount;
}

struct MoELayer::Carve {
    size_t slotStride = 0;
    char* subWs = nullptr;
    int32_t *sel = nullptr, *pos = nullptr, *rowExpert = nullptr, *sched = nullptr;
    RowTile* tiles = nullptr;
    int maxTiles = 0;
    void* countScratch = nullptr;
    float* gateScratch = nullptr;  // partial scores of the gating kernel's slices
    float *coeff = nullptr, *routedCoeff = nullptr, *routed = nullptr, *post = nullptr;
    float* rowStats = nullptr;  // (mean, reciprocal deviation) of every routed row, when the sub-layer asks for them
    size_t total = 0;
};

// Workspace layout (every block 256-byte aligned).  The max_concurrency weight slots of streamed experts,
// which the reference carves from the workspace (plugin/MoELayerPlugin.cc:243-245), are device memory of
// the layer here: they keep experts between calls, which memory that the caller may hand to others between
// calls cannot.
//   sub-layer scratch for T rows, shared by all experts because their rows are disjoint
//     (the reference sizes one full-T scratch per slot, :256-263)
//   sel[T] pos[T] rowExpert[T] | row tiles | scan scratch | coeff[T] routedCoeff[T] rowStats[T][2] | routed[T][d] | post[T][d]
//   (the reference also keeps the T x E score matrix, :246; the fused gating never stores it)
Status MoELayer::carve(int T, void* workspace, Carve* c) const {
    char* base = static_cast<char*>(workspace);
    size_t off = 0;
    auto take = [&](size_t bytes) {
        char* p = base ? base + off : nullptr;
        off += align_up(bytes);
        return p;
    };
    const int E = mParams.expertCount, d = mParams.embeddingSize;
    c->slotStride = align_up(mSublayer->weightSize());
    c->subWs = take(mSublayer->workspaceSize(T));
    c->sel = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * (size_t)T));
    c->pos = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * (size_t)T));
    c->rowExpert = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * (size_t)T));
    c->maxTiles = max_row_tiles(T, E, mSublayer->minRowTileHeight());  // room for the shortest tiles any call may be cut into
    c->tiles = reinterpret_cast<RowTile*>(take(sizeof(RowTile) * 2 * (size_t)c->maxTiles));
    c->sched = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * kSchedInts));
    c->countScratch = take(expert_count_scratch_bytes(T, E));
    c->gateScratch = reinterpret_cast<float*>(take(sizeof(float) * gate_scratch_floats(T, d, E)));
    c->coeff = reinterpret_cast<float*>(take(sizeof(float) * (size_t)T));
    c->routedCoeff = reinterpret_cast<float*>(take(sizeof(float) * (size_t)T));
    c->rowStats = mSublayer->rowStatsKind() != NORM_NONE ? reinterpret_cast<float*>(take(sizeof(float) * 2 * (size_t)T)) : nullptr;
    c->routed = reinterpret_cast<float*>(take(sizeof(float) * (size_t)T * d));
    c->post = reinterpret_cast<float*>(take(sizeof(float) * (size_t)T * d));
    c->total = off;
    return INFMOE_OK;
}

Status MoELayer::workspaceSize(const int32_t* dims, int32_t nbDims, size_t* bytes) const {
    int T = 0;
    INFMOE_TRY(checkDims(dims, nbDims, &T));
    if (bytes == nullptr) return fail(INFMOE_ERR_INVALID_ARGUMENT, "null output pointer");
    Carve c;
    INFMOE_TRY(carve(T, nullptr, &c));
    *bytes = c.total;
    return INFMOE_OK;
}

// ---------------------------------------------------------------- initialize / terminate

Status MoELayer::initialize() {
    if (mInitialized) return INFMOE_OK;
    // all or nothing: a failure half way (a weight array that is missing, an allocation that does not
    // fit) releases what the earlier steps created, so that a retry starts from a clean layer
    const Status s = initializeSteps();
    if (s != INFMOE_OK) {
        const std::string why = last_error_slot();
        (void)terminate();
        last_error_slot() = why;
    }
    return s;
}

// The launch geometry of the kernels is tuned for the part they are written for: workgroup ids are dealt
// round-robin to 8 accelerator dies (the row-tile schedule of the grouped expert launch and the slice map of
// the gating count on it) and one workgroup per compute unit means 256 of them.  No result depends on it: every
// workgroup finds its work from its id alone, whichever die runs it.  A device partitioned differently (an
// MI355X in CPX/DPX mode, another gfx950 part) computes the same bits with a worse balance, so it is told
// once per process, on stderr, and served.
static Status check_device_geometry() {
    int dev = 0, cus = 0, xccs = 0;
    INFMOE_HIP(hipGetDevice(&dev));
    INFMOE_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    if (hipDeviceGetAttribute(&xccs, hipDeviceAttributeNumberOfXccs, dev) != hipSuccess) {
        (void)hipGetLastError();
        xccs = kXcdCount;  // a runtime that cannot tell: the compute-unit count decides
    }
    static std::atomic<bool> told{false};
    if ((cus != 256 || xccs != kXcdCount) && !told.exchange(true))
        fprintf(stderr,
                "infmoe: device %d has %d compute units in %d accelerator dies; the launch schedules are tuned for 256 in %d "
                "(an MI355X in its single-partition mode): results are the same, the load balance is not\n",
                dev, cus, xccs, kXcdCount);
    return INFMOE_OK;
}

Status MoELayer::initializeSteps() {
    INFMOE_TRY(check_device_geometry());
    const int E = mParams.expertCount, d = mParams.embeddingSize;
    INFMOE_TRY(mSublayer->initialize());
    // plugin/MoELayerPlugin.cc:14-26 (done on the first enqueue there)
    INFMOE_HIP(hipMalloc(reinterpret_cast<void**>(&mCentroidsGpu), sizeof(float) * (size_t)E * d));
    INFMOE_HIP(hipMemcpy(mCentroidsGpu, mParams.centroids.data(), sizeof(float) * (size_t)E * d, hipMemcpyHostToDevice));
    if (!mParams.layernormWeight.empty()) {
        INFMOE_HIP(hipMalloc(reinterpret_cast<void**>(&mLayernormGpu), sizeof(float) * d));
        INFMOE_HIP(hipMemcpy(mLayernormGpu, mParams.layernormWeight.data(), sizeof(float) * d, hipMemcpyHostToDevice));
    }
    {   // what the gating kernel needs of (centroids, gamma) and would otherwise recompute per workgroup
        std::vector<float> folded((size_t)E * d + 2 * (size_t)E);
        const bool ln = mParams.flags.layernormOnInputBeforeScore;
        fold_centroids_host(d, E, mParams.centroids.data(), ln ? mParams.layernormWeight.data() : nullptr, folded.data(),
                            folded.data() + (size_t)E * d);
        INFMOE_HIP(hipMalloc(reinterpret_cast<void**>(&mFoldedGpu), sizeof(float) * folded.size()));
        INFMOE_HIP(hipMemcpy(mFoldedGpu, folded.data(), sizeof(float) * folded.size(), hipMemcpyHostToDevice));
    }
    const size_t routingInts = (size_t)2 * E + 1 + 4;
    INFMOE_HIP(hipMalloc(reinterpret_cast<void**>(&mRoutingGpu), sizeof(int32_t) * routingInts));
    INFMOE_HIP(hipMemset(mRoutingGpu, 0, sizeof(int32_t) * routingInts));
    // page-locked and visible to the device: the last int is the flag the gating sets when it meets a
    // token without an orderable score (the host reads it without waiting for the device)
    INFMOE_HIP(hipHostMalloc(reinterpret_cast<void**>(&mRoutingHost), sizeof(int32_t) * (routingInts + 1), hipHostMallocMapped));
    mNanFlagHost = mRoutingHost + routingInts;
    *mNanFlagHost = 0;
    INFMOE_HIP(hipHostGetDevicePointer(reinterpret_cast<void**>(&mNanFlagDev), mNanFlagHost, 0));
    INFMOE_HIP(hipEventCreateWithFlags(&mRoutingDone, hipEventDisableTiming));
    if (resident()) {
        INFMOE_TRY(mSublayer->makeResident());
    } else {
        // plugin/MoELayerPlugin.cc:182-195 creates max_concurrency streams; here one copy stream
        // feeds the slots and a few compute streams let consecutive experts overlap
        const size_t stride = align_up(mSublayer->weightSize());
        INFMOE_HIP(hipMalloc(reinterpret_cast<void**>(&mSlotPool), stride * (size_t)mParams.maxConcurrency));
        mSlotExpert.assign(mParams.maxConcurrency, -1);
        mSlotVersion = mSublayer->weightsVersion();
        INFMOE_HIP(hipMalloc(reinterpret_cast<void**>(&mSlotTableGpu), sizeof(int32_t) * E));
        INFMOE_HIP(hipHostMalloc(reinterpret_cast<void**>(&mSlotTableHost), sizeof(int32_t) * E, hipHostMallocDefault));
        mSlotTableSent.clear();
        INFMOE_HIP(hipStreamCreateWithFlags(&mCopyStream, hipStreamNonBlocking));
        mComputeStreams.resize(std::min(mParams.maxConcurrency, 4));
        for (auto& s : mComputeStreams) INFMOE_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
        mJoin.resize(mComputeStreams.size());
        for (auto& e : mJoin) INFMOE_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
        mCopyDone.resize(E);
        mComputeDone.resize(E);
        for (auto& e : mCopyDone) INFMOE_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
        for (auto& e : mComputeDone) INFMOE_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
        INFMOE_HIP(hipEventCreateWithFlags(&mFork, hipEventDisableTiming));
        INFMOE_HIP(hipEventCreateWithFlags(&mCallDone, hipEventDisableTiming));
        mHaveCallDone = false, mLastStream = nullptr;
        for (auto* v : {&mNeeded, &mOrder, &mSlotOf, &mSlotTableSent}) v->reserve(E);
        mStreamSlots.reserve(2 * (size_t)mParams.maxConcurrency);
        mLastUse.reserve(mParams.maxConcurrency);
    }
    mCallNumber = 0;
    mInitialized = true;
    if (!mScoreBias.empty()) INFMOE_TRY(setScoreBias(mScoreBias.data()));
    return INFMOE_OK;
}

Status MoELayer::terminate() {
    // plugin/MoELayerPlugin.cc:203-237.  The sub-layer is shared with clones and releases its
    // weights when its last owner goes away.
    if (mCentroidsGpu) (void)hipFree(mCentroidsGpu);
    if (mLayernormGpu) (void)hipFree(mLayernormGpu);
    if (mScoreBiasGpu) (void)hipFree(mScoreBiasGpu);
    if (mFoldedGpu) (void)hipFree(mFoldedGpu);
    mFoldedGpu = nullptr;
    if (mRoutingGpu) (void)hipFree(mRoutingGpu);
    if (mRoutingHost) (void)hipHostFree(mRoutingHost);
    mCentroidsGpu = mLayernormGpu = mScoreBiasGpu = nullptr;
    mRoutingGpu = mRoutingHost = nullptr;
    mNanFlagHost = mNanFlagDev = nullptr;
    if (mCopyStream) (void)hipStreamDestroy(mCopyStream);
    mCopyStream = nullptr;
    if (mSlotPool) (void)hipFree(mSlotPool);
    mSlotPool = nullptr;
    mSlotExpert.clear();
    if (mSlotTableGpu) (void)hipFree(mSlotTableGpu);
    if (mSlotTableHost) (void)hipHostFree(mSlotTableHost);
    mSlotTableGpu = mSlotTableHost = nullptr;
    mSlotTableSent.clear();
    for (auto s : mComputeStreams) (void)hipStreamDestroy(s);
    mComputeStreams.clear();
    for (auto* v : {&mCopyDone, &mComputeDone, &mJoin}) {
        for (auto e : *v) (void)hipEventDestroy(e);
        v->clear();
    }
    for (auto e : mMarks) (void)hipEventDestroy(e);
    mMarks.clear();
    mTimedCalls = 0;
    mTimingDepth = 0;
    if (mFork) (void)hipEventDestroy(mFork);
    if (mRoutingDone) (void)hipEventDestroy(mRoutingDone);
    if (mCallDone) (void)hipEventDestroy(mCallDone);
    mFork = mRoutingDone = mCallDone = nullptr;
    mHaveCallDone = false, mLastStream = nullptr;
    mInitialized = false;
    return INFMOE_OK;
}

// ---------------------------------------------------------------- enqueue

Status MoELayer::enqueue(const int32_t* dims, int32_t nbDims, const void* const* inputs, void* const* outputs,
                         void* workspace, hipStream_t stream) {
    int T = 0;
    INFMOE_TRY(checkDims(dims, nbDims, &T));
    if (!mInitialized) return fail(INFMOE_ERR_STATE, "enqueue before initialize");
    if (T == 0) return INFMOE_OK;  // an empty batch has nothing to read or write: its tensors may have no memory at all
    if (inputs == nullptr || outputs == nullptr || inputs[0] == nullptr || outputs[0] == nullptr)
        return fail(INFMOE_ERR_INVALID_ARGUMENT, "null input or output");
    if (workspace == nullptr || (reinterpret_cast<uintptr_t>(workspace) & 255))
        return fail(INFMOE_ERR_INVALID_ARGUMENT, "workspace must be non-null and 256-byte aligned");
    // An earlier call met a token without an orderable score (a NaN in its row) and the device has said so
    // since, by writing that call's number into the flag.  It is reported once, by the first call that sees it:
    // a deferred notice.  The present call is queued in full all the same, and its own output is not touched by
    // the notice.
    const int32_t earlierNan = __atomic_exchange_n(mNanFlagHost, 0, __ATOMIC_ACQ_REL);
    mCallNumber = mCallNumber == 0x7fffffff ? 1 : mCallNumber + 1;
    const int E = mParams.expertCount, d = mParams.embeddingSize;
    const float* x = static_cast<const float*>(inputs[0]);
    float* y = static_cast<float*>(outputs[0]);
    Carve c;
    INFMOE_TRY(carve(T, workspace, &c));
    int32_t* dCount = mRoutingGpu;
    int32_t* dOffset = dCount + E;
    int32_t* dStats = dOffset + E + 1;

    // Streamed experts: the weight slots (and the routing block the host reads) outlive the call.  Work of an
    // earlier call that uses them was joined into THAT call's stream; a call on another stream waits, on the
    // device, for its end before it queues anything.
    if (!resident() && mHaveCallDone && stream != mLastStream) INFMOE_HIP(hipStreamWaitEvent(stream, mCallDone, 0));
    // ... and this call's end is marked on every way out of it, a failure halfway included: what it has queued
    // by then uses the slots all the same.
    struct CallEnd {
        MoELayer* layer;
        hipStream_t stream;
        ~CallEnd() {
            if (layer != nullptr && hipEventRecord(layer->mCallDone, stream) == hipSuccess)
                layer->mHaveCallDone = true, layer->mLastStream = stream;
        }
    } callEnd{resident() ? nullptr : this, stream};

    const bool timed = mTiming && !mMarks.empty();
    hipEvent_t* marks = timed ? &mMarks[(size_t)(mTimedCalls % mTimingDepth) * (INFMOE_N_PHASES + 1)] : nullptr;
    auto mark = [&](int i) -> Status {
        if (timed) INFMOE_HIP(hipEventRecord(marks[i], stream));
        return INFMOE_OK;
    };
    INFMOE_TRY(mark(0));
    // 0-2. norm (cpm_2: for scoring only), scores, top-1          plugin/MoELayerPlugin.cc:312-345
    const bool ln = mParams.flags.layernormOnInputBeforeScore;
    bool histReady = false;  // the gating leaves the first pass of the counting sort behind when it can
    INFMOE_HIP(launch_gate_top1(T, d, E, x, mCentroidsGpu, ln ? mLayernormGpu : nullptr, ln ? mParams.normKind : NORM_NONE,
                                mScoreBias.empty() ? nullptr : mScoreBiasGpu, c.sel, c.coeff, dStats, stream, mFoldedGpu,
                                mFoldedGpu + (size_t)E * d, c.gateScratch, gate_scratch_floats(T, d, E),
                                /*zero_stats=*/true, mNanFlagDev, mCallNumber, static_cast<int*>(c.countScratch), &histReady));
    INFMOE_TRY(mark(1));
    // 3. count, sort, scatter                                      plugin/MoELayerPlugin.cc:349-355
    // (the row tiles of the grouped expert launch are made on either schedule: streamed experts that are all
    // still in their slots run from one set of launches too)
    const bool grouped = resident();
    const int skinnyMax = mSublayer->skinnyMaxRows(T);
    INFMOE_HIP(launch_expert_count(T, E, c.sel, c.pos, dCount, dOffset, c.countScratch, c.tiles, c.sched,
                                   mSublayer->rowTileHeightFor(T), skinnyMax, c.rowExpert, stream, histReady));
    INFMOE_TRY(mark(2));
    // experts see the raw input (:354); the statistics of their row norm are taken while the rows are copied
    INFMOE_HIP(launch_scatter(T, d, x, c.coeff, c.pos, c.routed, c.routedCoeff, stream, c.rowStats, mSublayer->rowStatsKind()));
    INFMOE_HIP(hipEventRecord(mRoutingDone, stream));
    INFMOE_TRY(mark(3));

    // 4. experts                                                   plugin/MoELayerPlugin.cc:360-402
    GroupedRun g;
    g.tokenCount = T, g.input = c.routed, g.output = c.post, g.workspace = c.subWs;
    g.count = dCount, g.offset = dOffset, g.rowExpert = c.rowExpert, g.rowStats = c.rowStats;
    g.tiles = c.tiles, g.sched = c.sched, g.stream = stream;
    g.maxTiles = std::min(c.maxTiles, max_row_tiles(T, E, mSublayer->rowTileHeightFor(T)));  // of this call's tile height
    if (skinnyMax > 0) {
        // Only experts with more than skinnyMax rows are cut into row tiles: at most T / (skinnyMax + 1)
        // of them, each with one tile more than its rows fill.  (T5_FF answers "every expert" for a decode call:
        // no expert is tiled then and its grouped run launches no matrix-core grid at all.)
        const int tall = T / (skinnyMax + 1);
        g.maxTiles = std::min(g.maxTiles, tall + T / mSublayer->rowTileHeightFor(T));
    }
    if (timed) g.afterNorm = marks[4], g.afterGemm1 = marks[5];
    if (grouped) {
        INFMOE_TRY(mSublayer->runGrouped(g));
    } else {
        mNanRowsSeen = 0;
        INFMOE_TRY(runStreamed(T, c, stream, g));
    }
    INFMOE_TRY(mark(6));

    // 6-7. mix (base_layer) and un-shuffle                         plugin/MoELayerPlugin.cc:404-412
    // (the post-expert rows are gathered; :411 of the public reference passes the pre-expert ones)
    if (mParams.flags.baseLayerOutputMix)
        INFMOE_HIP(launch_mix_gather(T, d, c.pos, c.routed, c.post, c.routedCoeff, y, stream));
    else
        INFMOE_HIP(launch_gather(T, d, c.post, c.pos, y, stream, c.routedCoeff));
    INFMOE_TRY(mark(7));
    if (timed) ++mTimedCalls;
    if (!grouped && mNanRowsSeen > 0) {
        // reported here, not again by the next call (the routing was waited for, so the flag is this call's)
        __atomic_store_n(mNanFlagHost, 0, __ATOMIC_RELEASE);
        return fail(INFMOE_ERR_NAN, "%d token(s) of this call (number %d on this layer) have no orderable score (NaN input?); "
                                    "their output rows are NaN", mNanRowsSeen, mCallNumber);
    }
    if (earlierNan != 0)
        return fail(INFMOE_ERR_NAN, "call number %d on this layer met token(s) with no orderable score (NaN input?) and wrote "
                                    "NaN output rows for them; this call (number %d) was queued in full and is not affected",
                    earlierNan, mCallNumber);
    return INFMOE_OK;
}

Status MoELayer::setTiming(int depth) {
    if (depth < 0 || depth > 4096) return fail(INFMOE_ERR_INVALID_ARGUMENT, "timing depth must be 0..4096");
    if (depth != mTimingDepth) {
        for (auto e : mMarks) (void)hipEventDestroy(e);
        mMarks.clear();
        mTimingDepth = 0;
        mTiming = false;
        std::vector<hipEvent_t> marks((size_t)depth * (INFMOE_N_PHASES + 1), nullptr);
        for (auto& e : marks) {
            // timestamps only: nothing waits on these events, so they need not publish memory beyond the device
            // (an event's system-wide release costs a few microseconds on the stream, eight times per call)
            const hipError_t err = hipEventCreateWithFlags(&e, hipEventDisableSystemFence);
            if (err != hipSuccess) {  // leave timing off rather than half built
                for (auto m : marks)
                    if (m) (void)hipEventDestroy(m);
                return hip_fail(err, "hipEventCreate");
            }
        }
        mMarks.swap(marks);
        mTimingDepth = depth;
    }
    mTiming = depth > 0;
    mTimedCalls = 0;
    return INFMOE_OK;
}

Status MoELayer::timingHistory(float* ms, int maxCalls, int* nCalls) {
    if (ms == nullptr || nCalls == nullptr || maxCalls < 0) return fail(INFMOE_ERR_INVALID_ARGUMENT, "null output");
    const long long kept = std::min<long long>(mTimedCalls, mTimingDepth);
    const int n = (int)std::min<long long>(kept, maxCalls);
    *nCalls = n;
    for (int j = 0; j < n; ++j) {  // oldest of the n first
        const long long call = mTimedCalls - n + j;
        hipEvent_t* marks = &mMarks[(size_t)(call % mTimingDepth) * (INFMOE_N_PHASES + 1)];
        INFMOE_HIP(hipEventSynchronize(marks[INFMOE_N_PHASES]));
        for (int i = 0; i < INFMOE_N_PHASES; ++i) {
            float* out = ms + (size_t)j * INFMOE_N_PHASES + i;
            *out = 0.f;
            // an Identity sub-layer or a streamed expert loop leaves some marks unrecorded
            if (hipEventElapsedTime(out, marks[i], marks[i + 1]) != hipSuccess) *out = 0.f;
        }
    }
    return INFMOE_OK;
}

Status MoELayer::lastTiming(float* ms) {
    if (mTimedCalls == 0) return fail(INFMOE_ERR_STATE, "no timed enqueue to report (infmoe_set_timing, then infmoe_enqueue)");
    int n = 0;
    return timingHistory(ms, 1, &n);
}

// Experts streamed through max_concurrency device slots (plugin/MoELayerPlugin.cc:360-402).
// The host learns the token counts once (one blocking copy of E integers), then queues every
// copy and every expert without blocking again:
//   copy stream:   [wait: the slot's previous expert done] copy expert into its slot, signal copyDone[k]
//   compute k%n:   [wait: copyDone[k]] run expert k from its slot,                     signal computeDone[k]
// so experts are prefetched while others compute (the reference prefetches one), and
// max_concurrency = 1 degenerates to copy, compute, copy, ... with no overlap.
//
// The slots are the layer's own device memory and keep their contents between calls, each slot
// remembering which expert it holds (the reference copies every active expert on every call,
// plugin/MoELayerPlugin.cc:365,385-387).  An expert that is still in a slot from an earlier call runs
// from there without a copy.  When the experts a call needs do not all fit, the ones already present
// with the most rows are retained, up to max_concurrency less the two slots the others are streamed
// through (copy of one under the compute of the other); the rest are copied, most rows first.  A change of
// any expert's weights (infmoe_set_expert_weights) empties the slots.  Which expert sits where has no
// influence on the arithmetic: the output is the same bit for bit.
Status MoELayer::runStreamed(int T, const Carve& c, hipStream_t stream, GroupedRun& g) {
    const int E = mParams.expertCount, d = mParams.embeddingSize, mc = mParams.maxConcurrency;
    const size_t routingInts = (size_t)2 * E + 1 + 4;
    INFMOE_HIP(hipMemcpyAsync(mRoutingHost, mRoutingGpu, sizeof(int32_t) * routingInts, hipMemcpyDeviceToHost, stream));
    INFMOE_HIP(hipStreamSynchronize(stream));
    const int32_t* count = mRoutingHost;
    const int32_t* offset = mRoutingHost + E;
    const int32_t* stats = offset + E + 1;
    // tokens without an orderable score do not stop the call: their rows come out as NaN, and enqueue
    // reports them when everything is queued (this schedule knows of them now; the resident one later)
    mNanRowsSeen = stats[1];

    if (mSublayer->weightsVersion() != mSlotVersion) {  // some expert's weights changed: nothing cached is valid
        std::fill(mSlotExpert.begin(), mSlotExpert.end(), -1);
        mSlotVersion = mSublayer->weightsVersion();
    }
    // Empty experts are skipped (:361-363,383-384).  The reference takes the others in ascending
    // index; here the ones with most rows go first (stable, so equal counts stay ascending): every
    // expert costs the same copy, and the compute that nothing can hide is the last expert's, so it
    // should be the shortest.  Rows of different experts are disjoint: the order cannot change a bit.
    // (the lists are members with room reserved in initialize(): nothing here touches the heap)
    std::vector<int>&needed = mNeeded, &order = mOrder, &slotOf = mSlotOf, &streamSlots = mStreamSlots, &lastUse = mLastUse;
    needed.clear();
    for (int e = 0; e < E; ++e)
        if (count[e] > 0) needed.push_back(e);
    // (an insertion sort: stable, in place - std::stable_sort takes a temporary buffer from the heap - and E is small)
    for (size_t i = 1; i < needed.size(); ++i) {
        const int e = needed[i];
        size_t j = i;
        for (; j > 0 && count[needed[j - 1]] < count[e]; --j) needed[j] = needed[j - 1];
        needed[j] = e;
    }
    slotOf.assign(E, -1);
    for (int s = 0; s < mc; ++s)
        if (mSlotExpert[s] >= 0) slotOf[mSlotExpert[s]] = s;
    // Experts still in a slot run first, from there and without a copy; the others follow, most rows first,
    // through the slots that are not retained.
    order.clear();
    for (const int e : needed)
        if (slotOf[e] >= 0) order.push_back(e);
    const int present = (int)order.size(), absent = (int)needed.size() - present;
    for (const int e : needed)
        if (slotOf[e] < 0) order.push_back(e);
    // Retained for the next call: of the experts present, those with most rows, leaving (at most) two slots
    // for the others to pass through - copy of one under the compute of the other.
    const int keep = absent == 0 ? present : std::min(present, std::max(0, mc - std::min(2, absent)));
    // Slots the absent experts pass through, in the order they become free: first those that hold nothing
    // this call needs, then those of the experts that run from them once more and are then given up (in the
    // order they run).  Slot numbers break ties, so the choice is deterministic.
    streamSlots.clear();
    for (int s = 0; s < mc; ++s)
        if (mSlotExpert[s] < 0 || count[mSlotExpert[s]] == 0) streamSlots.push_back(s);
    for (int k = keep; k < present; ++k) streamSlots.push_back(slotOf[order[k]]);
    mLastCopies = 0, mLastHits = present;
    if (absent == 0 && mSublayer->groupedFromSlots()) {
        // Every expert of the call is in a slot already: one set of launches over all of them, as when the
        // experts are resident, with a table that says which slot holds which expert.
        if (slotOf != mSlotTableSent) {
            memcpy(mSlotTableHost, slotOf.data(), sizeof(int32_t) * E);
            INFMOE_HIP(hipMemcpyAsync(mSlotTableGpu, mSlotTableHost, sizeof(int32_t) * E, hipMemcpyHostToDevice, stream));
            mSlotTableSent = slotOf;
        }
        g.weights = mSlotPool, g.weightStride = c.slotStride, g.expertSlot = mSlotTableGpu, g.expertSlotHost = slotOf.data();
        return mSublayer->runGrouped(g);
    }
    if (g.afterNorm) INFMOE_HIP(hipEventRecord(g.afterNorm, stream));  // the whole expert loop is reported as one phase
    INFMOE_HIP(hipEventRecord(mFork, stream));
    INFMOE_HIP(hipStreamWaitEvent(mCopyStream, mFork, 0));
    for (auto s : mComputeStreams) INFMOE_HIP(hipStreamWaitEvent(s, mFork, 0));
    lastUse.assign(mc, -1);  // position in `order` of the expert that last ran from the slot in this call
    // Whatever happens in the loop, the compute streams forked above are joined back into the caller's
    // stream before returning: an error half way must not leave work that nothing waits for.
    auto queueExperts = [&]() -> Status {
        int k = 0, turn = 0;
        for (const int e : order) {
            int slot = slotOf[e];
            hipStream_t cs = mComputeStreams[k % mComputeStreams.size()];
            if (slot < 0) {
                slot = streamSlots[turn++ % streamSlots.size()];
                // the slot's previous expert of this call must be done with it (earlier calls are: the copy
                // stream was forked from the caller's stream, into which they were joined)
                if (lastUse[slot] >= 0) INFMOE_HIP(hipStreamWaitEvent(mCopyStream, mComputeDone[lastUse[slot]], 0));
                mSlotExpert[slot] = -1;  // not valid until the copy has been queued without error
                INFMOE_TRY(mSublayer->copyWeights(mSlotPool + c.slotStride * (size_t)slot, e, mCopyStream));
                mSlotExpert[slot] = e;
                ++mLastCopies;
                INFMOE_HIP(hipEventRecord(mCopyDone[k], mCopyStream));
                INFMOE_HIP(hipStreamWaitEvent(cs, mCopyDone[k], 0));
            }
            char* slotPtr = mSlotPool + c.slotStride * (size_t)slot;
            // rows of different experts are disjoint, so each expert gets its own stretch of the
            // shared scratch (row stride applied: the public reference omits it at :373,391-392)
            INFMOE_TRY(mSublayer->runInLayer(T, count[e], slotPtr, c.routed + (size_t)offset[e] * d,
                                             c.post + (size_t)offset[e] * d,
                                             c.subWs + mSublayer->workspaceOffset(offset[e]), cs,
                                             c.rowStats ? c.rowStats + 2 * (size_t)offset[e] : nullptr));
            INFMOE_HIP(hipEventRecord(mComputeDone[k], cs));
            lastUse[slot] = k;
            ++k;
        }
        return INFMOE_OK;
    };
    const Status queued = queueExperts();
    auto join = [&]() -> Status {
        // the copy stream's last work is waited for by a compute stream unless the loop broke off in between
        if (queued != INFMOE_OK) {
            INFMOE_HIP(hipEventRecord(mFork, mCopyStream));
            INFMOE_HIP(hipStreamWaitEvent(stream, mFork, 0));
        }
        for (size_t i = 0; i < mComputeStreams.size(); ++i) {
            INFMOE_HIP(hipEventRecord(mJoin[i], mComputeStreams[i]));
            INFMOE_HIP(hipStreamWaitEvent(stream, mJoin[i], 0));
        }
        if (g.afterGemm1) INFMOE_HIP(hipEventRecord(g.afterGemm1, stream));
        return INFMOE_OK;
    };
    if (queued == INFMOE_OK) return join();
    const std::string why = last_error_slot();  // (the error path only: the message of the first failure is the one kept)
    (void)join();
    last_error_slot() = why;
    return queued;
}

Status MoELayer::lastRouting(int32_t* countHost, int32_t* statsHost) {
    if (!mInitialized) return fail(INFMOE_ERR_STATE, "no routing before initialize");
    const int E = mParams.expertCount;
    INFMOE_HIP(hipEventSynchronize(mRoutingDone));
    std::vector<int32_t> tmp((size_t)2 * E + 1 + 4);
    INFMOE_HIP(hipMemcpy(tmp.data(), mRoutingGpu, sizeof(int32_t) * tmp.size(), hipMemcpyDeviceToHost));
    if (countHost) memcpy(countHost, tmp.data(), sizeof(int32_t) * E);
    if (statsHost) memcpy(statsHost, tmp.data() + 2 * E + 1, sizeof(int32_t) * 3);
    // the caller has now been told of that call's NaN rows (stats[1]): the next enqueue does not repeat it
    if (tmp[2 * E + 1 + 1] > 0) *static_cast<volatile int32_t*>(mNanFlagHost) = 0;
    return INFMOE_OK;
}

Status MoELayer::lastStreaming(int32_t* copies, int32_t* hits) const {
    if (!mInitialized) return fail(INFMOE_ERR_STATE, "no call before initialize");
    if (copies) *copies = mLastCopies;
    if (hits) *hits = mLastHits;
    return INFMOE_OK;
}

// ---------------------------------------------------------------- serialisation
// Own little-endian format (the reference's has known defects, plugin/MoELayerPlugin.cc:131-140,
// 418-423,451-453, and is not reproduced):
//   u32 magic 'IMOE', u32 version = 1,
//   i32 E, d, h, mc, normKind, ffnKind, u32 flags (bit0 norm-before-score, bit1 base-layer mix),
//   u32 len(weight_file), len(sublayer_type), len(variant), n_centroids, n_layernorm,
//   the three strings (no terminator), zero padding to a multiple of 4, centroids, layernorm.
namespace {
constexpr uint32_t kMagic = 0x454F4D49u, kVersion = 1u;
constexpr size_t kHeaderWords = 14;
}

Status MoELayer::serializationSize(size_t* bytes) const {
    const size_t strings = mParams.weightFile.size() + mParams.sublayerType.size() + mParams.variant.size();
    *bytes = kHeaderWords * 4 + align_up(strings, 4) + 4 * (mParams.centroids.size() + mParams.layernormWeight.size());
    return INFMOE_OK;
}

Status MoELayer::serialize(void* buffer, size_t bytes) const {
    size_t need = 0;
    serializationSize(&need);
    if (buffer == nullptr || bytes < need) return fail(INFMOE_ERR_INVALID_ARGUMENT, "serialize needs %zu bytes", need);
    memset(buffer, 0, need);
    uint32_t* w = static_cast<uint32_t*>(buffer);
    const uint32_t head[kHeaderWords] = {kMagic, kVersion, (uint32_t)mParams.expertCount, (uint32_t)mParams.embeddingSize,
                                         (uint32_t)mParams.hiddenSize, (uint32_t)mParams.maxConcurrency, (uint32_t)mParams.normKind,
                                         (uint32_t)mParams.ffnKind,
                                         (mParams.flags.layernormOnInputBeforeScore ? 1u : 0u) | (mParams.flags.baseLayerOutputMix ? 2u : 0u),
                                         (uint32_t)mParams.weightFile.size(), (uint32_t)mParams.sublayerType.size(),
                                         (uint32_t)mParams.variant.size(), (uint32_t)mParams.centroids.size(),
                                         (uint32_t)mParams.layernormWeight.size()};
    memcpy(w, head, sizeof(head));
    char* p = static_cast<char*>(buffer) + sizeof(head);
    char* s = p;
    for (const std::string* str : {&mParams.weightFile, &mParams.sublayerType, &mParams.variant}) {
        if (!str->empty()) memcpy(s, str->data(), str->size());
        s += str->size();
    }
    p += align_up((size_t)(s - p), 4);
    // (an empty vector's data() may be null, which memcpy must not be given even for no bytes)
    if (!mParams.centroids.empty()) memcpy(p, mParams.centroids.data(), 4 * mParams.centroids.size());
    p += 4 * mParams.centroids.size();
    if (!mParams.layernormWeight.empty()) memcpy(p, mParams.layernormWeight.data(), 4 * mParams.layernormWeight.size());
    return INFMOE_OK;
}

Status MoELayer::deserialize(const char* layerName, const void* data, size_t bytes, std::unique_ptr<MoELayer>* out) {
    if (data == nullptr || bytes < kHeaderWords * 4) return fail(INFMOE_ERR_INVALID_ARGUMENT, "serialized layer is truncated");
    uint32_t head[kHeaderWords];
    memcpy(head, data, sizeof(head));
    if (head[0] != kMagic || head[1] != kVersion) return fail(INFMOE_ERR_INVALID_ARGUMENT, "not a serialized MoE layer of this version");
    MoEParams p;
    p.layerName = layerName ? layerName : "";
    p.expertCount = (int)head[2], p.embeddingSize = (int)head[3], p.hiddenSize = (int)head[4], p.maxConcurrency = (int)head[5];
    p.normKind = (int)head[6], p.ffnKind = (int)head[7];
    const size_t l1 = head[9], l2 = head[10], l3 = head[11], nc = head[12], nl = head[13];
    const size_t need = sizeof(head) + align_up(l1 + l2 + l3, 4) + 4 * (nc + nl);
    if (bytes < need) return fail(INFMOE_ERR_INVALID_ARGUMENT, "serialized layer is truncated: %zu of %zu bytes", bytes, need);
    const char* s = static_cast<const char*>(data) + sizeof(head);
    p.weightFile.assign(s, l1);
    p.sublayerType.assign(s + l1, l2);
    p.variant.assign(s + l1 + l2, l3);
    const char* f = s + align_up(l1 + l2 + l3, 4);
    p.centroids.resize(nc);
    if (nc > 0) memcpy(p.centroids.data(), f, 4 * nc);
    p.layernormWeight.resize(nl);
    if (nl > 0) memcpy(p.layernormWeight.data(), f + 4 * nc, 4 * nl);
    const uint32_t storedFlags = head[8];
    INFMOE_TRY(create(std::move(p), out));
    // the flags are a function of the variant string (plugin/MoELayerPlugin.cc:44-58); a blob whose flag
    // word says otherwise was not written by serialize()
    const MoEFlags& fl = (*out)->mParams.flags;
    if (storedFlags != ((fl.layernormOnInputBeforeScore ? 1u : 0u) | (fl.baseLayerOutputMix ? 2u : 0u))) {
        out->reset();
        return fail(INFMOE_ERR_INVALID_ARGUMENT, "serialized layer: flag word %u does not belong to its moe_variant", storedFlags);
    }
    return INFMOE_OK;
}

}  // namespace infmoe
