#include "t5ff_layer.h"

#include <cstring>

#include "../npz_reader.h"

namespace infmoe {

T5FFLayer::T5FFLayer(int expertCount, int embeddingSize, int hiddenSize, const char* weightFile, int maxConcurrency,
                     int normKind, int ffnKind)
    : MoESubLayer(expertCount, embeddingSize, hiddenSize, weightFile, maxConcurrency),
      mNormKind(normKind),
      mFfnKind(ffnKind) {}

T5FFLayer::~T5FFLayer() { terminate(); }

bool T5FFLayer::configureWithFormat(const Dims* in, int32_t nbInputs, const Dims* out, int32_t nbOutputs) {
    // plugin/sublayers/T5FFLayer.cc:20-36
    if (nbInputs != 1 || nbOutputs != 1) return false;
    if (in[0].nbDims != 3 || out[0].nbDims != 3) return false;
    for (int i = 0; i < 3; ++i)
        if (in[0].d[i] != out[0].d[i]) return false;
    return in[0].d[2] == mEmbeddingSize;
}

size_t T5FFLayer::weightBytes(int d, int h, int ffnKind) {
    const size_t mats = ffnKind == FFN_GATED_GELU ? 3 : 2;
    return sizeof(float) * ((size_t)d + mats * (size_t)d * (size_t)h);  // plugin/sublayers/T5FFLayer.cc:43
}

size_t T5FFLayer::workspaceBytes(int rows, int d, int h) {
    return sizeof(float) * (size_t)rows * ((size_t)d + (size_t)h);  // normed rows, hidden rows
}

size_t T5FFLayer::weightSize() { return weightBytes(mEmbeddingSize, mHiddenSize, mFfnKind); }

// Norm carried on the first product: hidden rows, then room for (-, rstd, -, -) per row, used when nobody hands
// the statistics over.  Norm as a launch of its own: normed rows, hidden rows.
size_t T5FFLayer::layerWorkspaceBytes(int rows) const {
    return folds() ? sizeof(float) * (size_t)rows * ((size_t)mHiddenSize + 4) : workspaceBytes(rows, mEmbeddingSize, mHiddenSize);
}

size_t T5FFLayer::workspaceSize(int32_t tokenCount) { return align_up(layerWorkspaceBytes(tokenCount)); }

int T5FFLayer::keyIndex(const char* key, size_t* off, size_t* cnt) const {
    const size_t d = mEmbeddingSize, dh = (size_t)mEmbeddingSize * mHiddenSize;
    if (strcmp(key, "layer_norm_weight") == 0) {
        *off = 0, *cnt = d;
        return 0;
    }
    if (mFfnKind == FFN_GATED_GELU) {
        if (strcmp(key, "wi_0_weight") == 0) return *off = d, *cnt = dh, 1;
        if (strcmp(key, "wi_1_weight") == 0) return *off = d + dh, *cnt = dh, 2;
        if (strcmp(key, "wo_weight") == 0) return *off = d + 2 * dh, *cnt = dh, 3;
    } else {
        if (strcmp(key, "wi_weight") == 0) return *off = d, *cnt = dh, 1;
        if (strcmp(key, "wo_weight") == 0) return *off = d + dh, *cnt = dh, 2;
    }
    return -1;
}

Status T5FFLayer::ensureHostStore() {
    if (mHostWeights != nullptr) return INFMOE_OK;
    // page-locked like the reference's npz store (plugin/thirdparty/cnpy/cnpy.h:27-39), so that
    // hipMemcpyAsync from it really is asynchronous
    INFMOE_HIP(hipHostMalloc(reinterpret_cast<void**>(&mHostWeights), hostStride() * (size_t)mExpertCount,
                             hipHostMallocDefault));
    mHave.assign((size_t)mExpertCount * (nMatrices() + 1), 0);
    return INFMOE_OK;
}

Status T5FFLayer::setWeights(int expert, const char* key, const float* host, size_t count) {
    if (expert < 0 || expert >= mExpertCount) return fail(INFMOE_ERR_INVALID_ARGUMENT, "expert %d out of range", expert);
    if (key == nullptr || host == nullptr) return fail(INFMOE_ERR_INVALID_ARGUMENT, "null key or data");
    size_t off = 0, cnt = 0;
    const int idx = keyIndex(key, &off, &cnt);
    if (idx < 0) return fail(INFMOE_ERR_UNKNOWN_FIELD, "unknown weight key for this ffn kind: %s", key);
    // the reference asserts on the byte count of every array (plugin/sublayers/T5FFLayer.cc:62,69,76,83)
    if (count != cnt) return fail(INFMOE_ERR_INVALID_ARGUMENT, "%s: expected %zu floats, got %zu", key, cnt, count);
    INFMOE_TRY(ensureHostStore());
    if (mCopiesQueued.exchange(false, std::memory_order_acq_rel)) {
        // streamed experts: a copy out of the host store that an earlier call queued may still be on its way,
        // and must not read half of the old and half of the new array (blocking; not a hot path)
        INFMOE_HIP(hipDeviceSynchronize());
    }
    float* slot = reinterpret_cast<float*>(reinterpret_cast<char*>(mHostWeights) + hostStride() * (size_t)expert);
    memcpy(slot + off, host, cnt * sizeof(float));
    mHave[(size_t)expert * (nMatrices() + 1) + idx] = 1;
    mVersion.fetch_add(1, std::memory_order_acq_rel);
    if (mDeviceWeights != nullptr) {
        // already resident: the device slot is made anew from the host store, because gamma may be multiplied
        // into the input-side matrices there and either may be the array that changed (blocking; not a hot path)
        INFMOE_HIP(hipDeviceSynchronize());
        INFMOE_TRY(copyWeights(static_cast<char*>(mDeviceWeights) + deviceStride() * (size_t)expert, expert, nullptr));
        INFMOE_HIP(hipStreamSynchronize(nullptr));
    }
    return INFMOE_OK;
}

Status T5FFLayer::loadFromFile() {
    NpzReader npz;
    INFMOE_TRY(npz.open(mWeightFile.c_str()));
    INFMOE_TRY(ensureHostStore());
    static const char* kGated[] = {"layer_norm_weight", "wi_0_weight", "wi_1_weight", "wo_weight"};
    static const char* kRelu[] = {"layer_norm_weight", "wi_weight", "wo_weight"};
    const char* const* keys = mFfnKind == FFN_GATED_GELU ? kGated : kRelu;
    const size_t d = mEmbeddingSize, h = mHiddenSize;
    for (int e = 0; e < mExpertCount; ++e) {
        float* slot = reinterpret_cast<float*>(reinterpret_cast<char*>(mHostWeights) + hostStride() * (size_t)e);
        for (int j = 0; j <= nMatrices(); ++j) {
            size_t off = 0, cnt = 0;
            keyIndex(keys[j], &off, &cnt);
            const std::string name = std::to_string(e) + "/" + keys[j];  // README.md:121
            if (!npz.has(name.c_str())) {
                // name the likely cause when the file holds the other FFN kind's arrays
                const std::string other = std::to_string(e) + (mFfnKind == FFN_GATED_GELU ? "/wi_weight" : "/wi_0_weight");
                if (npz.has(other.c_str()))
                    return fail(INFMOE_ERR_MISSING_FIELD,
                                "%s: no array named %s but %s exists: the file holds %s experts; set ffn_kind accordingly",
                                mWeightFile.c_str(), name.c_str(), other.c_str(),
                                mFfnKind == FFN_GATED_GELU ? "relu (wi, wo)" : "gated_gelu (wi_0, wi_1, wo)");
            }
            // shapes as python/infmoe/config.py:46-52 saves them: gamma (d,), input-side matrices (h, d), wo (d, h)
            const bool isWo = j == nMatrices();
            INFMOE_TRY(npz.read_f32(name.c_str(), slot + off, j == 0 ? d : (isWo ? d : h), j == 0 ? 0 : (isWo ? h : d)));
            mHave[(size_t)e * (nMatrices() + 1) + j] = 1;
        }
    }
    return INFMOE_OK;
}

Status T5FFLayer::initialize() {
    // plugin/sublayers/T5FFLayer.cc:143-147
    if (mHostWeights == nullptr) {
        if (mWeightFile.empty()) return fail(INFMOE_ERR_STATE, "T5_FF: no expert_weight_file and no weights given by pointer");
        const Status loaded = loadFromFile();
        if (loaded != INFMOE_OK) {  // leave no half-filled store behind: a retry reads the file again
            const std::string why = last_error_slot();
            terminate();
            last_error_slot() = why;
            return loaded;
        }
    }
    for (size_t i = 0; i < mHave.size(); ++i)
        if (!mHave[i])
            return fail(INFMOE_ERR_MISSING_FIELD, "T5_FF: expert %zu is missing weight array #%zu", i / (nMatrices() + 1),
                        i % (nMatrices() + 1));
    return INFMOE_OK;
}

void T5FFLayer::terminate() {
    // plugin/sublayers/T5FFLayer.cc:149-156
    if (mDeviceWeights) (void)hipFree(mDeviceWeights);
    mDeviceWeights = nullptr;
    if (mHostWeights) (void)hipHostFree(mHostWeights);
    mHostWeights = nullptr;
    mHave.clear();
}

Status T5FFLayer::makeResident() {
    if (mDeviceWeights != nullptr) return INFMOE_OK;
    if (mHostWeights == nullptr) return fail(INFMOE_ERR_STATE, "T5_FF: makeResident before initialize");
    INFMOE_HIP(hipMalloc(&mDeviceWeights, deviceStride() * (size_t)mExpertCount));
    for (int e = 0; e < mExpertCount; ++e) {
        const Status s = copyWeights(static_cast<char*>(mDeviceWeights) + deviceStride() * (size_t)e, e, nullptr);
        if (s != INFMOE_OK) {
            (void)hipFree(mDeviceWeights);
            mDeviceWeights = nullptr;
            return s;
        }
    }
    INFMOE_HIP(hipStreamSynchronize(nullptr));
    return INFMOE_OK;
}

Status T5FFLayer::copyWeights(void* dst, int expert, hipStream_t stream) {
    // plugin/sublayers/T5FFLayer.cc:55-88 issues four copies; the host store is already packed in slot order,
    // so one copy moves the expert.  Then, with the rms norm and on the same stream, the norm's gamma is
    // multiplied into the input-side matrices where they now lie: the first product of the expert then carries
    // the norm with it (a read and a write of those matrices in device memory, a few percent of what the copy
    // over the host link takes).
    if (mHostWeights == nullptr) return fail(INFMOE_ERR_STATE, "T5_FF: copyWeights before initialize");
    const char* src = reinterpret_cast<const char*>(mHostWeights) + hostStride() * (size_t)expert;
    const int d = mEmbeddingSize, h = mHiddenSize;
    INFMOE_HIP(hipMemcpyAsync(dst, src, weightBytes(d, h, mFfnKind), hipMemcpyHostToDevice, stream));
    mCopiesQueued.store(true, std::memory_order_release);
    if (!folds()) return INFMOE_OK;
    float* w = static_cast<float*>(dst);
    const size_t dh = (size_t)d * h;
    for (int m = 0; m < nMatrices() - 1; ++m) INFMOE_HIP(launch_fold_gamma(w + d + m * dh, w, h, d, stream));
    return INFMOE_OK;
}

// Few-row kernels are used for an expert only when the whole call is decode-like, and the rule
// depends on nothing but (tokens of the call, experts, rows of the expert), so that the grouped
// and the per-expert schedules pick the same kernel for the same expert and agree bit for bit.
// (Up to two tokens per expert.  With more, the matrix-core kernel for calls with few rows per expert, which runs
// two workgroups per compute unit, streams the weights faster than the few-row kernel and one more launch
// would: 128 tokens over 32 experts of 4096 x 10240 take 0.80 ms per launch against 0.95 ms.)
static bool decode_like(int layerTokens, int expertCount) { return layerTokens <= 2 * expertCount; }
constexpr int kAllRows = 1 << 30;

int T5FFLayer::skinnyMaxRows(int32_t tokenCount) const {
    // (every expert of a decode call, whatever its rows: the few-row kernel takes a taller one in runs of 8)
    return decode_like(tokenCount, mExpertCount) && mEmbeddingSize % 4 == 0 && mHiddenSize % 4 == 0 ? kAllRows : 0;
}

// folded (rms norm only): `weights` is a slot as copyWeights leaves it (gamma multiplied into the input-side
// matrices), the workspace is [H | statistics], and the norm rides on the first product; rowStats are the rows'
// (-, rstd) or null to compute them here.  Not folded: `weights` holds the arrays as they were given
// (plugin/sublayers/T5FFLayer.cc:100-131), the norm is a launch of its own into the workspace [LN | H].
Status T5FFLayer::runOne(int rows, int layerTokens, int expertCount, int d, int h, int normKind, int ffnKind,
                         const void* weights, const float* in, float* out, void* workspace, hipStream_t stream,
                         bool folded, const float* rowStats) {
    if (rows <= 0) return INFMOE_OK;
    const float* w = static_cast<const float*>(weights);
    const size_t dh = (size_t)d * h;
    const int nMat = ffnKind == FFN_GATED_GELU ? 3 : 2;
    GemmProblem g1{};  // plugin/sublayers/T5FFLayer.cc:99-126: norm, one or two products, activation
    float* hid = nullptr;
    if (folded) {
        hid = static_cast<float*>(workspace);
        if (rowStats == nullptr) {  // outside a layer call: nobody has looked at the rows yet
            float* stats = hid + (size_t)rows * h;
            INFMOE_HIP(launch_row_stats(stats, in, rows, d, normKind, stream));
            rowStats = stats;
        }
        g1.A = in, g1.row_stats = rowStats;
    } else {
        float* ln = static_cast<float*>(workspace);
        hid = ln + (size_t)rows * d;
        INFMOE_HIP(launch_row_norm(ln, in, rows, d, w, 0, nullptr, normKind, stream));
        g1.A = ln;
    }
    g1.B = w + d, g1.C = hid, g1.N = h, g1.K = d;
    g1.B1 = ffnKind == FFN_GATED_GELU ? w + d + dh : nullptr;
    g1.epilogue = ffnKind == FFN_GATED_GELU ? EPI_GATED_GELU : EPI_RELU;
    GemmProblem g2{};  // plugin/sublayers/T5FFLayer.cc:130-138 (residual instead of copy + beta = 1)
    g2.A = hid, g2.B = w + d + (size_t)(nMat - 1) * dh, g2.R = in, g2.C = out, g2.N = d, g2.K = h;
    g2.epilogue = EPI_RESIDUAL;
    const bool aligned = ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(g1.A) | reinterpret_cast<uintptr_t>(hid)) & 15) == 0;
    const bool skinny = decode_like(layerTokens, expertCount) && d % 4 == 0 && h % 4 == 0 && aligned;
    if (skinny) {
        INFMOE_HIP(launch_expert_skinny(g1, rows, stream));
        INFMOE_HIP(launch_expert_skinny(g2, rows, stream));
    } else {
        // both launches cut the rows, and pick their kernel, as the grouped schedule does (rowTileHeightFor())
        const bool smallTiles = gemm_small_tiles(layerTokens, expertCount, ffnKind);
        g1.small_tiles = g2.small_tiles = smallTiles ? 1 : 0;
        const int tileRows = smallTiles ? kGemmTileRowsSmall : (ffnKind == FFN_GATED_GELU ? kGemmTileRowsGated : kGemmTileRows);
        INFMOE_HIP(launch_expert_gemm(g1, rows, tileRows, stream));
        INFMOE_HIP(launch_expert_gemm(g2, rows, tileRows, stream));
    }
    return INFMOE_OK;
}

Status T5FFLayer::run(int32_t tokenCount, const void* weights, const void* input, void* output, void* workspace,
                      hipStream_t stream) {
    // outside a layer call the expert stands alone: a call of tokenCount tokens over one expert, on a slot
    // that copyWeights filled.  With up to kSkinnyMaxRows rows it is a decode call whatever the rule for
    // layers says of (tokens, 1 expert): one expert's column tiles would occupy a third of the compute units.
    return runOne(tokenCount, tokenCount <= kSkinnyMaxRows ? 1 : tokenCount, 1, mEmbeddingSize, mHiddenSize, mNormKind, mFfnKind, weights,
                  static_cast<const float*>(input), static_cast<float*>(output), workspace, stream, folds(), nullptr);
}

Status T5FFLayer::runInLayer(int32_t layerTokens, int32_t tokenCount, const void* weights, const void* input,
                             void* output, void* workspace, hipStream_t stream, const float* rowStats) {
    return runOne(tokenCount, layerTokens, mExpertCount, mEmbeddingSize, mHiddenSize, mNormKind, mFfnKind, weights,
                  static_cast<const float*>(input), static_cast<float*>(output), workspace, stream, folds(), rowStats);
}

Status T5FFLayer::runGrouped(const GroupedRun& g) {
    if (mDeviceWeights == nullptr && g.weights == nullptr) return fail(INFMOE_ERR_STATE, "T5_FF: runGrouped needs resident weights");
    const int T = g.tokenCount, d = mEmbeddingSize, h = mHiddenSize;
    const size_t dh = (size_t)d * h, stride = (g.weights ? g.weightStride : deviceStride()) / sizeof(float);
    const float* w = static_cast<const float*>(g.weights ? g.weights : mDeviceWeights);
    const int* slot = g.weights ? g.expertSlot : nullptr;
    float* hid = static_cast<float*>(g.workspace);
    GemmProblem g1{};
    g1.expert_slot = slot;
    if (folds()) {
        const float* stats = g.rowStats;
        if (stats == nullptr) {  // a caller that did not compute them with the scatter
            float* own = hid + (size_t)T * h;
            INFMOE_HIP(launch_row_stats(own, g.input, T, d, mNormKind, g.stream));
            stats = own;
        }
        g1.A = g.input, g1.row_stats = stats;
    } else {  // every routed row with the gamma of its own expert (plugin/sublayers/T5FFLayer.cc:99-103)
        float* ln = hid;
        hid = ln + (size_t)T * d;
        INFMOE_HIP(launch_row_norm(ln, g.input, T, d, w, stride, g.rowExpert, mNormKind, g.stream, slot));
        g1.A = ln;
    }
    g1.B = w + d, g1.C = hid, g1.N = h, g1.K = d;
    g1.B1 = mFfnKind == FFN_GATED_GELU ? w + d + dh : nullptr;
    g1.epilogue = mFfnKind == FFN_GATED_GELU ? EPI_GATED_GELU : EPI_RELU;
    GemmProblem g2{};
    g2.expert_slot = slot;
    g2.A = hid, g2.B = w + d + (mFfnKind == FFN_GATED_GELU ? 2 : 1) * dh, g2.R = g.input, g2.C = g.output, g2.N = d, g2.K = h;
    g2.epilogue = EPI_RESIDUAL;
    const bool skinny = skinnyMaxRows(T) > 0;
    g1.small_tiles = g2.small_tiles = gemm_small_tiles(T, mExpertCount, mFfnKind) ? 1 : 0;
    if (g.afterNorm) INFMOE_HIP(hipEventRecord(g.afterNorm, g.stream));
    if (skinny) {  // a decode call: every expert through the few-row kernel (as runOne does for it)
        INFMOE_HIP(launch_expert_skinny_grouped(g1, stride, g.count, g.offset, mExpertCount, g.stream));
        if (g.afterGemm1) INFMOE_HIP(hipEventRecord(g.afterGemm1, g.stream));
        INFMOE_HIP(launch_expert_skinny_grouped(g2, stride, g.count, g.offset, mExpertCount, g.stream));
        return INFMOE_OK;
    }
    if (!expert_gemm_grouped_ok(g1, stride) || !expert_gemm_grouped_ok(g2, stride)) {
        // sizes the matrix-core kernel does not take (d or h not a multiple of 32)
        INFMOE_HIP(launch_expert_gemm_any_shape_grouped(g1, stride, g.rowExpert, T, g.stream));
        if (g.afterGemm1) INFMOE_HIP(hipEventRecord(g.afterGemm1, g.stream));
        INFMOE_HIP(launch_expert_gemm_any_shape_grouped(g2, stride, g.rowExpert, T, g.stream));
        return INFMOE_OK;
    }
    INFMOE_HIP(launch_expert_gemm_grouped(g1, stride, g.tiles, g.sched, g.maxTiles, g.stream));
    if (g.afterGemm1) INFMOE_HIP(hipEventRecord(g.afterGemm1, g.stream));
    INFMOE_HIP(launch_expert_gemm_grouped(g2, stride, g.tiles, g.sched, g.maxTiles, g.stream));
    return INFMOE_OK;
}

}  // namespace infmoe
