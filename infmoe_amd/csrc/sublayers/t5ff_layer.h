// T5 feed-forward expert: out = in + FFN(norm(in)).  Same role as class T5FFLayer of the
// reference (plugin/sublayers/T5FFLayer.h:11-37, plugin/sublayers/T5FFLayer.cc:43-156).
//
// The reference's code and README disagree on both halves of that formula, so both are explicit:
//   norm: "centered" as coded (plugin/cuda/ops/layernorm.cu:149-161) or "rms" as documented
//         (README.md:115, comment at plugin/sublayers/T5FFLayer.cc:98);
//   ffn:  "gated_gelu" with wi_0, wi_1, wo as coded (plugin/sublayers/T5FFLayer.cc:105-138) or
//         "relu" with wi, wo (the dense_relu_dense the layer is named after).
// Device slot of one expert, as plugin/sublayers/T5FFLayer.cc:100,112,118-119,130-131:
//   [gamma d | wi h*d | wo d*h]  or  [gamma d | wi_0 h*d | wi_1 h*d | wo d*h]   (floats)
// With the rms norm, copyWeights leaves the input-side matrices multiplied by gamma: the norm then rides on the
// first product (rstd_r * x.w') and is no launch of its own.  Workspace for M rows: [H M*h | row statistics M*4]
// (the reference keeps the normed rows M*d and two M*h buffers; here the gelu*mul product is formed in the
// epilogue, so one hidden buffer is all; the statistics area is used when nobody hands them over).
// With the centered norm the slot holds the arrays as they are and the norm runs first, as a launch of its own,
// as in the reference: carried on the product it would subtract mu_r * (column sum of w') from x.w', two numbers
// that are large against their difference whenever a row's mean is large against its deviation.  Workspace
// [LN M*d | H M*h].  infmoe_t5ff_run, which takes the arrays as the caller made them, does the same for both norms.
#pragma once

#include <atomic>
#include <vector>

#include "sublayer.h"

namespace infmoe {

class T5FFLayer : public MoESubLayer {
   public:
    T5FFLayer(int expertCount, int embeddingSize, int hiddenSize, const char* weightFile, int maxConcurrency,
              int normKind, int ffnKind);
    ~T5FFLayer() override;

    bool configureWithFormat(const Dims* inputDims, int32_t nbInputs, const Dims* outputDims,
                             int32_t nbOutputs) override;
    size_t weightSize() override;
    size_t workspaceSize(int32_t tokenCount) override;
    size_t workspaceOffset(int32_t firstRow) override { return layerWorkspaceBytes(firstRow); }
    Status copyWeights(void* dst, int expert, hipStream_t stream) override;
    Status run(int32_t tokenCount, const void* weights, const void* input, void* output, void* workspace,
               hipStream_t stream) override;
    Status runInLayer(int32_t layerTokens, int32_t tokenCount, const void* weights, const void* input, void* output,
                      void* workspace, hipStream_t stream, const float* rowStats) override;
    int rowStatsKind() const override { return folds() ? NORM_RMS : NORM_NONE; }
    Status initialize() override;
    void terminate() override;

    Status setWeights(int expert, const char* key, const float* host, size_t count) override;
    uint64_t weightsVersion() const override { return mVersion.load(std::memory_order_acquire); }
    Status makeResident() override;
    const void* residentWeights() const override { return mDeviceWeights; }
    size_t residentStride() const override { return deviceStride(); }
    int skinnyMaxRows(int32_t tokenCount) const override;
    int rowTileHeight() const override { return mFfnKind == FFN_GATED_GELU ? kGemmTileRowsGated : kGemmTileRows; }
    int rowTileHeightFor(int32_t tokenCount) const override {
        return gemm_small_tiles(tokenCount, mExpertCount, mFfnKind) ? kGemmTileRowsSmall : rowTileHeight();
    }
    int minRowTileHeight() const override { return mFfnKind == FFN_GATED_GELU ? kGemmTileRowsGated : kGemmTileRowsSmall; }
    Status runGrouped(const GroupedRun& g) override;

    // used by the kernel-level C entry points
    static size_t weightBytes(int d, int h, int ffnKind);
    static size_t workspaceBytes(int rows, int d, int h);
    static Status runOne(int rows, int layerTokens, int expertCount, int d, int h, int normKind, int ffnKind,
                         const void* weights, const float* in, float* out, void* workspace, hipStream_t stream,
                         bool folded, const float* rowStats);

   private:
    int mNormKind, mFfnKind;
    int nMatrices() const { return mFfnKind == FFN_GATED_GELU ? 3 : 2; }
    bool folds() const { return mNormKind == NORM_RMS; }  // the norm rides on the first product
    size_t hostStride() const { return align_up(weightBytes(mEmbeddingSize, mHiddenSize, mFfnKind)); }
    size_t deviceStride() const { return hostStride(); }
    size_t layerWorkspaceBytes(int rows) const;
    int keyIndex(const char* key, size_t* offsetFloats, size_t* countFloats) const;
    Status ensureHostStore();
    Status loadFromFile();

    float* mHostWeights = nullptr;   // page-locked, E slots of hostStride() bytes
    std::vector<uint8_t> mHave;      // [E][nMatrices+1] which arrays have been provided
    void* mDeviceWeights = nullptr;  // E slots when resident
    std::atomic<uint64_t> mVersion{0};  // bumped by every setWeights
    std::atomic<bool> mCopiesQueued{false};  // a copy out of the host store may be in flight
};

}  // namespace infmoe
