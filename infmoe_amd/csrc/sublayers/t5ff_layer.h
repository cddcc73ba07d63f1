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
// Workspace for M rows: [LN M*d | H M*h] (the reference keeps two M*h buffers; the gelu*mul
// product is formed in the GEMM epilogue here, so one is enough).
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
    size_t workspaceOffset(int32_t firstRow) override { return workspaceBytes(firstRow, mEmbeddingSize, mHiddenSize); }
    Status copyWeights(void* dst, int expert, hipStream_t stream) override;
    Status run(int32_t tokenCount, const void* weights, const void* input, void* output, void* workspace,
               hipStream_t stream) override;
    Status runInLayer(int32_t layerTokens, int32_t tokenCount, const void* weights, const void* input, void* output,
                      void* workspace, hipStream_t stream) override;
    Status initialize() override;
    void terminate() override;

    Status setWeights(int expert, const char* key, const float* host, size_t count) override;
    uint64_t weightsVersion() const override { return mVersion.load(std::memory_order_acquire); }
    Status makeResident() override;
    const void* residentWeights() const override { return mDeviceWeights; }
    size_t residentStride() const override { return slotStride(); }
    int skinnyMaxRows(int32_t tokenCount) const override;
    int rowTileHeight() const override { return mFfnKind == FFN_GATED_GELU ? kGemmTileRowsGated : kGemmTileRows; }
    Status runGrouped(const GroupedRun& g) override;

    // used by the kernel-level C entry points
    static size_t weightBytes(int d, int h, int ffnKind);
    static size_t workspaceBytes(int rows, int d, int h);
    static Status runOne(int rows, int layerTokens, int expertCount, int d, int h, int normKind, int ffnKind,
                         const void* weights, const float* in, float* out, void* workspace, hipStream_t stream);

   private:
    int mNormKind, mFfnKind;
    int nMatrices() const { return mFfnKind == FFN_GATED_GELU ? 3 : 2; }
    size_t slotStride() const { return align_up(weightBytes(mEmbeddingSize, mHiddenSize, mFfnKind)); }
    int keyIndex(const char* key, size_t* offsetFloats, size_t* countFloats) const;
    Status ensureHostStore();
    Status loadFromFile();

    float* mHostWeights = nullptr;   // page-locked, E slots of slotStride() bytes
    std::vector<uint8_t> mHave;      // [E][nMatrices+1] which arrays have been provided
    void* mDeviceWeights = nullptr;  // E slots when resident
    std::atomic<uint64_t> mVersion{0};  // bumped by every setWeights
};

}  // namespace infmoe
