// The expert ("sub-layer") plug-in point: same role and method set as class MoESubLayer of the
// reference (plugin/sublayers/SubLayer.h:18-48) with HIP types instead of TensorRT / cuBLAS ones
// and a status return instead of asserts.  To add an expert type, subclass this, give it a name
// and add a branch to make_sublayer() (README.md:100-107 describes the same recipe).
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>
#include <memory>
#include <atomic>
#include <string>

#include "../kernels/kernels.h"
#include "../status.h"

namespace infmoe {

struct Dims {  // stands in for nvinfer1::Dims
    int32_t nbDims = 0;
    int32_t d[8] = {0, 0, 0, 0, 0, 0, 0, 0};
};

// Everything a sub-layer needs to run every expert of one layer call from a single set of
// launches.  Rows are the routed (expert-contiguous) rows; all pointers are device pointers.
struct GroupedRun {
    int32_t tokenCount = 0;
    const float* input = nullptr;   // routed rows [T][d]
    float* output = nullptr;        // post-expert rows [T][d]
    void* workspace = nullptr;      // workspaceSize(T) bytes
    const int32_t* count = nullptr;      // [E]
    const int32_t* offset = nullptr;     // [E+1]
    const int32_t* rowExpert = nullptr;  // [T]
    const RowTile* tiles = nullptr;      // scheduled row tiles of the experts with more than skinnyMax rows
    const int32_t* sched = nullptr;      // kSchedInts ints describing the schedule
    int32_t maxTiles = 0;                // max_row_tiles(T, E, rowTileHeight())
    hipStream_t stream = nullptr;
    // optional phase marks: recorded on `stream` after the norm and after the first GEMM
    hipEvent_t afterNorm = nullptr, afterGemm1 = nullptr;
};

class MoESubLayer {
   protected:
    int mExpertCount;
    int mEmbeddingSize;
    int mHiddenSize;
    int mMaxConcurrency;
    std::string mWeightFile;
    // Tokens of the whole layer call the next run() belongs to (only picks between two kernels of equal
    // results to rounding).  Clones share the sub-layer, as in the reference
    // (plugin/MoELayerPlugin.cc:100): atomic, so that clones driven from different threads do not race.
    std::atomic<int> mLayerTokenCount{0};

   public:
    MoESubLayer(int expertCount, int embeddingSize, int hiddenSize, const char* weightFile, int maxConcurrency)
        : mExpertCount(expertCount),
          mEmbeddingSize(embeddingSize),
          mHiddenSize(hiddenSize),
          mMaxConcurrency(maxConcurrency),
          mWeightFile(weightFile ? weightFile : "") {}
    virtual ~MoESubLayer() {}

    // ---- the reference's interface (plugin/sublayers/SubLayer.h:36-47)
    virtual bool configureWithFormat(const Dims* inputDims, int32_t nbInputs, const Dims* outputDims,
                                     int32_t nbOutputs) = 0;
    virtual size_t weightSize() = 0;                       // bytes of one expert's device slot
    virtual size_t workspaceSize(int32_t tokenCount) = 0;  // bytes of scratch for tokenCount rows
    // Where, inside a scratch of workspaceSize(T) bytes, the expert whose rows start at routed row
    // `firstRow` may work without touching another expert's stretch.
    virtual size_t workspaceOffset(int32_t /*firstRow*/) { return 0; }
    virtual Dims getOutputDimensions(const Dims* inputs) { return inputs[0]; }
    virtual Status copyWeights(void* dst, int expert, hipStream_t stream) = 0;
    virtual Status run(int32_t tokenCount, const void* weights, const void* input, void* output, void* workspace,
                       hipStream_t stream) = 0;
    virtual Status initialize() = 0;  // read weights to page-locked memory
    virtual void terminate() = 0;     // free them

    // ---- additions of this build
    // Weights handed over by pointer instead of through the npz file.
    virtual Status setWeights(int /*expert*/, const char* /*key*/, const float* /*host*/, size_t /*count*/) {
        return fail(INFMOE_ERR_UNSUPPORTED, "this sub-layer takes no weights");
    }
    // Keep every expert in device memory (called once when max_concurrency >= expert_count).
    virtual Status makeResident() { return INFMOE_OK; }
    virtual const void* residentWeights() const { return nullptr; }
    virtual size_t residentStride() const { return 0; }
    // Row-count threshold below which runGrouped handles an expert outside the row tiles.
    virtual int skinnyMaxRows(int32_t /*tokenCount*/) const { return 0; }
    // Tallest row tile runGrouped wants the dispatch scan to cut an expert's rows into.
    virtual int rowTileHeight() const { return kGemmTileRows; }
    virtual Status runGrouped(const GroupedRun& g) = 0;
    void setLayerTokenCount(int32_t tokens) { mLayerTokenCount.store(tokens, std::memory_order_relaxed); }
    int expertCount() const { return mExpertCount; }
};

enum class SubLayerKind { T5FF, Identity };

// Replaces MoELayerPlugin::createSublayer (plugin/MoELayerPlugin.cc:28-41).
Status make_sublayer(const char* type, int expertCount, int embeddingSize, int hiddenSize, const char* weightFile,
                     int maxConcurrency, int normKind, int ffnKind, std::shared_ptr<MoESubLayer>* out);

}  // namespace infmoe
