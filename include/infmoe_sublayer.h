/*
 * infmoe_sublayer.h - the expert ("sub-layer") plug-in point of the MI355X MoE layer, for C++.
 *
 * Same role and method set as class MoESubLayer of InfMoE (plugin/sublayers/SubLayer.h:18-48) with
 * HIP types in place of the TensorRT / cuBLAS ones and a status return in place of asserts.  The
 * reference's recipe for a new expert type (README.md:100-107: subclass MoESubLayer, give it a name,
 * add a branch to MoELayerPlugin::createSublayer, plugin/MoELayerPlugin.cc:28-41) becomes: subclass
 * infmoe::MoESubLayer, call infmoe::register_sublayer("Name", factory) once (for instance from a
 * static initialiser of a shared library loaded next to libinfmoe.so), and pass
 * expert_sublayer_type = "Name" to infmoe_create.  The header depends on the HIP runtime API header
 * and the C ABI header only; compile against it and link with libinfmoe.so.
 *
 * What the layer does with a sub-layer, per infmoe_enqueue (plugin/MoELayerPlugin.cc:360-402):
 *   experts streamed (max_concurrency < expert_count, weightSize() > 0): for every expert with rows,
 *     copyWeights(slot, expert, copy stream) then runInLayer(...) on that slot and the expert's rows;
 *   experts resident (otherwise): makeResident() once at initialize, then one runGrouped() per call.
 * Rows are the routed (expert-contiguous) rows; every pointer named input / output / workspace /
 * weights is a device pointer; everything is asynchronous on the given stream.
 */
#ifndef INFMOE_SUBLAYER_H
#define INFMOE_SUBLAYER_H

#include <hip/hip_runtime_api.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <memory>
#include <string>

#include "infmoe.h"

namespace infmoe {

using Status = int32_t; /* an infmoe_status */

/* Message slot behind infmoe_last_error() (one per thread; lives in libinfmoe.so). */
std::string& last_error_slot();

/* Records a message for infmoe_last_error() and returns `code`: `return fail(INFMOE_ERR_IO, "...", ...)`. */
inline Status fail(Status code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    last_error_slot() = buf;
    return code;
}

struct Dims { /* stands in for nvinfer1::Dims */
    int32_t nbDims = 0;
    int32_t d[8] = {0, 0, 0, 0, 0, 0, 0, 0};
};

/* A run of consecutive routed rows of one expert, at most rowTileHeight() of them: the unit of work of a
 * launch that covers all experts.  The dispatch step cuts every expert with more than skinnyMaxRows()
 * rows into such tiles on the device and orders them for the eight accelerator dies. */
struct RowTile {
    int32_t expert;
    int32_t row0; /* first routed row */
    int32_t rows; /* 1..tile height */
    int32_t pad;  /* place in its run | length of the run << 16 (a run: row tiles of one expert scheduled together); 0: by itself */
};

/* Everything a sub-layer needs to run every expert of one layer call from a single set of launches. */
struct GroupedRun {
    int32_t tokenCount = 0;
    const float* input = nullptr;       /* routed rows [T][d] */
    float* output = nullptr;            /* post-expert rows [T][d] */
    void* workspace = nullptr;          /* workspaceSize(T) bytes */
    const int32_t* count = nullptr;     /* device [E]: rows of every expert */
    const int32_t* offset = nullptr;    /* device [E+1]: first routed row of every expert */
    const int32_t* rowExpert = nullptr; /* device [T]: expert of every routed row */
    const float* rowStats = nullptr;    /* device [T][2]: (mean, reciprocal deviation) of every routed row, when rowStatsKind() asks for them */
    const RowTile* tiles = nullptr;     /* device: scheduled row tiles */
    const int32_t* sched = nullptr;     /* device, 16 ints: [0] number of tiles, [1 + x] first tile of die x's share */
    int32_t maxTiles = 0;               /* upper bound of [0], known on the host */
    /* Where the experts' weights are.  Null: the sub-layer's own resident copy (makeResident).  Else the base
     * of weight slots of `weightStride` bytes each, expert e in slot expertSlot[e] (device [E]; an entry is
     * only meaningful for an expert with rows): the layer's slots when every expert of a call with streamed
     * experts is already in one. */
    const void* weights = nullptr;
    size_t weightStride = 0;
    const int32_t* expertSlot = nullptr;
    const int32_t* expertSlotHost = nullptr; /* the same table in host memory */
    hipStream_t stream = nullptr;
    hipEvent_t afterNorm = nullptr, afterGemm1 = nullptr; /* optional phase marks to record on `stream` */
};

class MoESubLayer {
   protected:
    int mExpertCount;
    int mEmbeddingSize;
    int mHiddenSize;
    int mMaxConcurrency;
    std::string mWeightFile;

   public:
    MoESubLayer(int expertCount, int embeddingSize, int hiddenSize, const char* weightFile, int maxConcurrency)
        : mExpertCount(expertCount),
          mEmbeddingSize(embeddingSize),
          mHiddenSize(hiddenSize),
          mMaxConcurrency(maxConcurrency),
          mWeightFile(weightFile ? weightFile : "") {}
    virtual ~MoESubLayer() {}

    /* ---- the reference's interface (plugin/sublayers/SubLayer.h:36-47) */
    virtual bool configureWithFormat(const Dims* inputDims, int32_t nbInputs, const Dims* outputDims,
                                     int32_t nbOutputs) = 0;
    virtual size_t weightSize() = 0;                      /* bytes of one expert's device slot (0: no weights) */
    virtual size_t workspaceSize(int32_t tokenCount) = 0; /* bytes of scratch for tokenCount rows */
    virtual Dims getOutputDimensions(const Dims* inputs) { return inputs[0]; }
    virtual Status copyWeights(void* dst, int expert, hipStream_t stream) = 0;
    /* One expert on `tokenCount` rows, standing alone. */
    virtual Status run(int32_t tokenCount, const void* weights, const void* input, void* output, void* workspace,
                       hipStream_t stream) = 0;
    virtual Status initialize() = 0; /* read weights to page-locked memory */
    virtual void terminate() = 0;    /* free them */

    /* ---- additions of this library; every one has a default */
    /* One expert as part of a layer call of `layerTokens` tokens over expertCount() experts.  A sub-layer
     * that picks between kernels by the shape of the whole call does it here, from its arguments only, so
     * that layers that share the sub-layer (clones) cannot influence each other. */
    virtual Status runInLayer(int32_t /*layerTokens*/, int32_t tokenCount, const void* weights, const void* input,
                              void* output, void* workspace, hipStream_t stream, const float* /*rowStats*/ = nullptr) {
        return run(tokenCount, weights, input, output, workspace, stream);
    }
    /* Row statistics the layer's scatter computes while it copies the routed rows, for experts that start with
     * a row norm: INFMOE_NORM_NONE (none), INFMOE_NORM_RMS: (0, rsqrt(mean(x^2) + 1e-6)), INFMOE_NORM_CENTERED:
     * (mean, rsqrt(biased variance + 1e-6)).  They arrive as GroupedRun::rowStats and as runInLayer's last
     * argument (there for the expert's own rows). */
    virtual int rowStatsKind() const { return INFMOE_NORM_NONE; }
    /* Where, inside a scratch of workspaceSize(T) bytes, the expert whose rows start at routed row
     * `firstRow` may work without touching another expert's stretch. */
    virtual size_t workspaceOffset(int32_t /*firstRow*/) { return 0; }
    /* Weights handed over by pointer instead of through the weight file (infmoe_set_expert_weights). */
    virtual Status setWeights(int /*expert*/, const char* /*key*/, const float* /*host*/, size_t /*count*/) {
        return fail(INFMOE_ERR_UNSUPPORTED, "this sub-layer takes no weights");
    }
    /* A number that changes whenever any expert's weights change after initialize(); the layer then drops
     * the device copies of experts it has kept from earlier calls. */
    virtual uint64_t weightsVersion() const { return 0; }
    /* Keep every expert in device memory (called once, from infmoe_initialize, when the experts are not
     * streamed).  The default allocates expertCount() slots of weightSize() bytes (rounded up to 256) and
     * fills them with copyWeights. */
    virtual Status makeResident();
    virtual const void* residentWeights() const { return mResident; }
    virtual size_t residentStride() const { return mResidentStride; }
    /* Row count up to which runGrouped handles an expert outside the row tiles (0: every expert is tiled). */
    virtual int skinnyMaxRows(int32_t /*tokenCount*/) const { return 0; }
    /* Tallest row tile runGrouped wants an expert's rows cut into (a multiple of 16). */
    virtual int rowTileHeight() const { return 256; }
    /* All experts of one call, weights resident.  The default copies count / offset to the host (one wait
     * on the stream) and calls runInLayer once per expert with rows, in ascending index, on g.stream. */
    virtual Status runGrouped(const GroupedRun& g);
    /* Whether runGrouped honours g.weights / g.expertSlot (the default one does). */
    virtual bool groupedFromSlots() const { return true; }
    /* rowTileHeight() for a call of `tokenCount` tokens, for a sub-layer that cuts the rows of calls with few rows
     * per expert into shorter tiles (a multiple of 16, at most rowTileHeight(), at least minRowTileHeight()). */
    virtual int rowTileHeightFor(int32_t /*tokenCount*/) const { return rowTileHeight(); }
    virtual int minRowTileHeight() const { return rowTileHeight(); }
    int expertCount() const { return mExpertCount; }

   private:
    void* mResident = nullptr; /* owned by the default makeResident */
    size_t mResidentStride = 0;

   protected:
    void releaseResident(); /* frees what the default makeResident allocated; call from terminate() */
};

/* What a factory is given: the creation attributes of the layer that concern its experts. */
struct SubLayerConfig {
    int expertCount, embeddingSize, hiddenSize, maxConcurrency;
    const char* weightFile; /* null when none was given */
    int normKind, ffnKind;  /* INFMOE_NORM_*, INFMOE_FFN_* */
};
typedef std::shared_ptr<MoESubLayer> (*SubLayerFactory)(const SubLayerConfig&);

/* Makes `type` a value that expert_sublayer_type accepts (replaces the branch one adds to
 * MoELayerPlugin::createSublayer, plugin/MoELayerPlugin.cc:28-41).  "T5_FF" and "Identity" are built in;
 * registering a name again replaces its factory.  Thread-safe. */
Status register_sublayer(const char* type, SubLayerFactory factory);

} /* namespace infmoe */
#endif /* INFMOE_SUBLAYER_H */
