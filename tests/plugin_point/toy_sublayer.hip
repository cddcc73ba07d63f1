// An expert type built OUTSIDE the library, against include/infmoe_sublayer.h and libinfmoe.so only:
// what a user of the reference does by subclassing MoESubLayer and adding a branch to createSublayer
// (README.md:100-107).  Expert e computes out = in * (e + 2) + e / 2, with its two coefficients as "weights"
// that travel through copyWeights, so the streamed and the resident schedule both have something to move.
// It overrides the reference's methods only; the grouped run and the resident copy are the library's defaults.
// A second type, "ToyStandardize", has no weights and asks the layer for the centered statistics of its rows
// (rowStatsKind): out = (in - mean) * reciprocal deviation, with both numbers taken from what the layer's scatter
// computed on the way.
#include <hip/hip_runtime.h>

#include <vector>

#include "infmoe_sublayer.h"

namespace {

__global__ void affine_rows(const float* __restrict__ in, float* __restrict__ out, const float* __restrict__ w, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = in[i] * w[0] + w[1];
}

__global__ void standardize_rows(const float* __restrict__ in, float* __restrict__ out, const float* __restrict__ stats,
                                 int d, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = (in[i] - stats[2 * (i / d)]) * stats[2 * (i / d) + 1];
}

class AffineLayer : public infmoe::MoESubLayer {
    std::vector<float> mHost;  // [E][2]

   public:
    explicit AffineLayer(const infmoe::SubLayerConfig& c)
        : MoESubLayer(c.expertCount, c.embeddingSize, c.hiddenSize, c.weightFile, c.maxConcurrency) {}
    ~AffineLayer() override { terminate(); }
    bool configureWithFormat(const infmoe::Dims* in, int32_t nbIn, const infmoe::Dims* out, int32_t nbOut) override {
        return nbIn == 1 && nbOut == 1 && in[0].nbDims == 3 && out[0].nbDims == 3 && in[0].d[2] == mEmbeddingSize;
    }
    size_t weightSize() override { return 2 * sizeof(float); }
    size_t workspaceSize(int32_t) override { return 0; }
    infmoe::Status initialize() override {
        mHost.resize((size_t)2 * mExpertCount);
        for (int e = 0; e < mExpertCount; ++e) mHost[2 * e] = (float)(e + 2), mHost[2 * e + 1] = 0.5f * e;
        return INFMOE_OK;
    }
    void terminate() override {
        releaseResident();
        mHost.clear();
    }
    infmoe::Status copyWeights(void* dst, int expert, hipStream_t stream) override {
        if (mHost.empty()) return infmoe::fail(INFMOE_ERR_STATE, "ToyAffine: copyWeights before initialize");
        if (hipMemcpyAsync(dst, &mHost[(size_t)2 * expert], 2 * sizeof(float), hipMemcpyHostToDevice, stream) != hipSuccess)
            return infmoe::fail(INFMOE_ERR_HIP, "ToyAffine: copy failed");
        return INFMOE_OK;
    }
    infmoe::Status run(int32_t tokenCount, const void* weights, const void* input, void* output, void*,
                       hipStream_t stream) override {
        const size_t n = (size_t)tokenCount * mEmbeddingSize;
        if (n == 0) return INFMOE_OK;
        affine_rows<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(static_cast<const float*>(input), static_cast<float*>(output),
                                                                    static_cast<const float*>(weights), n);
        return hipGetLastError() == hipSuccess ? INFMOE_OK : infmoe::fail(INFMOE_ERR_HIP, "ToyAffine: launch failed");
    }
};

class StandardizeLayer : public infmoe::MoESubLayer {
   public:
    explicit StandardizeLayer(const infmoe::SubLayerConfig& c)
        : MoESubLayer(c.expertCount, c.embeddingSize, c.hiddenSize, c.weightFile, c.maxConcurrency) {}
    bool configureWithFormat(const infmoe::Dims* in, int32_t nbIn, const infmoe::Dims* out, int32_t nbOut) override {
        return nbIn == 1 && nbOut == 1 && in[0].nbDims == 3 && out[0].nbDims == 3 && in[0].d[2] == mEmbeddingSize;
    }
    size_t weightSize() override { return 0; }
    size_t workspaceSize(int32_t) override { return 0; }
    infmoe::Status initialize() override { return INFMOE_OK; }
    void terminate() override {}
    infmoe::Status copyWeights(void*, int, hipStream_t) override { return INFMOE_OK; }
    int rowStatsKind() const override { return INFMOE_NORM_CENTERED; }
    infmoe::Status run(int32_t, const void*, const void*, void*, void*, hipStream_t) override {
        return infmoe::fail(INFMOE_ERR_UNSUPPORTED, "ToyStandardize: runs inside a layer only (it needs the layer's row statistics)");
    }
    infmoe::Status runInLayer(int32_t, int32_t tokenCount, const void*, const void* input, void* output, void*,
                              hipStream_t stream, const float* rowStats) override {
        const size_t n = (size_t)tokenCount * mEmbeddingSize;
        if (n == 0) return INFMOE_OK;
        if (rowStats == nullptr) return infmoe::fail(INFMOE_ERR_STATE, "ToyStandardize: no row statistics handed over");
        standardize_rows<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(static_cast<const float*>(input), static_cast<float*>(output),
                                                                         rowStats, mEmbeddingSize, n);
        return hipGetLastError() == hipSuccess ? INFMOE_OK : infmoe::fail(INFMOE_ERR_HIP, "ToyStandardize: launch failed");
    }
};

std::shared_ptr<infmoe::MoESubLayer> make_affine(const infmoe::SubLayerConfig& c) { return std::make_shared<AffineLayer>(c); }

std::shared_ptr<infmoe::MoESubLayer> make_standardize(const infmoe::SubLayerConfig& c) { return std::make_shared<StandardizeLayer>(c); }

}  // namespace

extern "C" int toy_register(void) {
    const int s = infmoe::register_sublayer("ToyAffine", make_affine);
    return s != INFMOE_OK ? s : infmoe::register_sublayer("ToyStandardize", make_standardize);
}
