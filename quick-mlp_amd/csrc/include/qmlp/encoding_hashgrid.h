#pragma once

#include "iencoding.h"

QUICKMLP_NAMESPACE_BEGIN

/** How the features of the individual levels are combined. */
enum class LayerCombinationMode
{
    CONCAT,  // #output features = #per-level features * #levels
    ADD      // #output features = #per-level features
};

/** One level of the multi-resolution grid (offsets in parameter entries). */
struct HashGridLayerConfig
{
    int memoryOffset;
    int resolution;
    int hashGridSize;
    bool hashed;
};

/**
 * Multi-resolution hash grid 1D-6D. Per level a dense grid is used if it fits into
 * the hash-table budget, else the cells are hashed. The per-level features are
 * concatenated or added. Input coordinates are first mapped to the unit (hyper-)cube
 * by the bounding box (default: [-0.5, 0.5]^D).
 *
 * The trainable table is one flat tensor (fp32 by default; "parameter_precision":
 * "half" stores it as fp16, gradients stay fp32).
 */
class EncodingHashGrid : public IVolumetricEncoding
{
private:
    const int startChannel_;
    const int dimension_;
    const int numLevels_;
    const int numFeaturesPerLevel_;
    const int log2HashmapSize_;
    const int hashmapSize_;
    const int minResolution_;
    const int maxResolution_;
    const LayerCombinationMode combinationMode_;
    const std::vector<float> boundingBoxMin_;
    const std::vector<float> boundingBoxSize_;
    const std::vector<float> boundingBoxInvSize_;
    const Tensor::Precision parameterPrecision_;

    int numParameters_;
    std::vector<HashGridLayerConfig> layers_;
    Tensor parametersForward_;
    Tensor parametersGradients_;

public:
    EncodingHashGrid(int start_channel, int dimension, int num_levels, int num_features_per_level,
                     int log2_hashmap_size, int min_resolution, int max_resolution,
                     LayerCombinationMode combination_mode, const std::vector<float>& bounding_box_min,
                     const std::vector<float>& bounding_box_size,
                     Tensor::Precision parameter_precision = Tensor::FLOAT);
    explicit EncodingHashGrid(const json& cfg);

    [[nodiscard]] json toJson() const override;
    static std::string ID();
    [[nodiscard]] std::string id() const override;

    [[nodiscard]] int maxInputChannel() const override;
    [[nodiscard]] int numOutputChannels() const override;
    [[nodiscard]] std::string qualifiedName() const override;
    void fillCode(std::stringstream& code) const override;
    [[nodiscard]] bool hasParameters() const override;
    [[nodiscard]] std::string parameterName() const override;
    [[nodiscard]] Tensor::Precision parameterPrecision(Tensor::Usage usage) const override;
    [[nodiscard]] int parameterCount() const override;
    [[nodiscard]] int ldsGradientFloats(int maxBytes, int& levels) const override;
    [[nodiscard]] bool gradientSlices(GradientSliceLayout& layout) const override;
    [[nodiscard]] bool gradientColumns(const kernel::PointOrderKey& key, GradientColumnLayout& layout) const override;
    [[nodiscard]] int numSweptTables() const override { return numLevels_; }
    [[nodiscard]] int gatherRegistersPerPoint() const override;
    [[nodiscard]] bool pointOrderKey(kernel::PointOrderKey& key, long long numPoints = 0) const override;
    /** pointOrderKey() for grids that do not qualify through their dense levels: slabs of multi-level hashed grids. */
    [[nodiscard]] bool hashedPointOrderKey(kernel::PointOrderKey& key, long long numPoints) const;
    [[nodiscard]] int channelsWrittenTogether() const override { return numFeaturesPerLevel_; }
    void setParameter(const Tensor& tensor, Tensor::Usage usage) override;
    [[nodiscard]] bool hasParameterTensor(Tensor::Usage usage) const override
    {
        return usage == Tensor::INFERENCE ? parametersForward_.defined() : parametersGradients_.defined();
    }
    [[nodiscard]] int fillParameterMemory(char* dst, int dstSize) override;
    void zeroGradients() override;

    [[nodiscard]] int startChannel() const { return startChannel_; }
    [[nodiscard]] int ndim() const override { return dimension_; }
    [[nodiscard]] int numLevels() const { return numLevels_; }
    [[nodiscard]] int numFeaturesPerLevel() const { return numFeaturesPerLevel_; }
    [[nodiscard]] int log2HashmapSize() const { return log2HashmapSize_; }
    [[nodiscard]] int hashmapSize() const { return hashmapSize_; }
    [[nodiscard]] int minResolution() const { return minResolution_; }
    [[nodiscard]] int maxResolution() const { return maxResolution_; }
    [[nodiscard]] LayerCombinationMode combinationMode() const { return combinationMode_; }
    [[nodiscard]] const std::vector<HashGridLayerConfig>& levels() const { return layers_; }
    [[nodiscard]] std::vector<float> boundingBoxMin() const override { return boundingBoxMin_; }
    [[nodiscard]] std::vector<float> boundingBoxSize() const override { return boundingBoxSize_; }
    [[nodiscard]] std::vector<float> boundingBoxInvSize() const override { return boundingBoxInvSize_; }

    /**
     * Test aid: evaluates the device index code. indices / weights are device arrays with
     * N * numLevels() * 2^ndim() entries: table offset of feature 0 and interpolation
     * weight of every corner. mode 0: the index function on its own; 1: the table entries that
     * the gathers of the fused forward kernels use (needs a bound table); 2: the entries the
     * gradient scatter of the fused backward kernel adds to (nothing is added).
     */
    void corners(const Tensor& input, unsigned* indices, float* weights, stream_t stream, int mode = 0);
    /** Compiles the kernel of corners(.., mode); compileOnly: into the kernel cache only, which needs no GPU. */
    void precompileCorners(int mode, bool compileOnly);

private:
    [[nodiscard]] std::string configName() const;
    std::optional<KernelFunction> cornersKernel_[5];
};

QUICKMLP_NAMESPACE_END
