#pragma once

#include "iencoding.h"

QUICKMLP_NAMESPACE_BEGIN

/** How the samples along the ray are combined. */
enum class LineIntegrationBlendingMode
{
    ADDITIVE,  // sum of the samples
    AVERAGE    // sum divided by the number of steps
};

/**
 * Fixed-step line integration through a child volume encoding (3D only). The input
 * provides the ray start in channels [start_in, start_in+n_in) and the ray direction in
 * the n_in channels after that; the ray is clipped against the child's bounding box and
 * the child's features are summed (or averaged) at steps of `stepsize` in ray parameter.
 * All trainable parameters are the child's.
 *
 * JSON: {"id": "LineIntegration", "start_in", "n_in", "volume": {child encoding},
 * "stepsize", "blending": "additive"|"average"}; the child's start_in / n_in are
 * overwritten by 0 / n_in.
 *
 * Mirrors src_cpp/include/qmlp/encoding_line_integration.h:15-67 of the reference.
 */
class EncodingLineIntegration : public IVolumetricEncoding
{
    const int startChannel_;
    const int dimension_;
    const std::shared_ptr<IVolumetricEncoding> volume_;
    const float stepsizeWorld_;
    const LineIntegrationBlendingMode blendingMode_;

public:
    EncodingLineIntegration(int start_channel, int dimension, std::shared_ptr<IVolumetricEncoding> volume,
                            float stepsize, LineIntegrationBlendingMode blendingMode);
    explicit EncodingLineIntegration(const json& cfg);

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
    void setParameter(const Tensor& tensor, Tensor::Usage usage) override;
    [[nodiscard]] bool hasParameterTensor(Tensor::Usage usage) const override { return volume_->hasParameterTensor(usage); }
    [[nodiscard]] int fillParameterMemory(char* dst, int dstSize) override;
    void zeroGradients() override;

    /** Ray start + ray direction. */
    [[nodiscard]] int ndim() const override;
    [[nodiscard]] BoundingBoxVector_t boundingBoxMin() const override;
    [[nodiscard]] BoundingBoxVector_t boundingBoxSize() const override;
    [[nodiscard]] BoundingBoxVector_t boundingBoxInvSize() const override;

    [[nodiscard]] std::shared_ptr<IVolumetricEncoding> volume() const { return volume_; }
    [[nodiscard]] float stepsize() const { return stepsizeWorld_; }
    [[nodiscard]] LineIntegrationBlendingMode blendingMode() const { return blendingMode_; }
};

QUICKMLP_NAMESPACE_END
