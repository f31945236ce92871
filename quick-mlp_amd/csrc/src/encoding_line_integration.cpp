#include <qmlp/encoding_line_integration.h>

#include <qmlp/qmlp.h>

#include <cstring>

QUICKMLP_NAMESPACE_BEGIN

static LineIntegrationBlendingMode parseBlending(const json& j)
{
    const std::string s = j.get<std::string>();
    if (s == "additive") return LineIntegrationBlendingMode::ADDITIVE;
    if (s == "average") return LineIntegrationBlendingMode::AVERAGE;
    throw configuration_error("Unknown blending '%s', expected 'additive' or 'average'", s.c_str());
}

static std::shared_ptr<IVolumetricEncoding> parseChild(json cfg, int ndim)
{
    // the child always reads the sample position: channels 0..ndim-1
    cfg["start_in"] = 0;
    cfg["n_in"] = ndim;
    auto ptr = EncodingFactory::Instance().create(cfg);
    auto ptrCast = std::dynamic_pointer_cast<IVolumetricEncoding>(ptr);
    CHECK_ERROR(ptrCast != nullptr, "Child encoding for LineIntegration must be a volumetric encoding");
    return ptrCast;
}

EncodingLineIntegration::EncodingLineIntegration(int start_channel, int dimension,
                                                 std::shared_ptr<IVolumetricEncoding> volume, float stepsize,
                                                 LineIntegrationBlendingMode blendingMode)
    : startChannel_(start_channel)
    , dimension_(dimension)
    , volume_(std::move(volume))
    , stepsizeWorld_(stepsize)
    , blendingMode_(blendingMode)
{
    CHECK_ERROR(start_channel >= 0, "start_in must be non-negative but is ", start_channel);
    CHECK_ERROR(stepsize > 0, "Stepsize must be positive, but is ", stepsize);
    CHECK_ERROR(dimension_ == 3, "LineIntegration is only defined for 3D volumes, but n_in is ", dimension_);
    CHECK_ERROR(dimension_ == volume_->ndim(), "Dimension of the child volume doesn't match");
    CHECK_ERROR(volume_->hasParameters(), "Child volume needs trainable parameters");
}

EncodingLineIntegration::EncodingLineIntegration(const json& cfg)
    : EncodingLineIntegration(cfg.at("start_in").get<int>(), cfg.at("n_in").get<int>(),
                              parseChild(cfg.at("volume"), cfg.at("n_in").get<int>()),
                              cfg.at("stepsize").get<float>(), parseBlending(cfg.at("blending")))
{
}

json EncodingLineIntegration::toJson() const
{
    json j = json::object();
    j["id"] = id();
    j["start_in"] = startChannel_;
    j["n_in"] = dimension_;
    j["volume"] = volume_->toJson();
    j["stepsize"] = stepsizeWorld_;
    j["blending"] = blendingMode_ == LineIntegrationBlendingMode::ADDITIVE ? "additive" : "average";
    return j;
}

std::string EncodingLineIntegration::ID() { return "LineIntegration"; }

std::string EncodingLineIntegration::id() const { return ID(); }

int EncodingLineIntegration::maxInputChannel() const { return startChannel_ + dimension_ * 2 - 1; }

int EncodingLineIntegration::numOutputChannels() const { return volume_->numOutputChannels(); }

std::string EncodingLineIntegration::qualifiedName() const
{
    return format("qmlp::kernel::EncodingLineIntegration<%d, %d, qmlp::kernel::LineIntegrationBlendingMode::%s, %s>",
                  startChannel_, dimension_,
                  blendingMode_ == LineIntegrationBlendingMode::ADDITIVE ? "ADDITIVE" : "AVERAGE",
                  volume_->qualifiedName().c_str());
}

void EncodingLineIntegration::fillCode(std::stringstream& code) const
{
    volume_->fillCode(code);  // the child's definitions first
    code << KernelLoader::MainFile("qmlp/kernels/encoding_line_integration.h");
}

int EncodingLineIntegration::ndim() const { return dimension_ * 2; }

IVolumetricEncoding::BoundingBoxVector_t EncodingLineIntegration::boundingBoxMin() const { return volume_->boundingBoxMin(); }

IVolumetricEncoding::BoundingBoxVector_t EncodingLineIntegration::boundingBoxSize() const { return volume_->boundingBoxSize(); }

IVolumetricEncoding::BoundingBoxVector_t EncodingLineIntegration::boundingBoxInvSize() const
{
    return volume_->boundingBoxInvSize();
}

bool EncodingLineIntegration::hasParameters() const { return volume_->hasParameters(); }

std::string EncodingLineIntegration::parameterName() const
{
    return format("qmlp::kernel::LineIntegrationParams<%s, %d>", volume_->parameterName().c_str(), dimension_);
}

Tensor::Precision EncodingLineIntegration::parameterPrecision(Tensor::Usage usage) const
{
    return volume_->parameterPrecision(usage);
}

int EncodingLineIntegration::parameterCount() const { return volume_->parameterCount(); }

void EncodingLineIntegration::setParameter(const Tensor& tensor, Tensor::Usage usage)
{
    volume_->setParameter(tensor, usage);
}

int EncodingLineIntegration::fillParameterMemory(char* dst, int dstSize)
{
    // mirrors qmlp::kernel::LineIntegrationParams<Child, D>: the child's block (a multiple of
    // 8 bytes), then box minimum, box size and the step size as floats
    int index = volume_->fillParameterMemory(dst, dstSize);
    CHECK_ERROR(index % 8 == 0, "the child's parameter block must be a multiple of 8 bytes");
    const int needed = index + static_cast<int>((2 * dimension_ + 1) * sizeof(float));
    CHECK_ERROR(dstSize >= roundUp(needed, 8), "parameter buffer too small");
    const auto boxMin = boundingBoxMin();
    const auto boxSize = boundingBoxSize();
    std::memcpy(dst + index, boxMin.data(), dimension_ * sizeof(float));
    index += static_cast<int>(dimension_ * sizeof(float));
    std::memcpy(dst + index, boxSize.data(), dimension_ * sizeof(float));
    index += static_cast<int>(dimension_ * sizeof(float));
    std::memcpy(dst + index, &stepsizeWorld_, sizeof(float));
    index += static_cast<int>(sizeof(float));
    return roundUp(index, 8);
}

void EncodingLineIntegration::zeroGradients() { volume_->zeroGradients(); }

QUICKMLP_NAMESPACE_END
