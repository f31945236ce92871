#include <qmlp/encoding_identity.h>

QUICKMLP_NAMESPACE_BEGIN

EncodingIdentity::EncodingIdentity(const json& cfg)
    : EncodingIdentity(cfg.at("start_in").get<int>(), cfg.at("n_in").get<int>())
{
    if (startChannel_ < 0) throw configuration_error("Start channel must be non-negative, but is %d", startChannel_);
    if (numChannels_ <= 0) throw configuration_error("Num channels must be positive, but is %d", numChannels_);
}

json EncodingIdentity::toJson() const
{
    return json::object({{"id", id()}, {"start_in", startChannel_}, {"n_in", numChannels_}});
}

std::string EncodingIdentity::ID() { return "Identity"; }

std::string EncodingIdentity::id() const { return ID(); }

int EncodingIdentity::maxInputChannel() const { return startChannel_ + numChannels_ - 1; }

int EncodingIdentity::numOutputChannels() const { return numChannels_; }

std::string EncodingIdentity::qualifiedName() const
{
    return format("qmlp::kernel::EncodingIdentity<%d, %d>", startChannel_, numChannels_);
}

void EncodingIdentity::fillCode(std::stringstream& code) const
{
    code << KernelLoader::MainFile("qmlp/kernels/encoding_identity.h");
}

QUICKMLP_NAMESPACE_END
