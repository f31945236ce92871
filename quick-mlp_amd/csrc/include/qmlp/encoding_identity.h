#pragma once

#include "iencoding.h"

QUICKMLP_NAMESPACE_BEGIN

/** Copies 'n_in' input channels starting at 'start_in' into the network input. */
class EncodingIdentity : public IEncoding
{
    const int startChannel_;
    const int numChannels_;

public:
    EncodingIdentity(int startChannel, int numChannels) : startChannel_(startChannel), numChannels_(numChannels) {}
    explicit EncodingIdentity(const json& cfg);

    [[nodiscard]] json toJson() const override;
    static std::string ID();
    [[nodiscard]] std::string id() const override;
    [[nodiscard]] int maxInputChannel() const override;
    [[nodiscard]] int numOutputChannels() const override;
    [[nodiscard]] std::string qualifiedName() const override;
    void fillCode(std::stringstream& code) const override;

    [[nodiscard]] int startChannel() const { return startChannel_; }
};

QUICKMLP_NAMESPACE_END
