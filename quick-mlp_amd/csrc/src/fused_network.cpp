#include <qmlp/fused_network.h>
#include <qmlp/device_code.h>

#include <qmlp/encoding_identity.h>
#include <qmlp/qmlp.h>

#include "qmlp_hip.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>
#include <sstream>
#include <unordered_set>

QUICKMLP_NAMESPACE_BEGIN

namespace {
constexpr int TILE_POINTS = 64;          // points per wavefront tile
constexpr int DEFAULT_BLOCK_SIZE = 256;  // 4 wavefronts
constexpr int MAX_WEIGHT_UPDATE_SLICES = 512;  // batch slices with partial weight gradients
constexpr int STAGE_PAD = 8;             // halves of padding per staging row
constexpr int MAX_REGISTER_SHAPE_SCRATCH = 512;   // bytes per lane, see forwardKernelFor

int gfx950LdsBytes() { return 160 * 1024; }
} // namespace

int FusedNetwork::MaxSharedMemoryBytes()
{
    static const int value = [] {
        int count = 0;
        qmlp_hip_device_count(&count);
        if (count == 0) return gfx950LdsBytes();
        qmlp_hip_device_props props;
        QMLP_HIP_CALL(qmlp_hip_get_device_props(0, &props));
        if (props.wave_size != FusedNetwork::WARP_SIZE)
            throw configuration_error("The wavefront size of the device is %d, but the kernels are written for %d",
                                      props.wave_size, FusedNetwork::WARP_SIZE);
        QuickMLP::Instance().getLogger()->debug("LDS per workgroup on the current device in bytes: %d",
                                                props.lds_bytes_per_block);
        return props.lds_bytes_per_block;
    }();
    return value;
}

static bool offersSlices(const IEncoding& e, IEncoding::GradientSliceLayout* layout = nullptr)
{
    IEncoding::GradientSliceLayout local;
    return e.hasParameters() && e.gradientSlices(layout ? *layout : local);
}

FusedNetwork::FusedNetwork(const json& cfg, const std::filesystem::path& parent)
    : channelsIn_(cfg.at("num_inputs").get<int>())
    , channelsOut_(cfg.at("num_outputs").get<int>())
    , encodedChannels_(0)
    , networkInputPadding_(0)
    , numParameters_(0)
    , perEntryForwardMemoryBytes_(0)
    , adjointEvent_(nullptr)
    , streamsCreated_(false)
{
    auto loader = QuickMLP::Instance().kernelLoader();
    auto logger = QuickMLP::Instance().getLogger();

    if (channelsIn_ <= 0) throw configuration_error("num_inputs must be positive, but is %d", channelsIn_);
    if (channelsOut_ <= 0) throw configuration_error("num_outputs must be positive, but is %d", channelsOut_);

    //compile options
    if (cfg.contains("options")) {
        const json& options = cfg.at("options");
        compileOptions_.overwriteBlocksizeInference =
            options.value("overwrite_blocksize_inference", compileOptions_.overwriteBlocksizeInference);
        compileOptions_.overwriteBlocksizeForward =
            options.value("overwrite_blocksize_forward", compileOptions_.overwriteBlocksizeForward);
        compileOptions_.overwriteBlocksizeBackward =
            options.value("overwrite_blocksize_backward", compileOptions_.overwriteBlocksizeBackward);
        compileOptions_.overwriteBlocksizeWeightUpdate =
            options.value("overwrite_blocksize_weight_update", compileOptions_.overwriteBlocksizeWeightUpdate);
        compileOptions_.pointsPerLane = options.value("points_per_lane", compileOptions_.pointsPerLane);
        if (compileOptions_.pointsPerLane > 8)
            throw configuration_error("points_per_lane must be at most 8, but is %d", compileOptions_.pointsPerLane);
        compileOptions_.registerStaging = options.value("register_staging", compileOptions_.registerStaging);
        compileOptions_.sortPoints = options.value("sort_points", compileOptions_.sortPoints);
        compileOptions_.sortTraining = options.value("sort_training", compileOptions_.sortTraining);
        compileOptions_.directInput = options.value("direct_input", compileOptions_.directInput);
        compileOptions_.sliceGradients = options.value("slice_gradients", compileOptions_.sliceGradients);
        compileOptions_.inputDerivatives = options.value("input_derivatives", compileOptions_.inputDerivatives);
        compileOptions_.columnGradients = options.value("column_gradients", compileOptions_.columnGradients);
        compileOptions_.recomputeIntermediates = options.value("recompute_intermediates", compileOptions_.recomputeIntermediates);
        compileOptions_.fusedWeightUpdate = options.value("fused_weight_update", compileOptions_.fusedWeightUpdate);
        compileOptions_.skewSharedMemory = options.value("skew_shared_memory", compileOptions_.skewSharedMemory);
        compileOptions_.parallelWeightUpdate =
            options.value("parallel_weight_update", compileOptions_.parallelWeightUpdate);
    }

    //activations
    const json& activationSpecs = cfg.at("activation_specification");
    auto activationFactory = ActivationFactory(activationSpecs, parent, loader);

    //encodings
    const json& encodingSpecs = cfg.at("encodings");
    if (!encodingSpecs.is_array()) throw configuration_error("Illegal type for 'encodings', array expected");
    for (const auto& ecfg : encodingSpecs) {
        auto enc = EncodingFactory::Instance().create(ecfg);
        if (enc->maxInputChannel() >= channelsIn_)
            throw configuration_error("Input channels for encoding '%s' out of bounds (num channels=%d)",
                                      enc->id().c_str(), channelsIn_);
        encodedChannels_ += enc->numOutputChannels();
        encodings_.push_back(enc);
    }
    if (encodings_.empty()) {
        // no encoding given: the raw inputs are the network input
        encodings_.push_back(std::make_shared<EncodingIdentity>(0, channelsIn_));
        encodedChannels_ = channelsIn_;
    }

    //hidden layers
    const json& networkSpecs = cfg.at("network");
    if (!networkSpecs.is_array()) throw configuration_error("Expected a json-array for the network configuration");
    if (networkSpecs.empty()) throw configuration_error("Empty network!");

    // The first layer consumes the concatenated encoding outputs.
    int prevInput = encodedChannels_;
    for (const auto& e : networkSpecs) {
        try {
            LayerSpecification specs;
            specs.channelsIn = prevInput;
            specs.channelsOut = e.at("n_out").get<int>();
            specs.useBias = e.at("bias").get<bool>();
            specs.weightsStart = specs.biasStart = 0;
            if (specs.channelsOut <= 0) throw configuration_error("n_out must be positive, but is %d", specs.channelsOut);

            //either a single activation for all channels or one activation per channel
            const json& ae = e.at("activation");
            if (ae.is_string()) {
                specs.activations.push_back(activationFactory.get(ae.get<std::string>()));
            } else if (ae.is_array()) {
                if (static_cast<int>(ae.size()) != specs.channelsOut)
                    throw configuration_error(
                        "If you specify individual activations per channel, then the number of activations (%d) must match the number of output channels (%d)",
                        static_cast<int>(ae.size()), specs.channelsOut);
                for (const auto& e2 : ae) {
                    if (!e2.is_string()) throw configuration_error("Per-channel activations must be specified as a string");
                    specs.activations.push_back(activationFactory.get(e2.get<std::string>()));
                }
            } else {
                throw configuration_error("Unknown type for the activations, expected string or array");
            }

            prevInput = specs.channelsOut;
            layers_.push_back(specs);
        } catch (...) {
            std::throw_with_nested(configuration_error("Parser error when processing network layer %d",
                                                       static_cast<int>(layers_.size())));
        }
    }
    if (channelsOut_ != prevInput)
        throw configuration_error(
            "The channel count of the last layer (%d) does not match the number of outputs specified at the top of the config file (%d)",
            prevInput, channelsOut_);

    //padding: every width becomes a multiple of the matrix size
    for (size_t i = 0; i < layers_.size(); ++i) {
        const int currentIn = layers_[i].channelsIn;
        const int paddedIn = roundUp(currentIn, MATRIX_SIZE);
        if (currentIn == paddedIn) continue;
        if (i == 0) {
            networkInputPadding_ = paddedIn - currentIn;
            layers_[i].channelsIn = paddedIn;
            logger->warn("need to pad the network input channels from the encodings (%d channels)"
                         " to the next multiple of the matrix size (%d). "
                         "These extra channels are padded with zeros and are thus wasted. Consider increasing the input encoding.",
                         currentIn, paddedIn);
        } else {
            layers_[i].channelsIn = paddedIn;
            layers_[i - 1].channelsOut = paddedIn;
            logger->warn("The hidden channels between layer %d and %d is currently specified to be "
                         "%d channels wide. Matrix multiplications, however, are always performed in multiples of %d "
                         "channels. The network has been automatically increased in size to fit %d channels. "
                         "Consider updating the network specification to reflect this.",
                         static_cast<int>(i) - 1, static_cast<int>(i), currentIn, MATRIX_SIZE, paddedIn);
        }
    }
    {
        const int currentOut = layers_.rbegin()->channelsOut;
        const int paddedOut = roundUp(currentOut, MATRIX_SIZE);
        if (currentOut != paddedOut) {
            layers_.rbegin()->channelsOut = paddedOut;
            logger->debug("the last layer's output (%d channels) is padded to %d channels", currentOut, paddedOut);
        }
    }

    //prefix sum for the offsets of weight + bias: first all weights, then all biases
    numParameters_ = 0;
    for (auto& specs : layers_) {
        specs.weightsStart = numParameters_;
        numParameters_ += specs.channelsIn * specs.channelsOut;
    }
    for (auto& specs : layers_) {
        if (specs.useBias) {
            specs.biasStart = numParameters_;
            numParameters_ += specs.channelsOut;
        } else {
            specs.biasStart = 0;
        }
    }

    //tmp memory layout (channel prefixes; multiplied by the padded batch size at run time)
    backwardInfo_.resize(layers_.size());
    int offsetAdjOut = 0;
    int offsetFwd = layers_[0].channelsIn;   // region 0 of the forward tmp memory: the encoded input
    int offsetIn = 0;
    for (size_t i = 0; i < layers_.size(); ++i) {
        backwardInfo_[i].offsetAdjOut = offsetAdjOut;
        backwardInfo_[i].offsetIn = offsetIn;
        backwardInfo_[i].offsetPre = offsetFwd;
        offsetIn = offsetFwd;
        offsetAdjOut += layers_[i].channelsOut;
        offsetFwd += layers_[i].channelsOut;
    }
    perEntryForwardMemoryBytes_ = offsetFwd * static_cast<int>(sizeof(half));

    for (auto& perFlags : recomputeVerdict_) perFlags[0] = perFlags[1] = -1;
    // behind the intermediates: the position derivatives of the grids whose gradients take the slice kernels
    derivativeOffsets_.assign(encodings_.size(), -1);
    derivativeBytesPerPoint_ = 0;
    if (compileOptions_.inputDerivatives != 0 && hasSliceGradients()) {
        for (size_t i = 0; i < encodings_.size(); ++i) {
            IEncoding::GradientSliceLayout layout;
            if (!offersSlices(*encodings_[i], &layout) || layout.derivativeBytesPerPoint <= 0) continue;
            derivativeOffsets_[i] = derivativeBytesPerPoint_;
            derivativeBytesPerPoint_ += layout.derivativeBytesPerPoint;
        }
    }
}

bool FusedNetwork::recomputesFor(int numel, int flags) const
{
    if (compileOptions_.recomputeIntermediates == 0 || flags <= 0 || flags >= ADJOINT_MODE_MAX_COMBINATIONS) return false;
    if (!(flags & GRADIENTS_NETWORK_WEIGHTS)) return false;
    // the backward kernel of these flags sums the weight gradients of every layer itself ...
    const bool sliceGradients = useSliceGradients(numel, flags);
    for (bool fused : fusedWeightUpdateLayers(flags, sliceGradients))
        if (!fused) return false;
    // ... and has room for the weights in both operand orders and for a second tile per wavefront
    for (int p : weightPlacement(false))
        if (p != WEIGHTS_RESIDENT) return false;
    const int blockSize = forwardBlockSize(compileOptions_.overwriteBlocksizeBackward, true);
    std::vector<LdsGradients> unused;
    const int lds = roundUp(ldsGradientLayout(flags, blockSize, unused, sliceGradients, true), 16)
        + (blockSize / WARP_SIZE) * fusedWeightUpdateTransposeHalves(true) * static_cast<int>(sizeof(half));
    return lds <= MaxSharedMemoryBytes();
}

bool FusedNetwork::recomputes(int numel, int flags)
{
    if (!recomputesFor(numel, flags)) return false;
    const bool sliceGradients = useSliceGradients(numel, flags);
    int& verdict = recomputeVerdict_[flags][sliceGradients ? 1 : 0];
    if (verdict < 0) {
        compileBackwardKernel(flags, sliceGradients, false, true);
        const auto& kernel = backwardKernel_[flags][sliceGradients ? 1 : 0][1].value().adjoint;
        verdict = kernel.fun.scratchBytes() <= MAX_RECOMPUTE_SCRATCH ? 1 : 0;
        if (!verdict)
            QuickMLP::Instance().getLogger()->debug("the backward kernel that runs the layers again (flags %d) spills %d bytes per lane, not used",
                                                    flags, kernel.fun.scratchBytes());
    }
    return verdict == 1;
}

bool FusedNetwork::storesDerivatives(int numel, int flags) const
{
    if (derivativeBytesPerPoint_ <= 0) return false;
    if (compileOptions_.inputDerivatives > 0) return true;
    return (flags & GRADIENTS_INPUT) && useSliceGradients(numel, flags);
}

FusedNetwork::~FusedNetwork()
{
    for (auto& info : backwardInfo_) {
        if (info.stream) qmlp_hip_stream_destroy(info.stream);
        if (info.event) qmlp_hip_event_destroy(info.event);
    }
    if (adjointEvent_) qmlp_hip_event_destroy(adjointEvent_);
}

void FusedNetwork::ensureStreams()
{
    if (streamsCreated_) return;
    for (auto& info : backwardInfo_) {
        qmlp_hip_stream s = nullptr;
        qmlp_hip_event e = nullptr;
        QMLP_HIP_CALL(qmlp_hip_stream_create(&s));
        QMLP_HIP_CALL(qmlp_hip_event_create(&e, 0));
        info.stream = static_cast<stream_t>(s);
        info.event = static_cast<event_t>(e);
    }
    qmlp_hip_event e = nullptr;
    QMLP_HIP_CALL(qmlp_hip_event_create(&e, 0));
    adjointEvent_ = static_cast<event_t>(e);
    streamsCreated_ = true;
}

IEncoding_ptr FusedNetwork::encoding(int idx)
{
    if (idx < 0 || idx >= static_cast<int>(encodings_.size())) throw std::runtime_error("Array index out of bounds");
    return encodings_[idx];
}

int FusedNetwork::networkParameterCount() const { return numParameters_; }

Tensor::Precision FusedNetwork::networkParameterPrecision(Tensor::Usage usage) const
{
    switch (usage) {
    case Tensor::INFERENCE: return Tensor::HALF;
    case Tensor::GRADIENTS: return Tensor::FLOAT;
    default: throw std::runtime_error("Unknown usage");
    }
}

void FusedNetwork::setNetworkParameter(const Tensor& tensor, Tensor::Usage usage)
{
    if (tensor.defined()) {
        if (tensor.ndim() != 1 || tensor.sizes()[0] != numParameters_)
            throw std::runtime_error(format("Illegal tensor shape, 1D tensor with %d entries required", numParameters_));
        if (tensor.precision() != networkParameterPrecision(usage))
            throw std::runtime_error("Wrong data type for the parameter. See parameterPrecision() for the expected format");
        if (tensor.stride(0) != 1) throw std::runtime_error("The network parameters must be contiguous");
        if (reinterpret_cast<uintptr_t>(tensor.rawPtr()) % 16 != 0)
            throw std::runtime_error("The network parameters must be aligned to 16 bytes");
    }
    switch (usage) {
    case Tensor::INFERENCE: parametersInference_ = tensor; break;
    case Tensor::GRADIENTS: parametersGradients_ = tensor; break;
    }
}

void FusedNetwork::initializeInferenceParameters(std::default_random_engine& rng)
{
    if (!parametersInference_.defined())
        throw std::runtime_error("Inference parameters not defined, call setNetworkParameter(...) first");

    std::vector<half> dataHost(static_cast<size_t>(parametersInference_.numel()), static_cast<half>(0));
    for (int layer = 0; layer < numLayers(); ++layer) {
        const auto& l = layers_[layer];
        // std::sqrt of an int is evaluated in double, as in the reference (fused_network.cpp:294)
        const float bound = static_cast<float>(1.0f / std::sqrt(static_cast<double>(l.channelsIn)));
        std::uniform_real_distribution<float> distr1(-bound, +bound);
        Tensor weights = networkParameter(layer, false, dataHost.data(), Tensor::HALF);
        for (int32_t i = 0; i < weights.size(0); ++i)
            for (int32_t j = 0; j < weights.size(1); ++j)
                weights.dataPtr<half>()[weights.idx({i, j})] = static_cast<half>(distr1(rng));
        if (l.useBias) {
            Tensor bias = networkParameter(layer, true, dataHost.data(), Tensor::HALF);
            for (int32_t i = 0; i < bias.size(0); ++i) bias.dataPtr<half>()[bias.idx({i})] = static_cast<half>(distr1(rng));
        }
    }
    parametersInference_.copyFromHost(dataHost.data(), dataHost.size() * sizeof(half));
}

Tensor FusedNetwork::networkParameter(int layer, bool bias, void* rawPtr, Tensor::Precision precision)
{
    if (layer < 0 || layer >= static_cast<int>(layers_.size())) throw std::runtime_error("Layer index out of bounds");
    const auto& l = layers_[layer];
    int8_t* data = static_cast<int8_t*>(rawPtr);
    const int bytesPerEntry = Tensor::BytesPerEntry[precision];
    if (bias) {
        if (!l.useBias) return {};
        return Tensor(data + static_cast<ptrdiff_t>(bytesPerEntry) * l.biasStart, precision, {l.channelsOut}, {1});
    }
    //row-major
    return Tensor(data + static_cast<ptrdiff_t>(bytesPerEntry) * l.weightsStart, precision,
                  {l.channelsOut, l.channelsIn}, {l.channelsIn, 1});
}

Tensor FusedNetwork::networkParameter(int layer, bool bias, Tensor::Usage usage)
{
    auto& p = usage == Tensor::INFERENCE ? parametersInference_ : parametersGradients_;
    return networkParameter(layer, bias, p.rawPtr(), p.precision());
}

// ------------------------------------------------------------------ code generation

void FusedNetwork::fillEncodingsAndActivations(std::string& codeTemplate) const
{
    std::stringstream encodingIncludes;
    std::stringstream encodingParameters;
    for (size_t encodingIdx = 0; encodingIdx < encodings_.size(); ++encodingIdx) {
        const auto& e = encodings_[encodingIdx];
        e->fillCode(encodingIncludes);
        encodingIncludes << "\n";
        if (e->hasParameters())
            encodingParameters << ",\n    const " << e->parameterName() << " cEncoding" << encodingIdx;
    }
    replaceAll(codeTemplate, "$$INCLUDES$$", encodingIncludes.str());
    replaceAll(codeTemplate, "$$ENCODING_PARAMETERS$$", encodingParameters.str());

    replaceAll(codeTemplate, "$$DEFINE_ACTIVATIONS$$", activationDefinitions());

    replaceAll(codeTemplate, "$$NUM_INPUTS$$", std::to_string(channelsIn_));
    replaceAll(codeTemplate, "$$ENCODED_CHANNELS$$", std::to_string(encodedChannels_));
    replaceAll(codeTemplate, "$$CHANNELS_IN$$", std::to_string(layers_.begin()->channelsIn));
    replaceAll(codeTemplate, "$$CHANNELS_OUT$$", std::to_string(layers_.rbegin()->channelsOut));
}

static int ldsWeightHalves(int channelsIn, int channelsOut, bool adjoint)
{
    // matrix-core operand order, contraction width padded to 32 channels
    return adjoint ? channelsIn * roundUp(channelsOut, 32) : channelsOut * roundUp(channelsIn, 32);
}

std::vector<int> FusedNetwork::weightPlacement(bool adjoint) const
{
    const int L = static_cast<int>(layers_.size());
    std::vector<int> placement(L, WEIGHTS_RESIDENT);
    std::vector<long long> bytes(L);
    long long total = 0, biases = 0;
    for (int i = 0; i < L; ++i) {
        bytes[i] = static_cast<long long>(ldsWeightHalves(layers_[i].channelsIn, layers_[i].channelsOut, adjoint)) * sizeof(half);
        total += bytes[i];
        if (!adjoint && layers_[i].useBias) biases += layers_[i].channelsOut * sizeof(half);
    }
    const long long maxLds = MaxSharedMemoryBytes();
    // everything stays if four wavefronts still find room for their staging tiles
    if (total + biases + 16 + 4ll * stageBytesPerWave(adjoint) <= maxLds) return placement;

    // Otherwise the workgroup shares a stream buffer as large as the largest streamed layer; of
    // the layers that fit into such a buffer, the subset with the most bytes that still fits
    // beside it stays resident. Room is left for the staging tiles of eight wavefronts, or of
    // four if that lets a layer be streamed that would otherwise have to be read from global
    // memory by every wavefront.
    auto place = [&](int waves, std::vector<int>& out) {
        out.assign(L, WEIGHTS_RESIDENT);
        const long long budget = maxLds - biases - 16 - static_cast<long long>(waves) * stageBytesPerWave(adjoint);
        std::vector<int> candidates;
        int numGlobal = 0;
        for (int i = 0; i < L; ++i) {
            if (bytes[i] > budget) {
                out[i] = WEIGHTS_GLOBAL;
                ++numGlobal;
            } else {
                candidates.push_back(i);
            }
        }
        const int C = static_cast<int>(candidates.size());
        long long best = -1;
        unsigned bestMask = 0;
        const unsigned numMasks = C <= 16 ? (1u << C) : 1u;   // many layers: stream them all
        for (unsigned mask = 0; mask < numMasks; ++mask) {
            long long resident = 0, stream = 0;
            for (int k = 0; k < C; ++k) {
                if (mask & (1u << k)) resident += bytes[candidates[k]];
                else stream = std::max(stream, bytes[candidates[k]]);
            }
            if (resident + stream <= budget && resident > best) {
                best = resident;
                bestMask = mask;
            }
        }
        for (int k = 0; k < C; ++k) out[candidates[k]] = (bestMask >> k) & 1 ? WEIGHTS_RESIDENT : WEIGHTS_STREAMED;
        return numGlobal;
    };
    const int globalWithEight = place(8, placement);
    if (globalWithEight > 0) {
        std::vector<int> withFour;
        if (place(4, withFour) < globalWithEight) placement = withFour;
    }
    return placement;
}

int FusedNetwork::ldsLayout(bool adjoint, std::vector<int>& weightOffsets, std::vector<int>& biasOffsets,
                            int* streamOffset) const
{
    // Weights sit in LDS in matrix-core operand order, contraction width padded to 32
    // channels (forward: C_in, adjoint: C_out); the biases follow (forward only).
    weightOffsets.assign(layers_.size(), -1);
    biasOffsets.assign(layers_.size(), 0);
    const auto placement = weightPlacement(adjoint);
    int n = 0, streamHalves = 0;
    for (size_t i = 0; i < layers_.size(); ++i) {
        const auto& l = layers_[i];
        const int halves = ldsWeightHalves(l.channelsIn, l.channelsOut, adjoint);
        if (placement[i] == WEIGHTS_STREAMED) streamHalves = std::max(streamHalves, halves);
        if (placement[i] != WEIGHTS_RESIDENT) continue;
        weightOffsets[i] = n;
        n += halves;
    }
    if (!adjoint) {
        for (size_t i = 0; i < layers_.size(); ++i) {
            if (!layers_[i].useBias) continue;
            biasOffsets[i] = n;
            n += layers_[i].channelsOut;
        }
    }
    n = roundUp(n, 8);
    if (streamOffset) *streamOffset = streamHalves > 0 ? n : -1;
    for (size_t i = 0; i < layers_.size(); ++i)
        if (placement[i] == WEIGHTS_STREAMED) weightOffsets[i] = n;
    return roundUp(n + streamHalves, 8);
}

size_t FusedNetwork::transposedWeightLayout(int adjointFlags, std::vector<long long>& offsets) const
{
    offsets.assign(layers_.size(), -1);
    const auto placement = weightPlacement(true);
    const bool needsEncodingAdjoint = adjointFlags & (GRADIENTS_INPUT | GRADIENTS_INPUT_ENCODINGS);
    size_t n = 0;
    for (size_t i = 0; i < layers_.size(); ++i) {
        if (placement[i] != WEIGHTS_GLOBAL || (i == 0 && !needsEncodingAdjoint)) continue;
        offsets[i] = static_cast<long long>(n);
        n += static_cast<size_t>(layers_[i].channelsIn) * layers_[i].channelsOut;
    }
    return n;
}

std::string FusedNetwork::activationTypeName(int layer) const
{
    const auto& a = layers_[layer].activations;
    return a.size() == 1 ? a[0]->id() : "mixed_layer" + std::to_string(layer) + "_";
}

std::string FusedNetwork::activationDefinitions() const
{
    std::stringstream ss;
    std::unordered_set<std::string> ids;
    for (const auto& l : layers_)
        for (const auto& a : l.activations)
            if (ids.insert(a->id()).second) ss << a->code() << "\n";
    // One activation per output channel (the reference parses such lists and then rejects them,
    // fused_network.cpp:112-125,447): a composite that dispatches on the channel. Channels of
    // the padding use the activation of the last listed channel.
    for (size_t layer = 0; layer < layers_.size(); ++layer) {
        const auto& l = layers_[layer];
        if (l.activations.size() == 1) continue;
        std::vector<std::string> kinds;
        std::vector<int> kindOfChannel;
        for (const auto& a : l.activations) {
            auto it = std::find(kinds.begin(), kinds.end(), a->id());
            if (it == kinds.end()) {
                kinds.push_back(a->id());
                it = kinds.end() - 1;
            }
            kindOfChannel.push_back(static_cast<int>(it - kinds.begin()));
        }
        while (static_cast<int>(kindOfChannel.size()) < l.channelsOut) kindOfChannel.push_back(kindOfChannel.back());
        ss << "struct " << activationTypeName(static_cast<int>(layer)) << "\n{\n"
           << "    static constexpr bool PerChannel = true;\n"
           << "    static __device__ __forceinline__ int kind(int channel) {\n"
           << "        constexpr unsigned char kinds[" << kindOfChannel.size() << "] = {";
        for (size_t i = 0; i < kindOfChannel.size(); ++i) ss << (i ? "," : "") << kindOfChannel[i];
        ss << "};\n        return kinds[channel];\n    }\n"
           << "    static __device__ __forceinline__ half forwardAt(half x, int channel) {\n        switch (kind(channel)) {\n";
        for (size_t k = 0; k + 1 < kinds.size(); ++k)
            ss << "        case " << k << ": return " << kinds[k] << "::forward(x);\n";
        ss << "        default: return " << kinds.back() << "::forward(x);\n        }\n    }\n"
           << "    static __device__ __forceinline__ half adjointAt(half x, half adjz, int channel) {\n        switch (kind(channel)) {\n";
        for (size_t k = 0; k + 1 < kinds.size(); ++k)
            ss << "        case " << k << ": return " << kinds[k] << "::adjoint(x, adjz);\n";
        ss << "        default: return " << kinds.back() << "::adjoint(x, adjz);\n        }\n    }\n};\n";
    }
    return ss.str();
}

int FusedNetwork::ldsParamHalves(bool adjoint) const
{
    std::vector<int> w, b;
    return ldsLayout(adjoint, w, b);
}

std::string FusedNetwork::kernelAttributes(int blockSize) const
{
    // a workgroup of 8 wavefronts has that budget anyway
    if (blockSize >= 2 * DEFAULT_BLOCK_SIZE) return "";
    // Two wavefronts per SIMD at least: the register budget is then 256, all of them vector
    // registers, and the compiler keeps the matrix-core accumulators there (with up to 512 it
    // puts them into accumulation registers and copies every value out one by one). Layers
    // wider than 128 need more than 256 registers and keep the larger budget.
    int widest = 0;
    for (const auto& l : layers_) widest = std::max(widest, std::max(l.channelsIn, l.channelsOut));
    return widest <= 128 ? "__attribute__((amdgpu_waves_per_eu(2)))" : "";
}

int FusedNetwork::directInputStart() const
{
    if (!compileOptions_.directInput || encodings_.size() != 1) return -1;
    const auto* identity = dynamic_cast<const EncodingIdentity*>(encodings_[0].get());
    return identity ? identity->startChannel() : -1;
}

int FusedNetwork::stageBytesPerWave(bool adjoint) const
{
    // operands straight from the input rows: the forward kernel stages nothing
    if (!adjoint && directInputStart() >= 0) return 0;
    // the forward kernel rotates the chunks of rows of 32, 64 or 128 halves instead of padding them
    const int c = layers_[0].channelsIn;
    const bool rotated = !adjoint && (c == 32 || c == 64 || c == 128);
    return TILE_POINTS * (c + (rotated ? 0 : STAGE_PAD)) * static_cast<int>(sizeof(half));
}

int FusedNetwork::forwardBlockSize(int overwrite, bool adjoint, int* pointsPerLane, int fixedPointsPerLane) const
{
    int blockSize = DEFAULT_BLOCK_SIZE;
    if (overwrite > 0) {
        if (overwrite % WARP_SIZE != 0 || overwrite > 1024)
            throw configuration_error("The block size must be a multiple of %d and at most 1024, but is %d", WARP_SIZE,
                                      overwrite);
        blockSize = overwrite;
    }
    const int maxLds = MaxSharedMemoryBytes();
    const int paramBytes = ldsParamHalves(adjoint) * static_cast<int>(sizeof(half));
    if (paramBytes + stageBytesPerWave(adjoint) > maxLds)
        throw configuration_error("The network is too large for the fused kernels: its %d parameters plus one staging "
                                  "tile need %d bytes of LDS, the device offers %d",
                                  numParameters_, paramBytes + stageBytesPerWave(adjoint), maxLds);
    while (paramBytes + (blockSize / WARP_SIZE) * stageBytesPerWave(adjoint) > maxLds) blockSize -= WARP_SIZE;
    int ppl = 1;
    if (pointsPerLane) {
        // Grid encodings gather level by level over several points per lane; two workgroups
        // should still fit on a compute unit.
        bool gathers = false;
        for (const auto& e : encodings_) gathers = gathers || e->hasParameters();
        const int fixed = fixedPointsPerLane > 0 ? fixedPointsPerLane : compileOptions_.pointsPerLane;
        ppl = fixed > 0 ? fixed : (gathers ? 2 : 1);
        const int budget = fixed > 0 ? maxLds : maxLds / 2;
        while (ppl > 1 && paramBytes + (blockSize / WARP_SIZE) * ppl * stageBytesPerWave(adjoint) > budget) --ppl;
        *pointsPerLane = ppl;
    }
    if (overwrite <= 0) {
        // The weights in LDS are per workgroup: when they are large, a workgroup of 8 wavefronts
        // brings more wavefronts onto a compute unit than two of 4 would.
        auto wavesPerComputeUnit = [&](int block) {
            const int lds = paramBytes + (block / WARP_SIZE) * ppl * stageBytesPerWave(adjoint);
            if (lds > maxLds) return 0;
            return std::min(16, (maxLds / lds) * (block / WARP_SIZE));
        };
        // Input and output activations of a layer live in registers: one VGPR per channel each.
        // Above 128 channels a wave needs more than the 256 registers it gets in a workgroup
        // of 8 wavefronts.
        int widest = 0;
        for (const auto& l : layers_) widest = std::max(widest, std::max(l.channelsIn, l.channelsOut));
        if (widest <= 128 && wavesPerComputeUnit(2 * DEFAULT_BLOCK_SIZE) > wavesPerComputeUnit(blockSize))
            blockSize = 2 * DEFAULT_BLOCK_SIZE;
    }
    return blockSize;
}

int FusedNetwork::weightUpdateBlockSize() const
{
    int blockSize = DEFAULT_BLOCK_SIZE;
    if (compileOptions_.overwriteBlocksizeWeightUpdate > 0) {
        blockSize = compileOptions_.overwriteBlocksizeWeightUpdate;
        if (blockSize % WARP_SIZE != 0 || blockSize > 1024)
            throw configuration_error("The block size must be a multiple of %d and at most 1024, but is %d", WARP_SIZE, blockSize);
    }
    return blockSize;
}

int FusedNetwork::weightUpdateSlices(int numTiles) const
{
    const int waves = weightUpdateBlockSize() / WARP_SIZE;
    return std::max(1, std::min(divUp(numTiles, waves), MAX_WEIGHT_UPDATE_SLICES));
}

std::vector<bool> FusedNetwork::fusedWeightUpdateLayers(int adjointFlags, bool sliceGradients, bool* wideRegisters) const
{
    std::vector<bool> fused(layers_.size(), false);
    if (wideRegisters) *wideRegisters = false;
    if (compileOptions_.fusedWeightUpdate == 0 || !(adjointFlags & GRADIENTS_NETWORK_WEIGHTS)) return fused;
    // a backward kernel that gathers from or scatters into the tables of an encoding itself has no registers to spare
    // (32 -> 64 -> 64 -> 16 behind a hash grid: 320 bytes of scratch per lane without any gradient tile)
    for (const auto& e : encodings_) {
        if (!e->hasParameters() || !(adjointFlags & (GRADIENTS_INPUT | GRADIENTS_INPUT_ENCODINGS))) continue;
        if (!(sliceGradients && (adjointFlags & GRADIENTS_INPUT_ENCODINGS) && offersSlices(*e))) return fused;
    }
    for (int p : weightPlacement(true))
        if (p != WEIGHTS_RESIDENT) return fused;
    // a workgroup of 8 wavefronts leaves 128 registers to each: none to spare; nor do layers of more than 64
    // channels, whose activations fill 64 registers and more (16 -> 128 -> 64 -> 48 -> 16 with sine activations
    // and workgroups of 4 wavefronts: a train step of 1.27 instead of 0.67 ms with two layers summed in the kernel)
    const int blockSize = forwardBlockSize(compileOptions_.overwriteBlocksizeBackward, true);
    if (blockSize != DEFAULT_BLOCK_SIZE) return fused;
    for (const auto& l : layers_)
        if (std::max(l.channelsIn, l.channelsOut) > 64) return fused;
    // room for the transposed tiles beside the weights and staging rows (32 KiB are kept for the gradients of a coarse grid level)
    const int lds = ldsParamHalves(true) * static_cast<int>(sizeof(half))
        + (blockSize / WARP_SIZE) * (stageBytesPerWave(true) + fusedWeightUpdateTransposeHalves() * static_cast<int>(sizeof(half)));
    if (lds + 32 * 1024 > MaxSharedMemoryBytes()) return fused;
    // Four accumulator registers per gradient tile and lane, for as long as the kernel runs: the layers with the
    // fewest tiles first, up to 16 tiles (all 28 tiles of a 32 -> 64 -> 64 -> 16 network: 1 KB of scratch per lane
    // and a backward kernel of 116 instead of 31 us; the weight-update kernels it replaced took 62 us).
    int budget = compileOptions_.fusedWeightUpdate > 0 ? 32 : 16;
    std::vector<std::pair<int, int>> byTiles;
    int allTiles = 0;
    for (size_t i = 0; i < layers_.size(); ++i) {
        const int mt = layers_[i].channelsOut / MATRIX_SIZE, kt = layers_[i].channelsIn / MATRIX_SIZE;
        byTiles.push_back({mt * kt + (layers_[i].useBias ? 1 : 0), static_cast<int>(i)});   // the bias sums share a tile
        allTiles += byTiles.back().first;
    }
    // One wavefront per SIMD has 512 registers, half of them accumulation registers, where gradient tiles that are
    // only read once at the end of the kernel cost nothing: taken where that fuses *every* layer (no weight-update
    // kernel and no stored adjoints remain) and 16 tiles did not -- the kernel then runs half as many wavefronts.
    // Measured, backward + weight updates: 32 -> 64 -> 64 -> 16 (28 tiles) 39 + 25 -> 51 us; forward + backward of
    // 64 -> 64 -> 64 -> 16 (36 tiles) on 10^6 points 530 -> 505 us. Networks that 16 tiles fuse completely lose
    // 8-14 % with one wavefront per SIMD, 64 x 4 hidden layers (68 tiles, partly fused) gain nothing, and where 16
    // tiles leave out only a small layer (32 x 4 hidden layers: 16 of 18 tiles) the smaller kernel stays ahead
    // (forward + backward 300 against 317 us) -- unless the kernel that holds every tile may also run the layers
    // again, so that the training pass stores the encoded input only (layers of up to 32 channels, whose
    // pre-activations fit beside the tiles: 32 x 4 hidden layers 300 -> 230 us).
    std::sort(byTiles.begin(), byTiles.end());
    int within = 0;
    for (const auto& [count, layer] : byTiles) {
        if (within + count > budget) break;
        within += count;
    }
    if (wideRegisters) *wideRegisters = false;
    int widest = 0;
    for (const auto& l : layers_) widest = std::max(widest, std::max(l.channelsIn, l.channelsOut));
    const bool runsLayersAgain = compileOptions_.recomputeIntermediates != 0 && widest <= 32 && allTiles > within;
    if (compileOptions_.fusedWeightUpdate < 0 && allTiles <= 48 && (allTiles - within >= 12 || runsLayersAgain)) {
        budget = allTiles;
        if (wideRegisters) *wideRegisters = true;
    }
    int tiles = 0;
    for (const auto& [count, layer] : byTiles) {
        if (tiles + count > budget) break;
        tiles += count;
        fused[layer] = true;
    }
    return fused;
}

int FusedNetwork::fusedWeightUpdateTransposeHalves(bool recompute) const
{
    int widest = 0, widestIn = 0;
    for (const auto& l : layers_) {
        widest = std::max(widest, l.channelsOut);
        widestIn = std::max(widestIn, l.channelsIn);
    }
    // Layer::T_HALVES; behind it, where the layers run again in the backward kernel, the tile of a layer's input
    return (widest + (recompute ? widestIn : 0)) * (TILE_POINTS + 8);
}

int FusedNetwork::storedAdjointChannels(int adjointFlags, bool sliceGradients) const
{
    if (!(adjointFlags & GRADIENTS_NETWORK_WEIGHTS)) return 0;
    // (the regions of the layers keep their places while any of them is stored)
    bool allFused = true;
    for (bool f : fusedWeightUpdateLayers(adjointFlags, sliceGradients)) allFused = allFused && f;
    if (allFused) return 0;
    int channels = 0;
    for (const auto& l : layers_) channels += l.channelsOut;
    return channels;
}

static std::string layerTypedefs(const std::vector<std::string>& layerTypes)
{
    std::stringstream ss;
    for (size_t i = 0; i < layerTypes.size(); ++i) ss << "    typedef " << layerTypes[i] << " Layer" << i << ";\n";
    return ss.str();
}

std::string FusedNetwork::forwardSource(int blockSize, int pointsPerLane, bool registerStaging, bool derivatives, bool inputOnly) const
{
    auto kl = QuickMLP::Instance().kernelLoader();
    std::string code = kl->findFile("qmlp/kernels/network_forward.h").value();
    fillEncodingsAndActivations(code);
    replaceAll(code, "$$BLOCK_SIZE$$", std::to_string(blockSize));
    replaceAll(code, "$$POINTS_PER_LANE$$", std::to_string(pointsPerLane));
    replaceAll(code, "$$REGISTER_STAGING$$", registerStaging ? "true" : "false");
    replaceAll(code, "$$DIRECT_INPUT_START$$", std::to_string(directInputStart()));
    replaceAll(code, "$$KERNEL_ATTRIBUTES$$", kernelAttributes(blockSize));
    // rows in registers are indexed by the tile: that loop has to be unrolled
    replaceAll(code, "$$TILE_LOOP_PRAGMA$$", registerStaging ? "#pragma unroll" : "#pragma unroll 1");
    std::vector<int> ldsW, ldsB;
    int streamOffset = -1;
    replaceAll(code, "$$LDS_PARAM_HALVES$$", std::to_string(ldsLayout(false, ldsW, ldsB, &streamOffset)));
    replaceAll(code, "$$HAS_STREAMED_LAYERS$$", streamOffset >= 0 ? "true" : "false");
    const auto placement = weightPlacement(false);

    std::vector<std::string> layerTypes;
    for (const auto& l : layers_) {
        layerTypes.push_back(format("Layer<%d, %d, %s, activations::%s>", l.channelsIn, l.channelsOut,
                                    l.useBias ? "true" : "false",
                                    activationTypeName(static_cast<int>(&l - layers_.data())).c_str()));
    }

    std::stringstream stage;
    stage << layerTypedefs(layerTypes);
    for (size_t i = 0; i < layers_.size(); ++i) {
        const auto& l = layers_[i];
        if (placement[i] == WEIGHTS_RESIDENT)
            stage << "    Layer" << i << "::stageForward(networkParameters + " << l.weightsStart << ", sParams + "
                  << ldsW[i] << ", threadIdx.x, blockDim.x);\n";
        if (l.useBias)
            stage << "    for (int i = threadIdx.x; i < " << l.channelsOut << "; i += blockDim.x) sParams["
                  << ldsB[i] << " + i] = networkParameters[" << l.biasStart << " + i];\n";
    }
    replaceAll(code, "$$STAGE_PARAMETERS$$", stage.str());

    std::stringstream callEncodings;
    int encodingOffset = 0;
    replaceAll(code, "$$ENCODING_OUTPUT_ROWS$$",
               registerStaging ? "PackedRegisterRowsView<f16, PPL, CHANNELS_IN, 0> encodingOutput{encodedRegisters};"
                               : "StageRowArray<f16, CHANNELS_IN> encodingOutput[PPL];");
    for (size_t encodingIdx = 0; encodingIdx < encodings_.size(); ++encodingIdx) {
        const auto& e = encodings_[encodingIdx];
        if (registerStaging)
            callEncodings << "            {\n                PackedRegisterRowsView<f16, PPL, CHANNELS_IN, " << encodingOffset
                          << "> encodingOutputK{encodedRegisters};\n                ";
        else
            callEncodings << "            {\n                StageRowArray<f16, CHANNELS_IN> encodingOutputK[PPL];\n"
                          << "#pragma unroll\n                for (int q = 0; q < PPL; ++q) encodingOutputK[q] = encodingOutput[q] + "
                          << encodingOffset << ";\n                ";
        IEncoding::GradientSliceLayout sliceLayout;
        if (derivatives && derivativeOffsets_[encodingIdx] >= 0 && offersSlices(*e, &sliceLayout)) {
            // the lane's chunks of its first tile; the tiles of a wave follow one another
            callEncodings << "static_assert(STORE && DERIVATIVES, \"this source is that of the training pass that keeps position derivatives\");\n"
                          << "                typedef PositionDerivativeLayout<" << sliceLayout.configType << "> DerivativeLayout;\n"
                          << "                StorePositionDerivatives<" << sliceLayout.configType << "> derivatives{\n"
                          << "                    reinterpret_cast<DerivativeLayout::chunk_t*>(reinterpret_cast<unsigned char*>(forwardTmpMemoryH) + "
                          << (static_cast<long long>(perEntryForwardMemoryBytes_) + derivativeOffsets_[encodingIdx]) << "ll * numel64)\n"
                          << "                        + DerivativeLayout::chunkIndex(tile0 + tmpTileOffset, 0, 0, lane),\n"
                          << "                    numTiles - tile0};\n                ";
            callEncodings << e->qualifiedName() << "::template forwardBatch<PPL>(encodingInput, encodingOutputK, cEncoding" << encodingIdx
                          << ", derivatives);\n            }\n";
        } else {
            callEncodings << e->qualifiedName() << "::template forwardBatch<PPL>(encodingInput, encodingOutputK";
            if (e->hasParameters()) callEncodings << ", cEncoding" << encodingIdx;
            callEncodings << ");\n            }\n";
        }
        encodingOffset += e->numOutputChannels();
    }
    replaceAll(code, "$$CALL_ENCODINGS$$", callEncodings.str());

    std::stringstream callLayers;
    for (size_t i = 0; i < layers_.size(); ++i) {
        const auto& l = layers_[i];
        callLayers << "        f16x4 x" << (i + 1) << "[NT][Layer" << i << "::MT];\n";
        if (placement[i] == WEIGHTS_STREAMED)
            callLayers << "        materialize(x" << i << ");\n        __syncthreads();   // the stream buffer is free\n        Layer" << i
                       << "::stageForward(networkParameters + " << l.weightsStart << ", sParams + " << ldsW[i]
                       << ", threadIdx.x, blockDim.x);\n        __syncthreads();\n";
        // (inputOnly: of the intermediates a training pass keeps the encoded input only; the backward kernel runs the layers again)
        const char* storeLayer = inputOnly ? "false" : "STORE";
        if (placement[i] != WEIGHTS_GLOBAL)
            callLayers << "        Layer" << i << "::template forward<" << storeLayer << ", false, HAS_STREAMED_LAYERS>(sParams + " << ldsW[i] << ", ";
        else
            callLayers << "        Layer" << i << "::template forward<" << storeLayer << ", true, HAS_STREAMED_LAYERS>(networkParameters + " << l.weightsStart
                       << ", ";
        if (l.useBias)
            callLayers << "sParams + " << ldsB[i];
        else
            callLayers << "nullptr";
        callLayers << ", x" << i << ", x" << (i + 1) << ",\n            (STORE && tileValid) ? forwardTmpMemory + ("
                   << backwardInfo_[i].offsetPre << "ll * numel64 + static_cast<long long>(tmpTile) * ("
                   << l.channelsOut << " * TILE_POINTS)) : nullptr, lane);\n";
    }
    callLayers << "        auto& xOut = x" << layers_.size() << ";\n";
    replaceAll(code, "$$CALL_NETWORK_LAYERS$$", callLayers.str());
    return code;
}

bool FusedNetwork::hasSliceGradients() const
{
    if (compileOptions_.sliceGradients == 0) return false;
    for (const auto& e : encodings_)
        if (offersSlices(*e)) return true;
    return false;
}

int FusedNetwork::sliceGradientBytesPerPoint() const
{
    // the adjoint of the encoded rows, which the records kernels of the grids read
    return hasSliceGradients() ? layers_[0].channelsIn * static_cast<int>(sizeof(half)) : 0;
}

size_t FusedNetwork::sliceGradientWorkspaceBytes(long long numel) const
{
    if (!hasSliceGradients()) return 0;
    size_t bytes = 0;
    for (const auto& e : encodings_) {
        IEncoding::GradientSliceLayout layout;
        if (!offersSlices(*e, &layout)) continue;
        bytes += roundUp(static_cast<size_t>(layout.numBuckets() + 1) * sizeof(int), size_t(256));   // cursors, largest adjoint
        bytes += roundUp(static_cast<size_t>(layout.totalRecords(numel)) * layout.recordWords * sizeof(uint32_t), size_t(256));
    }
    return bytes;
}

bool FusedNetwork::useSliceGradients(int numel, int flags) const
{
    if (!(flags & GRADIENTS_INPUT_ENCODINGS) || !hasSliceGradients()) return false;
    if (compileOptions_.sliceGradients > 0 || numel >= SLICE_GRADIENTS_MIN_BATCH) return true;
    if (numel < SLICE_GRADIENTS_MIN_BATCH_MANY_LEVELS) return false;
    for (const auto& e : encodings_) {
        IEncoding::GradientSliceLayout layout;
        if (offersSlices(*e, &layout) && layout.slicesPerLevel.size() >= 8) return true;
    }
    return false;
}

int FusedNetwork::ldsGradientLayout(int adjointFlags, int blockSize, std::vector<LdsGradients>& perEncoding, bool sliceGradients,
                                    bool recompute) const
{
    perEncoding.assign(encodings_.size(), LdsGradients{});
    // (recompute: the weights in forward operand order and the biases behind the transposed weights)
    int bytes = (ldsParamHalves(true) + (recompute ? ldsParamHalves(false) : 0)) * static_cast<int>(sizeof(half))
        + (blockSize / WARP_SIZE) * stageBytesPerWave(true);
    if (!(adjointFlags & GRADIENTS_INPUT_ENCODINGS)) return bytes;
    // Up to 96 KiB of LDS per workgroup in total: a coarse level of a grid fits (16^3 cells with
    // 2 features: 32 KiB), and a second workgroup per compute unit stays possible.
    const int limit = std::min(MaxSharedMemoryBytes(), 96 * 1024);
    for (size_t i = 0; i < encodings_.size(); ++i) {
        if (!encodings_[i]->hasParameters()) continue;
        if (sliceGradients && offersSlices(*encodings_[i])) continue;   // summed by the slice kernel, not here
        bytes = roundUp(bytes, 16);
        LdsGradients g;
        g.floats = encodings_[i]->ldsGradientFloats(limit - bytes, g.levels);
        if (g.floats <= 0) continue;
        g.byteOffset = bytes;
        bytes += g.floats * static_cast<int>(sizeof(float));
        perEncoding[i] = g;
    }
    return bytes;
}

std::string FusedNetwork::backwardSource(int flags, int blockSize, bool sliceGradients, bool recompute, bool twoWavefrontsPerSimd) const
{
    const bool hasInputGradients = flags & GRADIENTS_INPUT;
    const bool hasNetworkGradients = flags & GRADIENTS_NETWORK_WEIGHTS;
    const bool hasEncodingGradients = flags & GRADIENTS_INPUT_ENCODINGS;

    auto kl = QuickMLP::Instance().kernelLoader();
    std::string code = kl->findFile("qmlp/kernels/network_backward.h").value();
    fillEncodingsAndActivations(code);
    replaceAll(code, "$$BLOCK_SIZE$$", std::to_string(blockSize));
    replaceAll(code, "$$HAS_OUTPUT_ORDER$$", trainsSortedBatches() ? "1" : "0");
    bool wideRegisters = false;
    (void)fusedWeightUpdateLayers(flags, sliceGradients, &wideRegisters);
    // (the pre-activations of all layers stay in registers beside the gradient tiles: 256 registers spilled 404 bytes
    // per lane for 16 -> 32 -> 32 -> 32 -> 16 with the run-time compiler that ships with torch 2.10; the offline compiler of
    // ROCm 7.2 needs 232 registers and no scratch for the same source, see compileBackwardKernel)
    wideRegisters = (wideRegisters || recompute) && !twoWavefrontsPerSimd;
    replaceAll(code, "$$KERNEL_ATTRIBUTES$$", wideRegisters ? std::string("__attribute__((amdgpu_waves_per_eu(1, 1)))") : kernelAttributes(blockSize));
    // (set below: input gradients that the kernels of the gradient slices compute are none of this kernel's)
    replaceAll(code, "$$HAS_NETWORK_GRADIENTS$$", hasNetworkGradients ? "true" : "false");
    replaceAll(code, "$$HAS_ENCODING_GRADIENTS$$", hasEncodingGradients ? "true" : "false");
    std::vector<int> ldsW, ldsB;
    int streamOffset = -1;
    const int adjointParamHalves = ldsLayout(true, ldsW, ldsB, &streamOffset);
    // recompute: the weights in forward operand order and the biases, behind the transposed weights
    std::vector<int> ldsWForward, ldsBForward;
    const int forwardParamHalves = recompute ? ldsLayout(false, ldsWForward, ldsBForward) : 0;
    replaceAll(code, "$$LDS_PARAM_HALVES$$", std::to_string(adjointParamHalves + forwardParamHalves));
    const auto placement = weightPlacement(true);

    std::vector<std::string> layerTypes;
    for (const auto& l : layers_) {
        layerTypes.push_back(format("Layer<%d, %d, %s, activations::%s>", l.channelsIn, l.channelsOut,
                                    l.useBias ? "true" : "false",
                                    activationTypeName(static_cast<int>(&l - layers_.data())).c_str()));
    }

    // the first layer's transposed weights are only needed when something consumes dX0
    const bool needsEncodingAdjoint = hasInputGradients || hasEncodingGradients;
    std::stringstream stage;
    stage << layerTypedefs(layerTypes);
    for (size_t i = 0; i < layers_.size(); ++i) {
        if ((i == 0 && !needsEncodingAdjoint) || placement[i] != WEIGHTS_RESIDENT) continue;
        const auto& l = layers_[i];
        stage << "    Layer" << i << "::stageAdjoint(networkParameters + " << l.weightsStart << ", sParams + "
              << ldsW[i] << ", threadIdx.x, blockDim.x);\n";
    }
    if (recompute) {
        for (size_t i = 0; i < layers_.size(); ++i) {
            const auto& l = layers_[i];
            stage << "    Layer" << i << "::stageForward(networkParameters + " << l.weightsStart << ", sParams + "
                  << (adjointParamHalves + ldsWForward[i]) << ", threadIdx.x, blockDim.x);\n";
            if (l.useBias)
                stage << "    for (int i = threadIdx.x; i < " << l.channelsOut << "; i += blockDim.x) sParams["
                      << (adjointParamHalves + ldsBForward[i]) << " + i] = networkParameters[" << l.biasStart << " + i];\n";
        }
    }
    replaceAll(code, "$$STAGE_PARAMETERS$$", stage.str());

    std::vector<long long> transposed;
    transposedWeightLayout(flags, transposed);
    std::stringstream callLayers, declareGradients, storeGradients;
    const std::vector<bool> fusedLayers = fusedWeightUpdateLayers(flags, sliceGradients);
    bool anyFused = false;
    for (bool f : fusedLayers) anyFused = anyFused || f;
    const int L = static_cast<int>(layers_.size());
    bool anyStreamed = false;
    for (int i = L - 1; i >= 0; --i) {
        const auto& l = layers_[i];
        const std::string dy = (i == L - 1) ? std::string("dyOut") : "dx" + std::to_string(i + 1);
        const bool needsWeights = i > 0 || needsEncodingAdjoint;
        const bool fused = fusedLayers[i];
        callLayers << "        f16x4 dx" << i << "[NT][Layer" << i << "::KT];\n";
        std::string weights = "sParams + " + std::to_string(ldsW[i]);
        if (placement[i] == WEIGHTS_GLOBAL)
            weights = transposed[i] >= 0 ? "transposedWeights + " + std::to_string(transposed[i]) : "nullptr";
        if (placement[i] == WEIGHTS_STREAMED && needsWeights) {
            anyStreamed = true;
            callLayers << "        materialize(" << dy << ");\n        __syncthreads();   // the stream buffer is free\n        Layer" << i
                       << "::stageAdjoint(networkParameters + " << l.weightsStart << ", sParams + " << ldsW[i]
                       << ", threadIdx.x, blockDim.x);\n        __syncthreads();\n";
        }
        if (recompute) {
            // (every layer is summed here: recomputesFor())
            const std::string inputActivation = i > 0 ? "activations::" + activationTypeName(i - 1) : std::string("activations::passthrough_");
            callLayers << "        Layer" << i << "::template adjointKept<" << (i == 0 ? "NEEDS_ENCODING_ADJOINT" : "true") << ">(" << weights << ", "
                       << dy << ", dx" << i << ", pre" << i << ", sTranspose, validMask, lane);\n"
                       << "        Layer" << i << "::stageInput(" << (i == 0 ? std::string("x0Kept") : "pre" + std::to_string(i - 1))
                       << ", sLayerInput, lane);\n"
                       << "        Layer" << i << "::template weightGradient<" << inputActivation << ", Layer" << i
                       << "::T_STRIDE>(sTranspose, sLayerInput, accW" << i << ", accB" << i << ", lane);\n";
            declareGradients << "    f32x4 accW" << i << "[Layer" << i << "::MT][Layer" << i << "::KT], accB" << i << " = {0.f, 0.f, 0.f, 0.f};\n"
                             << "    zeroTiles(accW" << i << ");\n";
            storeGradients << "    Layer" << i << "::template storeWeightGradient<WAVES>(accW" << i << ", accB" << i
                           << ", reinterpret_cast<float*>(sMemory),\n        partialGradients + (static_cast<long long>(blockIdx.x) * NUM_PARAMETERS + "
                           << l.weightsStart << "), partialGradients + (static_cast<long long>(blockIdx.x) * NUM_PARAMETERS + "
                           << (l.useBias ? l.biasStart : 0) << "), partialSlices, NUM_PARAMETERS, wave, lane);\n";
            continue;
        }
        callLayers << "        Layer" << i << "::template adjoint<" << (fused ? "true" : "STORE_DPRE") << ", "
                   << (i == 0 ? "NEEDS_ENCODING_ADJOINT" : "true") << (placement[i] == WEIGHTS_GLOBAL ? ", true" : ", false")
                   << ", HAS_STREAMED_LAYERS" << (fused ? ", Layer" + std::to_string(i) + "::T_STRIDE" : std::string()) << ">(" << weights << ", " << dy
                   << ", dx" << i << ",\n            forwardTmpMemory + (" << backwardInfo_[i].offsetPre
                   << "ll * numel64 + static_cast<long long>(tileRead) * (" << l.channelsOut << " * TILE_POINTS)),\n"
                   << "            ";
        if (fused) callLayers << "sTranspose";
        else callLayers << "(STORE_DPRE && tileValid) ? adjointTmpMemory + (" << backwardInfo_[i].offsetAdjOut
                        << "ll * numel64 + static_cast<long long>(tile) * (" << l.channelsOut << " * TILE_POINTS)) : nullptr";
        callLayers << ",\n            validMask, lane);\n";
        if (fused) {
            // the LDS tile now holds the adjoint of the pre-activations, zero outside the batch
            const std::string inputActivation = i > 0 ? "activations::" + activationTypeName(i - 1) : std::string("activations::passthrough_");
            callLayers << "        Layer" << i << "::template weightGradient<" << inputActivation << ">(sTranspose,\n"
                       << "            forwardTmpMemory + (" << backwardInfo_[i].offsetIn << "ll * numel64 + static_cast<long long>(tileRead) * ("
                       << l.channelsIn << " * TILE_POINTS)), accW" << i << ", accB" << i << ", lane);\n";
            declareGradients << "    f32x4 accW" << i << "[Layer" << i << "::MT][Layer" << i << "::KT], accB" << i << " = {0.f, 0.f, 0.f, 0.f};\n"
                             << "    zeroTiles(accW" << i << ");\n";
            storeGradients << "    Layer" << i << "::template storeWeightGradient<WAVES>(accW" << i << ", accB" << i
                           << ", reinterpret_cast<float*>(sMemory),\n        partialGradients + (static_cast<long long>(blockIdx.x) * NUM_PARAMETERS + "
                           << l.weightsStart << "), partialGradients + (static_cast<long long>(blockIdx.x) * NUM_PARAMETERS + "
                           << (l.useBias ? l.biasStart : 0) << "), partialSlices, NUM_PARAMETERS, wave, lane);\n";
        }
    }
    replaceAll(code, "$$FUSED_WEIGHT_UPDATE$$", anyFused ? "true" : "false");
    replaceAll(code, "$$NUM_PARAMETERS$$", std::to_string(numParameters_));
    replaceAll(code, "$$DECLARE_WEIGHT_GRADIENTS$$", declareGradients.str());
    replaceAll(code, "$$STORE_WEIGHT_GRADIENTS$$", storeGradients.str());
    {
        std::vector<LdsGradients> unused;
        replaceAll(code, "$$OFFSET_TRANSPOSE$$", std::to_string(roundUp(ldsGradientLayout(flags, blockSize, unused, sliceGradients, recompute), 16)));
        replaceAll(code, "$$TRANSPOSE_HALVES$$", std::to_string(anyFused ? fusedWeightUpdateTransposeHalves(recompute) : 0));
        replaceAll(code, "$$LAYER_INPUT_OFFSET$$", std::to_string(fusedWeightUpdateTransposeHalves(false)));
    }
    {
        // recompute: the encoded input of the tile as the forward kernel stored it (channel-major, four points per
        // load: the layout of the matrix-core operands of the first layer), then the layers, first to last
        std::stringstream forward;
        if (recompute) {
            forward << "        f16x4 x0Kept[NT][Layer0::KT];\n        {\n"
                    << "            const f16* encTile = forwardTmpMemory + static_cast<long long>(tileRead) * (CHANNELS_IN * TILE_POINTS);\n"
                    << "#pragma unroll\n            for (int t = 0; t < KT0; ++t)\n#pragma unroll\n                for (int i = 0; i < 4; ++i) {\n"
                    << "                    const f16x4 v = *reinterpret_cast<const f16x4*>(encTile + (16 * t + 4 * g + i) * TILE_POINTS + 4 * r);\n"
                    << "#pragma unroll\n                    for (int nt = 0; nt < NT; ++nt) x0Kept[nt][t][i] = v[nt];\n                }\n        }\n";
            for (int i = 0; i < L; ++i) {
                const auto& l = layers_[i];
                const std::string in = i == 0 ? std::string("x0Kept") : "act" + std::to_string(i);
                forward << "        f16x4 pre" << i << "[NT][Layer" << i << "::MT], act" << (i + 1) << "[NT][Layer" << i << "::MT];\n"
                        << "        Layer" << i << "::forwardKeep(sParams + " << (adjointParamHalves + ldsWForward[i]) << ", "
                        << (l.useBias ? "sParams + " + std::to_string(adjointParamHalves + ldsBForward[i]) : std::string("nullptr")) << ", " << in
                        << ", pre" << i << ", act" << (i + 1) << ", lane);\n";
            }
            forward << "        (void)act" << L << ";\n";
        }
        replaceAll(code, "$$RECOMPUTE_FORWARD$$", forward.str());
    }
    callLayers << "        auto& dxIn = dx0;\n        (void)dxIn;\n";
    replaceAll(code, "$$CALL_NETWORK_LAYERS$$", callLayers.str());
    replaceAll(code, "$$HAS_STREAMED_LAYERS$$", anyStreamed ? "true" : "false");

    std::stringstream callEncodings, callScatter, zeroLds, flushLds;
    std::vector<LdsGradients> ldsGradients;
    ldsGradientLayout(flags, blockSize, ldsGradients, sliceGradients);
    int encodingOffset = 0;
    bool storeEncodedAdjoint = false, gradientsInKernel = false, inputGradientsInKernel = false;
    for (size_t encodingIdx = 0; encodingIdx < encodings_.size(); ++encodingIdx) {
        const auto& e = encodings_[encodingIdx];
        bool parameterGradients = hasEncodingGradients && e->hasParameters();
        bool inputGradients = hasInputGradients;
        if (parameterGradients && sliceGradients && offersSlices(*e)) {
            // This kernel only stores the adjoint of the encoded rows; the records kernel of the gradient slices,
            // which walks the levels of every point anyway, also gathers for this grid's share of dL/dinput
            // (at 16 wavefronts per compute unit instead of the 8 this kernel's registers leave).
            parameterGradients = false;
            inputGradients = false;
            storeEncodedAdjoint = true;
        }
        gradientsInKernel = gradientsInKernel || parameterGradients;
        inputGradientsInKernel = inputGradientsInKernel || inputGradients;
        const std::string name = e->qualifiedName();
        const LdsGradients& lg = ldsGradients[encodingIdx];
        if (lg.levels > 0) {
            zeroLds << "    float* sGradients" << encodingIdx << " = reinterpret_cast<float*>(sMemory + " << lg.byteOffset
                    << ");\n    for (int e = threadIdx.x; e < " << lg.floats << "; e += blockDim.x) sGradients"
                    << encodingIdx << "[e] = 0.f;\n";
            flushLds << "    " << name << "::template flushLdsGradients<" << lg.levels << ">(sGradients" << encodingIdx
                     << ", cEncoding" << encodingIdx << ", threadIdx.x, blockDim.x);\n";
        }
        // encodings with a tile-wide scatter take their parameter gradients out of the per-point call
        const std::string perPointParameterGradients =
            parameterGradients ? "!" + name + "::HasTileScatter" : std::string("false");
        callEncodings << "                {\n                    auto adjEncodingOutputK = adjEncodingOutput + "
                      << encodingOffset << ";\n                    " << name << "::template adjoint<"
                      << (inputGradients ? "true" : "false") << ", " << perPointParameterGradients
                      << ">(encodingInput, adjEncodingOutputK, adjEncodingInput";
        if (e->hasParameters()) callEncodings << ", cEncoding" << encodingIdx;
        callEncodings << ");\n                }\n";
        if (parameterGradients) {
            callScatter << "            if constexpr (" << name << "::HasTileScatter)\n                " << name
                        << "::template scatterTile<" << lg.levels << ">(lane, static_cast<long long>(tile) * TILE_POINTS, numel, inputs,\n"
                        << "                    [&](int pt, int c) { return static_cast<float>(sStage[stageRow(pt) * STAGE_STRIDE + "
                        << encodingOffset << " + c]); },\n                    cEncoding" << encodingIdx;
            if (lg.levels > 0) callScatter << ", sGradients" << encodingIdx;
            callScatter << ");\n";
        }
        encodingOffset += e->numOutputChannels();
    }
    replaceAll(code, "$$CALL_ENCODINGS$$", callEncodings.str());
    replaceAll(code, "$$STORE_ENCODED_ADJOINT$$", storeEncodedAdjoint ? "true" : "false");
    {
        replaceAll(code, "$$OFFSET_ENCODED_ADJOINT$$", std::to_string(storedAdjointChannels(flags, sliceGradients)));
    }
    // the adjoint of the encoded rows goes through the staging rows only if a lane per point still needs it
    replaceAll(code, "$$NEEDS_STAGED_ADJOINT$$", (inputGradientsInKernel || gradientsInKernel) ? "true" : "false");
    replaceAll(code, "$$HAS_INPUT_GRADIENTS$$", inputGradientsInKernel ? "true" : "false");
    // layer 0 still has to produce the adjoint of the encoded rows for the kernels behind this one
    replaceAll(code, "$$NEEDS_ENCODING_ADJOINT$$", (hasInputGradients || hasEncodingGradients) ? "true" : "false");
    replaceAll(code, "$$CALL_ENCODING_SCATTER$$", callScatter.str());
    replaceAll(code, "$$ZERO_LDS_GRADIENTS$$", zeroLds.str());
    replaceAll(code, "$$FLUSH_LDS_GRADIENTS$$", flushLds.str().empty() ? std::string() : "    __syncthreads();\n" + flushLds.str());
    return code;
}

std::string FusedNetwork::weightUpdateSource(int blockSize) const
{
    auto kl = QuickMLP::Instance().kernelLoader();
    std::string code = kl->findFile("qmlp/kernels/network_weight_update.h").value();
    replaceAll(code, "$$DEFINE_ACTIVATIONS$$", activationDefinitions());
    replaceAll(code, "$$BLOCK_SIZE$$", std::to_string(blockSize));
    return code;
}

std::string FusedNetwork::weightUpdateKernelName(int layer, int& numChunks, int& tilesPerBlock) const
{
    const auto& l = layers_[layer];
    const int kt = l.channelsIn / MATRIX_SIZE, mt = l.channelsOut / MATRIX_SIZE;
    // A workgroup accumulates a block of mo x ki tiles of dW, at most 16 (64 accumulator
    // registers per lane; 32 tiles measured slower: half the waves per SIMD). Splitting the
    // output tiles makes every block read the whole input operand again and re-apply its
    // activation; splitting the input tiles makes every block read dpre again. Take the split
    // with the least traffic, the activation counted as half of another read.
    const double inputCost = layer > 0 ? 1.5 : 1.0;
    int moChunk = 1, kiChunk = 1;
    double best = -1;
    for (int mo = 1; mo <= mt; ++mo) {
        if (mt % mo != 0) continue;
        for (int ki = 1; ki <= kt; ++ki) {
            if (kt % ki != 0 || mo * ki > 16) continue;
            const double cost = l.channelsOut * static_cast<double>(kt / ki) + inputCost * l.channelsIn * (mt / mo);
            if (best < 0 || cost < best || (cost == best && mo * ki > moChunk * kiChunk)) {
                best = cost;
                moChunk = mo;
                kiChunk = ki;
            }
        }
    }
    numChunks = (mt / moChunk) * (kt / kiChunk);
    tilesPerBlock = moChunk * kiChunk + (l.useBias ? moChunk : 0);
    std::string inputActivation = "qmlp::kernel::activations::passthrough_";
    if (layer > 0) {
        inputActivation = "qmlp::kernel::activations::" + activationTypeName(layer - 1);
    }
    return format("qmlp::kernel::WeightUpdateKernel<%d, %d, %s, %s, %d, %d>", l.channelsIn, l.channelsOut,
                  l.useBias ? "true" : "false", inputActivation.c_str(), moChunk, kiChunk);
}

std::string FusedNetwork::generatedSource(const std::string& kind, int adjointFlags)
{
    if (kind == "inference" || kind == "forward") {
        int ppl = 1;
        const int blockSize = forwardBlockSize(kind == "forward" ? compileOptions_.overwriteBlocksizeForward
                                                                  : compileOptions_.overwriteBlocksizeInference, false, &ppl);
        return forwardSource(blockSize, ppl);
    }
    if (kind == "shapes") {
        // which shapes of the forward kernel this network may launch (diagnostics and tests)
        std::stringstream ss;
        ss << "[";
        for (int store = 0; store < 2; ++store) {
            const char* pass = store ? "forward" : "inference";
            auto add = [&](const char* name, int variant) {
                int blockSize = 0, pointsPerLane = 1;
                forwardShape(store != 0, variant, blockSize, pointsPerLane);
                if (ss.tellp() > 1) ss << ", ";
                ss << "{\"pass\": \"" << pass << "\", \"shape\": \"" << name << "\", \"block\": " << blockSize
                   << ", \"tiles_per_wave\": " << pointsPerLane << "}";
            };
            add("default", VARIANT_DEFAULT);
            int ppl = 1;
            forwardBlockSize(-1, false, &ppl);
            if (ppl > 1) add("narrow", VARIANT_NARROW);
            if (hasLargeVariant(store != 0)) add("large", VARIANT_LARGE);
            if (registerVariantTiles(store != 0) > 0) add("registers", VARIANT_REGISTERS);
        }
        ss << "]";
        return ss.str();
    }
    // the shape with the encoded rows in registers, whether or not the network would get it
    if (kind == "forward_registers") return forwardSource(2 * DEFAULT_BLOCK_SIZE, std::min(8, 256 / layers_[0].channelsIn), true);
    if (kind == "backward") return backwardSource(adjointFlags, forwardBlockSize(compileOptions_.overwriteBlocksizeBackward, true));
    if (kind == "backward_recompute")   // the variant that runs the layers again, for networks that have one at these flags
        return backwardSource(adjointFlags, forwardBlockSize(compileOptions_.overwriteBlocksizeBackward, true),
                              useSliceGradients(1 << 30, adjointFlags), true);
    if (kind == "weight_update") return weightUpdateSource(weightUpdateBlockSize());
    if (kind == "backward_resources" || kind == "backward_slices_resources") {
        // what the loaded backward kernel takes (needs a device): for tests of the register budget
        const bool slices = kind == "backward_slices_resources";
        // ("recompute": the kernel of a batch of that kind runs the layers again instead of reading their intermediates)
        const bool recompute = useSliceGradients(slices ? (1 << 30) : 1, adjointFlags) == slices && recomputes(slices ? (1 << 30) : 1, adjointFlags);
        compileBackwardKernel(adjointFlags, slices, false, recompute);
        const auto& ak = backwardKernel_[adjointFlags][slices ? 1 : 0][recompute ? 1 : 0].value();
        return format("{\"block\": %d, \"lds_bytes\": %d, \"registers\": %d, \"scratch_bytes\": %d, \"full_grid\": %d, \"recompute\": %s}",
                      ak.adjoint.blockSize, ak.adjoint.sharedMemorySize, ak.adjoint.fun.numVgprs(), ak.adjoint.fun.scratchBytes(),
                      ak.adjoint.fullGrid, recompute ? "true" : "false");
    }
    throw std::runtime_error("unknown kernel kind '" + kind + "'");
}

// ------------------------------------------------------------------ compilation

static int loaderFlags(bool compileOnly)
{
    int flags = QuickMLP::Instance().getCompileFlags();
    if (compileOnly) flags |= KernelLoader::CompileOnly;
    return flags;
}

bool FusedNetwork::hasLargeVariant(bool store) const
{
    const int overwrite = store ? compileOptions_.overwriteBlocksizeForward : compileOptions_.overwriteBlocksizeInference;
    if (overwrite > 0 || compileOptions_.pointsPerLane > 0) return false;
    bool gathers = false;
    for (const auto& e : encodings_) gathers = gathers || e->hasParameters();
    const int lds = ldsParamHalves(false) * static_cast<int>(sizeof(half)) + 8 * 4 * stageBytesPerWave(false);
    return gathers && lds <= MaxSharedMemoryBytes();
}

int FusedNetwork::registerVariantTiles(bool store) const
{
    const int overwrite = store ? compileOptions_.overwriteBlocksizeForward : compileOptions_.overwriteBlocksizeInference;
    if (overwrite > 0 || compileOptions_.pointsPerLane > 0 || !compileOptions_.registerStaging) return 0;
    bool gathers = false;
    int channelOffset = 0;
    for (const auto& e : encodings_) {
        const int offset = channelOffset;
        channelOffset += e->numOutputChannels();
        gathers = gathers || e->hasParameters();
        if (!e->hasParameters()) continue;
        // a register holds two channels: the features of a level have to fill whole registers
        if (offset % 2 != 0 || e->channelsWrittenTogether() % 2 != 0) return 0;
        // The shape pays through fewer sweeps over the tables of a multi-level grid (only
        // grids write their rows with indices that resolve to registers). The gathers of
        // all 8 points of a lane are in flight together: far beyond 64 registers for them
        // the compiler spills (fp32 entries, 128 registers: 32 spilled registers and 18 %
        // faster than the LDS shape; a dense 4-D grid with 8 features, 512 registers: 1.5 KB
        // of scratch per lane and 1.9 times the time of the LDS shape).
        if (e->numSweptTables() < 2 || 8 * e->gatherRegistersPerPoint() > 128) return 0;
    }
    if (!gathers) return 0;
    // a wavefront of a workgroup of 8 has 256 registers: half of them hold encoded rows (two
    // channels per register), the layers need the rest
    int widest = 0;
    for (const auto& l : layers_) widest = std::max(widest, std::max(l.channelsIn, l.channelsOut));
    if (widest > 64) return 0;
    for (int p : weightPlacement(false))
        if (p != WEIGHTS_RESIDENT) return 0;
    const int tiles = std::min(8, 256 / layers_[0].channelsIn);
    const int lds = ldsParamHalves(false) * static_cast<int>(sizeof(half)) + 8 * stageBytesPerWave(false);
    if (tiles < 8 || lds > MaxSharedMemoryBytes()) return 0;
    return tiles;
}

void FusedNetwork::forwardShape(bool store, int variant, int& blockSize, int& pointsPerLane) const
{
    // the narrow shape is sized like a network with one tile per wave (smaller workgroups when
    // the weights allow it: a small batch then spreads over more compute units)
    blockSize = forwardBlockSize(store ? compileOptions_.overwriteBlocksizeForward : compileOptions_.overwriteBlocksizeInference,
                                 false, &pointsPerLane, variant == VARIANT_NARROW ? 1 : 0);
    if (variant == VARIANT_LARGE) {
        blockSize = 2 * DEFAULT_BLOCK_SIZE;
        pointsPerLane = 4;
    }
    if (variant == VARIANT_REGISTERS) {
        blockSize = 2 * DEFAULT_BLOCK_SIZE;
        pointsPerLane = registerVariantTiles(store);
    }
}

void FusedNetwork::compileForwardKernel(bool store, int variant, bool compileOnly, bool derivatives, bool inputOnly)
{
    derivatives = derivatives && store;
    inputOnly = inputOnly && store;
    auto& slot = forwardKernels_[(derivatives ? 2 : store ? 1 : 0) + (inputOnly ? 2 : 0)][variant];
    if (slot.has_value() && !compileOnly) return;
    auto kl = QuickMLP::Instance().kernelLoader();
    CompiledKernel ck;
    forwardShape(store, variant, ck.blockSize, ck.pointsPerLane);
    const bool registerStaging = variant == VARIANT_REGISTERS;
    ck.sharedMemorySize = ldsParamHalves(false) * static_cast<int>(sizeof(half))
        + (ck.blockSize / WARP_SIZE) * (registerStaging ? 1 : ck.pointsPerLane) * stageBytesPerWave(false);
    ck.fun = kl->getKernel(derivatives ? "qmlp::kernel::NetworkKernelInferenceAndForward<true, true>"
                           : store     ? "qmlp::kernel::NetworkKernelInferenceAndForward<true>"
                                       : "qmlp::kernel::NetworkKernelInferenceAndForward<false>",
                           forwardSource(ck.blockSize, ck.pointsPerLane, registerStaging, derivatives, inputOnly), loaderFlags(compileOnly)).value();
    if (compileOnly) return;
    ck.fullGrid = ck.fun.fullGridSize(ck.blockSize, ck.sharedMemorySize);
    QuickMLP::Instance().getLogger()->debug(
        "%s kernel, %d tile(s) per wave: block %d, LDS %d bytes, %d VGPRs, %d bytes scratch, full grid %d",
        inputOnly ? (derivatives ? "forward (encoded input and position derivatives only)" : "forward (encoded input only)")
                  : derivatives ? "forward (with position derivatives)" : store ? "forward" : "inference", ck.pointsPerLane, ck.blockSize, ck.sharedMemorySize, ck.fun.numVgprs(),
        ck.fun.scratchBytes(), ck.fullGrid);
    slot = std::move(ck);
}

const FusedNetwork::CompiledKernel& FusedNetwork::forwardKernelFor(bool store, int numTiles, int* launchTiles, bool noAlloc, bool derivatives,
                                                                  bool inputOnly)
{
    derivatives = derivatives && store;
    inputOnly = inputOnly && store;
    const int s = (derivatives ? 2 : store ? 1 : 0) + (inputOnly ? 2 : 0);
    // loading a kernel allocates device memory: a call that must not allocate only takes what is loaded
    auto loaded = [&](int variant) -> const CompiledKernel& {
        if (noAlloc && !forwardKernels_[s][variant].has_value())
            throw std::runtime_error("The kernel for a batch of this size is not loaded yet, and loading allocates: run "
                                     "inference() once on a batch of the same size first");
        compileForwardKernel(store, variant, false, derivatives, inputOnly);
        return forwardKernels_[s][variant].value();
    };
    if (launchTiles) *launchTiles = numTiles;
    {
        int blockSize = 0, pointsPerLane = 1;
        forwardShape(store, VARIANT_DEFAULT, blockSize, pointsPerLane);
        if (pointsPerLane == 1) return loaded(VARIANT_DEFAULT);   // no gathers, or a pinned shape: one kernel
    }
    // Kernels that take more tiles per wave are faster per point, but the time grows in steps
    // of one workgroup per compute unit, whether all compute units have one or not. Measured on
    // a 16-level hash grid, per step: 4 waves x 1 tile 26 us (2^16 points), 8 waves x 2 tiles
    // 82 us (2^18 points), 8 waves x 4 tiles 153 us (2^19 points), 8 waves x 8 tiles with the
    // rows in registers 271 us (2^20 points). Estimated time of a shape = steps x points per
    // step x relative cost per point. A batch first gets whole steps of the cheapest shape
    // that it fills (at most two per launch, see gatherChunkPoints), what is left the shape
    // with the least estimated time; the caller comes back for the rest. Only shapes that
    // are used are compiled.
    struct Shape { int variant; long long stepTiles; double costPerPoint; };
    std::vector<Shape> shapes;
    const int computeUnits = KernelFunction::computeUnits();
    auto consider = [&](int variant, double costPerPoint) {
        int blockSize = 0, pointsPerLane = 1;
        forwardShape(store, variant, blockSize, pointsPerLane);
        shapes.push_back({variant, static_cast<long long>(computeUnits) * (blockSize / WARP_SIZE) * pointsPerLane, costPerPoint});
    };
    // measured 258 ps per point against 288 for 8 waves x 4 tiles (16-level hash grid, 2^20 points)
    if (registerVariantTiles(store) > 0 && !registerShapeSpills_[s]) consider(VARIANT_REGISTERS, 0.9);
    if (hasLargeVariant(store)) consider(VARIANT_LARGE, 1.0);
    consider(VARIANT_DEFAULT, 1.075);
    consider(VARIANT_NARROW, 1.39);
    auto wholeBatch = [&](long long tiles, int& variant) {
        double bestCost = 0;
        variant = -1;
        for (const auto& sh : shapes) {
            const double cost = static_cast<double>(divUp<long long>(tiles, sh.stepTiles)) * sh.stepTiles * sh.costPerPoint;
            if (variant < 0 || cost < bestCost) {
                variant = sh.variant;
                bestCost = cost;
            }
        }
        return tiles > 0 ? bestCost : 0.0;
    };
    int best = -1;
    double bestCost = wholeBatch(numTiles, best);
    for (const auto& sh : shapes) {
        const long long steps = numTiles / sh.stepTiles;
        if (steps < 1) continue;
        int unused = -1;
        const double cost = static_cast<double>(steps * sh.stepTiles) * sh.costPerPoint
            + wholeBatch(numTiles - steps * sh.stepTiles, unused);
        if (cost < bestCost) {
            best = sh.variant;
            bestCost = cost;
            if (launchTiles) *launchTiles = static_cast<int>(steps * sh.stepTiles);
        }
    }
    loaded(best);
    if (best == VARIANT_REGISTERS && forwardKernels_[s][best].value().fun.scratchBytes() > MAX_REGISTER_SHAPE_SCRATCH) {
        // the compiler did not get the rows and the gathers into the registers: a kernel that
        // spills this much is slower than the shapes that stage in LDS
        QuickMLP::Instance().getLogger()->debug("the forward kernel with rows in registers spills %d bytes per lane, not used",
                                                forwardKernels_[s][best].value().fun.scratchBytes());
        registerShapeSpills_[s] = true;
        return forwardKernelFor(store, numTiles, launchTiles, noAlloc, derivatives, inputOnly);
    }
    return forwardKernels_[s][best].value();
}

void FusedNetwork::compileBackwardKernel(int flags, bool sliceGradients, bool compileOnly, bool recompute)
{
    if (flags <= 0 || flags >= ADJOINT_MODE_MAX_COMBINATIONS) throw std::runtime_error("At least one derivative must be enabled");
    const int variant = sliceGradients ? 1 : 0;
    if (backwardKernel_[flags][variant][recompute ? 1 : 0].has_value() && !compileOnly) return;
    const bool hasNetworkGradients = flags & GRADIENTS_NETWORK_WEIGHTS;
    auto kl = QuickMLP::Instance().kernelLoader();
    auto logger = QuickMLP::Instance().getLogger();

    AdjointKernel ak;
    ak.adjoint.blockSize = forwardBlockSize(compileOptions_.overwriteBlocksizeBackward, true);
    {
        std::vector<LdsGradients> ldsGradients;
        ak.adjoint.sharedMemorySize = ldsGradientLayout(flags, ak.adjoint.blockSize, ldsGradients, sliceGradients, recompute);
    }
    ak.fusedLayers = fusedWeightUpdateLayers(flags, sliceGradients);
    ak.outputOrder = trainsSortedBatches();
    ak.fusedWeightUpdate = false;
    for (bool f : ak.fusedLayers) ak.fusedWeightUpdate = ak.fusedWeightUpdate || f;
    if (ak.fusedWeightUpdate) {
        // behind everything else: a tile per wavefront for Layer::weightGradient; after the last tile the gradient
        // tiles of one layer at a time are summed over the wavefronts from the start of the LDS
        int widestTiles = 0;
        for (size_t i = 0; i < layers_.size(); ++i) {
            const auto& l = layers_[i];
            const int mt = l.channelsOut / MATRIX_SIZE, kt = l.channelsIn / MATRIX_SIZE;
            if (ak.fusedLayers[i]) widestTiles = std::max(widestTiles, mt * kt + (l.useBias ? 1 : 0));
        }
        ak.adjoint.sharedMemorySize = std::max(roundUp(ak.adjoint.sharedMemorySize, 16) + (ak.adjoint.blockSize / WARP_SIZE)
                                                   * fusedWeightUpdateTransposeHalves(recompute) * static_cast<int>(sizeof(half)),
                                               widestTiles * 256 * static_cast<int>(sizeof(float)));
    }
    // Which compiler and how many registers. The run-time compiler is the one of the process (a Python process that
    // imported torch compiles with the libamd_comgr that torch ships, ROCm 7.0's under torch 2.10); where the installed
    // ROCm has an offline compiler, the kernels that hold gradient tiles are given to it:
    //  - the kernel that runs the layers again, within the 256 registers of two wavefronts per SIMD: BASELINE config 5
    //    needs 232 registers and no scratch there against 404 bytes of scratch from the run-time compiler, and takes
    //    135 instead of 233 us, also because no matrix result passes through accumulation registers. Taken if it does
    //    not spill; a pass that only fills the cache cannot know and compiles the next form as well.
    //  - kernels of one wavefront per SIMD with the matrix instructions in their vector-register form: a kernel that may
    //    use more than 256 registers otherwise gets every matrix result in an accumulation register and copies each
    //    value out (a quarter of the instructions of such a kernel's loop).
    std::string adjointSource;
    int adjointLoaderFlags = loaderFlags(compileOnly);
    std::vector<std::string> offlineOptions;
    bool wideByTiles = false;
    (void)fusedWeightUpdateLayers(flags, sliceGradients, &wideByTiles);
    const bool offlineCompiler = KernelLoader::hasOfflineCompiler() && (recompute || wideByTiles);
    bool chosen = false;
    if (recompute && offlineCompiler) {
        adjointSource = backwardSource(flags, ak.adjoint.blockSize, sliceGradients, true, true);
        auto fun = kl->getKernel("qmlp::kernel::NetworkKernelBackward", adjointSource, adjointLoaderFlags | KernelLoader::CompileOffline);
        if (fun.has_value() && !compileOnly && fun.value().scratchBytes() <= MAX_RECOMPUTE_SCRATCH) {
            ak.adjoint.fun = fun.value();
            adjointLoaderFlags |= KernelLoader::CompileOffline;
            chosen = true;
        } else if (fun.has_value() && !compileOnly) {
            logger->debug("the backward kernel that runs the layers again (flags %d) spills %d bytes per lane with two wavefronts per SIMD",
                          flags, fun.value().scratchBytes());
        }
    }
    if (!chosen) {
        adjointSource = backwardSource(flags, ak.adjoint.blockSize, sliceGradients, recompute);
        if (offlineCompiler) {
            adjointLoaderFlags |= KernelLoader::CompileOffline;
            offlineOptions = {"-mllvm", "-amdgpu-mfma-vgpr-form"};
        }
        ak.adjoint.fun = kl->getKernel("qmlp::kernel::NetworkKernelBackward", adjointSource, adjointLoaderFlags, offlineOptions).value();
    }
    {
        std::vector<long long> transposed;
        if (transposedWeightLayout(flags, transposed) > 0) {
            ak.transpose.blockSize = 256;
            ak.transpose.fun =
                kl->getKernel("qmlp::kernel::TransposeWeightsKernel", adjointSource, adjointLoaderFlags, offlineOptions).value();
        }
    }
    if (!compileOnly) {
        ak.adjoint.fullGrid = ak.adjoint.fun.fullGridSize(ak.adjoint.blockSize, ak.adjoint.sharedMemorySize);
        logger->debug("backward kernel (flags %d%s): block %d, LDS %d bytes, %d VGPRs, %d bytes scratch, full grid %d", flags,
                      recompute ? ", the layers run again" : "",
                      ak.adjoint.blockSize, ak.adjoint.sharedMemorySize, ak.adjoint.fun.numVgprs(),
                      ak.adjoint.fun.scratchBytes(), ak.adjoint.fullGrid);
    }
    ak.perEntryAdjointMemoryBytes = storedAdjointChannels(flags, sliceGradients) * static_cast<int>(sizeof(half));
    // behind the adjoint pre-activations: the adjoint of the encoded rows for the records kernels
    if (sliceGradients && (flags & GRADIENTS_INPUT_ENCODINGS)) ak.perEntryAdjointMemoryBytes += sliceGradientBytesPerPoint();

    if (sliceGradients && (flags & GRADIENTS_INPUT_ENCODINGS)) {
        int channelOffset = 0;
        for (size_t i = 0; i < encodings_.size(); ++i) {
            const auto& e = encodings_[i];
            const int offset = channelOffset;
            channelOffset += e->numOutputChannels();
            SliceGradientKernel sk;
            if (!offersSlices(*e, &sk.layout)) continue;
            const auto& layout = sk.layout;
            sk.encoding = static_cast<int>(i);
            std::stringstream source;
            e->fillCode(source);
            source << "\n" << KernelLoader::MainFile("qmlp/kernels/grid_gradient.h");
            sk.recordsSource = source.str();
            sk.channelOffset = offset;
            for (int points = layout.pointsPerWorkgroup; points >= std::min(128, layout.pointsPerWorkgroup); points /= 2) {
                sk.records.emplace_back();
                sk.recordsFromDerivatives.emplace_back();
            }
            sk.derivativeOffset = derivativeOffsets_[i];
            {
                // batches that train sorted by the slabs of this grid
                kernel::PointOrderKey key{};
                sk.columnsOffered = compileOptions_.columnGradients != 0 && compileOptions_.sortTraining && compileOptions_.sortPoints != 0
                    && channelsIn() <= 16 && e->pointOrderKey(key, 0) && e->gradientColumns(key, sk.columnLayout);
                if (sk.columnsOffered && compileOnly) {
                    compileColumnKernels(sk, flags, true);
                    if ((flags & GRADIENTS_INPUT) && sk.derivativeOffset >= 0) compileColumnKernels(sk, flags, true, true);
                }
            }
            if (compileOnly)
                for (size_t v = 0; v < sk.records.size(); ++v) {
                    compileRecordsKernel(sk, flags, v, true);
                    if ((flags & GRADIENTS_INPUT) && sk.derivativeOffset >= 0) compileRecordsKernel(sk, flags, v, true, true);
                }
            sk.kernel.blockSize = 1024;
            sk.kernel.sharedMemorySize = layout.sliceFloats * static_cast<int>(sizeof(long long));
            sk.kernel.fun = kl->getKernel(format("qmlp::kernel::GridGradientSlicesKernel<%s, %d>", layout.configType.c_str(), layout.sliceFloats),
                                          source.str(), loaderFlags(compileOnly)).value();
            if (!compileOnly) {
                static_assert(sizeof(IEncoding::GradientSlice) == 32, "eight 32-bit words, as in kernels/grid_gradient.h");
                sk.items = Tensor(Tensor::FLOAT, {static_cast<int32_t>(layout.items.size() * 8)});
                QMLP_HIP_CALL(qmlp_hip_memcpy_h2d(sk.items.rawPtr(), layout.items.data(), layout.items.size() * sizeof(layout.items[0]), nullptr));
                logger->debug("gradient slices of encoding %d: %d buckets, %d work items", sk.encoding, layout.numBuckets(),
                              static_cast<int>(layout.items.size()));
            }
            ak.sliceGradients.push_back(std::move(sk));
        }
    }

    if (hasNetworkGradients) {
        const int blockSize = weightUpdateBlockSize();
        const std::string source = weightUpdateSource(blockSize);
        ak.reduce.blockSize = 1024;
        ak.reduce.fun = kl->getKernel("qmlp::kernel::WeightUpdateReduceKernel", source, loaderFlags(compileOnly)).value();
        ak.layers.resize(layers_.size());
        for (size_t layer = 0; layer < ak.layers.size(); ++layer) {
            if (ak.fusedLayers[layer]) continue;   // summed by the adjoint kernel
            auto& wk = ak.layers[layer];
            int tiles = 0;
            const std::string name = weightUpdateKernelName(static_cast<int>(layer), wk.numChunks, tiles);
            wk.kernel.blockSize = blockSize;
            wk.kernel.sharedMemorySize = tiles * 256 * static_cast<int>(sizeof(float));
            if (wk.kernel.sharedMemorySize > MaxSharedMemoryBytes())
                throw configuration_error("Layer %d too large for block-wise weight update!", static_cast<int>(layer));
            wk.kernel.fun = kl->getKernel(name, source, loaderFlags(compileOnly)).value();
            if (!compileOnly) {
                wk.kernel.fullGrid = wk.kernel.fun.fullGridSize(blockSize, wk.kernel.sharedMemorySize);
                logger->debug("weight update kernel layer %d: %s, LDS %d bytes, %d VGPRs, full grid %d",
                              static_cast<int>(layer), name.c_str(), wk.kernel.sharedMemorySize,
                              wk.kernel.fun.numVgprs(), wk.kernel.fullGrid);
            }
        }
    }
    if (!compileOnly) backwardKernel_[flags][variant][recompute ? 1 : 0] = std::move(ak);
}

void FusedNetwork::compileRecordsKernel(SliceGradientKernel& sk, int flags, size_t variant, bool compileOnly, bool fromDerivatives)
{
    const auto& layout = sk.layout;
    const int points = layout.pointsPerWorkgroup >> variant;
    CompiledKernel ck;
    ck.blockSize = points;
    ck.sharedMemorySize = layout.recordsLdsBytes(points);
    ck.fun = QuickMLP::Instance().kernelLoader()->getKernel(
        // (last argument: no input gradients | from gathers of all corners | from the position derivatives of the forward pass)
        format("qmlp::kernel::GridGradientRecordsKernel<%s, %d, %d, %d, %d, %d>", layout.configType.c_str(), layers_[0].channelsIn,
               sk.channelOffset, layout.sliceFloats, points, !(flags & GRADIENTS_INPUT) ? 0 : fromDerivatives ? 2 : 1),
        sk.recordsSource, loaderFlags(compileOnly)).value();
    if (compileOnly) return;
    ck.fullGrid = ck.fun.fullGridSize(ck.blockSize, ck.sharedMemorySize);
    QuickMLP::Instance().getLogger()->debug("records kernel of encoding %d with %d points per workgroup%s: %d VGPRs, full grid %d",
                                            sk.encoding, points, fromDerivatives ? " (stored position derivatives)" : "",
                                            ck.fun.numVgprs(), ck.fullGrid);
    (fromDerivatives ? sk.recordsFromDerivatives : sk.records)[variant] = std::move(ck);
}

void FusedNetwork::compileColumnKernels(SliceGradientKernel& sk, int flags, bool compileOnly, bool fromDerivatives)
{
    fromDerivatives = fromDerivatives && (flags & GRADIENTS_INPUT) && sk.derivativeOffset >= 0;
    if (sk.columns[fromDerivatives ? 1 : 0].has_value() && !compileOnly) return;
    auto kl = QuickMLP::Instance().kernelLoader();
    std::stringstream source;
    encodings_[sk.encoding]->fillCode(source);
    source << "\n" << KernelLoader::MainFile("qmlp/kernels/grid_gradient_columns.h");
    const auto& layout = sk.columnLayout;
    CompiledKernel plan, columns;
    plan.blockSize = 1024;
    plan.fun = kl->getKernel(format("qmlp::kernel::GridGradientColumnsPlan<%s, %d>", layout.configType.c_str(), layout.cellsPerSlab),
                             source.str(), loaderFlags(compileOnly)).value();
    columns.blockSize = 512;
    columns.sharedMemorySize = layout.ldsBytes;
    columns.fun = kl->getKernel(format("qmlp::kernel::GridGradientColumnsKernel<%s, %d, %d, %d, %d, %d>", layout.configType.c_str(),
                                       layout.cellsPerSlab, layers_[0].channelsIn, sk.channelOffset,
                                       !(flags & GRADIENTS_INPUT) ? 0 : fromDerivatives ? 2 : 1, columns.blockSize),
                                source.str(), loaderFlags(compileOnly)).value();
    if (compileOnly) return;
    QuickMLP::Instance().getLogger()->debug("column kernel of encoding %d: %d x %d owners, LDS %d bytes, %d VGPRs, %d bytes scratch",
                                            sk.encoding, layout.owners, layout.owners, layout.ldsBytes, columns.fun.numVgprs(),
                                            columns.fun.scratchBytes());
    sk.columnsPlan = std::move(plan);
    sk.columns[fromDerivatives ? 1 : 0] = std::move(columns);
}

size_t FusedNetwork::columnWorkspaceBytes(const IEncoding::GradientColumnLayout& layout, long long numel, int* maxItems)
{
    // as kernels/grid_gradient_columns.h: an owner is split into parts of GRID_GRADIENT_COLUMNS_PART_POINTS points, and
    // every point is visited by at most four owners
    constexpr long long PART_POINTS = 24 * 1024;
    const long long items = static_cast<long long>(layout.owners) * layout.owners + 4 * numel / PART_POINTS + 4;
    if (maxItems) *maxItems = static_cast<int>(items);
    return roundUp(static_cast<size_t>(SORT_SLABS + 1 + 1) * sizeof(int), size_t(256)) + static_cast<size_t>(items) * 4 * sizeof(int);
}

const FusedNetwork::CompiledKernel& FusedNetwork::recordsKernelFor(SliceGradientKernel& sk, int flags, int numel, bool fromDerivatives)
{
    // The table entries that a workgroup gathers for the input gradients and the records it writes pass through
    // one compute unit's memory pipeline: a batch that fills fewer workgroups than there are compute units leaves
    // the rest of the chip idle. Measured on a 16-level hash grid (train step, ms; 1024 / 512 / 256 / 128 points):
    // 2^17 points 0.414 / 0.302 / 0.319 / 0.371, 2^16 points 0.290 / 0.233 / 0.215 / 0.244.
    const int computeUnits = KernelFunction::computeUnits();
    size_t variant = 0;
    while (variant + 1 < sk.records.size() && divUp(numel, sk.layout.pointsPerWorkgroup >> variant) < computeUnits) ++variant;
    auto& kernels = fromDerivatives ? sk.recordsFromDerivatives : sk.records;
    if (!kernels[variant].has_value()) compileRecordsKernel(sk, flags, variant, false, fromDerivatives);
    return kernels[variant].value();
}

void FusedNetwork::precompile(int adjointFlags)
{
    for (int store = 0; store < 2; ++store) {
        compileForwardKernel(store, VARIANT_DEFAULT, true);
        int ppl = 1;
        forwardBlockSize(-1, false, &ppl);
        if (ppl > 1) compileForwardKernel(store, VARIANT_NARROW, true);
        if (hasLargeVariant(store)) compileForwardKernel(store, VARIANT_LARGE, true);
        if (registerVariantTiles(store) > 0) compileForwardKernel(store, VARIANT_REGISTERS, true);
    }
    if (adjointFlags > 0) {
        // training passes that keep the encoded input only, and the backward kernels that run the layers again
        bool any = false;
        for (int numel : {1, 1 << 30}) {
            if (!recomputesFor(numel, adjointFlags)) continue;
            any = true;
            compileBackwardKernel(adjointFlags, useSliceGradients(numel, adjointFlags), true, true);
        }
        if (any)
            for (int derivatives = 0; derivatives <= (storesDerivatives(1 << 30, adjointFlags) ? 1 : 0); ++derivatives) {
                compileForwardKernel(true, VARIANT_DEFAULT, true, derivatives != 0, true);
                int ppl = 1;
                forwardBlockSize(-1, false, &ppl);
                if (ppl > 1) compileForwardKernel(true, VARIANT_NARROW, true, derivatives != 0, true);
                if (hasLargeVariant(true)) compileForwardKernel(true, VARIANT_LARGE, true, derivatives != 0, true);
                if (registerVariantTiles(true) > 0) compileForwardKernel(true, VARIANT_REGISTERS, true, derivatives != 0, true);
            }
    }
    if (adjointFlags > 0 && storesDerivatives(1 << 30, adjointFlags)) {
        // training passes that keep the position derivatives of their grids
        compileForwardKernel(true, VARIANT_DEFAULT, true, true);
        int ppl = 1;
        forwardBlockSize(-1, false, &ppl);
        if (ppl > 1) compileForwardKernel(true, VARIANT_NARROW, true, true);
        if (hasLargeVariant(true)) compileForwardKernel(true, VARIANT_LARGE, true, true);
        if (registerVariantTiles(true) > 0) compileForwardKernel(true, VARIANT_REGISTERS, true, true);
    }
    if (adjointFlags > 0) {
        if (compileOptions_.sliceGradients <= 0 || !hasSliceGradients() || !(adjointFlags & GRADIENTS_INPUT_ENCODINGS))
            compileBackwardKernel(adjointFlags, false, true);
        if ((adjointFlags & GRADIENTS_INPUT_ENCODINGS) && hasSliceGradients()) compileBackwardKernel(adjointFlags, true, true);
    }
    kernel::PointOrderKey key{};
    for (const auto& e : encodings_)
        // asked for, or chosen by itself for batches that are large enough
        if (compileOptions_.sortPoints != 0 && e->pointOrderKey(key, compileOptions_.sortPoints > 0 ? 0 : (1ll << 30))) {
            auto kl = QuickMLP::Instance().kernelLoader();
            const std::string source = KernelLoader::MainFile("qmlp/kernels/point_order.h");
            const std::string scatter = "PointOrderScatter<" + std::to_string(channelsIn_ <= 4 ? 4 : channelsIn_ <= 8 ? 8 : 16) + ">";
            for (const std::string& name : {std::string("PointOrderCount"), std::string("PointOrderScan"), scatter,
                                            std::string("PointOrderGatherAddRows")})
                kl->getKernel("qmlp::kernel::" + name, source, loaderFlags(true));
            break;
        }
}

// ------------------------------------------------------------------ launches

int FusedNetwork::gatherChunkPoints(const CompiledKernel& ck) const
{
    // The workgroups of a launch walk the levels of a grid side by side, which keeps the table
    // of the level in use in L2. Over many passes they drift apart and several level tables
    // compete for the L2: cfg2 at 2^24 points took 602 ps per point in one launch, against 288
    // at 2^20. Batches of a network that gathers are therefore cut into launches of two
    // passes each; a launch boundary brings the workgroups back in step. A single table (cfg5)
    // has nothing to compete with and stays in one launch (two launches cost 3 % there).
    int tables = 0;
    for (const auto& e : encodings_) tables = std::max(tables, e->numSweptTables());
    if (tables < 2) return std::numeric_limits<int>::max();
    const long long pass = static_cast<long long>(KernelFunction::computeUnits()) * (ck.blockSize / WARP_SIZE) * ck.pointsPerLane * TILE_POINTS;
    return static_cast<int>(std::min<long long>(2 * pass, std::numeric_limits<int>::max()));
}

std::vector<char> FusedNetwork::encodingArguments(std::vector<void*>& args, std::vector<std::vector<char>>& storage)
{
    storage.clear();
    storage.reserve(encodings_.size());
    for (auto& e : encodings_) {
        if (!e->hasParameters()) continue;
        storage.emplace_back(1024);
        int n = e->fillParameterMemory(storage.back().data(), static_cast<int>(storage.back().size()));
        (void)n;
        args.push_back(storage.back().data());
    }
    return {};
}

void FusedNetwork::checkEncodingParameters(Tensor::Usage usage) const
{
    for (size_t i = 0; i < encodings_.size(); ++i) {
        if (!encodings_[i]->hasParameters() || encodings_[i]->hasParameterTensor(usage)) continue;
        if (usage == Tensor::INFERENCE)
            throw std::runtime_error(format("Encoding %d has parameters, but no inference tensor is bound to it: call "
                                            "encoding(%d)->setParameter(tensor, INFERENCE) first", int(i), int(i)));
        throw std::runtime_error(format("Encoding gradients requested, but encoding %d has no gradient tensor: call "
                                        "encoding(%d)->setParameter(tensor, GRADIENTS) for every encoding with parameters",
                                        int(i), int(i)));
    }
}

void FusedNetwork::inference(const Tensor& input, Tensor& output, stream_t stream)
{
    CHECK_DIM(input, 2);
    CHECK_DIM(output, 2);
    CHECK_SIZE(input, 1, channelsIn());
    CHECK_SIZE(output, 1, channelsOut());
    int numel = input.size(0);
    CHECK_SIZE(output, 0, numel);
    CHECK_DTYPE(input, precisionIn());
    CHECK_DTYPE(output, precisionOut());
    CHECK_ERROR(parametersInference_.defined(), "Inference parameters not defined, call setNetworkParameter(...) first");
    checkEncodingParameters(Tensor::INFERENCE);
    if (numel == 0) return;

    launchForward(false, input, output, nullptr, stream);
}

void FusedNetwork::inferenceNoAlloc(const Tensor& input, Tensor& output, stream_t stream)
{
    CHECK_DIM(input, 2);
    CHECK_DIM(output, 2);
    CHECK_SIZE(input, 1, channelsIn());
    CHECK_SIZE(output, 1, channelsOut());
    int numel = input.size(0);
    CHECK_SIZE(output, 0, numel);
    CHECK_DTYPE(input, precisionIn());
    CHECK_DTYPE(output, precisionOut());
    CHECK_ERROR(parametersInference_.defined(), "Inference parameters not defined, call setNetworkParameter(...) first");
    checkEncodingParameters(Tensor::INFERENCE);
    if (numel == 0) return;

    launchForward(false, input, output, nullptr, stream, true);
}

void FusedNetwork::launchForward(bool store, const Tensor& input, Tensor& output, half* tmpMemory, stream_t stream, bool noAlloc, bool derivatives,
                                 bool inputOnly)
{
    const int numel = input.size(0);
    int tmpNumTiles = divUp(numel, TILE_POINTS);
    auto inputAll = input.accessor<kernel::Tensor2Read<float>>();
    const auto outputAll = output.accessor<kernel::Tensor2RW<float>>();
    // inference of a network with a large dense grid: rows of the input sorted by grid slab,
    // every row of the result written where its point stands in the caller's batch
    const int* orderAll = nullptr;
    // (a training pass keeps the sorted rows and the order in its forward memory, for the adjoint pass)
    void* sortedDestination = store && sortsTraining(numel) ? reinterpret_cast<char*>(tmpMemory) + sortedRowsOffset(numel) : nullptr;
    const bool sorted = (!store || sortedDestination != nullptr) && sortPoints(input, inputAll, orderAll, stream, noAlloc, sortedDestination);
    const half* networkParams = parametersInference_.dataPtr<half>();
    for (long long start = 0; start < numel;) {
        // the kernel shape for what is left; a network that gathers gets at most two steps of it per launch
        int launchTiles = 0;
        const auto& ck = forwardKernelFor(store, static_cast<int>(divUp<long long>(numel - start, TILE_POINTS)), &launchTiles, noAlloc, derivatives,
                                          inputOnly);
        int count = static_cast<int>(std::min<long long>(
            {static_cast<long long>(gatherChunkPoints(ck)), static_cast<long long>(launchTiles) * TILE_POINTS, numel - start}));
        auto inputAcc = inputAll;
        auto outputAcc = outputAll;
        inputAcc.data_ += start * inputAll.strides_[0];
        if (!sorted) outputAcc.data_ += start * outputAll.strides_[0];
        inputAcc.sizes_[0] = outputAcc.sizes_[0] = count;
        const int* order = sorted ? orderAll + start : nullptr;
        int tmpTileOffset = static_cast<int>(start / TILE_POINTS);
        const int waves = ck.blockSize / WARP_SIZE;
        const int grid = std::min(divUp(divUp(count, TILE_POINTS), waves * ck.pointsPerLane), ck.fullGrid);
        std::vector<void*> args = {&count, &inputAcc, &outputAcc, &networkParams, &tmpMemory, &tmpTileOffset, &tmpNumTiles, &order};
        std::vector<std::vector<char>> storage;
        encodingArguments(args, storage);
        ck.fun.launch(grid, ck.blockSize, ck.sharedMemorySize, stream, args.data());
        start += count;
    }
}

bool FusedNetwork::pointOrderFor(int numel, kernel::PointOrderKey& key) const
{
    if (compileOptions_.sortPoints == 0 || (compileOptions_.sortPoints < 0 && numel < SORT_POINTS_MIN_BATCH)) return false;
    if (channelsIn() > 16) return false;
    for (const auto& e : encodings_)
        if (e->pointOrderKey(key, compileOptions_.sortPoints < 0 ? numel : 0)) return true;
    return false;
}

void FusedNetwork::loadPointOrderKernels(bool rowMoves)
{
    auto& po = pointOrder_;
    auto kl = QuickMLP::Instance().kernelLoader();
    const std::string source = KernelLoader::MainFile("qmlp/kernels/point_order.h");
    if (!po.scatter.has_value()) {
        const int maxChannels = channelsIn_ <= 4 ? 4 : channelsIn_ <= 8 ? 8 : 16;
        po.scan = kl->getKernel("qmlp::kernel::PointOrderScan", source, loaderFlags(false)).value();
        po.count = kl->getKernel("qmlp::kernel::PointOrderCount", source, loaderFlags(false)).value();
        po.scatter = kl->getKernel("qmlp::kernel::PointOrderScatter<" + std::to_string(maxChannels) + ">", source, loaderFlags(false)).value();
    }
    if (rowMoves && !po.gatherAddRows.has_value())
        po.gatherAddRows = kl->getKernel("qmlp::kernel::PointOrderGatherAddRows", source, loaderFlags(false)).value();
}

void FusedNetwork::prepare(int numel, int adjointFlags)
{
    CHECK_ERROR(numel >= 0, "prepare(): the batch size must not be negative");
    CHECK_ERROR(adjointFlags >= 0 && adjointFlags < ADJOINT_MODE_MAX_COMBINATIONS, "prepare(): unknown adjoint flags ", adjointFlags);
    if (numel == 0) return;
    // the forward kernels that launchForward() takes for the pieces of a batch of this size
    if (adjointFlags > 0) announcedFlags_ = adjointFlags;
    for (int store = 0; store <= (adjointFlags > 0 ? 1 : 0); ++store)
        for (long long start = 0; start < numel;) {
            int launchTiles = 0;
            const auto& ck = forwardKernelFor(store != 0, static_cast<int>(divUp<long long>(numel - start, TILE_POINTS)), &launchTiles, false,
                                              store != 0 && storesDerivatives(numel, adjointFlags), store != 0 && recomputes(numel, adjointFlags));
            start += std::min<long long>({static_cast<long long>(gatherChunkPoints(ck)), static_cast<long long>(launchTiles) * TILE_POINTS,
                                          numel - start});
        }
    // the sort of a batch that is evaluated slab by slab: kernels, workspace, and the static buffer of inferenceNoAlloc()
    kernel::PointOrderKey key{};
    if (pointOrderFor(numel, key)) {
        loadPointOrderKernels(adjointFlags > 0 && sortsTraining(numel));
        constexpr long long SLABS = 1024, CHUNK = 4 * 1024;   // as in sortPoints()
        const long long words = (divUp<long long>(numel, CHUNK) + 1) * SLABS + static_cast<long long>(numel) * (channelsIn_ + 1);
        if (pointOrder_.capacityWords < words && words <= std::numeric_limits<int32_t>::max()) {
            pointOrder_.workspace = Tensor(Tensor::FLOAT, {static_cast<int32_t>(words)});
            pointOrder_.capacityWords = words;
        }
        void* scratch = nullptr;
        size_t scratchBytes = 0;
        std::string error;
        (void)device_code::staticScratch(&scratch, &scratchBytes, error);
    }
    if (adjointFlags > 0) {
        const bool sliceGradients = useSliceGradients(numel, adjointFlags);
        const bool recompute = recomputes(numel, adjointFlags);
        compileBackwardKernel(adjointFlags, sliceGradients, false, recompute);
        for (auto& sk : backwardKernel_[adjointFlags][sliceGradients ? 1 : 0][recompute ? 1 : 0].value().sliceGradients)
        {
            (void)recordsKernelFor(sk, adjointFlags, numel, storesDerivatives(numel, adjointFlags) && sk.derivativeOffset >= 0);
            if (sk.columnsOffered && sortsTraining(numel))
                compileColumnKernels(sk, adjointFlags, false, storesDerivatives(numel, adjointFlags) && sk.derivativeOffset >= 0);
        }
        // the streams and events on which the weight-update kernels of the layers run side by side
        if ((adjointFlags & GRADIENTS_NETWORK_WEIGHTS) && compileOptions_.parallelWeightUpdate && layers_.size() > 1) ensureStreams();
    }
}

bool FusedNetwork::trainsSortedBatches() const
{
    kernel::PointOrderKey key{};
    return compileOptions_.sortTraining && pointOrderFor(1 << 30, key);
}

bool FusedNetwork::sortsTraining(int numel) const
{
    kernel::PointOrderKey key{};
    return compileOptions_.sortTraining && pointOrderFor(numel, key);
}

size_t FusedNetwork::sortedRowsOffset(int numel) const
{
    return roundUp(forwardBytesPerPoint() * static_cast<size_t>(roundUp(numel, WARP_SIZE)), size_t(256));
}

size_t FusedNetwork::sortedTotalsOffset(int numel) const
{
    return sortedRowsOffset(numel) + roundUp(static_cast<size_t>(numel) * (channelsIn() + 1) * sizeof(float), size_t(256));
}

size_t FusedNetwork::sortedPlacementOffset(int numel) const
{
    return sortedTotalsOffset(numel) + SORT_SLABS * sizeof(int);
}

bool FusedNetwork::sortPoints(const Tensor& input, kernel::Tensor2Read<float>& sortedInput, const int*& order, stream_t stream,
                              bool noAlloc, void* destination)
{
    const int numel = input.size(0);
    kernel::PointOrderKey key{};
    if (!pointOrderFor(numel, key)) return false;
    const int channels = input.size(1);

    auto& po = pointOrder_;
    if (!po.scatter.has_value() && noAlloc)
        throw std::runtime_error("The kernels that order the batch are not loaded yet, and loading allocates: run "
                                 "inference() once on a batch of the same size first");
    loadPointOrderKernels(false);
    constexpr int SLABS = 1024, BLOCK = 1024, CHUNK = 4 * BLOCK;   // as in point_order.h
    // words: slab totals and one histogram per chunk; then (unless the caller has room for them) sorted inputs and order
    const long long histogramWords = (divUp(numel, CHUNK) + 1ll) * SLABS;
    const long long rowWords = static_cast<long long>(numel) * (channels + 1);
    const long long words = histogramWords + (destination ? 0 : rowWords);
    int* totals = nullptr;
    if (noAlloc) {
        // the workspace is the library's static device buffer; the kernels get its address
        // as the same arguments that otherwise point into the network's own workspace
        void* scratch = nullptr;
        size_t scratchBytes = 0;
        std::string error;
        if (device_code::staticScratch(&scratch, &scratchBytes, error) != 0) throw std::runtime_error(error);
        if (static_cast<unsigned long long>(words) * sizeof(float) > scratchBytes)
            throw std::runtime_error(format(
                "A batch of %d points with %d channels needs %lld bytes to be ordered by grid slab; the call that allocates "
                "nothing has a static buffer of %lld bytes (at most %lld points of this network): split the batch, or "
                "call inference()", numel, channels, words * static_cast<long long>(sizeof(float)),
                static_cast<long long>(scratchBytes),
                // per point: its row, its index and its share of the histogram of its chunk
                static_cast<long long>((scratchBytes / sizeof(float) - 2.0 * SLABS) / (channels + 1 + static_cast<double>(SLABS) / CHUNK))));
        if (device_code::claimStaticScratch(stream, error) != 0) throw std::runtime_error(error);
        totals = static_cast<int*>(scratch);
    } else {
        if (po.capacityWords < words) {
            if (words > std::numeric_limits<int32_t>::max()) return false;   // beyond one tensor: the batch stays as it is
            po.workspace = Tensor(Tensor::FLOAT, {static_cast<int32_t>(words)});
            po.capacityWords = words;
        }
        totals = reinterpret_cast<int*>(po.workspace.dataPtr<float>());
        // resolves the static buffer of inferenceNoAlloc() on this device while allocating is
        // still allowed (the first look-up loads the library's own code object)
        void* scratch = nullptr;
        size_t scratchBytes = 0;
        std::string error;
        (void)device_code::staticScratch(&scratch, &scratchBytes, error);
    }
    int* histogram = totals + SLABS;
    // the histograms are a multiple of 4 KiB: the sorted rows behind them stay 16-byte aligned
    float* sortedData = destination ? static_cast<float*>(destination) : reinterpret_cast<float*>(totals + histogramWords);
    int* orderData = reinterpret_cast<int*>(sortedData + static_cast<long long>(numel) * channels);
    // a training pass keeps the points per slab with its sorted rows: the adjoint pass may walk the batch slab by slab
    static_assert(SLABS == SORT_SLABS, "the slabs of kernels/point_order.h");
    if (destination) totals = reinterpret_cast<int*>(static_cast<char*>(destination) + (sortedTotalsOffset(numel) - sortedRowsOffset(numel)));
    // ... and for every point its place in the sorted order: rows computed in that order are gathered back with it
    int* placement = destination ? reinterpret_cast<int*>(static_cast<char*>(destination) + (sortedPlacementOffset(numel) - sortedRowsOffset(numel)))
                                 : nullptr;

    int count = numel;
    auto inputAcc = input.accessor<kernel::Tensor2Read<float>>();
    int chunks = divUp(numel, CHUNK);
    {
        void* args[] = {&count, &inputAcc, &key, &histogram};
        po.count.value().launch(chunks, BLOCK, 0, stream, args);
    }
    {
        void* args[] = {&chunks, &histogram, &totals};
        po.scan.value().launch(SLABS / 16, BLOCK, 0, stream, args);   // 16 slabs per workgroup (POINT_ORDER_SCAN_SLABS)
    }
    {
        void* args[] = {&count, &inputAcc, &key, &histogram, &totals, &sortedData, &orderData, &placement};
        po.scatter.value().launch(chunks, BLOCK, 0, stream, args);
    }
    sortedInput.data_ = sortedData;
    sortedInput.sizes_[0] = numel;
    sortedInput.sizes_[1] = channels;
    sortedInput.strides_[0] = channels;
    sortedInput.strides_[1] = 1;
    order = orderData;
    return true;
}

size_t FusedNetwork::forwardMemory(int numElements, AdjointModeFlags adjointFlags)
{
    // The size does not depend on the flags (a caller may size the memory once for several kinds of passes); they
    // announce what the adjoint pass will ask for, which decides whether forward() stores position derivatives.
    if (adjointFlags > 0 && adjointFlags < ADJOINT_MODE_MAX_COMBINATIONS) announcedFlags_ = adjointFlags;
    // a batch that trains in sorted order: its sorted rows and the order, behind the intermediates and the derivatives
    if (sortsTraining(numElements))
        return sortedPlacementOffset(numElements) + roundUp(static_cast<size_t>(numElements) * sizeof(int), size_t(256));
    numElements = roundUp(numElements, WARP_SIZE);
    return forwardBytesPerPoint() * static_cast<size_t>(numElements);
}

size_t FusedNetwork::forwardMemory(const Tensor& input, AdjointModeFlags adjointFlags)
{
    CHECK_DIM(input, 2);
    CHECK_SIZE(input, 1, channelsIn());
    return forwardMemory(input.size(0), adjointFlags);
}

void FusedNetwork::forward(const Tensor& input, Tensor& output, void* tmpMemory, stream_t stream)
{
    CHECK_DIM(input, 2);
    CHECK_DIM(output, 2);
    CHECK_SIZE(input, 1, channelsIn());
    CHECK_SIZE(output, 1, channelsOut());
    int numel = input.size(0);
    CHECK_SIZE(output, 0, numel);
    CHECK_DTYPE(input, precisionIn());
    CHECK_DTYPE(output, precisionOut());
    CHECK_ERROR(parametersInference_.defined(), "Inference parameters not defined, call setNetworkParameter(...) first");
    checkEncodingParameters(Tensor::INFERENCE);
    if (numel == 0) return;
    CHECK_ERROR(tmpMemory != nullptr, "forward() needs temporary memory of forwardMemory() bytes");
    CHECK_ERROR(reinterpret_cast<uintptr_t>(tmpMemory) % 16 == 0, "The temporary memory must be aligned to 16 bytes");

    const bool derivatives = storesDerivatives(numel, announcedFlags_);
    const bool inputOnly = recomputes(numel, announcedFlags_);
    if (derivatives || inputOnly) forwardRecords_[tmpMemory] = ForwardRecord{numel, derivatives, inputOnly};
    else forwardRecords_.erase(tmpMemory);
    launchForward(true, input, output, static_cast<half*>(tmpMemory), stream, false, derivatives, inputOnly);
}

void FusedNetwork::zeroGradients()
{
    if (parametersGradients_.defined()) parametersGradients_.zero_();
    for (auto& e : encodings_) e->zeroGradients();
}

size_t FusedNetwork::adjointMemory(int numElements, AdjointModeFlags adjointFlags)
{
    const size_t bytes = adjointMemoryAsGiven(numElements, adjointFlags);
    return bytes + sortedAdjointBytes(numElements, adjointFlags, bytes);
}

size_t FusedNetwork::adjointMemoryAsGiven(int numElements, AdjointModeFlags adjointFlags) const
{
    if (adjointFlags <= 0 || adjointFlags >= ADJOINT_MODE_MAX_COMBINATIONS)
        throw std::runtime_error("At least one derivative must be enabled");
    // batches that take the gradient slice kernels: the adjoint of the encoded rows, which the records kernels read
    const bool sliceGradients = useSliceGradients(numElements, adjointFlags);
    int perEntry = storedAdjointChannels(adjointFlags, sliceGradients) * static_cast<int>(sizeof(half));
    if (sliceGradients) perEntry += sliceGradientBytesPerPoint();
    numElements = roundUp(numElements, WARP_SIZE);
    size_t bytes = static_cast<size_t>(perEntry) * static_cast<size_t>(numElements);
    // behind the adjoint pre-activations: the partial weight gradients of the batch slices
    if (adjointFlags & GRADIENTS_NETWORK_WEIGHTS)
        bytes += static_cast<size_t>(weightUpdateSlices(numElements / TILE_POINTS)) * numParameters_ * sizeof(float);
    // last: transposed copies of the weights the adjoint kernel cannot keep in LDS
    std::vector<long long> transposed;
    bytes += roundUp(transposedWeightLayout(adjointFlags, transposed) * sizeof(half), size_t(16));
    // last: bucket cursors and records of the gradient slice kernels
    if (sliceGradients) bytes = roundUp(bytes, size_t(256)) + sliceGradientWorkspaceBytes(numElements);
    return bytes;
}

size_t FusedNetwork::sortedAdjointBytes(int numElements, AdjointModeFlags adjointFlags, size_t bytesInFront) const
{
    // A batch that trains in sorted order: the input gradients in that order before they are added to the caller's
    // rows (dense, 256-byte aligned, behind everything else).
    if (!sortsTraining(numElements) || !(adjointFlags & GRADIENTS_INPUT)) return 0;
    size_t bytes = roundUp(bytesInFront, size_t(256)) - bytesInFront;
    bytes += roundUp(static_cast<size_t>(numElements) * channelsIn() * sizeof(float), size_t(256));
    return bytes;
}

size_t FusedNetwork::adjointMemory(const Tensor& input, AdjointModeFlags adjointFlags)
{
    CHECK_DIM(input, 2);
    CHECK_SIZE(input, 1, channelsIn());
    return adjointMemory(input.size(0), adjointFlags);
}

void FusedNetwork::adjoint(const Tensor& input, const Tensor& adjOutput, AdjointModeFlags adjointFlags,
                           Tensor& adjInput, const void* tmpMemoryForward, void* tmpMemoryAdjoint, stream_t stream)
{
    CHECK_DIM(input, 2);
    CHECK_DIM(adjOutput, 2);
    CHECK_SIZE(input, 1, channelsIn());
    CHECK_SIZE(adjOutput, 1, channelsOut());
    int numel = input.size(0);
    CHECK_SIZE(adjOutput, 0, numel);
    CHECK_DTYPE(input, precisionIn());
    CHECK_DTYPE(adjOutput, precisionOut());
    if (adjointFlags <= 0 || adjointFlags >= ADJOINT_MODE_MAX_COMBINATIONS)
        throw std::runtime_error("At least one derivative must be enabled");

    const bool hasInputGradients = adjointFlags & GRADIENTS_INPUT;
    const bool hasNetworkGradients = adjointFlags & GRADIENTS_NETWORK_WEIGHTS;
    const bool hasEncodingGradients = adjointFlags & GRADIENTS_INPUT_ENCODINGS;

    if (hasInputGradients) {
        CHECK_ERROR(adjInput.defined(), "Input gradients requested, but adjInput is undefined");
        CHECK_DIM(adjInput, 2);
        CHECK_SIZE(adjInput, 1, channelsIn());
        CHECK_SIZE(adjInput, 0, numel);
        CHECK_DTYPE(adjInput, precisionIn());
    }
    if (hasNetworkGradients)
        CHECK_ERROR(parametersGradients_.defined(),
                    "Network gradients requested, but no gradient tensor was set via setNetworkParameter(..., GRADIENTS)");
    CHECK_ERROR(parametersInference_.defined(), "Inference parameters not defined, call setNetworkParameter(...) first");
    checkEncodingParameters(Tensor::INFERENCE);
    // the kernel adds the gradients of every encoding that has parameters: each needs a tensor to add into
    if (hasEncodingGradients) checkEncodingParameters(Tensor::GRADIENTS);
    if (numel == 0) return;
    CHECK_ERROR(tmpMemoryForward != nullptr, "adjoint() needs the temporary memory written by forward()");
    std::vector<long long> transposedOffsets;
    const size_t transposedHalves = transposedWeightLayout(adjointFlags, transposedOffsets);
    if (hasNetworkGradients || transposedHalves > 0 || useSliceGradients(numel, adjointFlags) || sortsTraining(numel)) {
        CHECK_ERROR(tmpMemoryAdjoint != nullptr, "adjoint() needs temporary memory of adjointMemory() bytes");
        CHECK_ERROR(reinterpret_cast<uintptr_t>(tmpMemoryAdjoint) % 16 == 0, "The temporary memory must be aligned to 16 bytes");
    }

    const bool sliceGradients = useSliceGradients(numel, adjointFlags);
    CHECK_ERROR(!sliceGradients || numel < (1 << 27), "batches of 2^27 points or more: set options.slice_gradients to 0");
    announcedFlags_ = adjointFlags;
    // what the forward pass that wrote this forward memory left there: the position derivatives of the grids? Of the
    // intermediates the encoded input only?
    bool derivativesStored = false, recompute = false;
    {
        const auto it = forwardRecords_.find(tmpMemoryForward);
        if (it != forwardRecords_.end() && it->second.numel == numel) {
            derivativesStored = hasInputGradients && sliceGradients && it->second.derivatives;
            if (it->second.inputOnly) {
                if (recomputes(numel, adjointFlags)) {
                    recompute = true;
                } else {
                    // Announced otherwise: the kernels of these flags read intermediates that the training pass did not
                    // keep. The forward pass runs again into the same memory, this time storing them (a batch that
                    // trains in sorted order is sorted again: rows, order and slab totals are rewritten together).
                    QuickMLP::Instance().getLogger()->debug("adjoint(flags %d): the forward pass kept the encoded input only; it runs again", adjointFlags);
                    Tensor scratchOutput(precisionOut(), {numel, channelsOut()});
                    const bool derivatives = it->second.derivatives;
                    it->second.inputOnly = false;
                    launchForward(true, input, scratchOutput, static_cast<half*>(const_cast<void*>(tmpMemoryForward)), stream, false, derivatives, false);
                }
            }
        }
    }
    const bool sortedPoints = sortsTraining(numel);
    compileBackwardKernel(adjointFlags, sliceGradients, false, recompute);
    auto& ak = backwardKernel_[adjointFlags][sliceGradients ? 1 : 0][recompute ? 1 : 0].value();

    const int numTiles = divUp(numel, TILE_POINTS);
    const long long numel64 = static_cast<long long>(numTiles) * TILE_POINTS;
    // a batch that the forward pass evaluated in sorted order: the rows as it sorted them, and for every row its
    // place in the caller's batch (rows of dL/dy are read, rows of the input gradients written through it)
    auto sortedInput = input.accessor<kernel::Tensor2Read<float>>();
    auto sortedAdjOutput = adjOutput.accessor<kernel::Tensor2Read<float>>();
    kernel::Tensor2RW<float> sortedAdjInput;
    std::memset(&sortedAdjInput, 0, sizeof(sortedAdjInput));
    if (hasInputGradients) sortedAdjInput = adjInput.accessor<kernel::Tensor2RW<float>>();
    const int* pointOrder = nullptr;
    const int* adjOutputOrder = nullptr;
    if (sortedPoints) {
        const float* rows = reinterpret_cast<const float*>(static_cast<const char*>(tmpMemoryForward) + sortedRowsOffset(numel));
        sortedInput.data_ = rows;
        sortedInput.strides_[0] = channelsIn();
        sortedInput.strides_[1] = 1;
        pointOrder = reinterpret_cast<const int*>(rows + static_cast<long long>(numel) * channelsIn());
        // The backward kernel reads its rows of dL/dy through the order (one index and one row of C_out floats per point
        // and tile: BASELINE config 5, rows of 8 bytes, kernel 135 -> 151 us against a gather kernel of 34 us in front
        // of it). The input gradients go the other way through dense rows behind the adjoint memory and one streaming
        // kernel: scattered 16-byte read-modify-writes from inside the kernels cost more than that kernel's 44 us.
        adjOutputOrder = pointOrder;
        loadPointOrderKernels(true);
        char* staging = static_cast<char*>(tmpMemoryAdjoint) + roundUp(adjointMemoryAsGiven(numel, adjointFlags), size_t(256));
        if (hasInputGradients) {
            float* adjInputRows = reinterpret_cast<float*>(staging);
            QMLP_HIP_CALL(qmlp_hip_memset_async(adjInputRows, 0, static_cast<size_t>(numel) * channelsIn() * sizeof(float), stream));
            sortedAdjInput.data_ = adjInputRows;
            sortedAdjInput.strides_[0] = channelsIn();
            sortedAdjInput.strides_[1] = 1;
        }
    }
    const half* transposedWeights = nullptr;
    if (transposedHalves > 0) {
        size_t offset = static_cast<size_t>(ak.perEntryAdjointMemoryBytes) * static_cast<size_t>(numel64);
        if (hasNetworkGradients) offset += static_cast<size_t>(weightUpdateSlices(numTiles)) * numParameters_ * sizeof(float);
        half* dstBase = reinterpret_cast<half*>(static_cast<char*>(tmpMemoryAdjoint) + offset);
        transposedWeights = dstBase;
        for (size_t layer = 0; layer < layers_.size(); ++layer) {
            if (transposedOffsets[layer] < 0) continue;
            const auto& ls = layers_[layer];
            const half* src = parametersInference_.dataPtr<half>() + ls.weightsStart;
            half* dst = dstBase + transposedOffsets[layer];
            int cout = ls.channelsOut, cin = ls.channelsIn;
            void* args[] = {&src, &dst, &cout, &cin};
            const int tiles = (cout / MATRIX_SIZE) * (cin / MATRIX_SIZE);
            ak.transpose.fun.launch(std::min(tiles, 1024), ak.transpose.blockSize, 0, stream, args);
        }
    }
    {
        const auto& ck = ak.adjoint;
        const int waves = ck.blockSize / WARP_SIZE;
        int grid = std::min(divUp(numTiles, waves), ck.fullGrid);
        // every workgroup stores its sums of the weight gradients as one of the slices of the batch that the
        // reduction adds up (and zeroes its share of the slices beyond the grid)
        int partialSlices = weightUpdateSlices(numTiles);
        if (ak.fusedWeightUpdate) grid = std::min(grid, partialSlices);
        auto inputAcc = sortedInput;
        auto adjOutputAcc = sortedAdjOutput;
        auto adjInputAcc = sortedAdjInput;
        const half* networkParams = parametersInference_.dataPtr<half>();
        const half* forwardTmpMemory = static_cast<const half*>(tmpMemoryForward);
        half* adjointTmpMemory = static_cast<half*>(tmpMemoryAdjoint);
        float* partialGradients = reinterpret_cast<float*>(static_cast<char*>(tmpMemoryAdjoint)
                                                           + static_cast<size_t>(ak.perEntryAdjointMemoryBytes) * static_cast<size_t>(numel64));
        std::vector<void*> args = {&numel, &inputAcc, &adjOutputAcc, &adjInputAcc, &networkParams,
                                   &forwardTmpMemory, &adjointTmpMemory, &transposedWeights, &partialGradients, &partialSlices};
        CHECK_ERROR(ak.outputOrder || adjOutputOrder == nullptr, "a batch trains in sorted order but the backward kernel does not take the order");
        if (ak.outputOrder) args.push_back(&adjOutputOrder);
        std::vector<std::vector<char>> storage;
        encodingArguments(args, storage);
        ck.fun.launch(grid, ck.blockSize, ck.sharedMemorySize, stream, args.data());
    }
    // parameter gradients of the grids, slice by slice, from the adjoint of the encoded rows the kernel above stored
    if (!ak.sliceGradients.empty()) {
        const half* adjEncoded = static_cast<const half*>(tmpMemoryAdjoint) + static_cast<ptrdiff_t>(storedAdjointChannels(adjointFlags, true)) * numel64;
        // the workspace is the last part of the adjoint memory: everything in front of it
        size_t offset = static_cast<size_t>(ak.perEntryAdjointMemoryBytes) * static_cast<size_t>(numel64);
        if (hasNetworkGradients) offset += static_cast<size_t>(weightUpdateSlices(numTiles)) * numParameters_ * sizeof(float);
        offset += roundUp(transposedHalves * sizeof(half), size_t(16));
        char* workspace = static_cast<char*>(tmpMemoryAdjoint) + roundUp(offset, size_t(256));
        auto inputAcc = sortedInput;
        for (auto& sk : ak.sliceGradients) {
            const auto& layout = sk.layout;
            kernel::PointOrderKey sortKey{};
            if (sortedPoints && sk.columnsOffered && pointOrderFor(numel, sortKey)) {
                IEncoding::GradientColumnLayout sortedFor;
                if (encodings_[sk.encoding]->gradientColumns(sortKey, sortedFor)
                    && columnWorkspaceBytes(sk.columnLayout, numel) <= sliceGradientWorkspaceBytes(numel64)) {
                    // the batch is sorted by the slabs of this grid: its gradients owner by owner, without records
                    const bool fromDerivatives = derivativesStored && sk.derivativeOffset >= 0;
                    compileColumnKernels(sk, adjointFlags, false, fromDerivatives);
                    int maxItems = 0;
                    (void)columnWorkspaceBytes(sk.columnLayout, numel, &maxItems);
                    int* starts = reinterpret_cast<int*>(workspace);
                    int* itemCount = starts + SORT_SLABS + 1;
                    void* items = workspace + roundUp(static_cast<size_t>(SORT_SLABS + 1 + 1) * sizeof(int), size_t(256));
                    const int* totals = reinterpret_cast<const int*>(static_cast<const char*>(tmpMemoryForward) + sortedTotalsOffset(numel));
                    int slabs0 = sortKey.slabs0, slabs1 = sortKey.slabs1;
                    std::vector<char> params(1024);
                    int n = encodings_[sk.encoding]->fillParameterMemory(params.data(), static_cast<int>(params.size()));
                    (void)n;
                    {
                        void* args[] = {&numel, &totals, &slabs0, &slabs1, &starts, &items, &itemCount, &maxItems};
                        sk.columnsPlan.value().fun.launch(1, sk.columnsPlan.value().blockSize, 0, stream, args);
                    }
                    {
                        const int* startsRead = starts;
                        const void* itemsRead = items;
                        const int* itemCountRead = itemCount;
                        auto adjInputAcc = sortedAdjInput;
                        const void* derivatives = static_cast<const char*>(tmpMemoryForward)
                            + (static_cast<long long>(perEntryForwardMemoryBytes_) + std::max(0ll, sk.derivativeOffset)) * numel64;
                        void* args[] = {&numel, &inputAcc, &adjEncoded, params.data(), &startsRead, &slabs0, &slabs1, &itemsRead, &itemCountRead,
                                        &adjInputAcc, &derivatives};
                        const auto& ck = sk.columns[fromDerivatives ? 1 : 0].value();
                        ck.fun.launch(maxItems, ck.blockSize, ck.sharedMemorySize, stream, args);
                    }
                    // (the room of this encoding's cursors and records stays where it is for the encodings behind it)
                    workspace += roundUp(static_cast<size_t>(layout.numBuckets() + 1) * sizeof(int), size_t(256))
                        + roundUp(static_cast<size_t>(layout.totalRecords(numel64)) * layout.recordWords * sizeof(uint32_t), size_t(256));
                    continue;
                }
            }
            int* cursors = reinterpret_cast<int*>(workspace);
            const size_t cursorBytes = roundUp(static_cast<size_t>(layout.numBuckets() + 1) * sizeof(int), size_t(256));
            uint32_t* records = reinterpret_cast<uint32_t*>(workspace + cursorBytes);
            workspace += cursorBytes + roundUp(static_cast<size_t>(layout.totalRecords(numel64)) * layout.recordWords * sizeof(uint32_t), size_t(256));
            QMLP_HIP_CALL(qmlp_hip_memset_async(cursors, 0, cursorBytes, stream));
            std::vector<char> params(1024);
            int n = encodings_[sk.encoding]->fillParameterMemory(params.data(), static_cast<int>(params.size()));
            (void)n;
            int numelPadded = static_cast<int>(numel64);   // the layout of the buckets is that of adjointMemory()
            {
                // the records kernel walks over the real points, but lays its buckets out for the padded batch
                auto adjInputAcc = sortedAdjInput;   // this grid's share of dL/dinput (zeros in it if none is asked for: unused)
                const bool fromDerivatives = derivativesStored && sk.derivativeOffset >= 0;
                const void* derivatives = static_cast<const char*>(tmpMemoryForward)
                    + (static_cast<long long>(perEntryForwardMemoryBytes_) + std::max(0ll, sk.derivativeOffset)) * numel64;
                void* args[] = {&numel, &numelPadded, &inputAcc, &adjEncoded, params.data(), &records, &cursors, &adjInputAcc, &derivatives};
                const CompiledKernel& rk = recordsKernelFor(sk, adjointFlags, numel, fromDerivatives);
                rk.fun.launch(std::min(divUp(numel, rk.blockSize), rk.fullGrid), rk.blockSize, rk.sharedMemorySize, stream, args);
            }
            const uint32_t* recordsRead = records;
            const int* cursorsRead = cursors;
            float* gradients = nullptr;
            std::memcpy(&gradients, params.data() + sizeof(void*), sizeof(void*));   // HashGridParams: forward table, gradient table, ...
            const void* items = sk.items.rawPtr();
            void* args[] = {&numelPadded, &recordsRead, &cursorsRead, &gradients, &items};
            sk.kernel.fun.launch(static_cast<int>(layout.items.size()), sk.kernel.blockSize, sk.kernel.sharedMemorySize, stream, args);
        }
    }

    // the input gradients of a batch that trained in sorted order: back to the caller's rows
    if (sortedPoints && hasInputGradients) {
        long long elements = static_cast<long long>(numel) * channelsIn();
        int channels = channelsIn();
        const float* src = sortedAdjInput.data_;
        auto dst = adjInput.accessor<kernel::Tensor2RW<float>>();
        const int* placement = reinterpret_cast<const int*>(static_cast<const char*>(tmpMemoryForward) + sortedPlacementOffset(numel));
        void* args[] = {&elements, &channels, &src, &placement, &dst};
        pointOrder_.gatherAddRows.value().launch(static_cast<int>(std::min<long long>(divUp<long long>(elements, 1024), 1 << 16)), 1024, 0,
                                                  stream, args);
    }

    if (!hasNetworkGradients) return;

    const bool parallel = compileOptions_.parallelWeightUpdate && layers_.size() > 1;
    if (parallel) {
        ensureStreams();
        QMLP_HIP_CALL(qmlp_hip_event_record(adjointEvent_, stream));
    }
    const int slices = weightUpdateSlices(numTiles);
    float* partial = reinterpret_cast<float*>(static_cast<char*>(tmpMemoryAdjoint)
                                              + static_cast<size_t>(ak.perEntryAdjointMemoryBytes) * static_cast<size_t>(numel64));
    for (size_t layer = 0; layer < layers_.size(); ++layer) {
        if (ak.fusedLayers[layer]) continue;
        const auto& ls = layers_[layer];
        const auto& ali = backwardInfo_[layer];
        const auto& wk = ak.layers[layer];

        float* outAdjWeights = partial + ls.weightsStart;
        float* outAdjBias = ls.useBias ? partial + ls.biasStart : nullptr;
        int sliceStride = numParameters_;
        const half* aIn = static_cast<const half*>(tmpMemoryAdjoint) + static_cast<ptrdiff_t>(ali.offsetAdjOut) * numel64;
        const half* bIn = static_cast<const half*>(tmpMemoryForward) + static_cast<ptrdiff_t>(ali.offsetIn) * numel64;

        stream_t layerStream = stream;
        if (parallel) {
            layerStream = ali.stream;
            QMLP_HIP_CALL(qmlp_hip_stream_wait_event(ali.stream, adjointEvent_));
        }
        int numTilesArg = numTiles;
        void* args[] = {&numTilesArg, &outAdjWeights, &outAdjBias, &sliceStride, &aIn, &bIn};
        wk.kernel.fun.launch(slices * wk.numChunks, wk.kernel.blockSize, wk.kernel.sharedMemorySize, layerStream, args);
        if (parallel) {
            QMLP_HIP_CALL(qmlp_hip_event_record(ali.event, ali.stream));
            QMLP_HIP_CALL(qmlp_hip_stream_wait_event(stream, ali.event));
        }
    }
    {
        int count = numParameters_, numSlices = slices;
        const float* partialArg = partial;
        float* gradBase = parametersGradients_.dataPtr<float>();
        void* args[] = {&count, &numSlices, &partialArg, &gradBase};
        ak.reduce.fun.launch(divUp(numParameters_, WARP_SIZE), ak.reduce.blockSize, 0, stream, args);
    }
}

void FusedNetwork::clearCachedKernels()
{
    for (auto& perStore : forwardKernels_)
        for (auto& k : perStore) k = {};
    for (int i = 0; i < ADJOINT_MODE_MAX_COMBINATIONS; ++i)
        for (auto& perSlices : backwardKernel_[i])
            for (auto& k : perSlices) k = {};
    for (auto& perFlags : recomputeVerdict_) perFlags[0] = perFlags[1] = -1;
    pointOrder_.scan = {};
    pointOrder_.count = {};
    pointOrder_.scatter = {};
    pointOrder_.gatherAddRows = {};
}

QUICKMLP_NAMESPACE_END
