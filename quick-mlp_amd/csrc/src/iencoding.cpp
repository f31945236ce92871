#include <qmlp/iencoding.h>

#include <qmlp/encoding_hashgrid.h>
#include <qmlp/encoding_line_integration.h>
#include <qmlp/encoding_identity.h>
#include <qmlp/qmlp.h>

#include <cctype>
#include <cstring>

QUICKMLP_NAMESPACE_BEGIN

namespace {

// Kernel arguments of the standalone kernels: fixed ones plus the optional parameter struct.
struct ArgPack
{
    std::vector<void*> ptrs;
    std::vector<char> paramBytes;
};

std::string standaloneSource(const IEncoding& e, const std::string& callForward, const std::string& callAdjoint,
                             const std::string& callCorners = "", const std::string& callScatter = "",
                             const std::string& callTraceGather = "", const std::string& callTraceScatter = "")
{
    auto kl = QuickMLP::Instance().kernelLoader();
    std::string codeTemplate = kl->findFile("qmlp/kernels/encoding_kernels.h").value();
    std::stringstream includes;
    e.fillCode(includes);
    includes << "\n";
    replaceAll(codeTemplate, "$$INCLUDES$$", includes.str());
    replaceAll(codeTemplate, "$$ENCODING_PARAMETERS$$",
               e.hasParameters() ? ", const " + e.parameterName() + " cEncoding" : std::string());
    replaceAll(codeTemplate, "$$CALL_ENCODINGS_FORWARD$$", callForward);
    replaceAll(codeTemplate, "$$CALL_ENCODINGS_ADJOINT$$", callAdjoint);
    replaceAll(codeTemplate, "$$CALL_ENCODINGS_CORNERS$$", callCorners);
    replaceAll(codeTemplate, "$$CALL_ENCODINGS_SCATTER$$", callScatter);
    replaceAll(codeTemplate, "$$CALL_ENCODINGS_TRACE_GATHER$$", callTraceGather);
    replaceAll(codeTemplate, "$$CALL_ENCODINGS_TRACE_SCATTER$$", callTraceScatter);
    return codeTemplate;
}

} // namespace

std::string IEncoding::forwardKernelSource() const
{
    std::stringstream call;
    call << qualifiedName() << "::forward(encodingInput, encodingOutput";
    if (hasParameters()) call << ", cEncoding";
    call << ");\n";
    return standaloneSource(*this, call.str(), "");
}

std::string IEncoding::adjointKernelSource(int adjointMode) const
{
    const bool hasInputGradients = adjointMode & INPUT_GRADIENTS;
    const bool hasParamGradients = (adjointMode & PARAM_GRADIENTS) && hasParameters();
    // encodings with a tile-wide scatter take their parameter gradients out of the per-point call
    std::stringstream call, scatter;
    call << qualifiedName() << "::template adjoint<" << (hasInputGradients ? "true" : "false") << ", "
         << (hasParamGradients ? "!" + qualifiedName() + "::HasTileScatter" : std::string("false"))
         << ">(encodingInput, encodingAdjOutput, encodingAdjInput";
    if (hasParameters()) call << ", cEncoding";
    call << ");\n";
    if (hasParamGradients)
        scatter << "if constexpr (" << qualifiedName() << "::HasTileScatter)\n            " << qualifiedName()
                << "::scatterTile(lane, tileBase, numel, inputs, [&](int pt, int c) { return adjOutputs.data_[(tileBase + pt)"
                   " * adjOutputs.strides_[0] + static_cast<long long>(c) * adjOutputs.strides_[1]]; }, cEncoding);\n";
    return standaloneSource(*this, "", call.str(), "", scatter.str());
}

void IEncoding::precompile(int adjointMode)
{
    auto kl = QuickMLP::Instance().kernelLoader();
    const int flags = QuickMLP::Instance().getCompileFlags() | KernelLoader::CompileOnly;
    kl->getKernel("qmlp::kernel::EncodingForwardKernel", forwardKernelSource(), flags);
    if (adjointMode > 0) {
        CHECK_ERROR(adjointMode <= ALL_GRADIENTS, "Illegal adjoint mode");
        kl->getKernel("qmlp::kernel::EncodingAdjointKernel", adjointKernelSource(adjointMode), flags);
    }
}

void IEncoding::forward(const Tensor& input, Tensor& output, stream_t stream,
                        const std::optional<const Tensor>& parametersForward)
{
    CHECK_DIM(input, 2);
    CHECK_DIM(output, 2);
    CHECK_DTYPE(input, Tensor::FLOAT);
    CHECK_DTYPE(output, Tensor::FLOAT);
    CHECK_SIZE(output, 0, input.size(0));
    CHECK_ERROR(input.size(1) > maxInputChannel());
    CHECK_ERROR(output.size(1) >= numOutputChannels());
    CHECK_ERROR(output.strides()[1] == 1, "The output stride along the channels must be 1");
    long long numel = input.size(0);
    if (hasParameters())
        CHECK_ERROR((parametersForward.has_value() && parametersForward.value().defined()) || hasParameterTensor(Tensor::INFERENCE),
                    "The encoding has parameters, but no inference tensor is bound or passed");
    if (numel == 0) return;

    if (!forwardKernel_.has_value())
        forwardKernel_ = QuickMLP::Instance().kernelLoader()->getKernel(
            "qmlp::kernel::EncodingForwardKernel", forwardKernelSource(), QuickMLP::Instance().getCompileFlags()).value();
    auto& fun = forwardKernel_.value();

    std::vector<char> paramBytes(4096);
    if (hasParameters()) {
        if (parametersForward.has_value()) setParameter(parametersForward.value(), Tensor::INFERENCE);
        int n = fillParameterMemory(paramBytes.data(), static_cast<int>(paramBytes.size()));
        (void)n;
    }

    const int block = 256;
    const int grid = static_cast<int>(std::min<long long>(divUp<long long>(numel, block), fun.fullGridSize(block, 0)));
    auto inputAcc = input.accessor<kernel::Tensor2Read<float>>();
    auto outputAcc = output.accessor<kernel::Tensor2RW<float>>();
    std::vector<void*> args = {&numel, &inputAcc, &outputAcc};
    if (hasParameters()) args.push_back(paramBytes.data());
    fun.launch(grid, block, 0, stream, args.data());

    if (hasParameters() && parametersForward.has_value()) setParameter({}, Tensor::INFERENCE);
}

void IEncoding::adjoint(const Tensor& input, const Tensor& adjOutput, Tensor& adjInput, stream_t stream,
                        const std::optional<const Tensor>& parametersForward,
                        const std::optional<const Tensor>& parametersGradients, int adjointMode)
{
    CHECK_DIM(input, 2);
    CHECK_DIM(adjOutput, 2);
    CHECK_DIM(adjInput, 2);
    CHECK_DTYPE(input, Tensor::FLOAT);
    CHECK_DTYPE(adjOutput, Tensor::FLOAT);
    CHECK_DTYPE(adjInput, Tensor::FLOAT);
    CHECK_SIZE(adjOutput, 0, input.size(0));
    CHECK_SIZE(adjInput, 0, input.size(0));
    CHECK_ERROR(input.size(1) > maxInputChannel());
    CHECK_ERROR(adjOutput.size(1) >= numOutputChannels());
    CHECK_ERROR(adjInput.size(1) == input.size(1));
    CHECK_ERROR(adjointMode >= 1 && adjointMode <= ALL_GRADIENTS, "Illegal adjoint mode");
    long long numel = input.size(0);
    if (hasParameters()) {
        CHECK_ERROR((parametersForward.has_value() && parametersForward.value().defined()) || hasParameterTensor(Tensor::INFERENCE),
                    "The encoding has parameters, but no inference tensor is bound or passed");
        CHECK_ERROR(!(adjointMode & PARAM_GRADIENTS) || (parametersGradients.has_value() && parametersGradients.value().defined())
                        || hasParameterTensor(Tensor::GRADIENTS),
                    "Parameter gradients requested, but no gradient tensor is bound or passed");
    }
    if (numel == 0) return;

    if (!adjointKernel_[adjointMode].has_value())
        adjointKernel_[adjointMode] = QuickMLP::Instance().kernelLoader()->getKernel(
            "qmlp::kernel::EncodingAdjointKernel", adjointKernelSource(adjointMode),
            QuickMLP::Instance().getCompileFlags()).value();
    auto& fun = adjointKernel_[adjointMode].value();

    std::vector<char> paramBytes(4096);
    if (hasParameters()) {
        if (parametersForward.has_value()) setParameter(parametersForward.value(), Tensor::INFERENCE);
        if (parametersGradients.has_value()) setParameter(parametersGradients.value(), Tensor::GRADIENTS);
        int n = fillParameterMemory(paramBytes.data(), static_cast<int>(paramBytes.size()));
        (void)n;
    }

    const int block = 256;
    const int grid = static_cast<int>(std::min<long long>(divUp<long long>(numel, block), fun.fullGridSize(block, 0)));
    auto inputAcc = input.accessor<kernel::Tensor2Read<float>>();
    auto adjOutputAcc = adjOutput.accessor<kernel::Tensor2Read<float>>();
    auto adjInputAcc = adjInput.accessor<kernel::Tensor2RW<float>>();
    std::vector<void*> args = {&numel, &inputAcc, &adjOutputAcc, &adjInputAcc};
    if (hasParameters()) args.push_back(paramBytes.data());
    fun.launch(grid, block, 0, stream, args.data());

    if (hasParameters() && parametersForward.has_value()) setParameter({}, Tensor::INFERENCE);
    if (hasParameters() && parametersGradients.has_value()) setParameter({}, Tensor::GRADIENTS);
}

void EncodingHashGrid::corners(const Tensor& input, unsigned* indices, float* weights, stream_t stream, int mode)
{
    CHECK_DIM(input, 2);
    CHECK_DTYPE(input, Tensor::FLOAT);
    CHECK_ERROR(input.size(1) > maxInputChannel());
    CHECK_ERROR(mode >= 0 && mode <= 4, "mode 0: the index function, 1: the gathers of the forward pass, 2: the gradient scatter, "
                                        "3: the gradient records of the slice kernels, 4: the sums of the column kernel");
    CHECK_ERROR(mode != 2 || (numFeaturesPerLevel_ & (numFeaturesPerLevel_ - 1)) == 0 && numFeaturesPerLevel_ <= 32,
                "the tile-wide gradient scatter exists for 1, 2, 4 .. 32 features per level");
    CHECK_ERROR(mode == 0 || hasParameterTensor(Tensor::INFERENCE), "the traces read the table: bind one first");
    long long numel = input.size(0);
    if (numel == 0) return;
    if (!cornersKernel_[mode].has_value()) precompileCorners(mode, false);
    auto& fun = cornersKernel_[mode].value();
    std::vector<char> paramBytes(4096);
    int n = fillParameterMemory(paramBytes.data(), static_cast<int>(paramBytes.size()));
    (void)n;
    const int block = 256;
    // modes 0 and 1: a lane per point; mode 2: a wavefront per 64 points
    const int grid = static_cast<int>(std::min<long long>(divUp<long long>(numel, block), fun.fullGridSize(block, 0)));
    auto inputAcc = input.accessor<kernel::Tensor2Read<float>>();
    int perPoint = numLevels() * (1 << ndim());
    if (mode == 3 || mode == 4) {
        void* args[] = {&numel, &inputAcc, &indices, &weights, paramBytes.data()};
        fun.launch(grid, block, 0, stream, args);
        return;
    }
    void* args[] = {&numel, &inputAcc, &indices, &weights, &perPoint, paramBytes.data()};
    fun.launch(grid, block, 0, stream, args);
}

void EncodingHashGrid::precompileCorners(int mode, bool compileOnly)
{
    CHECK_ERROR(mode >= 0 && mode <= 4, "mode 0: the index function, 1: the gathers of the forward pass, 2: the gradient scatter, "
                                        "3: the gradient records of the slice kernels, 4: the sums of the column kernel");
    if (mode == 3) {
        // the record building of kernels/grid_gradient.h with the slice size the fused network uses for this grid
        GradientSliceLayout layout;
        CHECK_ERROR(gradientSlices(layout), "this grid has no gradient slices");
        std::stringstream source;
        fillCode(source);
        source << "\n" << KernelLoader::MainFile("qmlp/kernels/grid_gradient.h");
        const int flags = QuickMLP::Instance().getCompileFlags() | (compileOnly ? KernelLoader::CompileOnly : 0);
        auto kernel = QuickMLP::Instance().kernelLoader()->getKernel(
            "qmlp::kernel::GridGradientTraceKernel<" + layout.configType + ", " + std::to_string(layout.sliceFloats) + ">",
            source.str(), flags);
        if (!compileOnly) cornersKernel_[mode] = kernel.value();
        return;
    }
    if (mode == 4) {
        // the index arithmetic of kernels/grid_gradient_columns.h for the slabs by which the fused network sorts for this grid
        kernel::PointOrderKey key{};
        GradientColumnLayout layout;
        CHECK_ERROR(pointOrderKey(key, 0) && gradientColumns(key, layout), "this grid has no gradient columns");
        std::stringstream source;
        fillCode(source);
        source << "\n" << KernelLoader::MainFile("qmlp/kernels/grid_gradient_columns.h");
        const int flags = QuickMLP::Instance().getCompileFlags() | (compileOnly ? KernelLoader::CompileOnly : 0);
        auto kernel = QuickMLP::Instance().kernelLoader()->getKernel(
            "qmlp::kernel::GridGradientColumnsTraceKernel<" + layout.configType + ", " + std::to_string(layout.cellsPerSlab) + ">",
            source.str(), flags);
        if (!compileOnly) cornersKernel_[mode] = kernel.value();
        return;
    }
    {
        const std::string name = qualifiedName();
        const std::string source = standaloneSource(
            *this, "", "", name + "::corners(encodingInput, cEncoding, cornerIndices, cornerWeights);\n", "",
            name + "::traceGather(encodingInput, cEncoding, cornerIndices, cornerWeights);\n",
            name + "::traceScatter(lane, tileBase, numel, inputs, cEncoding, indices, weights);\n");
        const char* kernels[] = {"qmlp::kernel::EncodingCornersKernel", "qmlp::kernel::EncodingTraceKernel<1>",
                                 "qmlp::kernel::EncodingTraceKernel<2>"};
        const int flags = QuickMLP::Instance().getCompileFlags() | (compileOnly ? KernelLoader::CompileOnly : 0);
        auto kernel = QuickMLP::Instance().kernelLoader()->getKernel(kernels[mode], source, flags);
        if (!compileOnly) cornersKernel_[mode] = kernel.value();
    }
}

EncodingFactory::EncodingFactory()
{
    encodings_[EncodingIdentity::ID()] = [](const json& cfg) { return std::make_shared<EncodingIdentity>(cfg); };
    encodings_[EncodingHashGrid::ID()] = [](const json& cfg) { return std::make_shared<EncodingHashGrid>(cfg); };
    encodings_[EncodingLineIntegration::ID()] = [](const json& cfg) { return std::make_shared<EncodingLineIntegration>(cfg); };
}

EncodingFactory& EncodingFactory::Instance()
{
    static EncodingFactory INSTANCE;
    return INSTANCE;
}

static std::string lowerCase(std::string s)
{
    for (auto& c : s) c = static_cast<char>(std::tolower(static_cast<unsigned char>(c)));
    return s;
}

IEncoding_ptr EncodingFactory::create(const json& cfg)
{
    const std::string id = cfg.at("id").get<std::string>();
    auto it = encodings_.find(id);
    if (it == encodings_.end()) {
        // The reference matches the id exactly, but its own sample specifications write
        // "identity" for "Identity" (network_configs/test1.json:9, README.md:76): match
        // without regard to case.
        for (auto jt = encodings_.begin(); jt != encodings_.end(); ++jt)
            if (lowerCase(jt->first) == lowerCase(id)) it = jt;
    }
    if (it == encodings_.end()) throw configuration_error("No encoding with id '%s' found", id.c_str());
    return it->second(cfg);
}

QUICKMLP_NAMESPACE_END
