#include <qmlp/activation.h>

#include <qmlp/errors.h>
#include <qmlp/qmlp.h>

#include <cctype>
#include <fstream>
#include <regex>
#include <sstream>

QUICKMLP_NAMESPACE_BEGIN

static std::string withoutSpaces(const std::string& s)
{
    std::string o;
    for (char c : s)
        if (!std::isspace(static_cast<unsigned char>(c))) o += c;
    return o;
}

/**
 * Packed form of snippets that are recognised literally (after removing white space): the
 * kernels apply it to four values at once (two packed instructions) instead of calling the
 * scalar snippet four times. Unknown snippets have none.
 */
static std::string packedForward(const std::string& forward)
{
    const std::string f = withoutSpaces(forward);
    if (f == "z=__hgt(x,hZERO())?x:hZERO()")   // ReLU: v_pk_max_f16 (NaN -> 0 like the comparison)
        return "        return __builtin_elementwise_max(x, f16x4{0, 0, 0, 0});\n";
    if (f == "z=x") return "        return x;\n";
    return "";
}

static std::string generateCode(const std::string& id, const std::string& forward, const std::string& adjoint)
{
    static const char* TEMPLATE = R"code(
struct %s
{
    static __device__ __forceinline__ half forward(half x) {
        half z;
        %s ;
        return z;
    }
    static __device__ __forceinline__ half adjoint(half x, half adjz) {
        half adjx;
        %s ;
        return adjx;
    }
%s};
    )code";

    static const std::regex CPP_IDENTIFIER_REGEX("^[a-zA-Z_][a-zA-Z0-9_]*$");
    if (!std::regex_match(id, CPP_IDENTIFIER_REGEX))
        throw configuration_error("id of the activation function is not a valid C++ identifier: %s", id.c_str());
    std::string packed = packedForward(forward);
    if (!packed.empty())
        packed = "    static __device__ __forceinline__ f16x4 forward4(f16x4 x) {\n" + packed + "    }\n";
    return format(TEMPLATE, id.c_str(), forward.c_str(), adjoint.c_str(), packed.c_str());
}

Activation::Activation(const std::string& id, const std::string& forward, const std::string& adjoint)
    : id_(id), forward_(forward), adjoint_(adjoint), code_(generateCode(id, forward, adjoint))
{}

Activation::Activation(const json& cfg)
    : Activation(cfg.at("id").get<std::string>(), cfg.at("forward").get<std::string>(),
                 cfg.at("adjoint").get<std::string>())
{}

json Activation::toJson() const
{
    return json::object({{"id", id()}, {"forward", forward()}, {"adjoint", adjoint()}});
}

static KernelFunction compileActivationKernel(const Activation& a, const char* kernelName, int extraFlags = 0)
{
    auto kl = QuickMLP::Instance().kernelLoader();
    std::string codeTemplate = kl->findFile("qmlp/kernels/activation_kernels.h").value();
    replaceAll(codeTemplate, "$$DEFINE_ACTIVATIONS$$", a.code());
    replaceAll(codeTemplate, "$$ACTIVATION_ID$$", a.id());
    return kl->getKernel(kernelName, codeTemplate, QuickMLP::Instance().getCompileFlags() | extraFlags).value();
}

void Activation::precompile()
{
    compileActivationKernel(*this, "qmlp::kernel::ActivationForwardKernel", KernelLoader::CompileOnly);
    compileActivationKernel(*this, "qmlp::kernel::ActivationAdjointKernel", KernelLoader::CompileOnly);
}

void Activation::forward(const Tensor& input, Tensor& output, stream_t stream)
{
    CHECK_DIM(input, 2);
    CHECK_DIM(output, 2);
    CHECK_DTYPE(input, Tensor::HALF);
    CHECK_DTYPE(output, Tensor::HALF);
    CHECK_SIZE(output, 0, input.size(0));
    CHECK_SIZE(output, 1, input.size(1));
    const long long numel = static_cast<long long>(input.size(0)) * input.size(1);
    if (numel == 0) return;

    if (!forwardKernel_.has_value())
        forwardKernel_ = compileActivationKernel(*this, "qmlp::kernel::ActivationForwardKernel");
    auto& fun = forwardKernel_.value();

    const int block = 256;
    const int grid = static_cast<int>(std::min<long long>(divUp<long long>(numel, block), fun.fullGridSize(block, 0)));
    auto inputAcc = input.accessor<kernel::Tensor2Read<half>>();
    auto outputAcc = output.accessor<kernel::Tensor2RW<half>>();
    fun.call(grid, block, 0, stream, static_cast<int>(input.size(0)), static_cast<int>(input.size(1)), inputAcc, outputAcc);
}

void Activation::adjoint(const Tensor& input, const Tensor& adjOutput, Tensor& adjInput, stream_t stream)
{
    CHECK_DIM(input, 2);
    CHECK_DIM(adjOutput, 2);
    CHECK_DIM(adjInput, 2);
    CHECK_DTYPE(input, Tensor::HALF);
    CHECK_DTYPE(adjOutput, Tensor::HALF);
    CHECK_DTYPE(adjInput, Tensor::HALF);
    CHECK_SIZE(adjOutput, 0, input.size(0));
    CHECK_SIZE(adjOutput, 1, input.size(1));
    CHECK_SIZE(adjInput, 0, input.size(0));
    CHECK_SIZE(adjInput, 1, input.size(1));
    const long long numel = static_cast<long long>(input.size(0)) * input.size(1);
    if (numel == 0) return;

    if (!adjointKernel_.has_value())
        adjointKernel_ = compileActivationKernel(*this, "qmlp::kernel::ActivationAdjointKernel");
    auto& fun = adjointKernel_.value();

    const int block = 256;
    const int grid = static_cast<int>(std::min<long long>(divUp<long long>(numel, block), fun.fullGridSize(block, 0)));
    auto inputAcc = input.accessor<kernel::Tensor2Read<half>>();
    auto adjOutputAcc = adjOutput.accessor<kernel::Tensor2Read<half>>();
    auto adjInputAcc = adjInput.accessor<kernel::Tensor2RW<half>>();
    fun.call(grid, block, 0, stream, static_cast<int>(input.size(0)), static_cast<int>(input.size(1)),
             inputAcc, adjOutputAcc, adjInputAcc);
}

ActivationFactory::ActivationFactory(const json& cfg, const std::filesystem::path& parent, KernelLoader_ptr loader)
{
    if (!cfg.is_array()) throw configuration_error("The activation specification tag must contain an array");

    for (const auto& element : cfg) {
        if (element.is_string()) {
            const std::string filename = element.get<std::string>();
            std::filesystem::path path = filename;
            std::error_code ec;
            //1. Direct
            if (std::filesystem::is_regular_file(path, ec)) {
                parseFile(path);
                continue;
            }
            if (path.is_absolute())
                throw configuration_error(
                    "Absolute path '%s' does not exist. Can't continue resolving the activation file, relative path required",
                    filename.c_str());
            //2. Relative to parent
            path = parent / filename;
            if (std::filesystem::is_regular_file(path, ec)) {
                parseFile(path);
                continue;
            }
            //3. built-in activations
            auto content = loader->findFile(filename);
            if (content.has_value()) {
                parseFile(json::parse(content.value()));
                continue;
            }
            throw configuration_error("Path to activation file '%s' could not be resolved. Is the filename correct?",
                                      filename.c_str());
        } else if (element.is_object()) {
            parseActivation(element, true);   //inline specification
        } else {
            const std::string es = element.dump();
            throw configuration_error(
                "Unknown type of element '%s', only filenames (strings) or in-place specifications (objects) supported.",
                es.c_str());
        }
    }
}

ActivationFactory::ActivationFactory(KernelLoader_ptr loader)
{
    auto content = loader->findFile("qmlp/builtin-activations.json");
    if (!content.has_value()) throw configuration_error("File with builtin activations not found");
    parseFile(json::parse(content.value()));
}

Activation_ptr ActivationFactory::get(const std::string& key) const
{
    auto it = activations_.find(key);
    if (it == activations_.end()) throw configuration_error("No activation with id '%s' found!", key.c_str());
    return it->second;
}

Activation_ptr ActivationFactory::getOrInline(const std::string& key)
{
    if (key.empty()) throw std::runtime_error("empty key");
    if (key[0] == '{') return parseActivation(json::parse(key), false);
    return get(key);
}

void ActivationFactory::parseFile(const std::filesystem::path& file)
{
    std::ifstream in(file);
    std::stringstream ss;
    ss << in.rdbuf();
    json j = json::parse(ss.str());
    if (!j.is_array())
        throw configuration_error("Activation file '%s' is expected to contain an array object as the root element",
                                  file.c_str());
    parseFile(j);
}

void ActivationFactory::parseFile(const json& j)
{
    if (!j.is_array()) throw configuration_error("Activation specifications are expected to be an array");
    for (const auto& element : j) parseActivation(element, true);
}

Activation_ptr ActivationFactory::parseActivation(const json& cfg, bool emplace)
{
    try {
        Activation_ptr a = std::make_shared<Activation>(cfg);
        if (emplace) activations_[a->id()] = a;
        return a;
    } catch (const std::exception&) {
        std::throw_with_nested(configuration_error("Parsing the activation configuration failed."));
    }
}

QUICKMLP_NAMESPACE_END
