// C ABI of the fused operators (include/qmlp_capi.h): thin exception-to-status wrappers
// around the C++ host classes.
#include "qmlp_capi.h"

#include <qmlp/activation.h>
#include <qmlp/encoding_hashgrid.h>
#include <qmlp/fused_network.h>
#include <qmlp/iencoding.h>
#include <qmlp/qmlp.h>
#include <qmlp/utils.h>

#include <cstdlib>
#include <cstring>
#include <random>

using namespace qmlp;

struct qmlp_network_s
{
    FusedNetwork_ptr network;
    std::vector<std::unique_ptr<qmlp_encoding_s>> encodings;
};
struct qmlp_encoding_s
{
    IEncoding_ptr encoding;
};
struct qmlp_activation_s
{
    Activation_ptr activation;
};

namespace {

thread_local std::string g_error;

int handleException()
{
    try {
        throw;
    } catch (const configuration_error& e) {
        g_error = describeException(e);
        return 1;
    } catch (const json::parse_error& e) {
        g_error = describeException(e);
        return 1;
    } catch (const json::type_error& e) {
        g_error = describeException(e);
        return 1;
    } catch (const json::out_of_range& e) {
        g_error = describeException(e);
        return 1;
    } catch (const hip_error& e) {
        g_error = describeException(e);
        return 3;
    } catch (const std::exception& e) {
        g_error = describeException(e);
        return 2;
    } catch (...) {
        g_error = "unknown error";
        return 2;
    }
}

#define QMLP_API_BEGIN try {
#define QMLP_API_END \
    return 0;        \
    }                \
    catch (...) { return handleException(); }

Tensor wrap(const qmlp_tensor* t)
{
    if (!t || t->ndim <= 0) return {};
    bool empty = false;
    for (int i = 0; i < t->ndim && i < 4; ++i) empty = empty || t->sizes[i] == 0;
    if (t->data == nullptr && !empty) return {};   // a null pointer is only a tensor if it has no entries
    if (t->ndim > 4) throw std::runtime_error("tensors with more than 4 dimensions are not supported");
    if (t->precision < 0 || t->precision > QMLP_DOUBLE) throw std::runtime_error("unknown tensor precision");
    std::vector<int32_t> sizes(t->sizes, t->sizes + t->ndim), strides(t->strides, t->strides + t->ndim);
    return Tensor(t->data, static_cast<Tensor::Precision>(t->precision), sizes, strides);
}

void unwrap(const Tensor& t, qmlp_tensor* out)
{
    std::memset(out, 0, sizeof(*out));
    if (!t.defined()) return;
    out->data = const_cast<void*>(t.rawPtr());
    out->precision = static_cast<int32_t>(t.precision());
    out->ndim = t.ndim();
    for (int i = 0; i < t.ndim(); ++i) {
        out->sizes[i] = t.size(i);
        out->strides[i] = t.stride(i);
    }
}

char* dupString(const std::string& s)
{
    char* p = static_cast<char*>(std::malloc(s.size() + 1));
    std::memcpy(p, s.c_str(), s.size() + 1);
    return p;
}

Tensor::Usage usageOf(int usage)
{
    if (usage == QMLP_INFERENCE) return Tensor::INFERENCE;
    if (usage == QMLP_GRADIENTS) return Tensor::GRADIENTS;
    throw std::runtime_error("unknown usage");
}

std::optional<const Tensor> optionalTensor(const qmlp_tensor* t)
{
    Tensor w = wrap(t);
    if (!w.defined()) return {};
    return std::optional<const Tensor>(w);
}

EncodingHashGrid& asHashGrid(qmlp_encoding_t e)
{
    auto* g = dynamic_cast<EncodingHashGrid*>(e->encoding.get());
    if (!g) throw std::runtime_error("the encoding is not a HashGrid");
    return *g;
}

} // namespace

extern "C" {

const char* qmlp_last_error(void) { return g_error.c_str(); }
void qmlp_free_string(char* s) { std::free(s); }

int qmlp_is_gpu_available(int* available)
{
    QMLP_API_BEGIN
    *available = QuickMLP::Instance().isHipAvailable() ? 1 : 0;
    QMLP_API_END
}

int qmlp_set_log_level(const char* level_name)
{
    QMLP_API_BEGIN
    QuickMLP::Instance().setLogLevel(std::string(level_name));
    QMLP_API_END
}

int qmlp_set_compile_debug_mode(int enable)
{
    QMLP_API_BEGIN
    QuickMLP::Instance().setCompileDebugMode(enable != 0);
    QMLP_API_END
}

int qmlp_is_compile_debug_mode(int* enabled)
{
    QMLP_API_BEGIN
    *enabled = QuickMLP::Instance().isCompileDebugMode() ? 1 : 0;
    QMLP_API_END
}

int qmlp_set_kernel_cache_dir(const char* directory)
{
    QMLP_API_BEGIN
    auto kl = QuickMLP::Instance().kernelLoader();
    if (!directory || !*directory) kl->disableCache();
    else kl->setCacheDir(directory);
    QMLP_API_END
}

int qmlp_kernel_cache_stats(int* compilations, int* disk_hits)
{
    QMLP_API_BEGIN
    auto kl = QuickMLP::Instance().kernelLoader();
    if (compilations) *compilations = kl->numCompilations();
    if (disk_hits) *disk_hits = kl->numDiskHits();
    QMLP_API_END
}

int qmlp_kernel_compiler_stats(int* has_offline_compiler, int* offline_compilations)
{
    QMLP_API_BEGIN
    auto kl = QuickMLP::Instance().kernelLoader();
    if (has_offline_compiler) *has_offline_compiler = KernelLoader::hasOfflineCompiler() ? 1 : 0;
    if (offline_compilations) *offline_compilations = kl->numOfflineCompilations();
    QMLP_API_END
}

// ---------------------------------------------------------------- network

int qmlp_network_create(const char* cfg_json, const char* parent_directory, qmlp_network_t* network)
{
    QMLP_API_BEGIN
    *network = nullptr;
    json cfg = json::parse(cfg_json);
    auto n = std::make_unique<qmlp_network_s>();
    n->network = std::make_shared<FusedNetwork>(cfg, parent_directory ? parent_directory : ".");
    for (int i = 0; i < n->network->numEncodings(); ++i) {
        n->encodings.push_back(std::make_unique<qmlp_encoding_s>());
        n->encodings.back()->encoding = n->network->encoding(i);
    }
    *network = n.release();
    QMLP_API_END
}

int qmlp_network_destroy(qmlp_network_t network)
{
    QMLP_API_BEGIN
    delete network;
    QMLP_API_END
}

#define QMLP_NETWORK_GETTER(fn, expr)             \
    int fn(qmlp_network_t network, int* value)    \
    {                                             \
        QMLP_API_BEGIN                            \
        *value = (expr);                          \
        QMLP_API_END                              \
    }
QMLP_NETWORK_GETTER(qmlp_network_channels_in, network->network->channelsIn())
QMLP_NETWORK_GETTER(qmlp_network_channels_out, network->network->channelsOut())
QMLP_NETWORK_GETTER(qmlp_network_num_layers, network->network->numLayers())
QMLP_NETWORK_GETTER(qmlp_network_num_encodings, network->network->numEncodings())
QMLP_NETWORK_GETTER(qmlp_network_parameter_count, network->network->networkParameterCount())
QMLP_NETWORK_GETTER(qmlp_network_is_parallel_streams, network->network->isParallelStreams() ? 1 : 0)

int qmlp_network_encoding(qmlp_network_t network, int index, qmlp_encoding_t* encoding)
{
    QMLP_API_BEGIN
    if (index < 0 || index >= static_cast<int>(network->encodings.size()))
        throw std::runtime_error("Array index out of bounds");
    *encoding = network->encodings[index].get();
    QMLP_API_END
}

int qmlp_network_parameter_precision(qmlp_network_t network, int usage, int* precision)
{
    QMLP_API_BEGIN
    *precision = static_cast<int>(network->network->networkParameterPrecision(usageOf(usage)));
    QMLP_API_END
}

int qmlp_network_matrix_size(int* value)
{
    *value = FusedNetwork::MATRIX_SIZE;
    return 0;
}

int qmlp_network_warp_size(int* value)
{
    *value = FusedNetwork::WARP_SIZE;
    return 0;
}

int qmlp_network_max_shared_memory_bytes(int* value)
{
    QMLP_API_BEGIN
    *value = FusedNetwork::MaxSharedMemoryBytes();
    QMLP_API_END
}

int qmlp_network_set_parallel_streams(qmlp_network_t network, int enabled)
{
    QMLP_API_BEGIN
    network->network->setParallelStreams(enabled != 0);
    QMLP_API_END
}

int qmlp_network_set_parameter(qmlp_network_t network, const qmlp_tensor* tensor, int usage)
{
    QMLP_API_BEGIN
    network->network->setNetworkParameter(wrap(tensor), usageOf(usage));
    QMLP_API_END
}

int qmlp_network_initialize_inference_parameters(qmlp_network_t network, uint32_t seed)
{
    QMLP_API_BEGIN
    std::default_random_engine rng(seed);
    network->network->initializeInferenceParameters(rng);
    QMLP_API_END
}

int qmlp_network_parameter_view(qmlp_network_t network, int layer, int bias, void* raw_pointer, int precision,
                                qmlp_tensor* view)
{
    QMLP_API_BEGIN
    if (precision != QMLP_FLOAT && precision != QMLP_HALF) throw std::runtime_error("precision must be float or half");
    Tensor t = network->network->networkParameter(layer, bias != 0, raw_pointer, static_cast<Tensor::Precision>(precision));
    unwrap(t, view);
    QMLP_API_END
}

int qmlp_network_inference(qmlp_network_t network, const qmlp_tensor* input, const qmlp_tensor* output, void* stream)
{
    QMLP_API_BEGIN
    Tensor out = wrap(output);
    network->network->inference(wrap(input), out, static_cast<stream_t>(stream));
    QMLP_API_END
}

int qmlp_network_inference_noalloc(qmlp_network_t network, const qmlp_tensor* input, const qmlp_tensor* output, void* stream)
{
    QMLP_API_BEGIN
    Tensor out = wrap(output);
    network->network->inferenceNoAlloc(wrap(input), out, static_cast<stream_t>(stream));
    QMLP_API_END
}

int qmlp_network_forward_memory(qmlp_network_t network, int num_elements, int adjoint_flags, size_t* bytes)
{
    QMLP_API_BEGIN
    *bytes = network->network->forwardMemory(num_elements, adjoint_flags);
    QMLP_API_END
}

int qmlp_network_forward(qmlp_network_t network, const qmlp_tensor* input, const qmlp_tensor* output,
                         void* tmp_memory, void* stream)
{
    QMLP_API_BEGIN
    Tensor out = wrap(output);
    network->network->forward(wrap(input), out, tmp_memory, static_cast<stream_t>(stream));
    QMLP_API_END
}

int qmlp_network_zero_gradients(qmlp_network_t network)
{
    QMLP_API_BEGIN
    network->network->zeroGradients();
    QMLP_API_END
}

int qmlp_network_adjoint_memory(qmlp_network_t network, int num_elements, int adjoint_flags, size_t* bytes)
{
    QMLP_API_BEGIN
    *bytes = network->network->adjointMemory(num_elements, adjoint_flags);
    QMLP_API_END
}

int qmlp_network_adjoint(qmlp_network_t network, const qmlp_tensor* input, const qmlp_tensor* adj_output,
                         int adjoint_flags, const qmlp_tensor* adj_input, const void* tmp_memory_forward,
                         void* tmp_memory_adjoint, void* stream)
{
    QMLP_API_BEGIN
    Tensor adjIn = wrap(adj_input);
    network->network->adjoint(wrap(input), wrap(adj_output), adjoint_flags, adjIn, tmp_memory_forward,
                              tmp_memory_adjoint, static_cast<stream_t>(stream));
    QMLP_API_END
}

int qmlp_network_clear_cached_kernels(qmlp_network_t network)
{
    QMLP_API_BEGIN
    network->network->clearCachedKernels();
    QMLP_API_END
}

int qmlp_network_precompile(qmlp_network_t network, int adjoint_flags)
{
    QMLP_API_BEGIN
    network->network->precompile(adjoint_flags);
    QMLP_API_END
}

int qmlp_network_prepare(qmlp_network_t network, int numel, int adjoint_flags)
{
    QMLP_API_BEGIN
    network->network->prepare(numel, adjoint_flags);
    QMLP_API_END
}

int qmlp_network_generated_source(qmlp_network_t network, const char* kind, int adjoint_flags, char** source)
{
    QMLP_API_BEGIN
    *source = dupString(network->network->generatedSource(kind, adjoint_flags));
    QMLP_API_END
}

// ---------------------------------------------------------------- encodings

int qmlp_encoding_create(const char* cfg_json, qmlp_encoding_t* encoding)
{
    QMLP_API_BEGIN
    *encoding = nullptr;
    json cfg = json::parse(cfg_json);
    auto e = std::make_unique<qmlp_encoding_s>();
    e->encoding = EncodingFactory::Instance().create(cfg);
    *encoding = e.release();
    QMLP_API_END
}

int qmlp_encoding_destroy(qmlp_encoding_t encoding)
{
    QMLP_API_BEGIN
    delete encoding;
    QMLP_API_END
}

int qmlp_encoding_to_json(qmlp_encoding_t encoding, char** out)
{
    QMLP_API_BEGIN
    *out = dupString(encoding->encoding->toJson().dump());
    QMLP_API_END
}

int qmlp_encoding_id(qmlp_encoding_t encoding, char** id)
{
    QMLP_API_BEGIN
    *id = dupString(encoding->encoding->id());
    QMLP_API_END
}

#define QMLP_ENCODING_GETTER(fn, expr)              \
    int fn(qmlp_encoding_t encoding, int* value)    \
    {                                               \
        QMLP_API_BEGIN                              \
        *value = (expr);                            \
        QMLP_API_END                                \
    }
QMLP_ENCODING_GETTER(qmlp_encoding_max_input_channel, encoding->encoding->maxInputChannel())
QMLP_ENCODING_GETTER(qmlp_encoding_num_output_channels, encoding->encoding->numOutputChannels())
QMLP_ENCODING_GETTER(qmlp_encoding_has_parameters, encoding->encoding->hasParameters() ? 1 : 0)
QMLP_ENCODING_GETTER(qmlp_encoding_parameter_count, encoding->encoding->parameterCount())

int qmlp_encoding_parameter_precision(qmlp_encoding_t encoding, int usage, int* precision)
{
    QMLP_API_BEGIN
    *precision = static_cast<int>(encoding->encoding->parameterPrecision(usageOf(usage)));
    QMLP_API_END
}

int qmlp_encoding_set_parameter(qmlp_encoding_t encoding, const qmlp_tensor* tensor, int usage)
{
    QMLP_API_BEGIN
    encoding->encoding->setParameter(wrap(tensor), usageOf(usage));
    QMLP_API_END
}

int qmlp_encoding_zero_gradients(qmlp_encoding_t encoding)
{
    QMLP_API_BEGIN
    encoding->encoding->zeroGradients();
    QMLP_API_END
}

int qmlp_encoding_forward(qmlp_encoding_t encoding, const qmlp_tensor* input, const qmlp_tensor* output,
                          void* stream, const qmlp_tensor* parameters_forward)
{
    QMLP_API_BEGIN
    Tensor out = wrap(output);
    encoding->encoding->forward(wrap(input), out, static_cast<stream_t>(stream), optionalTensor(parameters_forward));
    QMLP_API_END
}

int qmlp_encoding_adjoint(qmlp_encoding_t encoding, const qmlp_tensor* input, const qmlp_tensor* adj_output,
                          const qmlp_tensor* adj_input, void* stream, const qmlp_tensor* parameters_forward,
                          const qmlp_tensor* parameters_gradients, int adjoint_mode)
{
    QMLP_API_BEGIN
    Tensor adjIn = wrap(adj_input);
    encoding->encoding->adjoint(wrap(input), wrap(adj_output), adjIn, static_cast<stream_t>(stream),
                                optionalTensor(parameters_forward), optionalTensor(parameters_gradients),
                                adjoint_mode);
    QMLP_API_END
}

int qmlp_encoding_hashgrid_levels(qmlp_encoding_t encoding, int capacity, int* num_levels, int* memory_offset,
                                  int* resolution, int* hash_grid_size, int* hashed)
{
    QMLP_API_BEGIN
    const auto& g = asHashGrid(encoding);
    const auto& levels = g.levels();
    *num_levels = static_cast<int>(levels.size());
    for (int l = 0; l < std::min<int>(capacity, static_cast<int>(levels.size())); ++l) {
        if (memory_offset) memory_offset[l] = levels[l].memoryOffset;
        if (resolution) resolution[l] = levels[l].resolution;
        if (hash_grid_size) hash_grid_size[l] = levels[l].hashGridSize;
        if (hashed) hashed[l] = levels[l].hashed ? 1 : 0;
    }
    QMLP_API_END
}

int qmlp_encoding_precompile(qmlp_encoding_t encoding, int adjoint_mode)
{
    QMLP_API_BEGIN
    encoding->encoding->precompile(adjoint_mode);
    QMLP_API_END
}

int qmlp_encoding_hashgrid_corners(qmlp_encoding_t encoding, const qmlp_tensor* input, uint32_t* indices,
                                   float* weights, void* stream)
{
    QMLP_API_BEGIN
    asHashGrid(encoding).corners(wrap(input), indices, weights, static_cast<stream_t>(stream));
    QMLP_API_END
}

int qmlp_encoding_hashgrid_trace(qmlp_encoding_t encoding, const qmlp_tensor* input, int mode, uint32_t* indices,
                                 float* weights, void* stream)
{
    QMLP_API_BEGIN
    if (input == nullptr)
        asHashGrid(encoding).precompileCorners(mode, true);
    else
        asHashGrid(encoding).corners(wrap(input), indices, weights, static_cast<stream_t>(stream), mode);
    QMLP_API_END
}

// ---------------------------------------------------------------- activations

int qmlp_activation_create(const char* key_or_json, qmlp_activation_t* activation)
{
    QMLP_API_BEGIN
    *activation = nullptr;
    ActivationFactory factory(QuickMLP::Instance().kernelLoader());
    auto a = std::make_unique<qmlp_activation_s>();
    a->activation = factory.getOrInline(key_or_json);
    *activation = a.release();
    QMLP_API_END
}

int qmlp_activation_destroy(qmlp_activation_t activation)
{
    QMLP_API_BEGIN
    delete activation;
    QMLP_API_END
}

int qmlp_activation_to_json(qmlp_activation_t activation, char** out)
{
    QMLP_API_BEGIN
    *out = dupString(activation->activation->toJson().dump());
    QMLP_API_END
}

int qmlp_activation_forward(qmlp_activation_t activation, const qmlp_tensor* input, const qmlp_tensor* output,
                            void* stream)
{
    QMLP_API_BEGIN
    Tensor out = wrap(output);
    activation->activation->forward(wrap(input), out, static_cast<stream_t>(stream));
    QMLP_API_END
}

int qmlp_activation_adjoint(qmlp_activation_t activation, const qmlp_tensor* input, const qmlp_tensor* adj_output,
                            const qmlp_tensor* adj_input, void* stream)
{
    QMLP_API_BEGIN
    Tensor adjIn = wrap(adj_input);
    activation->activation->adjoint(wrap(input), wrap(adj_output), adjIn, static_cast<stream_t>(stream));
    QMLP_API_END
}

int qmlp_activation_precompile(qmlp_activation_t activation)
{
    QMLP_API_BEGIN
    activation->activation->precompile();
    QMLP_API_END
}

int qmlp_utils_pullpush_forward(const qmlp_tensor* mask, const qmlp_tensor* data, const qmlp_tensor* output,
                                void* stream)
{
    QMLP_API_BEGIN
    Tensor out = wrap(output);
    Utils::fractionalPullpush(wrap(mask), wrap(data), out, static_cast<stream_t>(stream));
    QMLP_API_END
}

int qmlp_utils_pullpush_adjoint(const qmlp_tensor* mask, const qmlp_tensor* data, const qmlp_tensor* adj_output,
                                const qmlp_tensor* adj_mask, const qmlp_tensor* adj_data, void* stream)
{
    QMLP_API_BEGIN
    Tensor adjMask = wrap(adj_mask), adjData = wrap(adj_data);
    Utils::adjointFractionalPullpush(wrap(mask), wrap(data), wrap(adj_output), adjMask, adjData,
                                     static_cast<stream_t>(stream));
    QMLP_API_END
}

int qmlp_utils_pullpush_precompile(int precision)
{
    QMLP_API_BEGIN
    if (precision != QMLP_FLOAT && precision != QMLP_DOUBLE) throw std::runtime_error("precision must be float or double");
    Utils::precompile(static_cast<Tensor::Precision>(precision));
    QMLP_API_END
}

} // extern "C"
