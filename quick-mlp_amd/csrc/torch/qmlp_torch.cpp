// torch custom classes torch.classes.qmlp_cu.{QuickMLP, Activation, Encoding, Network, utils}
// with the names, arguments and pickling of the reference's binding
// (src_cpp/pytorch-bindings/src/bindings.cpp:102-122, bind_activation.cpp:80-98,
// bind_encoding.cpp:165-197, bind_network.cpp:346-411, bind_utils.cpp:68-87), written on the C ABI
// of libqmlp.so (include/qmlp_capi.h): torch provides tensors, the current stream and autograd,
// every computation is a call through that ABI. Scripted / traced modules that hold these
// classes can be saved and loaded like with the reference.
#include <torch/custom_class.h>
#include <torch/script.h>
#include <c10/hip/HIPStream.h>

#include "qmlp_capi.h"

#include <mutex>
#include <string>
#include <tuple>
#include <vector>

namespace {

#define QMLP_CHECK(call) TORCH_CHECK((call) == 0, qmlp_last_error())

qmlp_tensor wrap(const torch::Tensor& t)
{
    qmlp_tensor d{};
    if (!t.defined()) return d;
    TORCH_CHECK(t.is_cuda(), "QuickMLP tensors must live on the GPU");
    TORCH_CHECK(t.dim() >= 1 && t.dim() <= 4, "tensors must have 1 to 4 dimensions");
    switch (t.scalar_type()) {
        case torch::kFloat32: d.precision = QMLP_FLOAT; break;
        case torch::kFloat16: d.precision = QMLP_HALF; break;
        case torch::kFloat64: d.precision = QMLP_DOUBLE; break;
        default: TORCH_CHECK(false, "unsupported dtype ", t.scalar_type());
    }
    d.data = t.data_ptr();
    d.ndim = static_cast<int32_t>(t.dim());
    for (int i = 0; i < d.ndim; ++i) {
        d.sizes[i] = static_cast<int32_t>(t.size(i));
        d.strides[i] = static_cast<int32_t>(t.stride(i));
    }
    return d;
}

void* currentStream() { return c10::hip::getCurrentHIPStream().stream(); }

torch::ScalarType dtypeOf(int precision)
{
    return precision == QMLP_HALF ? torch::kFloat16 : precision == QMLP_DOUBLE ? torch::kFloat64 : torch::kFloat32;
}

std::string takeString(char* s)
{
    std::string r = s ? s : "";
    qmlp_free_string(s);
    return r;
}

torch::Tensor createOutput(const torch::Tensor& input, int channels)
{
    TORCH_CHECK(input.dim() == 2, "input must be a tensor with 2 dimensions (batch, channels)");
    return torch::empty({input.size(0), channels}, input.options());
}

// ------------------------------------------------------------------------------------- QuickMLP
struct QuickMLPBindings : torch::CustomClassHolder
{
    static void setCompileDebugMode(bool enable) { QMLP_CHECK(qmlp_set_compile_debug_mode(enable ? 1 : 0)); }
    static bool isCompileDebugMode()
    {
        int v = 0;
        QMLP_CHECK(qmlp_is_compile_debug_mode(&v));
        return v != 0;
    }
    static void setLogLevel(const std::string& level) { QMLP_CHECK(qmlp_set_log_level(level.c_str())); }
    static bool isCudaAvailable()
    {
        int v = 0;
        QMLP_CHECK(qmlp_is_gpu_available(&v));
        return v != 0;
    }
};

// ------------------------------------------------------------------------------------- Activation
struct ActivationBindings;
using ActivationBindings_ptr = c10::intrusive_ptr<ActivationBindings>;

struct ActivationBindings : torch::CustomClassHolder
{
    std::string cfg_;
    qmlp_activation_t handle_ = nullptr;

    explicit ActivationBindings(std::string cfg) : cfg_(std::move(cfg)) { QMLP_CHECK(qmlp_activation_create(cfg_.c_str(), &handle_)); }
    ~ActivationBindings() override
    {
        if (handle_) qmlp_activation_destroy(handle_);
    }
    std::string cfg() const { return cfg_; }

    torch::Tensor inference(const torch::Tensor& input)
    {
        auto output = torch::empty_like(input);
        const qmlp_tensor in = wrap(input), out = wrap(output);
        QMLP_CHECK(qmlp_activation_forward(handle_, &in, &out, currentStream()));
        return output;
    }
    torch::Tensor adjoint(const torch::Tensor& input, const torch::Tensor& adjOutput)
    {
        auto adjInput = torch::empty_like(input);
        const qmlp_tensor in = wrap(input), adjOut = wrap(adjOutput), adjIn = wrap(adjInput);
        QMLP_CHECK(qmlp_activation_adjoint(handle_, &in, &adjOut, &adjIn, currentStream()));
        return adjInput;
    }
    static torch::Tensor forward(const ActivationBindings_ptr& self, const torch::Tensor& input);
};

struct ActivationFunction : torch::autograd::Function<ActivationFunction>
{
    static torch::Tensor forward(torch::autograd::AutogradContext* ctx, const torch::Tensor& input,
                                 const ActivationBindings_ptr& activ)
    {
        ctx->save_for_backward({input});
        ctx->saved_data["activ"] = activ;
        return activ->inference(input);
    }
    static torch::autograd::tensor_list backward(torch::autograd::AutogradContext* ctx, torch::autograd::tensor_list gradOutputs)
    {
        auto activ = ctx->saved_data["activ"].toCustomClass<ActivationBindings>();
        return {activ->adjoint(ctx->get_saved_variables()[0], gradOutputs[0].contiguous()), torch::Tensor()};
    }
};

torch::Tensor ActivationBindings::forward(const ActivationBindings_ptr& self, const torch::Tensor& input)
{
    return ActivationFunction::apply(input, self);
}

// ------------------------------------------------------------------------------------- Encoding
struct NetworkBindings;
struct EncodingBindings;
using EncodingBindings_ptr = c10::intrusive_ptr<EncodingBindings>;

struct EncodingBindings : torch::CustomClassHolder
{
    std::string cfg_;
    qmlp_encoding_t handle_ = nullptr;
    c10::intrusive_ptr<torch::CustomClassHolder> owner_;   // the network a borrowed handle belongs to

    explicit EncodingBindings(std::string cfg) : cfg_(std::move(cfg)) { QMLP_CHECK(qmlp_encoding_create(cfg_.c_str(), &handle_)); }
    EncodingBindings(qmlp_encoding_t borrowed, c10::intrusive_ptr<torch::CustomClassHolder> owner)
        : handle_(borrowed), owner_(std::move(owner))
    {
        cfg_ = toJson();
    }
    ~EncodingBindings() override
    {
        if (handle_ && !owner_) qmlp_encoding_destroy(handle_);
    }

    std::string cfg() const { return cfg_; }
    std::string toJson() const
    {
        char* s = nullptr;
        QMLP_CHECK(qmlp_encoding_to_json(handle_, &s));
        return takeString(s);
    }
    int64_t getInt(int (*fn)(qmlp_encoding_t, int*)) const
    {
        int v = 0;
        QMLP_CHECK(fn(handle_, &v));
        return v;
    }
    int64_t maxInputChannel() const { return getInt(qmlp_encoding_max_input_channel); }
    int64_t numOutputChannels() const { return getInt(qmlp_encoding_num_output_channels); }
    bool hasParameters() const { return getInt(qmlp_encoding_has_parameters) != 0; }
    int64_t parameterCount() const { return getInt(qmlp_encoding_parameter_count); }
    torch::ScalarType parameterDtype(bool gradients) const
    {
        int p = 0;
        QMLP_CHECK(qmlp_encoding_parameter_precision(handle_, gradients ? QMLP_GRADIENTS : QMLP_INFERENCE, &p));
        return dtypeOf(p);
    }
    torch::Tensor createParameters(bool gradients) const
    {
        TORCH_CHECK(hasParameters(), "the encoding has no parameters");
        return torch::empty({parameterCount()}, torch::TensorOptions().dtype(parameterDtype(gradients)).device(torch::kCUDA));
    }
    torch::Tensor createInferenceParameters() { return createParameters(false); }
    torch::Tensor createGradientParameters() { return createParameters(true); }

    torch::Tensor inference(const torch::Tensor& input)
    {
        TORCH_CHECK(!hasParameters(), "Encoding has parameters, call the variation of 'inference' with parameters");
        auto output = createOutput(input, static_cast<int>(numOutputChannels()));
        const qmlp_tensor in = wrap(input), out = wrap(output);
        QMLP_CHECK(qmlp_encoding_forward(handle_, &in, &out, currentStream(), nullptr));
        return output;
    }
    torch::Tensor inferenceWithParameter(const torch::Tensor& input, const torch::Tensor& parameter)
    {
        TORCH_CHECK(hasParameters(), "Encoding doesn't have parameters, call the variation of 'inference' without parameters");
        auto output = createOutput(input, static_cast<int>(numOutputChannels()));
        const qmlp_tensor in = wrap(input), out = wrap(output), par = wrap(parameter);
        QMLP_CHECK(qmlp_encoding_forward(handle_, &in, &out, currentStream(), &par));
        return output;
    }
    torch::Tensor adjoint(const torch::Tensor& input, const torch::Tensor& adjOutput)
    {
        TORCH_CHECK(!hasParameters(), "Encoding has parameters, call the variation of 'adjoint' with parameters");
        auto adjInput = torch::zeros_like(input);
        const qmlp_tensor in = wrap(input), adjOut = wrap(adjOutput), adjIn = wrap(adjInput);
        QMLP_CHECK(qmlp_encoding_adjoint(handle_, &in, &adjOut, &adjIn, currentStream(), nullptr, nullptr,
                                         QMLP_ENCODING_INPUT_GRADIENTS | QMLP_ENCODING_PARAM_GRADIENTS));
        return adjInput;
    }
    std::tuple<torch::Tensor, torch::Tensor> adjointWithParameterAndFlags(const torch::Tensor& input, const torch::Tensor& parameter,
                                                                          const torch::Tensor& adjOutput, int64_t flags)
    {
        TORCH_CHECK(hasParameters(), "Encoding doesn't have parameters, call the variation of 'adjoint' without parameters");
        auto adjInput = torch::zeros_like(input);
        auto adjParameter = torch::zeros(parameter.sizes(), parameter.options().dtype(parameterDtype(true)));
        const qmlp_tensor in = wrap(input), adjOut = wrap(adjOutput), adjIn = wrap(adjInput), par = wrap(parameter),
                          adjPar = wrap(adjParameter);
        QMLP_CHECK(qmlp_encoding_adjoint(handle_, &in, &adjOut, &adjIn, currentStream(), &par, &adjPar, static_cast<int>(flags)));
        return {adjInput, adjParameter.to(parameter.scalar_type())};
    }
    std::tuple<torch::Tensor, torch::Tensor> adjointWithParameter(const torch::Tensor& input, const torch::Tensor& parameter,
                                                                  const torch::Tensor& adjOutput)
    {
        return adjointWithParameterAndFlags(input, parameter, adjOutput,
                                            QMLP_ENCODING_INPUT_GRADIENTS | QMLP_ENCODING_PARAM_GRADIENTS);
    }
    static torch::Tensor forward(const EncodingBindings_ptr& self, const torch::Tensor& input);
    static torch::Tensor forwardWithParameter(const EncodingBindings_ptr& self, const torch::Tensor& input,
                                              const torch::Tensor& parameter);
};

struct EncodingFunction : torch::autograd::Function<EncodingFunction>
{
    static torch::Tensor forward(torch::autograd::AutogradContext* ctx, const torch::Tensor& input, const EncodingBindings_ptr& enc)
    {
        ctx->save_for_backward({input});
        ctx->saved_data["enc"] = enc;
        return enc->inference(input);
    }
    static torch::autograd::tensor_list backward(torch::autograd::AutogradContext* ctx, torch::autograd::tensor_list gradOutputs)
    {
        auto enc = ctx->saved_data["enc"].toCustomClass<EncodingBindings>();
        return {enc->adjoint(ctx->get_saved_variables()[0], gradOutputs[0].contiguous()), torch::Tensor()};
    }
};

struct EncodingFunctionWithParameter : torch::autograd::Function<EncodingFunctionWithParameter>
{
    static torch::Tensor forward(torch::autograd::AutogradContext* ctx, const torch::Tensor& input, const torch::Tensor& parameter,
                                 const EncodingBindings_ptr& enc)
    {
        ctx->save_for_backward({input, parameter});
        ctx->saved_data["enc"] = enc;
        ctx->saved_data["flags"] = static_cast<int64_t>((input.requires_grad() ? QMLP_ENCODING_INPUT_GRADIENTS : 0)
                                                        | (parameter.requires_grad() ? QMLP_ENCODING_PARAM_GRADIENTS : 0));
        return enc->inferenceWithParameter(input, parameter);
    }
    static torch::autograd::tensor_list backward(torch::autograd::AutogradContext* ctx, torch::autograd::tensor_list gradOutputs)
    {
        const int64_t flags = ctx->saved_data["flags"].toInt();
        if (flags == 0) return {torch::Tensor(), torch::Tensor(), torch::Tensor()};
        auto enc = ctx->saved_data["enc"].toCustomClass<EncodingBindings>();
        const auto saved = ctx->get_saved_variables();
        auto grads = enc->adjointWithParameterAndFlags(saved[0], saved[1], gradOutputs[0].contiguous(), flags);
        return {(flags & QMLP_ENCODING_INPUT_GRADIENTS) ? std::get<0>(grads) : torch::Tensor(),
                (flags & QMLP_ENCODING_PARAM_GRADIENTS) ? std::get<1>(grads) : torch::Tensor(), torch::Tensor()};
    }
};

torch::Tensor EncodingBindings::forward(const EncodingBindings_ptr& self, const torch::Tensor& input)
{
    TORCH_CHECK(!self->hasParameters(), "Encoding has parameters, call the variation of 'forward' with parameters");
    return EncodingFunction::apply(input, self);
}
torch::Tensor EncodingBindings::forwardWithParameter(const EncodingBindings_ptr& self, const torch::Tensor& input,
                                                     const torch::Tensor& parameter)
{
    TORCH_CHECK(self->hasParameters(), "Encoding doesn't have parameters, call the variation of 'forward' without parameters");
    return EncodingFunctionWithParameter::apply(input, parameter, self);
}

// ------------------------------------------------------------------------------------- Network
struct NetworkBindings;
using NetworkBindings_ptr = c10::intrusive_ptr<NetworkBindings>;

struct NetworkBindings : torch::CustomClassHolder
{
    std::string cfg_, parent_;
    qmlp_network_t handle_ = nullptr;
    std::mutex mutex_;   // the native object keeps the current parameter tensors: one call at a time (bind_network.h:20)

    NetworkBindings(std::string cfg, std::string parent) : cfg_(std::move(cfg)), parent_(std::move(parent))
    {
        QMLP_CHECK(qmlp_network_create(cfg_.c_str(), parent_.c_str(), &handle_));
    }
    ~NetworkBindings() override
    {
        if (handle_) qmlp_network_destroy(handle_);
    }
    std::string cfg() const { return cfg_; }
    std::string parent() const { return parent_; }

    static int64_t staticInt(int (*fn)(int*))
    {
        int v = 0;
        QMLP_CHECK(fn(&v));
        return v;
    }
    static int64_t MatrixSize() { return staticInt(qmlp_network_matrix_size); }
    static int64_t WarpSize() { return staticInt(qmlp_network_warp_size); }
    static int64_t MaxSharedMemoryBytes() { return staticInt(qmlp_network_max_shared_memory_bytes); }

    int64_t getInt(int (*fn)(qmlp_network_t, int*)) const
    {
        int v = 0;
        QMLP_CHECK(fn(handle_, &v));
        return v;
    }
    int64_t numEncodings() const { return getInt(qmlp_network_num_encodings); }
    int64_t channelsIn() const { return getInt(qmlp_network_channels_in); }
    int64_t channelsOut() const { return getInt(qmlp_network_channels_out); }
    int64_t numLayers() const { return getInt(qmlp_network_num_layers); }
    int64_t networkParameterCount() const { return getInt(qmlp_network_parameter_count); }
    bool isParallelStreams() const { return getInt(qmlp_network_is_parallel_streams) != 0; }
    void setParallelStreams(bool enabled) { QMLP_CHECK(qmlp_network_set_parallel_streams(handle_, enabled ? 1 : 0)); }

    qmlp_encoding_t encodingHandle(int64_t index) const
    {
        qmlp_encoding_t e = nullptr;
        QMLP_CHECK(qmlp_network_encoding(handle_, static_cast<int>(index), &e));
        return e;
    }
    bool encodingHasParameters(int64_t index) const
    {
        int v = 0;
        QMLP_CHECK(qmlp_encoding_has_parameters(encodingHandle(index), &v));
        return v != 0;
    }
    static EncodingBindings_ptr encoding(const NetworkBindings_ptr& self, int64_t index)
    {
        return c10::make_intrusive<EncodingBindings>(self->encodingHandle(index), self);
    }

    torch::Tensor createInferenceParameters() const
    {
        return torch::empty({networkParameterCount()}, torch::TensorOptions().dtype(torch::kFloat16).device(torch::kCUDA));
    }
    void initializeInferenceParameters(torch::Tensor dst)
    {
        std::lock_guard<std::mutex> lock(mutex_);
        const qmlp_tensor d = wrap(dst);
        QMLP_CHECK(qmlp_network_set_parameter(handle_, &d, QMLP_INFERENCE));
        const auto seed = static_cast<uint32_t>(torch::randint(0x7fffffff, {1}, torch::kInt64).item<int64_t>());
        QMLP_CHECK(qmlp_network_initialize_inference_parameters(handle_, seed));
    }
    torch::Tensor view(int64_t layer, bool bias, torch::Tensor parameters)
    {
        TORCH_CHECK(parameters.scalar_type() == torch::kFloat32 || parameters.scalar_type() == torch::kFloat16,
                    "parameters must be float or half");
        TORCH_CHECK(parameters.dim() == 1 && parameters.size(0) == networkParameterCount(),
                    "The tensor must be of shape (num_parameters, )");
        qmlp_tensor v{};
        QMLP_CHECK(qmlp_network_parameter_view(handle_, static_cast<int>(layer), bias ? 1 : 0, parameters.data_ptr(),
                                               parameters.scalar_type() == torch::kFloat32 ? QMLP_FLOAT : QMLP_HALF, &v));
        if (v.ndim == 0) return torch::Tensor();
        const int64_t offset = (static_cast<char*>(v.data) - static_cast<char*>(parameters.data_ptr())) / parameters.element_size();
        std::vector<int64_t> sizes(v.sizes, v.sizes + v.ndim), strides(v.strides, v.strides + v.ndim);
        return parameters.as_strided(sizes, strides, parameters.storage_offset() + offset);
    }

    /** Binds the inference parameters of the network and its encodings (mutex held by the caller). */
    void bindParameters(const torch::Tensor& networkParameters, const std::vector<torch::Tensor>& encodingParameters)
    {
        const qmlp_tensor p = wrap(networkParameters);
        QMLP_CHECK(qmlp_network_set_parameter(handle_, &p, QMLP_INFERENCE));
        const int64_t n = std::min<int64_t>(numEncodings(), static_cast<int64_t>(encodingParameters.size()));
        for (int64_t i = 0; i < n; ++i) {
            if (!encodingParameters[i].defined() || !encodingHasParameters(i)) continue;
            const qmlp_tensor e = wrap(encodingParameters[i]);
            QMLP_CHECK(qmlp_encoding_set_parameter(encodingHandle(i), &e, QMLP_INFERENCE));
        }
    }

    torch::Tensor inference(const torch::Tensor& input, const torch::Tensor& networkParameters,
                            const std::vector<torch::Tensor>& encodingParameters)
    {
        auto output = createOutput(input, static_cast<int>(channelsOut()));
        const auto p16 = networkParameters.scalar_type() == torch::kFloat16 ? networkParameters : networkParameters.to(torch::kFloat16);
        std::lock_guard<std::mutex> lock(mutex_);
        bindParameters(p16, encodingParameters);
        const qmlp_tensor in = wrap(input), out = wrap(output);
        QMLP_CHECK(qmlp_network_inference(handle_, &in, &out, currentStream()));
        return output;
    }
    static torch::Tensor forward(const NetworkBindings_ptr& self, const torch::Tensor& input, const torch::Tensor& networkParameters,
                                 const std::vector<torch::Tensor>& encodingParameters);
};

/** Differentiable fused forward pass; the inputs are (input, network parameters, one tensor per encoding). */
struct NetworkFunction : torch::autograd::Function<NetworkFunction>
{
    static torch::Tensor forward(torch::autograd::AutogradContext* ctx, const NetworkBindings_ptr& net, int64_t flags,
                                 const torch::Tensor& input, const torch::Tensor& networkParameters,
                                 at::TensorList encodingParameterList)
    {
        const std::vector<torch::Tensor> encodingParameters = encodingParameterList.vec();
        const auto p16 = networkParameters.scalar_type() == torch::kFloat16 ? networkParameters : networkParameters.to(torch::kFloat16);
        size_t bytes = 0;
        QMLP_CHECK(qmlp_network_forward_memory(net->handle_, static_cast<int>(input.size(0)), static_cast<int>(flags), &bytes));
        auto tmpForward = torch::empty({static_cast<int64_t>(std::max<size_t>(bytes, 16))},
                                       torch::TensorOptions().dtype(torch::kUInt8).device(input.device()));
        auto output = createOutput(input, static_cast<int>(net->channelsOut()));
        {
            std::lock_guard<std::mutex> lock(net->mutex_);
            net->bindParameters(p16, encodingParameters);
            const qmlp_tensor in = wrap(input), out = wrap(output);
            QMLP_CHECK(qmlp_network_forward(net->handle_, &in, &out, tmpForward.data_ptr(), currentStream()));
        }
        torch::autograd::variable_list saved = {input, p16, tmpForward};
        saved.insert(saved.end(), encodingParameters.begin(), encodingParameters.end());
        ctx->save_for_backward(saved);
        ctx->saved_data["net"] = net;
        ctx->saved_data["flags"] = flags;
        ctx->saved_data["param_dtype"] = static_cast<int64_t>(networkParameters.scalar_type());
        std::vector<int64_t> needs;
        for (const auto& t : encodingParameters) needs.push_back(t.defined() && t.requires_grad() ? 1 : 0);
        ctx->saved_data["enc_needs_grad"] = c10::IValue(needs);
        return output;
    }

    static torch::autograd::variable_list backward(torch::autograd::AutogradContext* ctx, torch::autograd::variable_list gradOutputs)
    {
        auto net = ctx->saved_data["net"].toCustomClass<NetworkBindings>();
        const int flags = static_cast<int>(ctx->saved_data["flags"].toInt());
        const auto paramDtype = static_cast<torch::ScalarType>(ctx->saved_data["param_dtype"].toInt());
        const auto needs = ctx->saved_data["enc_needs_grad"].toIntVector();
        const auto saved = ctx->get_saved_variables();
        const torch::Tensor& input = saved[0];
        const torch::Tensor& p16 = saved[1];
        const torch::Tensor& tmpForward = saved[2];
        const std::vector<torch::Tensor> encodingParameters(saved.begin() + 3, saved.end());
        const auto gradOutput = gradOutputs[0].contiguous();

        torch::Tensor adjInput, adjNetwork;
        std::vector<torch::Tensor> adjEncodings(encodingParameters.size());
        if (flags & QMLP_GRADIENTS_INPUT) adjInput = torch::zeros_like(input);
        {
            std::lock_guard<std::mutex> lock(net->mutex_);
            net->bindParameters(p16, encodingParameters);
            if (flags & QMLP_GRADIENTS_NETWORK_WEIGHTS) {
                adjNetwork = torch::zeros(p16.sizes(), p16.options().dtype(torch::kFloat32));
                const qmlp_tensor g = wrap(adjNetwork);
                QMLP_CHECK(qmlp_network_set_parameter(net->handle_, &g, QMLP_GRADIENTS));
            }
            if (flags & QMLP_GRADIENTS_INPUT_ENCODINGS) {
                for (size_t i = 0; i < encodingParameters.size(); ++i) {
                    // the kernel adds the gradients of every encoding with parameters: a frozen one gets a
                    // zero tensor as well, which is dropped afterwards (bind_network.cpp:277-290)
                    if (!net->encodingHasParameters(static_cast<int64_t>(i))) continue;
                    int precision = QMLP_FLOAT;
                    QMLP_CHECK(qmlp_encoding_parameter_precision(net->encodingHandle(static_cast<int64_t>(i)), QMLP_GRADIENTS, &precision));
                    adjEncodings[i] = torch::zeros(encodingParameters[i].sizes(), encodingParameters[i].options().dtype(dtypeOf(precision)));
                    const qmlp_tensor g = wrap(adjEncodings[i]);
                    QMLP_CHECK(qmlp_encoding_set_parameter(net->encodingHandle(static_cast<int64_t>(i)), &g, QMLP_GRADIENTS));
                }
            }
            size_t bytes = 0;
            QMLP_CHECK(qmlp_network_adjoint_memory(net->handle_, static_cast<int>(input.size(0)), flags, &bytes));
            auto tmpAdjoint = torch::empty({static_cast<int64_t>(std::max<size_t>(bytes, 16))},
                                           torch::TensorOptions().dtype(torch::kUInt8).device(input.device()));
            const qmlp_tensor in = wrap(input), adjOut = wrap(gradOutput), adjIn = wrap(adjInput);
            const int rc = qmlp_network_adjoint(net->handle_, &in, &adjOut, flags, &adjIn, tmpForward.data_ptr(),
                                                tmpAdjoint.data_ptr(), currentStream());
            // no dangling gradient bindings, whatever happened
            qmlp_network_set_parameter(net->handle_, nullptr, QMLP_GRADIENTS);
            for (size_t i = 0; i < adjEncodings.size(); ++i)
                if (adjEncodings[i].defined())
                    qmlp_encoding_set_parameter(net->encodingHandle(static_cast<int64_t>(i)), nullptr, QMLP_GRADIENTS);
            QMLP_CHECK(rc);
        }
        if (adjNetwork.defined()) adjNetwork = adjNetwork.to(paramDtype);
        torch::autograd::variable_list grads = {torch::Tensor(), torch::Tensor(), adjInput, adjNetwork};
        for (size_t i = 0; i < adjEncodings.size(); ++i)
            grads.push_back(adjEncodings[i].defined() && needs[i] ? adjEncodings[i].to(encodingParameters[i].scalar_type())
                                                                   : torch::Tensor());
        return grads;
    }
};

torch::Tensor NetworkBindings::forward(const NetworkBindings_ptr& self, const torch::Tensor& input,
                                       const torch::Tensor& networkParameters, const std::vector<torch::Tensor>& encodingParameters)
{
    int64_t flags = 0;
    if (input.requires_grad()) flags |= QMLP_GRADIENTS_INPUT;
    if (networkParameters.requires_grad()) flags |= QMLP_GRADIENTS_NETWORK_WEIGHTS;
    const int64_t numEncodings = self->numEncodings();
    for (int64_t i = 0; i < std::min<int64_t>(numEncodings, static_cast<int64_t>(encodingParameters.size())); ++i)
        if (encodingParameters[i].defined() && encodingParameters[i].requires_grad() && self->encodingHasParameters(i))
            flags |= QMLP_GRADIENTS_INPUT_ENCODINGS;
    if (flags == 0 || !torch::GradMode::is_enabled()) return self->inference(input, networkParameters, encodingParameters);
    // encodings without parameters get a placeholder so that the positions line up
    torch::autograd::variable_list filled;
    for (int64_t i = 0; i < numEncodings; ++i) {
        const bool given = i < static_cast<int64_t>(encodingParameters.size()) && encodingParameters[i].defined();
        if (given && self->encodingHasParameters(i)) filled.push_back(encodingParameters[i]);
        else filled.push_back(torch::zeros({1}, input.options()));
    }
    return NetworkFunction::apply(self, flags, input, networkParameters, at::TensorList(filled));
}

// ------------------------------------------------------------------------------------- utils
struct UtilsBindings : torch::CustomClassHolder
{
    static torch::Tensor pullpushForward(const torch::Tensor& mask, const torch::Tensor& data)
    {
        auto output = torch::empty_like(data);
        const qmlp_tensor m = wrap(mask), d = wrap(data), o = wrap(output);
        QMLP_CHECK(qmlp_utils_pullpush_forward(&m, &d, &o, currentStream()));
        return output;
    }
    static std::tuple<torch::Tensor, torch::Tensor> pullpushAdjoint(const torch::Tensor& mask, const torch::Tensor& data,
                                                                    const torch::Tensor& adjOutput)
    {
        auto gradMask = torch::zeros_like(mask);
        auto gradData = torch::zeros_like(data);
        const qmlp_tensor m = wrap(mask), d = wrap(data), a = wrap(adjOutput), gm = wrap(gradMask), gd = wrap(gradData);
        QMLP_CHECK(qmlp_utils_pullpush_adjoint(&m, &d, &a, &gm, &gd, currentStream()));
        return {gradMask, gradData};
    }
    static torch::Tensor pullpush(const torch::Tensor& mask, const torch::Tensor& data);
};

struct PushPullFunction : torch::autograd::Function<PushPullFunction>
{
    static torch::Tensor forward(torch::autograd::AutogradContext* ctx, const torch::Tensor& mask, const torch::Tensor& data)
    {
        ctx->save_for_backward({mask, data});
        return UtilsBindings::pullpushForward(mask, data);
    }
    static torch::autograd::tensor_list backward(torch::autograd::AutogradContext* ctx, torch::autograd::tensor_list gradOutputs)
    {
        const auto saved = ctx->get_saved_variables();
        auto grads = UtilsBindings::pullpushAdjoint(saved[0], saved[1], gradOutputs[0].contiguous());
        return {std::get<0>(grads), std::get<1>(grads)};
    }
};

torch::Tensor UtilsBindings::pullpush(const torch::Tensor& mask, const torch::Tensor& data) { return PushPullFunction::apply(mask, data); }

} // namespace

TORCH_LIBRARY(qmlp_cu, m)
{
    m.class_<QuickMLPBindings>("QuickMLP")
        .def_static("set_compile_debug_mode", &QuickMLPBindings::setCompileDebugMode)
        .def_static("is_compile_debug_mode", &QuickMLPBindings::isCompileDebugMode)
        .def_static("set_log_level", &QuickMLPBindings::setLogLevel)
        .def_static("is_cuda_available", &QuickMLPBindings::isCudaAvailable);

    m.class_<ActivationBindings>("Activation")
        .def(torch::init<std::string>())
        .def("cfg", &ActivationBindings::cfg)
        .def("inference", &ActivationBindings::inference)
        .def("adjoint", &ActivationBindings::adjoint)
        .def("forward", [](const ActivationBindings_ptr& self, const torch::Tensor& input) { return ActivationBindings::forward(self, input); })
        .def_pickle([](const ActivationBindings_ptr& self) -> std::string { return self->cfg(); },
                    [](std::string state) -> ActivationBindings_ptr { return c10::make_intrusive<ActivationBindings>(std::move(state)); });

    m.class_<EncodingBindings>("Encoding")
        .def(torch::init<std::string>())
        .def("cfg", &EncodingBindings::cfg)
        .def("max_input_channel", &EncodingBindings::maxInputChannel)
        .def("num_output_channels", &EncodingBindings::numOutputChannels)
        .def("has_parameters", &EncodingBindings::hasParameters)
        .def("to_json", &EncodingBindings::toJson)
        .def("create_inference_parameters", &EncodingBindings::createInferenceParameters)
        .def("create_gradient_parameters", &EncodingBindings::createGradientParameters)
        .def("inference", &EncodingBindings::inference)
        .def("adjoint", &EncodingBindings::adjoint)
        .def("inference_with_parameter", &EncodingBindings::inferenceWithParameter)
        .def("adjoint_with_parameter", &EncodingBindings::adjointWithParameter)
        .def("forward", [](const EncodingBindings_ptr& self, const torch::Tensor& input) { return EncodingBindings::forward(self, input); })
        .def("forward_with_parameter", [](const EncodingBindings_ptr& self, const torch::Tensor& input, const torch::Tensor& parameter) {
            return EncodingBindings::forwardWithParameter(self, input, parameter);
        })
        .def_pickle([](const EncodingBindings_ptr& self) -> std::string { return self->cfg(); },
                    [](std::string state) -> EncodingBindings_ptr { return c10::make_intrusive<EncodingBindings>(std::move(state)); });

    m.class_<NetworkBindings>("Network")
        .def(torch::init<std::string, std::string>(), "", {torch::arg("cfg"), torch::arg("parent") = "."})
        .def("cfg", &NetworkBindings::cfg)
        .def("parent", &NetworkBindings::parent)
        .def_static("MatrixSize", &NetworkBindings::MatrixSize)
        .def_static("WarpSize", &NetworkBindings::WarpSize)
        .def_static("MaxSharedMemoryBytes", &NetworkBindings::MaxSharedMemoryBytes)
        .def("is_parallel_streams", &NetworkBindings::isParallelStreams)
        .def("set_parallel_streams", &NetworkBindings::setParallelStreams)
        .def("num_encodings", &NetworkBindings::numEncodings)
        .def("encoding", [](const NetworkBindings_ptr& self, int64_t index) { return NetworkBindings::encoding(self, index); })
        .def("channels_in", &NetworkBindings::channelsIn)
        .def("channels_out", &NetworkBindings::channelsOut)
        .def("num_layers", &NetworkBindings::numLayers)
        .def("num_network_parameters", &NetworkBindings::networkParameterCount)
        .def("create_inference_parameters", &NetworkBindings::createInferenceParameters)
        .def("initialize_inference_parameters", &NetworkBindings::initializeInferenceParameters)
        .def("parameter_view", &NetworkBindings::view)
        .def("inference", &NetworkBindings::inference, "",
             {torch::arg("input"), torch::arg("network_parameters"), torch::arg("encoding_parameters") = std::vector<torch::Tensor>()})
        .def("forward",
             [](const NetworkBindings_ptr& self, const torch::Tensor& input, const torch::Tensor& networkParameters,
                const std::vector<torch::Tensor>& encodingParameters) {
                 return NetworkBindings::forward(self, input, networkParameters, encodingParameters);
             },
             "", {torch::arg("input"), torch::arg("network_parameters"), torch::arg("encoding_parameters") = std::vector<torch::Tensor>()})
        .def_pickle([](const NetworkBindings_ptr& self) -> std::vector<std::string> { return {self->cfg(), self->parent()}; },
                    [](std::vector<std::string> state) -> NetworkBindings_ptr {
                        TORCH_CHECK(state.size() == 2, "Corrupt state");
                        return c10::make_intrusive<NetworkBindings>(std::move(state[0]), std::move(state[1]));
                    });

    m.class_<UtilsBindings>("utils")
        .def_static("pullpush_forward", &UtilsBindings::pullpushForward)
        .def_static("pullpush_backward", &UtilsBindings::pullpushAdjoint)
        .def_static("pullpush", &UtilsBindings::pullpush);
}
