#pragma once

#include "common.h"
#include "json.h"
#include "kernel_loader.h"
#include "tensor.h"

#include <filesystem>
#include <optional>
#include <string>
#include <unordered_map>

QUICKMLP_NAMESPACE_BEGIN

/**
 * Defines an activation function by two code snippets acting point-wise:
 *
 * Forward function (inference): input <code>half x</code>, output <code>half z</code>,
 *   e.g. ReLU: <code>z = __hgt(x, hZERO()) ? x : hZERO()</code>
 * Adjoint function (training): input <code>half x, adjz</code>, output <code>half adjx</code>,
 *   e.g. ReLU: <code>adjx = __hgt(x, hZERO()) ? adjz : hZERO()</code>
 *
 * The snippets are device code and may use the half intrinsics of hip_fp16.h.
 */
class Activation
{
    const std::string id_;
    const std::string forward_;
    const std::string adjoint_;
    const std::string code_;

public:
    Activation(const std::string& id, const std::string& forward, const std::string& adjoint);
    explicit Activation(const json& cfg);

    [[nodiscard]] json toJson() const;
    [[nodiscard]] const std::string& id() const { return id_; }
    [[nodiscard]] const std::string& forward() const { return forward_; }
    [[nodiscard]] const std::string& adjoint() const { return adjoint_; }

    /**
     * The device code of this activation:
     * <code>struct {id()} { static half forward(half x); static half adjoint(half x, half adjz); };</code>
     */
    [[nodiscard]] std::string code() const { return code_; }

    /**
     * Standalone forward pass through the activation function (half precision).
     * \param input shape (B, C), \param output shape (B, C)
     */
    void forward(const Tensor& input, Tensor& output, stream_t stream);

    /**
     * Standalone adjoint pass. All tensors of shape (B, C), half precision.
     */
    void adjoint(const Tensor& input, const Tensor& adjOutput, Tensor& adjInput, stream_t stream);

    /** Compiles the two standalone kernels into the kernel cache; needs no GPU. */
    void precompile();

private:
    std::optional<KernelFunction> forwardKernel_;
    std::optional<KernelFunction> adjointKernel_;
};
typedef std::shared_ptr<Activation> Activation_ptr;

/**
 * Loader for activations from Json specifications
 */
class ActivationFactory
{
public:
    /**
     * Loads the activations from an activation specification tag: an array of file
     * names (each file holds an array of activation specifications) and/or inline
     * objects {"id","forward","adjoint"}.
     *
     * Search order for files: direct (relative to the working directory or absolute),
     * relative to 'parent', then the built-in files of the kernel loader.
     */
    ActivationFactory(const json& cfg, const std::filesystem::path& parent, KernelLoader_ptr loader);

    /** Loads the built-in activations only */
    explicit ActivationFactory(KernelLoader_ptr loader);

    /** Returns the activation with the given identifier; throws if unknown. */
    [[nodiscard]] Activation_ptr get(const std::string& key) const;

    /**
     * Like get(), but a key starting with '{' is parsed as an inline activation
     * definition with the tags 'id', 'forward' and 'adjoint'.
     */
    [[nodiscard]] Activation_ptr getOrInline(const std::string& key);

private:
    void parseFile(const std::filesystem::path& file);
    void parseFile(const json& j);
    Activation_ptr parseActivation(const json& cfg, bool emplace);

    std::unordered_map<std::string, Activation_ptr> activations_;
};
typedef std::shared_ptr<ActivationFactory> ActivationFactory_ptr;

QUICKMLP_NAMESPACE_END
