#pragma once

#include "common.h"
#include "kernel_loader.h"
#include "logger.h"

#include <memory>
#include <string>

QUICKMLP_NAMESPACE_BEGIN

/**
 * The entry class into quick-mlp (singleton): logger, kernel loader, compile mode.
 */
class QuickMLP : public NonAssignable
{
private:
    static std::unique_ptr<QuickMLP> INSTANCE;

    const logger_t logger_;
    const KernelLoader_ptr kl_;
    bool enableCompileDebugMode_;

    QuickMLP();

public:
    /** Returns the global quick-mlp instance */
    static QuickMLP& Instance();

    /** Deletes the global quick-mlp instance */
    static void DeleteInstance();

    /**
     * Tests if a GPU is available. If this is false, all kernel launches fail with
     * an exception (kernels can still be generated and compiled).
     */
    [[nodiscard]] bool isHipAvailable() const;
    /** Same query under the name the reference API uses. */
    [[nodiscard]] bool isCudaAvailable() const { return isHipAvailable(); }

    /** Tests if a GPU is available and if not, throws a hip_error. */
    void checkHipAvailable() const;
    void checkCudaAvailable() const { checkHipAvailable(); }

    /** Returns the logger instance used to report compile logs (debug) or errors */
    [[nodiscard]] logger_t getLogger() const;

    void setLogLevel(Logger::Level level);

    /**
     * Sets the log level by name: "off", "debug", "info", "warn", "error".
     * The kernel loader logs source code at debug, compilations at info, compile
     * errors at error.
     */
    void setLogLevel(const std::string& levelName);

    /** The kernel loader used to compile and load the generated kernels. */
    [[nodiscard]] KernelLoader_ptr kernelLoader() const;

    /**
     * Enable (true) or disable (false) debug compilation mode (debug info, reduced
     * optimization). Default: off.
     */
    void setCompileDebugMode(bool enable);
    [[nodiscard]] bool isCompileDebugMode() const { return enableCompileDebugMode_; }

    /** Returns the compile flags for the kernel loader. */
    [[nodiscard]] int getCompileFlags() const;

    /** Directory next to the library that holds the device sources. */
    [[nodiscard]] static std::filesystem::path LocateKernelDirectory();
};

QUICKMLP_NAMESPACE_END
